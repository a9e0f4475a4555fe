// Decode over the factored KV cache for gfx950: a few query tokens against a long cache, split
// over key ranges, built to be bound by HBM bandwidth.
//
// The cache is never expanded to per-head K/V.  With Qm[h, :] = (c / (Rq Rk)) sum_i qa[i, h] qb[i, :]
// the logits are  s[h, t] = sum_j a_k[t, j, h] * (Qm[h, :] . b_k[t, j, :])  and the output is
// o[h, :] = (1/Rk) sum_t sum_j (p[h, t] a_v[t, j, h]) b_v[t, j, :]  (the rank-shared products of
// the non-materialising form, tpa/tpa.py:333-359,398-413), so the rows b_k[(t, j), :] and
// b_v[(t, j), :] are plain row-major matrices that feed two skinny MFMA contractions with the
// heads as the N dimension.  Every cache byte is read from HBM exactly once for all heads.
//
// A workgroup has 4 independent waves; each streams its own range of 32-row blocks
// (32 / Rk tokens) with fully coalesced 16-byte loads that stay in flight in registers two
// blocks ahead, stages the block in its private LDS region (XOR-swizzled so that both the
// 16-byte operand reads and the transposed reads are bank-conflict free), and keeps a private
// online softmax (tpa/tpa.py:389-424).  The waves are merged through LDS, the key ranges
// through a workspace and a small second kernel, both with the rule of _lse_accum
// (tpa/tpa.py:228-242).
#include <mutex>
#include <type_traits>

#include "tpa_common.h"

namespace tpa {
namespace {

constexpr int kWaves = 4;
constexpr int kRowsPerBlock = 32;


struct DecodeParams {
  TpaFactor qa, qb, ka, kb, va, vb;
  float* part_o;  // [B, lq, S, H, D] fp32, unnormalised
  float* part_m;  // [B, lq, S, H] running max (log2 domain)
  float* part_l;  // [B, lq, S, H] sum of exp2
  const int32_t* kvlen;  // [B] keys per batch entry, or null (= lk)
  const int32_t* page_table;  // paged cache: [B, pages_per_seq] physical page of each logical page
  int page_size, pages_per_seq;  // tokens per page; table row length
  int B, lq, lk, H, rq;
  int climit;      // query row qi sees its first qi + climit keys (causal: offset + 1; otherwise lk, no limit)
  int cbr;         // causal, last query aligned with the last key of each batch entry: climit counts from len - lq_total
  int row0;        // this call serves query rows row0 .. row0 + lq - 1 of lq_total (outputs are indexed with them)
  int lq_total;
  int S;           // key ranges
  float qscale;    // sm_scale * log2(e) / (rq * rk)
};

template <int D>
struct DecodeLds {
  static constexpr int kB = kRowsPerBlock * D;       // elements of one B tile
  static constexpr int kA = kRowsPerBlock * 32;      // elements of one A tile (32 heads)
  static constexpr int kWave = 2 * kB + 2 * kA;      // elements per wave
  static constexpr int kRedStride = D + 4;           // fp32 row stride of the wave-merge staging (spreads the banks)
  static constexpr int kReduce = 32 * kRedStride * 2 + 128;  // fp32 O^T + m + l, in uint16 units
  static constexpr int kPerWave = kWave > kReduce ? kWave : kReduce;
  static constexpr size_t kBytes = (size_t)kWaves * kPerWave * sizeof(uint16_t);
  // with NQ > 1 query rows per workgroup: plus their Q fragments (NQ rows x D/16 steps x 64 lanes x 16 bytes)
  static constexpr size_t bytes(int nq) { return kBytes + (nq > 1 ? (size_t)nq * (D / 16) * 64 * 16 : 0); }
};

template <int D, int RK, bool PAGED, int NQ>
__global__ __launch_bounds__(kWaves * 64) void decode_kernel(DecodeParams p) {
  constexpr int CPR = D / 8;               // 16-byte chunks per B row
  constexpr int RPI = 64 / CPR;            // B rows per load instruction
  constexpr int NLB = kRowsPerBlock / RPI; // load instructions per B tile
  constexpr int NKS = D / 16;
  constexpr int NDB = D / 32;
  constexpr int NTOK = RK <= 4 ? 16 / RK : 32 / RK;  // tokens whose rows this lane holds, per block
  constexpr int NV = RK <= 4 ? RK : RK / 2;          // rows of one token held by this half of the wave
  static_assert(RK == 1 || RK == 2 || RK == 4 || RK == 8 || RK == 16 || RK == 32, "a block of 32 rows holds whole tokens");

  extern __shared__ __attribute__((aligned(16))) uint16_t smem[];

  const int S = p.S;
  // workgroup id -> (key range x, query row qi): ids are dealt to the 8 XCDs round-robin, and the
  // rows of one query token group read the same cache slice, so they get ids that are 8 apart
  // (same XCD, same L2) and next to each other in launch order (resident together)
  // A workgroup serves NQ query rows from one pass over its cache blocks (each staged block is
  // used NQ times); with an odd row count the last group's second row repeats the first and is
  // not stored.
  const int nqg = (p.lq + NQ - 1) / NQ;  // groups of NQ query rows
  const int gid = blockIdx.x, grp = gid / (8 * nqg), rem = gid - grp * 8 * nqg;
  const int qi0 = NQ * (rem >> 3), x = grp * 8 + (rem & 7);
  if (x >= p.B * S) return;  // the grid is rounded up to whole groups of 8 ranges
  const int b = x / S, split = x % S;
  const int h0 = blockIdx.y * 32;
  const int tid = threadIdx.x;
  const int w = tid >> 6, l = tid & 63, i = l & 31, g = l >> 5;
  const int hl = min(h0 + i, p.H - 1);  // this lane's head (clamped: lanes past H idle along)

  uint16_t* lds = smem + w * DecodeLds<D>::kPerWave;
  uint16_t* lds_bk = lds;
  uint16_t* lds_bv = lds + DecodeLds<D>::kB;
  uint16_t* lds_ak = lds + 2 * DecodeLds<D>::kB;
  uint16_t* lds_av = lds_ak + DecodeLds<D>::kA;

  // ---- Qm^T fragments (B operand of S'^T = B_k Qm^T): lane (h, g) holds Qm[h][16ks + 8g + 0..7].
  // Called after the first cache loads are in flight so that their latency is not exposed.
  // With one query row they stay in registers; with NQ rows wave r builds row r's fragments once
  // and parks them in LDS behind the waves' staging regions (fragment (r, ks) of lane l at
  // [(r NKS + ks) 64 + l]), from where every wave reads them as it needs them: the registers go to
  // the NQ accumulator sets instead.
  bf16x8 qf[NQ == 1 ? NKS : 1];
  u32x4* const lds_q = reinterpret_cast<u32x4*>(smem + kWaves * DecodeLds<D>::kPerWave);
  auto build_q = [&]() {
    const int qi = NQ == 1 ? qi0 : min(qi0 + w, p.lq - 1);
    const uint16_t* ap = static_cast<const uint16_t*>(p.qa.ptr) + b * p.qa.stride_b + (int64_t)qi * p.qa.stride_l + hl;
    const uint16_t* bp = static_cast<const uint16_t*>(p.qb.ptr) + b * p.qb.stride_b + (int64_t)qi * p.qb.stride_l + 8 * g;
    if constexpr (NQ == 1) {
      build_q_fragments<NKS, 6>(ap, p.qa.stride_r, bp, p.qb.stride_r, p.rq, p.qscale, qf);
    } else {
      if (w < NQ) {
        bf16x8 tmp[NKS];
        build_q_fragments<NKS, 6>(ap, p.qa.stride_r, bp, p.qb.stride_r, p.rq, p.qscale, tmp);
#pragma unroll
        for (int ks = 0; ks < NKS; ++ks) lds_q[(w * NKS + ks) * 64 + l] = __builtin_bit_cast(u32x4, tmp[ks]);
      }
      __syncthreads();
    }
  };

  // ---- this wave's blocks: part, part + nparts, part + 2 nparts, ... (dealt round robin, so the
  // waves of the grid, which advance in step, read neighbouring addresses at any one time)
  const int nparts = S * kWaves;
  const int part = split * kWaves + w;
  // keys of this batch entry that each query row sees, and the most any of them sees
  const int len_all = p.kvlen ? min(p.kvlen[b], p.lk) : p.lk;
  int row_last[NQ], len_b = 0;
#pragma unroll
  for (int r = 0; r < NQ; ++r) {
    const int len_r = max(0, min(len_all, min(qi0 + r, p.lq - 1) + p.climit + (p.cbr ? len_all - p.lq_total : 0)));
    row_last[r] = len_r * RK - 1;
    len_b = max(len_b, len_r);
  }
  const int blk_begin = part;
  const int blk_end = (len_b * RK + kRowsPerBlock - 1) / kRowsPerBlock;  // 32-row blocks of its cache
  const int blk_step = nparts;
  const int last_row = len_b * RK - 1;

  // rows of the cache matrices: row = token * RK + rank, row stride = stride_r
  // (paged cache: the arrays are page pools, stride_b = elements between pages, and a block of 32
  // rows lies inside one page, which the page table of this batch entry locates)
  const int64_t boff = PAGED ? 0 : b;
  const uint16_t* kb_base = static_cast<const uint16_t*>(p.kb.ptr) + boff * p.kb.stride_b;
  const uint16_t* vb_base = static_cast<const uint16_t*>(p.vb.ptr) + boff * p.vb.stride_b;
  const uint16_t* ka_base = static_cast<const uint16_t*>(p.ka.ptr) + boff * p.ka.stride_b + h0;
  const uint16_t* va_base = static_cast<const uint16_t*>(p.va.ptr) + boff * p.va.stride_b + h0;
  const int rpp = PAGED ? p.page_size * RK : 1;  // rows per page
  const int a_chunks = min(4, (p.H - h0) / 8);  // valid 16-byte chunks of an A row in this head block

  // loader lane roles
  const int lb_row = l / CPR, lb_c = l % CPR;             // B tiles: row within the instruction, chunk
  const int la_row = l >> 2, la_c = min(l & 3, a_chunks - 1);  // A tiles: 16 rows per instruction

  // two register sets: while one block is staged and consumed, two more are in flight (one set
  // with NQ rows, whose accumulators take the room and whose blocks take NQ times as long to
  // consume).  The cache is read exactly once per call, so the loads are marked non-temporal
  // (measured on the whole call: 5.1 -> 5.75 TB/s)
  constexpr int NSETS = NQ == 1 ? 2 : 1;
  u32x4 rbk[NSETS][NLB], rbv[NSETS][NLB], rak[NSETS][2], rav[NSETS][2];
  // Paged cache: the page a block lies in is looked up one visit of its register set ahead (when the set's
  // previous block is requested), so that no request waits for a page-table entry
  int32_t page_ahead[NSETS] = {};
  auto lookup = [&](int blk) __attribute__((always_inline)) -> int32_t {
    return PAGED && blk < blk_end ? p.page_table[(int64_t)b * p.pages_per_seq + blk * kRowsPerBlock / rpp] : 0;
  };
  // One row group per cache slice: each byte is used once and the loads are marked non-temporal.  Several
  // (more query rows than a workgroup serves): the groups' workgroups run side by side on one XCD and the
  // later one is meant to find the slice in its L2, so the loads stay ordinary (four rows at the c4 shape:
  // 1022 MB fetched with non-temporal loads, 676 MB = the cache once with ordinary ones).
  auto load16 = [&](const uint16_t* ptr, auto nt_c) __attribute__((always_inline)) -> u32x4 {
    if constexpr (decltype(nt_c)::value) return __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(ptr));
    else return *reinterpret_cast<const u32x4*>(ptr);
  };
  auto issue_as = [&](auto set_c, int blk, auto nt_c) __attribute__((always_inline)) {
    constexpr int set = decltype(set_c)::value;
    const int row0 = blk * kRowsPerBlock;
    // element offsets that take a logical row of this block to its place in the page pool
    int64_t pkb = 0, pvb = 0, pka = 0, pva = 0;
    if constexpr (PAGED) {
      const int page = row0 / rpp;
      const int64_t phys = page_ahead[set];
      page_ahead[set] = lookup(blk + NSETS * blk_step);
      const int64_t first = (int64_t)page * rpp;  // first logical row of the page
      pkb = phys * p.kb.stride_b - first * p.kb.stride_r;
      pvb = phys * p.vb.stride_b - first * p.vb.stride_r;
      pka = phys * p.ka.stride_b - first * p.ka.stride_r;
      pva = phys * p.va.stride_b - first * p.va.stride_r;
    }
#pragma unroll
    for (int n = 0; n < NLB; ++n) {
      const int row = min(row0 + n * RPI + lb_row, last_row);
      rbk[set][n] = load16(kb_base + pkb + (int64_t)row * p.kb.stride_r + 8 * lb_c, nt_c);
      rbv[set][n] = load16(vb_base + pvb + (int64_t)row * p.vb.stride_r + 8 * lb_c, nt_c);
    }
#pragma unroll
    for (int n = 0; n < 2; ++n) {
      const int row = min(row0 + 16 * n + la_row, last_row);
      rak[set][n] = load16(ka_base + pka + (int64_t)row * p.ka.stride_r + 8 * la_c, nt_c);
      rav[set][n] = load16(va_base + pva + (int64_t)row * p.va.stride_r + 8 * la_c, nt_c);
    }
  };
  auto issue = [&](auto set_c, int blk) {
    if constexpr (NQ == 1) {
      issue_as(set_c, blk, std::true_type{});
    } else {
      if (nqg == 1) issue_as(set_c, blk, std::true_type{});
      else issue_as(set_c, blk, std::false_type{});
    }
  };
  auto stage = [&](auto set_c) {
    constexpr int set = decltype(set_c)::value;
#pragma unroll
    for (int n = 0; n < NLB; ++n) {
      const int row = n * RPI + lb_row;
      const int pos = lb_c ^ (row & (CPR - 1));
      *reinterpret_cast<u32x4*>(lds_bk + row * D + 8 * pos) = rbk[set][n];
      *reinterpret_cast<u32x4*>(lds_bv + row * D + 8 * pos) = rbv[set][n];
    }
#pragma unroll
    for (int n = 0; n < 2; ++n) {
      const int row = 16 * n + la_row;
      *reinterpret_cast<u32x4*>(lds_ak + row * 32 + 8 * (l & 3)) = rak[set][n];
      *reinterpret_cast<u32x4*>(lds_av + row * 32 + 8 * (l & 3)) = rav[set][n];
    }
  };

  f32x16 o[NQ][NDB];
  float m[NQ], lsum[NQ];
#pragma unroll
  for (int r = 0; r < NQ; ++r) {
#pragma unroll
    for (int db = 0; db < NDB; ++db)
#pragma unroll
      for (int v = 0; v < 16; ++v) o[r][db][v] = 0.f;
    m[r] = -INFINITY;
    lsum[r] = 0.f;
  }

  const int lp = l & 15, dhalf = (l >> 4) & 1;

  using Set0 = std::integral_constant<int, 0>;
  using Set1 = std::integral_constant<int, 1>;
  page_ahead[0] = lookup(blk_begin);
  if constexpr (NSETS == 2) page_ahead[1] = lookup(blk_begin + blk_step);
  if (blk_begin < blk_end) issue(Set0{}, blk_begin);
  if constexpr (NSETS == 2) {
    if (blk_begin + blk_step < blk_end) issue(Set1{}, blk_begin + blk_step);
  }
  build_q();

  auto compute = [&](int blk) {
    // ---- a_k / a_v of this lane's head for its 16 rows (rows 8q + 4g + 0..3, q = 0..3)
    float ak[16], av[16];
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const int arow = 8 * q + 4 * g + (lp >> 2);
      const s16x4 tk = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
          (s16x4 __attribute__((address_space(3)))*)(lds_ak + arow * 32 + 16 * dhalf + 4 * (lp & 3)));
      const s16x4 tv = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
          (s16x4 __attribute__((address_space(3)))*)(lds_av + arow * 32 + 16 * dhalf + 4 * (lp & 3)));
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        ak[4 * q + j] = bf16bits_to_f32((uint16_t)tk[j]);
        av[4 * q + j] = bf16bits_to_f32((uint16_t)tv[j]);
      }
    }
    const int row0 = blk * kRowsPerBlock;

#pragma unroll
    for (int r = 0; r < NQ; ++r) {
      // keep the rows' instruction streams apart: interleaved, their temporaries do not fit the registers
      if constexpr (NQ > 1) __builtin_amdgcn_sched_barrier(0);
      // ---- S'^T[row, h] = sum_d B_k[row, d] Qm[h, d]
      f32x16 sp;
#pragma unroll
      for (int v = 0; v < 16; ++v) sp[v] = 0.f;
#pragma unroll
      for (int ks = 0; ks < NKS; ++ks) {
        const int pos = (2 * ks + g) ^ (i & (CPR - 1));
        const bf16x8 kf = *reinterpret_cast<const bf16x8*>(lds_bk + i * D + 8 * pos);
        if constexpr (NQ == 1) {
          sp = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf, qf[ks], sp, 0, 0, 0);
        } else {
          const bf16x8 qv = __builtin_bit_cast(bf16x8, lds_q[(r * NKS + ks) * 64 + l]);
          sp = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf, qv, sp, 0, 0, 0);
        }
      }

      // ---- logits per token (log2 domain), masked past the keys this query row sees
      // (a token's RK rows are registers v0 .. v0 + NV - 1; from rank 8 on they span both halves of
      // the wave, which then hold the same tokens and exchange their partial sums)
      float st[NTOK];
      float tmax = -INFINITY;
#pragma unroll
      for (int t = 0; t < NTOK; ++t) {
        const int v0 = t * NV;
        float acc = 0.f;
#pragma unroll
        for (int j = 0; j < NV; ++j) acc += ak[v0 + j] * sp[v0 + j];
        if constexpr (RK >= 8) acc = halves_sum(acc);
        const int row = RK >= 8 ? row0 + RK * t : row0 + 8 * (v0 >> 2) + 4 * g + (v0 & 3);  // the token's first row
        if (row > row_last[r]) acc = -INFINITY;
        st[t] = acc;
        tmax = fmaxf(tmax, acc);
      }
      tmax = halves_max(tmax);
      // finite with one query row (row0 itself is always inside its keys); a row that sees fewer
      // keys than its neighbour can meet a block with none of its keys, before any or after all.
      // The reference is a whole number (the running maximum rounded up): 2^(s - m) then has the same
      // significand whatever m is, so the bf16 rounding of P' below does not depend on how the keys are
      // split over waves and ranges, and every rescaling factor (here, in the wave merge, in the merge of
      // the key ranges) is an exact power of two
      const float m_new = fmaxf(m[r], __builtin_ceilf(tmax));
      const float m_use = NQ > 1 && m_new == -INFINITY ? 0.f : m_new;
      if (__any(m_new > m[r])) {
        const float alpha = __builtin_amdgcn_exp2f(m[r] - m_use);
        lsum[r] *= alpha;
#pragma unroll
        for (int db = 0; db < NDB; ++db)
#pragma unroll
          for (int v = 0; v < 16; ++v) o[r][db][v] *= alpha;
        m[r] = m_new;
      }

      // ---- P'^T[row, h] = p[h, token(row)] * a_v[row, h], packed as the B operand of the PV product
      float pp[16];
#pragma unroll
      for (int t = 0; t < NTOK; ++t) {
        const float pt = __builtin_amdgcn_exp2f(st[t] - m_use);
        lsum[r] += RK >= 8 ? 0.5f * pt : pt;  // both halves hold the token: each adds half of it
#pragma unroll
        for (int j = 0; j < NV; ++j) pp[t * NV + j] = pt * av[t * NV + j];
      }
      bf16x8 pf[2];
#pragma unroll
      for (int kk = 0; kk < 2; ++kk) {
        u32x4 pk;
#pragma unroll
        for (int j = 0; j < 4; ++j) pk[j] = pack_bf16(pp[8 * kk + 2 * j], pp[8 * kk + 2 * j + 1]);
        pf[kk] = __builtin_bit_cast(bf16x8, pk);
      }

      // ---- O^T[d, h] += sum_row B_v[row, d] P'^T[row, h]; slot (g, j) = row 16kk + 8(j/4) + 4g + j%4
#pragma unroll
      for (int kk = 0; kk < 2; ++kk) {
        const int r_lo = 16 * kk + 4 * g + (lp >> 2);
        const int r_hi = r_lo + 8;
#pragma unroll
        for (int db = 0; db < NDB; ++db) {
          const int chunk = 4 * db + 2 * dhalf + ((lp & 3) >> 1);
          const int sub = 4 * (lp & 1);
          const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
              (s16x4 __attribute__((address_space(3)))*)(lds_bv + r_lo * D + 8 * (chunk ^ (r_lo & (CPR - 1))) + sub));
          const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
              (s16x4 __attribute__((address_space(3)))*)(lds_bv + r_hi * D + 8 * (chunk ^ (r_hi & (CPR - 1))) + sub));
          const bf16x8 vf = __builtin_bit_cast(bf16x8, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
          o[r][db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf, pf[kk], o[r][db], 0, 0, 0);
        }
      }
    }
  };

  if constexpr (NSETS == 2) {
    for (int blk = blk_begin; blk < blk_end; blk += 2 * blk_step) {
      stage(Set0{});  // waits for this block's loads only; its registers are then free again
      if (blk + 2 * blk_step < blk_end) issue(Set0{}, blk + 2 * blk_step);
      compute(blk);
      if (blk + blk_step < blk_end) {
        stage(Set1{});
        if (blk + 3 * blk_step < blk_end) issue(Set1{}, blk + 3 * blk_step);
        compute(blk + blk_step);
      }
    }
  } else {
    for (int blk = blk_begin; blk < blk_end; blk += blk_step) {
      stage(Set0{});
      if (blk + blk_step < blk_end) issue(Set0{}, blk + blk_step);
      compute(blk);
    }
  }

  // ---- merge the 4 waves through LDS (each wave reuses its own staging region), row by row
  constexpr int RS = DecodeLds<D>::kRedStride;
  float* red_o = reinterpret_cast<float*>(lds);  // [32 heads][RS]
  float* red_m = red_o + 32 * RS;
  float* red_l = red_m + 32;
  const int nh = min(32, p.H - h0);
#pragma unroll
  for (int r = 0; r < NQ; ++r) {
    if (qi0 + r >= p.lq) break;  // uniform: the repeated row of an odd count
    const float ltot = halves_sum(lsum[r]);
    __syncthreads();  // the staging (or the previous row's merge) has been read by every wave
#pragma unroll
    for (int db = 0; db < NDB; ++db)
#pragma unroll
      for (int vq = 0; vq < 4; ++vq)
        *reinterpret_cast<f32x4*>(red_o + i * RS + 32 * db + 8 * vq + 4 * g) =
            f32x4{o[r][db][4 * vq], o[r][db][4 * vq + 1], o[r][db][4 * vq + 2], o[r][db][4 * vq + 3]};
    if (g == 0) {
      red_m[i] = m[r];
      red_l[i] = ltot;
    }
    __syncthreads();

    const int64_t pbase = (((int64_t)b * p.lq + qi0 + r) * S + split) * p.H + h0;
    for (int idx = tid; idx < nh * D; idx += kWaves * 64) {
      const int hh = idx / D, d = idx % D;
      float mw[kWaves], mmax = -INFINITY;
#pragma unroll
      for (int ww = 0; ww < kWaves; ++ww) {
        mw[ww] = reinterpret_cast<const float*>(smem + ww * DecodeLds<D>::kPerWave)[32 * RS + hh];
        mmax = fmaxf(mmax, mw[ww]);
      }
      float acc = 0.f, lacc = 0.f;
#pragma unroll
      for (int ww = 0; ww < kWaves; ++ww) {
        const float* ro = reinterpret_cast<const float*>(smem + ww * DecodeLds<D>::kPerWave);
        const float f = mw[ww] == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(mw[ww] - mmax);
        acc += f * ro[hh * RS + d];
        lacc += f * ro[32 * RS + 32 + hh];
      }
      p.part_o[(pbase + hh) * D + d] = acc;
      if (d == 0) {
        p.part_m[pbase + hh] = mmax;
        p.part_l[pbase + hh] = lacc;
      }
    }
  }
}

// ---------------------------------------------------------------------------------------------
// The same decode for an fp32 cache (the reference's default dtype): fp32 MFMA contractions
// (v_mfma_f32_32x32x2_f32) on fp32 rows.  Same decomposition and the same workspace; what differs
// is the operand order a two-index fp32 step asks for: over d, wave half g takes d = 8m + 4g + e
// (one 16-byte LDS read feeds four steps); over the block's rows, half g takes the row its S'^T
// register belongs to, and the 32 rows of block db of O^T are d = (D/32) i + db, so one 16-byte
// read of B_v[row][(D/32) i ...] feeds every block.  One block of loads is in flight in registers
// (128 of them for D = 128) while the previous block is consumed; the head factors a_k, a_v are
// read straight into the registers of the logits they multiply.
template <int D>
struct DecodeF32Lds {
  static constexpr int RS = D + 4;                   // row stride (floats)
  static constexpr int kTile = kRowsPerBlock * RS;   // one B tile
  static constexpr int kPerWave = 2 * kTile;         // B_k and B_v; the wave merge reuses it (32 x RS + 64 floats)
  static constexpr size_t kBytes = (size_t)kWaves * kPerWave * sizeof(float);
};

template <int D, int RK, bool PAGED>
__global__ __launch_bounds__(kWaves * 64) void decode_f32_kernel(DecodeParams p) {
  constexpr int CPR = D / 4;               // 16-byte chunks per B row
  constexpr int RPI = 64 / CPR;            // B rows per load instruction
  constexpr int NLB = kRowsPerBlock / RPI; // load instructions per B tile
  constexpr int NDB = D / 32;
  constexpr int NTOK = RK <= 4 ? 16 / RK : 32 / RK;  // tokens whose rows this lane holds, per block
  constexpr int NV = RK <= 4 ? RK : RK / 2;          // rows of one token held by this half of the wave
  constexpr int RS = DecodeF32Lds<D>::RS;
  static_assert(RK == 1 || RK == 2 || RK == 4 || RK == 8 || RK == 16 || RK == 32, "a block of 32 rows holds whole tokens");
  typedef __attribute__((ext_vector_type(NDB))) float f32xN;

  extern __shared__ __attribute__((aligned(16))) float smem_dec_f32[];

  const int S = p.S;
  // workgroup id -> (key range x, query row qi): ids are dealt to the 8 XCDs round-robin, and the
  // rows of one query token group read the same cache slice, so they get ids that are 8 apart
  // (same XCD, same L2) and next to each other in launch order (resident together)
  const int gid = blockIdx.x, grp = gid / (8 * p.lq), rem = gid - grp * 8 * p.lq;
  const int qi = rem >> 3, x = grp * 8 + (rem & 7);
  if (x >= p.B * S) return;  // the grid is rounded up to whole groups of 8 ranges
  const int b = x / S, split = x % S;
  const int h0 = blockIdx.y * 32;
  const int tid = threadIdx.x;
  const int w = tid >> 6, l = tid & 63, i = l & 31, g = l >> 5;
  const int hl = min(h0 + i, p.H - 1);  // this lane's head (clamped: lanes past H idle along)

  float* const lds = smem_dec_f32 + w * DecodeF32Lds<D>::kPerWave;
  float* const lds_bk = lds;
  float* const lds_bv = lds + DecodeF32Lds<D>::kTile;

  const int nparts = S * kWaves;
  const int part = split * kWaves + w;
  const int len_all = p.kvlen ? min(p.kvlen[b], p.lk) : p.lk;
  const int len_b = max(0, min(len_all, qi + p.climit + (p.cbr ? len_all - p.lq_total : 0)));
  const int blk_begin = part;
  const int blk_end = (len_b * RK + kRowsPerBlock - 1) / kRowsPerBlock;
  const int blk_step = nparts;
  const int last_row = len_b * RK - 1;

  // (paged cache: the arrays are page pools, stride_b = elements between pages, and a block of 32
  // rows lies inside one page, which the page table of this batch entry locates)
  const int64_t boff = PAGED ? 0 : b;
  const float* const kb_base = static_cast<const float*>(p.kb.ptr) + boff * p.kb.stride_b;
  const float* const vb_base = static_cast<const float*>(p.vb.ptr) + boff * p.vb.stride_b;
  const float* const ka_base = static_cast<const float*>(p.ka.ptr) + boff * p.ka.stride_b + hl;
  const float* const va_base = static_cast<const float*>(p.va.ptr) + boff * p.va.stride_b + hl;
  const int rpp = PAGED ? p.page_size * RK : 1;  // rows per page
  const int lb_row = l / CPR, lb_c = l % CPR;

  // one register set: the block after the one being consumed
  f32x4 rbk[NLB], rbv[NLB];
  float rak[16], rav[16];
  // (paged cache: a block's page is looked up while the block before it is requested)
  auto lookup = [&](int blk) __attribute__((always_inline)) -> int32_t {
    return PAGED && blk < blk_end ? p.page_table[(int64_t)b * p.pages_per_seq + blk * kRowsPerBlock / rpp] : 0;
  };
  int32_t page_ahead = lookup(blk_begin);
  auto issue = [&](int blk) {
    const int row0 = blk * kRowsPerBlock;
    // element offsets that take a logical row of this block to its place in the page pool
    int64_t pkb = 0, pvb = 0, pka = 0, pva = 0;
    if constexpr (PAGED) {
      const int page = row0 / rpp;
      const int64_t phys = page_ahead;
      page_ahead = lookup(blk + blk_step);
      const int64_t first = (int64_t)page * rpp;  // first logical row of the page
      pkb = phys * p.kb.stride_b - first * p.kb.stride_r;
      pvb = phys * p.vb.stride_b - first * p.vb.stride_r;
      pka = phys * p.ka.stride_b - first * p.ka.stride_r;
      pva = phys * p.va.stride_b - first * p.va.stride_r;
    }
#pragma unroll
    for (int n = 0; n < NLB; ++n) {
      const int row = min(row0 + n * RPI + lb_row, last_row);
      rbk[n] = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(kb_base + pkb + (int64_t)row * p.kb.stride_r + 4 * lb_c));
      rbv[n] = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(vb_base + pvb + (int64_t)row * p.vb.stride_r + 4 * lb_c));
    }
    // a[row][head of this lane] for the 16 rows this lane's S'^T registers belong to
#pragma unroll
    for (int v = 0; v < 16; ++v) {
      const int row = min(row0 + 8 * (v >> 2) + 4 * g + (v & 3), last_row);
      rak[v] = ka_base[pka + (int64_t)row * p.ka.stride_r];
      rav[v] = va_base[pva + (int64_t)row * p.va.stride_r];
    }
  };
  float ak[16], av[16];
  auto stage = [&]() {
#pragma unroll
    for (int n = 0; n < NLB; ++n) {
      const int row = n * RPI + lb_row;
      *reinterpret_cast<f32x4*>(lds_bk + row * RS + 4 * lb_c) = rbk[n];
      *reinterpret_cast<f32x4*>(lds_bv + row * RS + 4 * lb_c) = rbv[n];
    }
#pragma unroll
    for (int v = 0; v < 16; ++v) { ak[v] = rak[v]; av[v] = rav[v]; }
  };

  if (blk_begin < blk_end) issue(blk_begin);

  // ---- Qm (B operand of S'^T = B_k Qm^T): qf[4m + e] = qscale * sum_r qa[r][h] qb[r][8m + 4g + e]
  float qf[D / 2];
#pragma unroll
  for (int j = 0; j < D / 2; ++j) qf[j] = 0.f;
  {
    const float* ap = static_cast<const float*>(p.qa.ptr) + b * p.qa.stride_b + (int64_t)qi * p.qa.stride_l + hl;
    const float* bp = static_cast<const float*>(p.qb.ptr) + b * p.qb.stride_b + (int64_t)qi * p.qb.stride_l + 4 * g;
    for (int r = 0; r < p.rq; ++r) {
      const float a = ap[r * p.qa.stride_r];
#pragma unroll
      for (int m = 0; m < D / 8; ++m) {
        const f32x4 bv = *reinterpret_cast<const f32x4*>(bp + r * p.qb.stride_r + 8 * m);
#pragma unroll
        for (int e = 0; e < 4; ++e) qf[4 * m + e] += a * bv[e];
      }
    }
#pragma unroll
    for (int j = 0; j < D / 2; ++j) qf[j] *= p.qscale;
  }

  f32x16 o[NDB];
#pragma unroll
  for (int db = 0; db < NDB; ++db)
#pragma unroll
    for (int v = 0; v < 16; ++v) o[db][v] = 0.f;
  float m = -INFINITY, lsum = 0.f;

  auto compute = [&](int blk) {
    // ---- S'^T[row, h] = sum_d B_k[row, d] Qm[h, d]; two accumulation chains, added at the end
    f32x16 sp, sp2;
#pragma unroll
    for (int v = 0; v < 16; ++v) { sp[v] = 0.f; sp2[v] = 0.f; }
#pragma unroll
    for (int mm = 0; mm < D / 8; ++mm) {
      const f32x4 kf = *reinterpret_cast<const f32x4*>(lds_bk + i * RS + 8 * mm + 4 * g);
      sp = __builtin_amdgcn_mfma_f32_32x32x2f32(kf[0], qf[4 * mm], sp, 0, 0, 0);
      sp2 = __builtin_amdgcn_mfma_f32_32x32x2f32(kf[1], qf[4 * mm + 1], sp2, 0, 0, 0);
      sp = __builtin_amdgcn_mfma_f32_32x32x2f32(kf[2], qf[4 * mm + 2], sp, 0, 0, 0);
      sp2 = __builtin_amdgcn_mfma_f32_32x32x2f32(kf[3], qf[4 * mm + 3], sp2, 0, 0, 0);
    }
#pragma unroll
    for (int v = 0; v < 16; ++v) sp[v] += sp2[v];

    // ---- logits per token (log2 domain), masked past the end of the cache
    // (a token's RK rows are registers v0 .. v0 + NV - 1; from rank 8 on they span both halves of
    // the wave, which then hold the same tokens and exchange their partial sums)
    float st[NTOK];
    float tmax = -INFINITY;
    const int row0 = blk * kRowsPerBlock;
#pragma unroll
    for (int t = 0; t < NTOK; ++t) {
      const int v0 = t * NV;
      float acc = 0.f;
#pragma unroll
      for (int j = 0; j < NV; ++j) acc += ak[v0 + j] * sp[v0 + j];
      if constexpr (RK >= 8) acc = halves_sum(acc);
      const int row = RK >= 8 ? row0 + RK * t : row0 + 8 * (v0 >> 2) + 4 * g + (v0 & 3);  // the token's first row
      if (row > last_row) acc = -INFINITY;
      st[t] = acc;
      tmax = fmaxf(tmax, acc);
    }
    tmax = halves_max(tmax);
    const float m_new = fmaxf(m, tmax);  // finite: row0 itself is always inside the cache
    if (__any(m_new > m)) {
      const float alpha = __builtin_amdgcn_exp2f(m - m_new);
      lsum *= alpha;
#pragma unroll
      for (int db = 0; db < NDB; ++db)
#pragma unroll
        for (int v = 0; v < 16; ++v) o[db][v] *= alpha;
      m = m_new;
    }

    // ---- P'^T[row, h] = p[h, token(row)] * a_v[row, h], in place of the logits' registers
    float pp[16];
#pragma unroll
    for (int t = 0; t < NTOK; ++t) {
      const float pt = __builtin_amdgcn_exp2f(st[t] - m);
      lsum += RK >= 8 ? 0.5f * pt : pt;  // both halves hold the token: each adds half of it
#pragma unroll
      for (int j = 0; j < NV; ++j) pp[t * NV + j] = pt * av[t * NV + j];
    }

    // ---- O^T[d, h] += sum_row B_v[row, d] P'^T[row, h]
#pragma unroll
    for (int v = 0; v < 16; ++v) {
      const int row = 8 * (v >> 2) + 4 * g + (v & 3);
      const f32xN vf = *reinterpret_cast<const f32xN*>(lds_bv + row * RS + NDB * i);
#pragma unroll
      for (int db = 0; db < NDB; ++db) o[db] = __builtin_amdgcn_mfma_f32_32x32x2f32(vf[db], pp[v], o[db], 0, 0, 0);
    }
  };

  for (int blk = blk_begin; blk < blk_end; blk += blk_step) {
    stage();  // waits for this block's loads; its registers are then free again
    if (blk + blk_step < blk_end) issue(blk + blk_step);
    compute(blk);
  }

  // ---- merge the 4 waves through LDS (each wave reuses its own staging region)
  const float ltot = halves_sum(lsum);
  float* red_o = lds;  // [32 heads][RS]: row 8 (v/4) + 4 g + v%4 of block db is d = NDB * row + db
  float* red_m = red_o + 32 * RS;
  float* red_l = red_m + 32;
#pragma unroll
  for (int v = 0; v < 16; ++v) {
    const int row = 8 * (v >> 2) + 4 * g + (v & 3);
    f32xN out;
#pragma unroll
    for (int db = 0; db < NDB; ++db) out[db] = o[db][v];
    *reinterpret_cast<f32xN*>(red_o + i * RS + NDB * row) = out;
  }
  if (g == 0) {
    red_m[i] = m;
    red_l[i] = ltot;
  }
  __syncthreads();

  const int nh = min(32, p.H - h0);
  const int64_t pbase = (((int64_t)b * p.lq + qi) * S + split) * p.H + h0;
  for (int idx = tid; idx < nh * D; idx += kWaves * 64) {
    const int hh = idx / D, d = idx % D;
    float mw[kWaves], mmax = -INFINITY;
#pragma unroll
    for (int ww = 0; ww < kWaves; ++ww) {
      mw[ww] = (smem_dec_f32 + ww * DecodeF32Lds<D>::kPerWave)[32 * RS + hh];
      mmax = fmaxf(mmax, mw[ww]);
    }
    float acc = 0.f, lacc = 0.f;
#pragma unroll
    for (int ww = 0; ww < kWaves; ++ww) {
      const float* ro = smem_dec_f32 + ww * DecodeF32Lds<D>::kPerWave;
      const float f = mw[ww] == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(mw[ww] - mmax);
      acc += f * ro[hh * RS + d];
      lacc += f * ro[32 * RS + 32 + hh];
    }
    p.part_o[(pbase + hh) * D + d] = acc;
    if (d == 0) {
      p.part_m[pbase + hh] = mmax;
      p.part_l[pbase + hh] = lacc;
    }
  }
}

// Merge the key ranges: o = sum_s f_s O_s / (Rk sum_s f_s l_s), f_s = 2^(m_s - max m); lse = ln of the total.
template <int D, typename TO>
__global__ __launch_bounds__(D) void decode_merge_kernel(const float* part_o, const float* part_m, const float* part_l,
                                                         TO* o, float* lse, int S, int H, int lq, float inv_rk, int row0, int lq_total) {
  const int bq = blockIdx.x;  // b * lq + qi
  const int h = blockIdx.y;
  const int d = threadIdx.x;
  // ranges are taken eight at a time with all their loads in flight together (one round trip
  // to memory for the usual S <= 8); a running (max, sum, acc) triple carries across groups
  float mmax = -INFINITY, acc = 0.f, lacc = 0.f;
  for (int s0 = 0; s0 < S; s0 += 8) {
    float ms[8], ls[8], os[8];
#pragma unroll
    for (int q = 0; q < 8; ++q) {
      const int s = min(s0 + q, S - 1);
      const int64_t idx = ((int64_t)bq * S + s) * H + h;
      ms[q] = s0 + q < S ? part_m[idx] : -INFINITY;
      ls[q] = part_l[idx];
      os[q] = part_o[idx * D + d];
    }
    float gmax = mmax;
#pragma unroll
    for (int q = 0; q < 8; ++q) gmax = fmaxf(gmax, ms[q]);
    const float carry = mmax == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(mmax - gmax);
    acc *= carry;
    lacc *= carry;
#pragma unroll
    for (int q = 0; q < 8; ++q) {
      const float f = ms[q] == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(ms[q] - gmax);
      acc += f * os[q];
      lacc += f * ls[q];
    }
    mmax = gmax;
  }
  // this call's rows are row0 .. row0 + lq - 1 of the lq_total rows of o and lse
  const int b = bq / lq, qi = bq % lq;
  store_from_f32(o + (((int64_t)b * lq_total + row0 + qi) * H + h) * D + d, acc * inv_rk / lacc);
  if (lse && d == 0) lse[((int64_t)b * H + h) * lq_total + row0 + qi] = (mmax + __builtin_amdgcn_logf(lacc)) * kLn2;
}

size_t workspace_bytes(int B, int lq, int H, int D, int S) {
  return (size_t)B * lq * S * H * (D + 2) * sizeof(float);
}

// `rows` = {row0, lq_total}: the call serves a->lq query rows that are rows row0 .. of lq_total (a->qa / a->qb point at
// row row0; a->o and a->lse at row 0); a plain call has {0, a->lq}
struct RowWindow { int row0, lq_total; };

template <int D, int RK, bool PAGED, int NQ>
int launch_decode_t(const TpaFwdArgs* a, int S, hipStream_t stream, RowWindow rows) {
  DecodeParams p{};
  p.qa = a->qa; p.qb = a->qb; p.ka = a->ka; p.kb = a->kb; p.va = a->va; p.vb = a->vb;
  float* ws = static_cast<float*>(a->workspace);
  const size_t no = (size_t)a->B * a->lq * S * a->H * D;
  const size_t nm = (size_t)a->B * a->lq * S * a->H;
  p.part_o = ws; p.part_m = ws + no; p.part_l = ws + no + nm;
  p.B = a->B; p.lq = a->lq; p.lk = a->lk; p.H = a->H; p.rq = a->rq; p.S = S;
  p.kvlen = a->kv_lengths;
  p.climit = a->causal ? causal_offset_of(a) + 1 + rows.row0 : a->lk;
  p.cbr = a->causal == TPA_CAUSAL_BOTTOM_RIGHT;
  p.row0 = rows.row0; p.lq_total = rows.lq_total;
  p.page_table = a->page_table; p.page_size = a->page_size; p.pages_per_seq = a->pages_per_seq;
  p.qscale = a->sm_scale * kLog2e / ((float)a->rq * (float)RK);
  auto kern = decode_kernel<D, RK, PAGED, NQ>;
  static bool configured[kMaxDevices] = {};
  if (int rc = raise_lds_limit(configured, reinterpret_cast<const void*>(kern), DecodeLds<D>::bytes(NQ)); rc != TPA_OK) return rc;
  dim3 grid((a->B * S + 7) / 8 * 8 * ((a->lq + NQ - 1) / NQ), (a->H + 31) / 32);
  hipLaunchKernelGGL(kern, grid, dim3(kWaves * 64), DecodeLds<D>::bytes(NQ), stream, p);
  if (hipGetLastError() != hipSuccess) return TPA_ERR_LAUNCH;
  hipLaunchKernelGGL((decode_merge_kernel<D, uint16_t>), dim3(a->B * a->lq, a->H), dim3(D), 0, stream, p.part_o, p.part_m, p.part_l,
                     static_cast<uint16_t*>(a->o), a->lse, S, a->H, a->lq, 1.f / (float)RK, rows.row0, rows.lq_total);
  return hipGetLastError() == hipSuccess ? TPA_OK : TPA_ERR_LAUNCH;
}

template <int D, int RK, bool PAGED>
int launch_decode_f32_t(const TpaFwdArgs* a, int S, hipStream_t stream, RowWindow rows) {
  DecodeParams p{};
  p.qa = a->qa; p.qb = a->qb; p.ka = a->ka; p.kb = a->kb; p.va = a->va; p.vb = a->vb;
  float* ws = static_cast<float*>(a->workspace);
  const size_t no = (size_t)a->B * a->lq * S * a->H * D, nm = (size_t)a->B * a->lq * S * a->H;
  p.part_o = ws; p.part_m = ws + no; p.part_l = ws + no + nm;
  p.B = a->B; p.lq = a->lq; p.lk = a->lk; p.H = a->H; p.rq = a->rq; p.S = S;
  p.kvlen = a->kv_lengths;
  p.climit = a->causal ? causal_offset_of(a) + 1 + rows.row0 : a->lk;
  p.cbr = a->causal == TPA_CAUSAL_BOTTOM_RIGHT;
  p.row0 = rows.row0; p.lq_total = rows.lq_total;
  p.page_table = a->page_table; p.page_size = a->page_size; p.pages_per_seq = a->pages_per_seq;
  p.qscale = a->sm_scale * kLog2e / ((float)a->rq * (float)RK);
  auto kern = decode_f32_kernel<D, RK, PAGED>;
  static bool configured[kMaxDevices] = {};
  if (int rc = raise_lds_limit(configured, reinterpret_cast<const void*>(kern), DecodeF32Lds<D>::kBytes); rc != TPA_OK) return rc;
  dim3 grid((a->B * S + 7) / 8 * 8 * a->lq, (a->H + 31) / 32);
  hipLaunchKernelGGL(kern, grid, dim3(kWaves * 64), DecodeF32Lds<D>::kBytes, stream, p);
  if (hipGetLastError() != hipSuccess) return TPA_ERR_LAUNCH;
  hipLaunchKernelGGL((decode_merge_kernel<D, float>), dim3(a->B * a->lq, a->H), dim3(D), 0, stream, p.part_o, p.part_m, p.part_l,
                     static_cast<float*>(a->o), a->lse, S, a->H, a->lq, 1.f / (float)RK, rows.row0, rows.lq_total);
  return hipGetLastError() == hipSuccess ? TPA_OK : TPA_ERR_LAUNCH;
}

template <int D, int RK>
int launch_decode_f32(const TpaFwdArgs* a, int S, hipStream_t stream, RowWindow rows) {
  if (a->page_table) {
    if (a->page_size <= 0 || (a->page_size * RK) % kRowsPerBlock != 0 ||
        (int64_t)a->pages_per_seq * a->page_size < a->lk)
      return TPA_ERR_SHAPE;
    return launch_decode_f32_t<D, RK, true>(a, S, stream, rows);
  }
  return launch_decode_f32_t<D, RK, false>(a, S, stream, rows);
}

template <int D, int RK>
int launch_decode(const TpaFwdArgs* a, int S, hipStream_t stream, RowWindow rows) {
  if (a->page_table) {
    // a block of 32 (token, rank) rows must not straddle pages, and the table must cover lk
    if (a->page_size <= 0 || (a->page_size * RK) % kRowsPerBlock != 0 ||
        (int64_t)a->pages_per_seq * a->page_size < a->lk)
      return TPA_ERR_SHAPE;
    return a->lq >= 2 ? launch_decode_t<D, RK, true, 2>(a, S, stream, rows) : launch_decode_t<D, RK, true, 1>(a, S, stream, rows);
  }
  return a->lq >= 2 ? launch_decode_t<D, RK, false, 2>(a, S, stream, rows) : launch_decode_t<D, RK, false, 1>(a, S, stream, rows);
}

bool aligned16(const void* ptr) { return (reinterpret_cast<uintptr_t>(ptr) & 15) == 0; }

int default_splits(int B, int lq, int lk, int H, int rows_per_group = 2) {
  // one workgroup per CU is resident (the kernel keeps a block of loads in flight in registers),
  // so aim for a whole number of waves of 256 workgroups and at least 4 blocks per wave.
  // The bf16 kernel serves two query rows per workgroup, which is what callers are told to size
  // the workspace for; the fp32 kernel serves one, launches twice the workgroups per range and so
  // asks for at most as many ranges (and never more workspace).
  const int groups = B * ((lq + rows_per_group - 1) / rows_per_group) * ((H + 31) / 32);
  int S = (256 + groups - 1) / groups;
  if (groups >= 256) S = 1;
  const int max_s = (lk + 4 * kWaves * 16 - 1) / (4 * kWaves * 16);
  if (S > max_s) S = max_s;
  if (S < 1) S = 1;
  return S;
}

}  // namespace
}  // namespace tpa

extern "C" int32_t tpa_decode_default_splits(int32_t B, int32_t lq, int32_t lk, int32_t H) {
  if (B <= 0 || lq <= 0 || lk <= 0 || H <= 0) return 0;
  return tpa::default_splits(B, lq, lk, H);
}

extern "C" size_t tpa_decode_workspace_bytes(int32_t B, int32_t lq, int32_t lk, int32_t H, int32_t dv, int32_t num_splits) {
  if (B <= 0 || lq <= 0 || lk <= 0 || H <= 0 || dv <= 0) return 0;
  const int S = num_splits > 0 ? num_splits : tpa::default_splits(B, lq, lk, H);
  return tpa::workspace_bytes(B, lq, H, dv, S);
}

int tpa_decode_mfma_supported(const TpaFwdArgs* a) {
  using namespace tpa;
  if (a->dtype != TPA_DTYPE_BF16) return 0;
  if (a->dk != a->dv || (a->dk != 64 && a->dk != 128)) return 0;
  if (a->rk != 1 && a->rk != 2 && a->rk != 4 && a->rk != 8 && a->rk != 16 && a->rk != 32) return 0;
  if (a->H % 8 != 0) return 0;
  if (a->lq > 64) return 0;
  if (a->q_segment_ids || a->kv_segment_ids) return 0;
  // rows (token, rank) must be uniformly strided: stride_l == rk * stride_r
  const TpaFactor* fs[4] = {&a->ka, &a->kb, &a->va, &a->vb};
  for (const TpaFactor* f : fs) {
    if (f->stride_l != (int64_t)a->rk * f->stride_r) return 0;
    if (!aligned16(f->ptr) || f->stride_r % 8 != 0 || f->stride_b % 8 != 0) return 0;
  }
  if (!aligned16(a->qb.ptr) || a->qb.stride_r % 8 != 0 || a->qb.stride_l % 8 != 0 || a->qb.stride_b % 8 != 0) return 0;
  return 1;
}

int tpa_decode_mfma_launch(const TpaFwdArgs* a, hipStream_t stream) { return tpa_decode_mfma_launch_rows(a, stream, 0, a->lq); }

int tpa_decode_mfma_launch_rows(const TpaFwdArgs* a, hipStream_t stream, int row0, int lq_total) {
  using namespace tpa;
  const RowWindow rows{row0, lq_total};
  const int S = a->num_splits > 0 ? a->num_splits : default_splits(a->B, a->lq, a->lk, a->H);
  if (S > 65535 || (int64_t)a->B * S > 2147483647LL) return TPA_ERR_SHAPE;
  if (!a->workspace || a->workspace_bytes < workspace_bytes(a->B, a->lq, a->H, a->dv, S)) return TPA_ERR_WORKSPACE;
  if (!aligned16(a->workspace)) return TPA_ERR_ALIGN;
  if (a->dk == 128) {
    switch (a->rk) {
      case 1: return launch_decode<128, 1>(a, S, stream, rows);
      case 2: return launch_decode<128, 2>(a, S, stream, rows);
      case 4: return launch_decode<128, 4>(a, S, stream, rows);
      case 8: return launch_decode<128, 8>(a, S, stream, rows);
      case 16: return launch_decode<128, 16>(a, S, stream, rows);
      default: return launch_decode<128, 32>(a, S, stream, rows);
    }
  }
  switch (a->rk) {
    case 1: return launch_decode<64, 1>(a, S, stream, rows);
    case 2: return launch_decode<64, 2>(a, S, stream, rows);
    case 4: return launch_decode<64, 4>(a, S, stream, rows);
    case 8: return launch_decode<64, 8>(a, S, stream, rows);
    case 16: return launch_decode<64, 16>(a, S, stream, rows);
    default: return launch_decode<64, 32>(a, S, stream, rows);
  }
}

int tpa_decode_f32_supported(const TpaFwdArgs* a) {
  using namespace tpa;
  if (a->dtype != TPA_DTYPE_F32) return 0;
  if (a->dk != a->dv || (a->dk != 64 && a->dk != 128)) return 0;
  if (a->rk != 1 && a->rk != 2 && a->rk != 4 && a->rk != 8 && a->rk != 16 && a->rk != 32) return 0;
  if (a->lq > 64) return 0;
  if (a->q_segment_ids || a->kv_segment_ids) return 0;
  // rows (token, rank) must be uniformly strided: stride_l == rk * stride_r; B rows are read as 16-byte vectors
  const TpaFactor* fs[4] = {&a->ka, &a->kb, &a->va, &a->vb};
  for (const TpaFactor* f : fs)
    if (f->stride_l != (int64_t)a->rk * f->stride_r) return 0;
  const TpaFactor* bs[3] = {&a->kb, &a->vb, &a->qb};
  for (const TpaFactor* f : bs)
    if (!aligned16(f->ptr) || f->stride_r % 4 != 0 || f->stride_l % 4 != 0 || f->stride_b % 4 != 0) return 0;
  return 1;
}

int tpa_decode_f32_launch(const TpaFwdArgs* a, hipStream_t stream) { return tpa_decode_f32_launch_rows(a, stream, 0, a->lq); }

int tpa_decode_f32_launch_rows(const TpaFwdArgs* a, hipStream_t stream, int row0, int lq_total) {
  using namespace tpa;
  const RowWindow rows{row0, lq_total};
  const int S = a->num_splits > 0 ? a->num_splits : default_splits(a->B, a->lq, a->lk, a->H, 1);
  if (S > 65535 || (int64_t)a->B * S > 2147483647LL) return TPA_ERR_SHAPE;
  if (!a->workspace || a->workspace_bytes < workspace_bytes(a->B, a->lq, a->H, a->dv, S)) return TPA_ERR_WORKSPACE;
  if (!aligned16(a->workspace)) return TPA_ERR_ALIGN;
  if (a->dk == 128) {
    switch (a->rk) {
      case 1: return launch_decode_f32<128, 1>(a, S, stream, rows);
      case 2: return launch_decode_f32<128, 2>(a, S, stream, rows);
      case 4: return launch_decode_f32<128, 4>(a, S, stream, rows);
      case 8: return launch_decode_f32<128, 8>(a, S, stream, rows);
      case 16: return launch_decode_f32<128, 16>(a, S, stream, rows);
      default: return launch_decode_f32<128, 32>(a, S, stream, rows);
    }
  }
  switch (a->rk) {
    case 1: return launch_decode_f32<64, 1>(a, S, stream, rows);
    case 2: return launch_decode_f32<64, 2>(a, S, stream, rows);
    case 4: return launch_decode_f32<64, 4>(a, S, stream, rows);
    case 8: return launch_decode_f32<64, 8>(a, S, stream, rows);
    case 16: return launch_decode_f32<64, 16>(a, S, stream, rows);
    default: return launch_decode_f32<64, 32>(a, S, stream, rows);
  }
}

// ---------------------------------------------------------------------------------------------
// tpa_decode for callers that cannot allocate device memory (code under HIP graph capture, tight
// serving loops): the split partials go to a fixed array in this code object instead of a caller
// workspace.  Every device the library runs on holds its own copy of the array until the process
// ends.  Host code must not use the array's name as an address (in host code the name is a
// stand-in for the symbol, not device memory); the device address is looked up once per device
// and kept.
namespace tpa {
namespace {

static __device__ __align__(256) unsigned char scratch[TPA_DECODE_NOALLOC_SCRATCH_BYTES];

void* g_scratch_ptr[kMaxDevices] = {};
std::mutex g_scratch_mutex;

// Device address of `scratch` on the current device (looked up on the first call per device).
int scratch_of_current_device(void** out) {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return TPA_ERR_LAUNCH;
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (!g_scratch_ptr[dev]) {
    void* ptr = nullptr;
    if (hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)) != hipSuccess || !ptr) return TPA_ERR_LAUNCH;
    g_scratch_ptr[dev] = ptr;
  }
  *out = g_scratch_ptr[dev];
  return TPA_OK;
}

}  // namespace
}  // namespace tpa

extern "C" int tpa_decode_noalloc(const TpaFwdArgs* a, void* stream) {
  using namespace tpa;
  const int rc = tpa_validate_fwd_args(a);
  if (rc != TPA_OK) return rc;
  if (a->q_segment_ids) return TPA_ERR_UNSUPPORTED;
  const bool bf16 = tpa_decode_mfma_supported(a), f32 = !bf16 && tpa_decode_f32_supported(a);
  if (a->kernel == TPA_KERNEL_GENERIC || (!bf16 && !f32)) return TPA_ERR_UNSUPPORTED;  // the split-key kernels only
  const int S = a->num_splits > 0 ? a->num_splits : default_splits(a->B, a->lq, a->lk, a->H, bf16 ? 2 : 1);
  if (S > 65535 || (int64_t)a->B * S > 2147483647LL) return TPA_ERR_SHAPE;
  if (workspace_bytes(a->B, a->lq, a->H, a->dv, S) > (size_t)TPA_DECODE_NOALLOC_SCRATCH_BYTES) return TPA_ERR_WORKSPACE;  // partials exceed the fixed array
  void* ptr = nullptr;
  if (int rc2 = scratch_of_current_device(&ptr); rc2 != TPA_OK) return rc2;
  // every (batch entry, query row, key range, head) slot that the merge kernel reads is written by
  // the decode kernel of the same call, so nothing of the previous call's contents has to be cleared
  TpaFwdArgs b = *a;
  b.workspace = ptr;
  b.workspace_bytes = TPA_DECODE_NOALLOC_SCRATCH_BYTES;
  b.num_splits = S;
  return bf16 ? tpa_decode_mfma_launch(&b, static_cast<hipStream_t>(stream)) : tpa_decode_f32_launch(&b, static_cast<hipStream_t>(stream));
}
