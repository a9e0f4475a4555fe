// Backward pass of dense flash attention on the matrix cores (bf16 MFMA, fp32 accumulation),
// used for the dense baseline (tpa/mha.py:40-65) and - between a reconstruction of dense Q, K, V
// from the rank factors and a projection of the dense gradients back onto them - for tensor
// product attention (tpa/tpa.py:546-962).
//
// The softmax matrix is recomputed from the saved logsumexp, as in the forward kernel with the
// roles of the MFMA operands chosen so that nothing ever goes through LDS between two
// contractions (v_mfma_f32_32x32x16_bf16; "lane" = the accumulator column a lane owns):
//
//   bwd_dq_kernel   one workgroup = 256 query rows of one head, a wave owns 32 rows, lane = row
//     S^T  = K Q^T            A = K rows (LDS),      B = Q (registers, pre-scaled), addend -lse
//     dP^T = V dO^T           A = V rows (LDS),      B = dO (registers),            addend -delta
//     dS^T = exp2(S^T) * dP^T  in registers, packed to bf16 in place
//     dQ^T += K^T dS^T        A = K^T (transposed LDS reads), B = dS^T
//
//   bwd_dkv_kernel  one workgroup = 32 keys per wave of one head, lane = key
//     S  = Q K^T              A = Q rows (LDS),      B = K (registers, pre-scaled), addend -lse[row]
//     dP = dO V^T             A = dO rows (LDS),     B = V (registers; at D = 128 a per-lane LDS slot), addend -delta[row]
//     dV^T += dO^T P          A = dO^T (transposed LDS reads), B = P
//     dK^T += Q^T dS          A = Q^T  (transposed LDS reads), B = dS
//
// with p = exp(x - lse), ds = sm_scale * p * (dp - delta) (tpa/tpa.py:765-781, tpa/mha.py:57-63).
// Rows without a visible key carry lse = -inf and contribute nothing (tpa/tpa.py:675-676).
#include <type_traits>
#include <utility>

#include "tpa_common.h"

namespace tpa {
namespace {

constexpr int kTile = 64;  // keys (dq kernel) or query rows (dkv kernel) per LDS tile

struct BwdParams {
  const uint16_t* q;    // [B, lq, H, D] bf16
  const uint16_t* k;    // [B, lk, H, D]
  const uint16_t* v;    // [B, lk, H, D]
  const uint16_t* d_o;  // [B, lq, H, D]
  const float* lse;     // [B, H, lq] natural log
  const float* delta;   // [B, H, lq]
  const int32_t* qseg;  // [B, lq] or null
  const int32_t* kvseg; // [B, lk] or null
  float* dq;            // [B, lq, H, D] fp32
  float* dk;            // [B, lk, H, D]
  float* dv;            // [B, lk, H, D]
  int B, lq, lk, H;
  float sm_scale;
  int causal;
  int coff;  // with causal: row i sees keys <= i + coff
  int nblk;    // row blocks (dq) or key blocks (dkv) per (batch, head)
  int npairs;  // nblk * B
  int pair_group;  // (batch, head) pairs of an XCD whose blocks run side by side
};

__device__ __forceinline__ void lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

template <typename F, int... I>
__device__ __forceinline__ void static_for_impl(F&& f, std::integer_sequence<int, I...>) {
  (f(std::integral_constant<int, I>{}), ...);
}
template <int N, typename F>
__device__ __forceinline__ void static_for(F&& f) {
  static_for_impl(f, std::make_integer_sequence<int, N>{});
}

constexpr int kRsrcFlags = 0x00020000;  // raw 32-bit data format

// Row stride (elements) of the LDS tiles.  Every tile is read both by rows (16-byte reads of 16
// consecutive rows) and transposed (8-byte reads of 4 consecutive rows); no padding serves both
// without bank conflicts, these leave the row reads conflict-free and the transposed ones two-way.
constexpr int tile_stride(int d) { return d == 128 ? d + 24 : d + 8; }

// dK/dV kernel at D = 128: K, V and both accumulators of a wave's 32 keys are 192 of its 256 registers, and
// with S, dP, the rows on their way to LDS and the addresses the compiler spilled 26 of them and reloaded 15
// per tile (scratch reads in the loop: 4.2 M wave-level loads per launch at B = 4, T = 4096, H = 16).  The V
// fragments therefore live in LDS - each lane parks its own eight 16-byte B operands once and reads them back
// where dP = dO V^T needs them (one more 16-byte LDS read per matrix instruction of that product; LDS was busy
// a third of the time).  No scratch is left, and the kernel takes a fifth less (0.666 -> 0.54 ms at that shape).
constexpr bool dkv_v_in_lds(int d) { return d == 128; }

// A-operand fragment of rows 32 mb .. 32 mb + 31 of a row-major tile (row stride S elements),
// contraction columns 16 kk .. 16 kk + 15: lane (i, g) reads 8 elements of row 32 mb + i.
template <int S>
__device__ __forceinline__ bf16x8 rows_frag(const uint16_t* tile, int mb, int kk, int i, int g) {
  return *reinterpret_cast<const bf16x8*>(tile + (32 * mb + i) * S + 16 * kk + 8 * g);
}
// A-operand fragment of the TRANSPOSED tile: output rows = tile columns 32 db .. 32 db + 31,
// contraction = tile rows 16 kk .. 16 kk + 15 in the slot order an accumulator column already has
// (slot (g, j) = tile row 16 kk + 8 (j / 4) + 4 g + j % 4).
template <int S>
__device__ __forceinline__ bf16x8 cols_frag(const uint16_t* tile, int kk, int db, int g, int lp, int dhalf) {
  const uint16_t* row = tile + (16 * kk + 4 * g + (lp >> 2)) * S + 16 * dhalf + 4 * (lp & 3) + 32 * db;
  const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3)))*)(row));
  const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3)))*)(row + 8 * S));
  return __builtin_bit_cast(bf16x8, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
}

// 16 fp32 values of one accumulator block -> two B-operand fragments (contraction steps 2 mb, 2 mb + 1)
__device__ __forceinline__ void pack_block(const f32x16& x, bf16x8& f0, bf16x8& f1) {
  u32x4 a, b;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    a[j] = pack_bf16(x[2 * j], x[2 * j + 1]);
    b[j] = pack_bf16(x[8 + 2 * j], x[8 + 2 * j + 1]);
  }
  f0 = __builtin_bit_cast(bf16x8, a);
  f1 = __builtin_bit_cast(bf16x8, b);
}

__device__ __forceinline__ f32x16 splat16(float x) {
  f32x16 r;
#pragma unroll
  for (int v = 0; v < 16; ++v) r[v] = x;
  return r;
}


// Packed sequences (tpa/tpa.py:369-375 compares ids pairwise): an element of `other` can only
// pair with this workgroup's elements if its id lies within [min, max] of the workgroup's own ids
// `mine[0 .. n_mine)`.  Returns the first and last such index of other[0 .. n_other) (last = -1 if
// there is none): exact for ids that do not decrease along the sequence, conservative otherwise
// (the per-pair mask still decides).  `red` = 4 ints of LDS; every thread of the workgroup calls.
template <int NT>
__device__ __forceinline__ void id_window(const int32_t* mine, int n_mine, const int32_t* other, int n_other, int32_t* red,
                                          int tid, int& first, int& last) {
  if (tid == 0) { red[0] = INT32_MAX; red[1] = INT32_MIN; red[2] = INT32_MAX; red[3] = -1; }
  __syncthreads();
  {  // one atomic per wave: the lanes' values are reduced in registers first
    int32_t smin = INT32_MAX, smax = INT32_MIN;
    for (int t = tid; t < n_mine; t += NT) {
      const int32_t sid = mine[t];
      smin = min(smin, sid); smax = max(smax, sid);
    }
    smin = wave_min(smin); smax = wave_max(smax);
    if ((tid & 63) == 0 && smin <= smax) {
      __hip_atomic_fetch_min(&red[0], smin, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
      __hip_atomic_fetch_max(&red[1], smax, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    }
  }
  __syncthreads();
  const int32_t lo_id = red[0], hi_id = red[1];
  int lo = INT32_MAX, hi = -1;
  for (int t = tid; t < n_other; t += NT) {
    const int32_t sid = other[t];
    if (sid >= lo_id && sid <= hi_id) { lo = min(lo, t); hi = max(hi, t); }
  }
  lo = wave_min(lo); hi = wave_max(hi);
  if ((tid & 63) == 0 && hi >= 0) {
    __hip_atomic_fetch_min(&red[2], lo, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    __hip_atomic_fetch_max(&red[3], hi, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
  }
  __syncthreads();
  first = red[2];
  last = red[3];
  __syncthreads();  // the tiles reuse this memory
}

// ============================================================================================
// dQ
// ============================================================================================
template <int D, int NW, int NB, bool SEG>
__global__ __launch_bounds__(NW * 64) void bwd_dq_kernel(BwdParams p) {
  // a wave owns NB blocks of 32 query rows: every operand fragment read from LDS feeds NB MFMAs
  constexpr int NT = NW * 64, S = tile_stride(D), CPR = D / 8, TPP = NT / CPR, NPASS = kTile / TPP;
  constexpr int NKS = D / 16, NDB = D / 32, kWQ = 32 * NB, kBQ = NW * kWQ;
  static_assert(kTile % TPP == 0 && NPASS >= 1, "loader shape");
  extern __shared__ __attribute__((aligned(16))) uint16_t smem[];
  uint16_t* const lds_k = smem;                  // [2][64][S]
  uint16_t* const lds_v = smem + 2 * kTile * S;  // [2][64][S]
  int32_t* const lds_seg = reinterpret_cast<int32_t*>(smem + 4 * kTile * S);  // [2][64]

  // Workgroup ids are dealt round-robin to the 8 XCDs.  The dense arrays of one (batch, head) are what
  // workgroups can share, so an XCD owns whole (batch, head) pairs and runs their blocks heaviest first,
  // the same block of all its pairs side by side: neighbouring blocks of a pair walk the same tiles at
  // about the same time and find them in that XCD's L2.
  // Pairs are taken in groups of `pair_group` (launch_dq): with every pair of an XCD side by side and many pairs the
  // resident workgroups would all belong to different pairs and share nothing.
  const int id = blockIdx.x, xcd = id & 7, slot = id >> 3;
  const int per_xcd = (p.B * p.H + 7) / 8, per_group = p.pair_group * p.nblk;
  const int grp = slot / per_group, rem = slot - grp * per_group;
  const int pair_local = grp * p.pair_group + rem % p.pair_group;
  const int bh = pair_local * 8 + xcd;
  if (pair_local >= per_xcd || bh >= p.B * p.H) return;
  const int qblk = p.nblk - 1 - rem / p.pair_group, b = bh / p.H, h = bh % p.H;  // heaviest causal blocks first
  const int tid = threadIdx.x, w = tid >> 6, l = tid & 63, i = l & 31, g = l >> 5;
  const int lp = l & 15, dhalf = (l >> 4) & 1;
  const int q0 = qblk * kBQ, wrow0 = q0 + kWQ * w;
  const float c = p.sm_scale * kLog2e;

  // this lane's rows: Q (scaled) and dO as B-operand fragments, -lse (log2 domain) and -delta
  f32x16 nlse[NB], ndelta[NB];
  bf16x8 qf[NB][NKS], gf[NB][NKS];
  int32_t qseg[NB];
#pragma unroll
  for (int nb = 0; nb < NB; ++nb) {
    const int qrow = wrow0 + 32 * nb + i, qrow_ld = min(qrow, p.lq - 1);
    const float lse_r = p.lse[((int64_t)b * p.H + h) * p.lq + qrow_ld];
    const bool live = qrow < p.lq && lse_r > -INFINITY;
    nlse[nb] = splat16(live ? -lse_r * kLog2e : -INFINITY);
    ndelta[nb] = splat16(-p.delta[((int64_t)b * p.H + h) * p.lq + qrow_ld]);
    const uint16_t* qp = p.q + (((int64_t)b * p.lq + qrow_ld) * p.H + h) * D;
    const uint16_t* gp = p.d_o + (((int64_t)b * p.lq + qrow_ld) * p.H + h) * D;
#pragma unroll
    for (int ks = 0; ks < NKS; ++ks) {
      const u32x4 raw = *reinterpret_cast<const u32x4*>(qp + 16 * ks + 8 * g);
      u32x4 sc, gr = *reinterpret_cast<const u32x4*>(gp + 16 * ks + 8 * g);
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        sc[j] = pack_bf16(bf16lo_to_f32(raw[j]) * c, bf16hi_to_f32(raw[j]) * c);
        if (!live) gr[j] = 0u;  // the upstream gradient of a row without a visible key may be NaN
      }
      qf[nb][ks] = __builtin_bit_cast(bf16x8, sc);
      gf[nb][ks] = __builtin_bit_cast(bf16x8, gr);
    }
    qseg[nb] = SEG ? p.qseg[(int64_t)b * p.lq + qrow_ld] : 0;
  }

  // keys [kpos0, kend) are visited; tiles and key positions below count from kpos0
  int kpos0 = 0, kend = p.causal ? max(1, min(p.lk, min(q0 + kBQ, p.lq) + p.coff)) : p.lk;  // at least one (then fully masked) tile
  if constexpr (SEG) {
    int first, lastk;
    id_window<NT>(p.qseg + (int64_t)b * p.lq + q0, min(kBQ, p.lq - q0), p.kvseg + (int64_t)b * p.lk, kend,
                  reinterpret_cast<int32_t*>(smem), tid, first, lastk);
    if (lastk >= 0) { kpos0 = first / kTile * kTile; kend = lastk + 1; }
    else kend = min(kend, kTile);  // nothing visible: one fully masked tile
  }
  const int lk_r = kend - kpos0, wrow_r = wrow0 + p.coff - kpos0;  // rows on the key scale: row r sees keys <= r_r
  const int ntiles = (lk_r + kTile - 1) / kTile, last = ntiles - 1;
  const int wave_last_tile = p.causal ? min(last, max(wrow_r + kWQ - 1, 0) / kTile) : last;

  // tile loader: raw buffer loads one tile ahead (rows past kend read as zero), stored to LDS later
  const int lt = tid / CPR, lc = tid % CPR;
  const int64_t tok_stride = (int64_t)p.H * D;
  const int bytes = (int)(((int64_t)(lk_r - 1) * tok_stride + D) * 2);
  const __amdgpu_buffer_rsrc_t k_rs = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint16_t*>(p.k + (((int64_t)b * p.lk + kpos0) * p.H + h) * D), 0, bytes, kRsrcFlags);
  const __amdgpu_buffer_rsrc_t v_rs = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint16_t*>(p.v + (((int64_t)b * p.lk + kpos0) * p.H + h) * D), 0, bytes, kRsrcFlags);
  const int voff = (int)((lt * tok_stride + 8 * lc) * 2);
  u32x4 kreg[NPASS], vreg[NPASS];
  int32_t seg_pending = 0;
  auto issue = [&](int tile) __attribute__((always_inline)) {
#pragma unroll
    for (int ps = 0; ps < NPASS; ++ps) {
      const int soff = (int)((int64_t)(tile * kTile + ps * TPP) * tok_stride * 2);
      kreg[ps] = __builtin_amdgcn_raw_buffer_load_b128(k_rs, voff, soff, 0);
      vreg[ps] = __builtin_amdgcn_raw_buffer_load_b128(v_rs, voff, soff, 0);
    }
    if constexpr (SEG)
      if (tid < kTile) seg_pending = p.kvseg[(int64_t)b * p.lk + kpos0 + min(tile * kTile + tid, lk_r - 1)];
  };
  auto commit = [&](int tile) __attribute__((always_inline)) {
    uint16_t* kd = lds_k + (tile & 1) * kTile * S;
    uint16_t* vd = lds_v + (tile & 1) * kTile * S;
#pragma unroll
    for (int ps = 0; ps < NPASS; ++ps) {
      const int t = ps * TPP + lt;
      *reinterpret_cast<u32x4*>(kd + t * S + 8 * lc) = kreg[ps];
      *reinterpret_cast<u32x4*>(vd + t * S + 8 * lc) = vreg[ps];
    }
    if constexpr (SEG)
      if (tid < kTile) lds_seg[(tile & 1) * kTile + tid] = seg_pending;
  };

  f32x16 acc[NB][NDB];
#pragma unroll
  for (int nb = 0; nb < NB; ++nb)
#pragma unroll
    for (int db = 0; db < NDB; ++db) acc[nb][db] = splat16(0.f);

  auto compute = [&](int j) __attribute__((always_inline)) {
    const uint16_t* ks = lds_k + (j & 1) * kTile * S;
    const uint16_t* vs = lds_v + (j & 1) * kTile * S;
    const int k0 = j * kTile;
    const bool need_mask = (k0 + kTile > lk_r) || (p.causal && (k0 + kTile - 1 > wrow_r));
    static_for<2>([&](auto mb_c) __attribute__((always_inline)) {
      constexpr int mb = decltype(mb_c)::value;
      f32x16 s[NB], dp[NB];
#pragma unroll
      for (int nb = 0; nb < NB; ++nb) { s[nb] = nlse[nb]; dp[nb] = ndelta[nb]; }
      // The two chains are independent: they alternate, and their operands are requested two steps ahead.  The
      // order is pinned (left alone, the compiler runs one chain after the other and reads each operand right
      // before the instruction that takes it: 1 % of the call at B = 4, T = 4096, H = 16, more where blocks are long).
      __builtin_amdgcn_sched_barrier(0);
      static_for<NKS>([&](auto kk_c) __attribute__((always_inline)) {
        constexpr int kk = decltype(kk_c)::value;
        const bf16x8 a = rows_frag<S>(ks, mb, kk, i, g);
        const bf16x8 a2 = rows_frag<S>(vs, mb, kk, i, g);
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) {
          s[nb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, qf[nb][kk], s[nb], 0, 0, 0);
          dp[nb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a2, gf[nb][kk], dp[nb], 0, 0, 0);
        }
      });
      __builtin_amdgcn_sched_group_barrier(0x100, 4, 0);
#pragma unroll
      for (int n = 0; n < NKS - 2; ++n) {
        __builtin_amdgcn_sched_group_barrier(0x008, 2 * NB, 0);
        __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
      }
      __builtin_amdgcn_sched_group_barrier(0x008, 4 * NB, 0);
      __builtin_amdgcn_sched_barrier(0);
      bf16x8 df[NB][2];
#pragma unroll
      for (int nb = 0; nb < NB; ++nb) {
        if (need_mask) {
          const int qrow_r = wrow_r + 32 * nb + i;
          const int limit = p.causal ? min(qrow_r, lk_r - 1) : lk_r - 1;  // largest visible key index
#pragma unroll
          for (int v = 0; v < 16; ++v)
            if (k0 + 32 * mb + 8 * (v >> 2) + 4 * g + (v & 3) > limit) s[nb][v] = -INFINITY;
        }
        if constexpr (SEG) {
          const int32_t* ids_p = lds_seg + (j & 1) * kTile + 32 * mb + 4 * g;
#pragma unroll
          for (int vq = 0; vq < 4; ++vq) {
            const int4 ids = *reinterpret_cast<const int4*>(ids_p + 8 * vq);
            if (ids.x != qseg[nb]) s[nb][4 * vq] = -INFINITY;
            if (ids.y != qseg[nb]) s[nb][4 * vq + 1] = -INFINITY;
            if (ids.z != qseg[nb]) s[nb][4 * vq + 2] = -INFINITY;
            if (ids.w != qseg[nb]) s[nb][4 * vq + 3] = -INFINITY;
          }
        }
#pragma unroll
        for (int v = 0; v < 16; ++v) s[nb][v] = __builtin_amdgcn_exp2f(s[nb][v]) * dp[nb][v];  // p * (dp - delta)
        pack_block(s[nb], df[nb][0], df[nb][1]);
      }
      static_for<2 * NDB>([&](auto n_c) __attribute__((always_inline)) {
        constexpr int db = decltype(n_c)::value / 2, half = decltype(n_c)::value % 2;
        const bf16x8 a = cols_frag<S>(ks, 2 * mb + half, db, g, lp, dhalf);
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) acc[nb][db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, df[nb][half], acc[nb][db], 0, 0, 0);
      });
    });
  };

  issue(0);
  commit(0);
  issue(min(1, last));
  __syncthreads();
  for (int j = 0; j < ntiles; ++j) {
    if (j <= wave_last_tile) compute(j);
    if (j + 1 < ntiles) {
      commit(j + 1);
      issue(min(j + 2, last));
    }
    lds_barrier();
  }

#pragma unroll
  for (int nb = 0; nb < NB; ++nb) {
    const int qrow = wrow0 + 32 * nb + i;
    if (qrow < p.lq) {
      float* op = p.dq + (((int64_t)b * p.lq + qrow) * p.H + h) * D;
#pragma unroll
      for (int db = 0; db < NDB; ++db)
#pragma unroll
        for (int vq = 0; vq < 4; ++vq) {
          f32x4 out;
#pragma unroll
          for (int e = 0; e < 4; ++e) out[e] = acc[nb][db][4 * vq + e] * p.sm_scale;
          *reinterpret_cast<f32x4*>(op + 32 * db + 8 * vq + 4 * g) = out;
        }
    }
  }
}

// ============================================================================================
// dK, dV
// ============================================================================================
template <int D, int NW, int NB, bool SEG>
__global__ __launch_bounds__(NW * 64) void bwd_dkv_kernel(BwdParams p) {
  // a wave owns NB blocks of 32 keys: every operand fragment read from LDS feeds NB MFMAs
  constexpr int NT = NW * 64, S = tile_stride(D), CPR = D / 8, TPP = NT / CPR, NPASS = kTile / TPP;
  constexpr int NKS = D / 16, NDB = D / 32, kWK = 32 * NB, kBK = NW * kWK;
  static_assert(kTile % TPP == 0 && NPASS >= 1, "loader shape");
  extern __shared__ __attribute__((aligned(16))) uint16_t smem[];
  uint16_t* const lds_q = smem;                  // [2][64][S]
  uint16_t* const lds_g = smem + 2 * kTile * S;  // [2][64][S]  upstream gradient rows
  float* const lds_nlse = reinterpret_cast<float*>(smem + 4 * kTile * S);  // [2][64]  -lse * log2(e), -inf for dead rows
  float* const lds_ndel = lds_nlse + 2 * kTile;                            // [2][64]  -delta
  int32_t* const lds_seg = reinterpret_cast<int32_t*>(lds_ndel + 2 * kTile);  // [2][64]
  u32x4* const lds_vf = reinterpret_cast<u32x4*>(lds_seg + 2 * kTile);  // [NW][NB][NKS][64 lanes]: V of the wave's keys as B operands

  // (batch, head) pairs per XCD, blocks heaviest first: see bwd_dq_kernel
  const int id = blockIdx.x, xcd = id & 7, slot = id >> 3;
  const int per_xcd = (p.B * p.H + 7) / 8, per_group = p.pair_group * p.nblk;
  const int grp = slot / per_group, rem = slot - grp * per_group;
  const int pair_local = grp * p.pair_group + rem % p.pair_group;
  const int bh = pair_local * 8 + xcd;
  if (pair_local >= per_xcd || bh >= p.B * p.H) return;
  const int kblk = rem / p.pair_group, b = bh / p.H, h = bh % p.H;  // under the causal mask the first key blocks are the heaviest
  const int tid = threadIdx.x, w = tid >> 6, l = tid & 63, i = l & 31, g = l >> 5;
  const int lp = l & 15, dhalf = (l >> 4) & 1;
  const int k0 = kblk * kBK, wkey0 = k0 + kWK * w;
  const float c = p.sm_scale * kLog2e;

  constexpr bool VLDS = dkv_v_in_lds(D);
  bf16x8 kf[NB][NKS], vf[VLDS ? 1 : NB][VLDS ? 1 : NKS];
  int32_t kseg[NB];
#pragma unroll
  for (int nb = 0; nb < NB; ++nb) {
    const int key_ld = min(wkey0 + 32 * nb + i, p.lk - 1);
    const uint16_t* kp = p.k + (((int64_t)b * p.lk + key_ld) * p.H + h) * D;
    const uint16_t* vp = p.v + (((int64_t)b * p.lk + key_ld) * p.H + h) * D;
#pragma unroll
    for (int ks = 0; ks < NKS; ++ks) {
      const u32x4 raw = *reinterpret_cast<const u32x4*>(kp + 16 * ks + 8 * g);
      u32x4 sc;
#pragma unroll
      for (int j = 0; j < 4; ++j) sc[j] = pack_bf16(bf16lo_to_f32(raw[j]) * c, bf16hi_to_f32(raw[j]) * c);
      kf[nb][ks] = __builtin_bit_cast(bf16x8, sc);
      if constexpr (VLDS) lds_vf[((w * NB + nb) * NKS + ks) * 64 + l] = *reinterpret_cast<const u32x4*>(vp + 16 * ks + 8 * g);
      else vf[nb][ks] = *reinterpret_cast<const bf16x8*>(vp + 16 * ks + 8 * g);
    }
    kseg[nb] = SEG ? p.kvseg[(int64_t)b * p.lk + key_ld] : 0;
  }

  // query tiles tile0 .. : under the causal mask rows before this block's first key see none of
  // its keys; rows from lq_r on are not visited
  int tile0 = p.causal ? max(k0 - p.coff, 0) / kTile : 0, lq_r = p.lq;
  if constexpr (SEG) {
    int first, lastq;
    const int rbeg = min(tile0 * kTile, p.lq);
    id_window<NT>(p.kvseg + (int64_t)b * p.lk + k0, min(kBK, p.lk - k0), p.qseg + (int64_t)b * p.lq + rbeg, p.lq - rbeg,
                  reinterpret_cast<int32_t*>(smem), tid, first, lastq);
    if (lastq >= 0) { tile0 = (rbeg + first) / kTile; lq_r = rbeg + lastq + 1; }
    else lq_r = 0;  // no row can see a key of this block
  }
  const int ntiles = max(0, (lq_r + kTile - 1) / kTile - tile0), last = ntiles - 1;
  const int wave_first_tile = p.causal ? max(max(wkey0 - p.coff, 0) / kTile - tile0, 0) : 0;

  const int lt = tid / CPR, lc = tid % CPR;
  const int64_t tok_stride = (int64_t)p.H * D;
  const int bytes = (int)(((int64_t)(max(lq_r, 1) - 1) * tok_stride + D) * 2);
  const __amdgpu_buffer_rsrc_t q_rs = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint16_t*>(p.q + ((int64_t)b * p.lq * p.H + h) * D), 0, bytes, kRsrcFlags);
  const __amdgpu_buffer_rsrc_t g_rs = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint16_t*>(p.d_o + ((int64_t)b * p.lq * p.H + h) * D), 0, bytes, kRsrcFlags);
  const int voff = (int)((lt * tok_stride + 8 * lc) * 2);
  const float* lse_b = p.lse + ((int64_t)b * p.H + h) * p.lq;
  const float* del_b = p.delta + ((int64_t)b * p.H + h) * p.lq;
  u32x4 qreg[NPASS], greg[NPASS];
  float row_lse[NPASS];   // lse of the rows this thread stages (their upstream gradient is zeroed if dead)
  float aux_pending = 0.f;
  auto issue = [&](int tile) __attribute__((always_inline)) {
    const int r0 = (tile0 + tile) * kTile;
#pragma unroll
    for (int ps = 0; ps < NPASS; ++ps) {
      const int soff = (int)((int64_t)(r0 + ps * TPP) * tok_stride * 2);
      qreg[ps] = __builtin_amdgcn_raw_buffer_load_b128(q_rs, voff, soff, 0);
      greg[ps] = __builtin_amdgcn_raw_buffer_load_b128(g_rs, voff, soff, 0);
      const int r = r0 + ps * TPP + lt;
      row_lse[ps] = r < lq_r ? lse_b[r] : -INFINITY;
    }
    // threads 0..63: -lse, 64..127: -delta, 128..191: segment id of row r0 + tid % 64
    if (tid < 3 * kTile) {
      const int r = r0 + (tid & (kTile - 1));
      const int rl = min(r, p.lq - 1);
      if (tid < kTile) {
        const float x = lse_b[rl];
        aux_pending = (r < lq_r && x > -INFINITY) ? -x * kLog2e : -INFINITY;
      } else if (tid < 2 * kTile) {
        aux_pending = -del_b[rl];
      } else if (SEG) {
        aux_pending = __int_as_float(p.qseg[(int64_t)b * p.lq + rl]);
      }
    }
  };
  auto commit = [&](int tile) __attribute__((always_inline)) {
    uint16_t* qd = lds_q + (tile & 1) * kTile * S;
    uint16_t* gd = lds_g + (tile & 1) * kTile * S;
#pragma unroll
    for (int ps = 0; ps < NPASS; ++ps) {
      const int t = ps * TPP + lt;
      u32x4 gr = greg[ps];
      if (!(row_lse[ps] > -INFINITY)) gr = u32x4{0u, 0u, 0u, 0u};  // a dead row's upstream gradient may be NaN
      *reinterpret_cast<u32x4*>(qd + t * S + 8 * lc) = qreg[ps];
      *reinterpret_cast<u32x4*>(gd + t * S + 8 * lc) = gr;
    }
    if (tid < kTile) lds_nlse[(tile & 1) * kTile + tid] = aux_pending;
    else if (tid < 2 * kTile) lds_ndel[(tile & 1) * kTile + tid - kTile] = aux_pending;
    else if (SEG && tid < 3 * kTile) lds_seg[(tile & 1) * kTile + tid - 2 * kTile] = __float_as_int(aux_pending);
  };

  f32x16 dk_acc[NB][NDB], dv_acc[NB][NDB];
#pragma unroll
  for (int nb = 0; nb < NB; ++nb)
#pragma unroll
    for (int db = 0; db < NDB; ++db) { dk_acc[nb][db] = splat16(0.f); dv_acc[nb][db] = splat16(0.f); }

  auto compute = [&](int j) __attribute__((always_inline)) {
    const uint16_t* qs = lds_q + (j & 1) * kTile * S;
    const uint16_t* gs = lds_g + (j & 1) * kTile * S;
    const float* nl = lds_nlse + (j & 1) * kTile;
    const float* nd = lds_ndel + (j & 1) * kTile;
    const int r0 = (tile0 + j) * kTile;
    const bool need_mask = p.causal && (r0 + p.coff < wkey0 + kWK - 1);  // a row of the tile lies before a key of this wave
    static_for<2>([&](auto mb_c) __attribute__((always_inline)) {
      constexpr int mb = decltype(mb_c)::value;
      // accumulator rows of this lane: 32 mb + 8 vq + 4 g + (0..3)
      f32x16 s[NB], dp[NB];
#pragma unroll
      for (int vq = 0; vq < 4; ++vq) {
        const f32x4 a = *reinterpret_cast<const f32x4*>(nl + 32 * mb + 8 * vq + 4 * g);
        const f32x4 d4 = *reinterpret_cast<const f32x4*>(nd + 32 * mb + 8 * vq + 4 * g);
#pragma unroll
        for (int nb = 0; nb < NB; ++nb)
#pragma unroll
          for (int e = 0; e < 4; ++e) { s[nb][4 * vq + e] = a[e]; dp[nb][4 * vq + e] = d4[e]; }
      }
      // the two independent chains alternate with their operands requested ahead, in a pinned order (see bwd_dq_kernel);
      // the index of the parked V fragments passes through an empty asm per row block: the compiler would otherwise keep
      // the first block's fragments for the second, which is the register pressure parking them is meant to take away
      int vf_idx = w * NB * NKS * 64 + l;  // (the index, not the pointer: a pointer out of an asm has lost its address space)
      asm volatile("" : "+v"(vf_idx));
      __builtin_amdgcn_sched_barrier(0);
      static_for<NKS>([&](auto kk_c) __attribute__((always_inline)) {
        constexpr int kk = decltype(kk_c)::value;
        const bf16x8 a = rows_frag<S>(qs, mb, kk, i, g);
        const bf16x8 a2 = rows_frag<S>(gs, mb, kk, i, g);
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) {
          s[nb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, kf[nb][kk], s[nb], 0, 0, 0);
          if constexpr (VLDS) {
            const bf16x8 vfrag = __builtin_bit_cast(bf16x8, lds_vf[vf_idx + (nb * NKS + kk) * 64]);
            dp[nb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a2, vfrag, dp[nb], 0, 0, 0);
          } else {
            dp[nb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a2, vf[nb][kk], dp[nb], 0, 0, 0);
          }
        }
      });
      {
        constexpr int RD = VLDS ? 2 + NB : 2;  // LDS reads per step
        constexpr int AHEAD = VLDS ? 1 : 2;    // steps whose operands are in flight (registers decide)
        __builtin_amdgcn_sched_group_barrier(0x100, AHEAD * RD, 0);
#pragma unroll
        for (int n = 0; n < NKS - AHEAD; ++n) {
          __builtin_amdgcn_sched_group_barrier(0x008, 2 * NB, 0);
          __builtin_amdgcn_sched_group_barrier(0x100, RD, 0);
        }
        __builtin_amdgcn_sched_group_barrier(0x008, 2 * AHEAD * NB, 0);
      }
      __builtin_amdgcn_sched_barrier(0);
      bf16x8 pf[NB][2], df[NB][2];
#pragma unroll
      for (int nb = 0; nb < NB; ++nb) {
        if (need_mask) {
          const int key = wkey0 + 32 * nb + i - p.coff;  // first row that sees this lane's key
#pragma unroll
          for (int v = 0; v < 16; ++v)
            if (r0 + 32 * mb + 8 * (v >> 2) + 4 * g + (v & 3) < key) s[nb][v] = -INFINITY;
        }
        if constexpr (SEG) {
          const int32_t* ids_p = lds_seg + (j & 1) * kTile + 32 * mb + 4 * g;
#pragma unroll
          for (int vq = 0; vq < 4; ++vq) {
            const int4 ids = *reinterpret_cast<const int4*>(ids_p + 8 * vq);
            if (ids.x != kseg[nb]) s[nb][4 * vq] = -INFINITY;
            if (ids.y != kseg[nb]) s[nb][4 * vq + 1] = -INFINITY;
            if (ids.z != kseg[nb]) s[nb][4 * vq + 2] = -INFINITY;
            if (ids.w != kseg[nb]) s[nb][4 * vq + 3] = -INFINITY;
          }
        }
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          s[nb][v] = __builtin_amdgcn_exp2f(s[nb][v]);  // p
          dp[nb][v] *= s[nb][v];                        // p * (dp - delta)
        }
        pack_block(s[nb], pf[nb][0], pf[nb][1]);
        pack_block(dp[nb], df[nb][0], df[nb][1]);
      }
      static_for<2 * NDB>([&](auto n_c) __attribute__((always_inline)) {
        constexpr int db = decltype(n_c)::value / 2, half = decltype(n_c)::value % 2;
        const bf16x8 a = cols_frag<S>(gs, 2 * mb + half, db, g, lp, dhalf);
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) dv_acc[nb][db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, pf[nb][half], dv_acc[nb][db], 0, 0, 0);
      });
      static_for<2 * NDB>([&](auto n_c) __attribute__((always_inline)) {
        constexpr int db = decltype(n_c)::value / 2, half = decltype(n_c)::value % 2;
        const bf16x8 a = cols_frag<S>(qs, 2 * mb + half, db, g, lp, dhalf);
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) dk_acc[nb][db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, df[nb][half], dk_acc[nb][db], 0, 0, 0);
      });
    });
  };

  if (ntiles > 0) {
    issue(0);
    commit(0);
    issue(min(1, last));
    __syncthreads();
    for (int j = 0; j < ntiles; ++j) {
      if (j >= wave_first_tile) compute(j);
      if (j + 1 < ntiles) {
        commit(j + 1);
        issue(min(j + 2, last));
      }
      lds_barrier();
    }
  }

#pragma unroll
  for (int nb = 0; nb < NB; ++nb) {
    const int key = wkey0 + 32 * nb + i;
    if (key < p.lk) {
      float* okp = p.dk + (((int64_t)b * p.lk + key) * p.H + h) * D;
      float* ovp = p.dv + (((int64_t)b * p.lk + key) * p.H + h) * D;
#pragma unroll
      for (int db = 0; db < NDB; ++db)
#pragma unroll
        for (int vq = 0; vq < 4; ++vq) {
          f32x4 ok, ov;
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            ok[e] = dk_acc[nb][db][4 * vq + e] * p.sm_scale;
            ov[e] = dv_acc[nb][db][4 * vq + e];
          }
          *reinterpret_cast<f32x4*>(okp + 32 * db + 8 * vq + 4 * g) = ok;
          *reinterpret_cast<f32x4*>(ovp + 32 * db + 8 * vq + 4 * g) = ov;
        }
    }
  }
}

// (batch, head) pairs of an XCD that run side by side: enough of them for about 64 workgroups (two rounds of an XCD's 32
// compute units, so that the heaviest blocks of a group start together) and eight pairs where there are as many (these
// kernels wait for LDS more than for memory: with fewer pairs side by side they lose 1 % at B = 4, T = 4096, H = 16),
// but not all pairs of the XCD where they are many (the workgroups resident together would all belong to different
// pairs and share nothing: B = 16, T = 1024, H = 16 takes 0.574 ms with 16 of its 32 pairs side by side, 0.620 with all;
// B = 8, T = 2048, H = 64, D = 64 not causal 2.25 against 2.44 ms)
inline int pair_group_of(int per_xcd, int nblk) {
  int g = (64 + nblk - 1) / nblk;
  if (g < 8) g = 8;
  return g < per_xcd ? g : per_xcd;
}

template <int D, int NW, int NB, bool SEG>
int launch_dq(const BwdParams& base, hipStream_t stream) {
  BwdParams p = base;
  p.nblk = (p.lq + NW * NB * 32 - 1) / (NW * NB * 32);
  p.npairs = p.nblk * p.B;
  const int per_xcd = (p.B * p.H + 7) / 8;
  p.pair_group = pair_group_of(per_xcd, p.nblk);
  const int64_t nwg = (int64_t)((per_xcd + p.pair_group - 1) / p.pair_group) * p.pair_group * p.nblk * 8;
  if (nwg > 2147483647LL) return TPA_ERR_SHAPE;
  auto kern = bwd_dq_kernel<D, NW, NB, SEG>;
  const size_t smem = (size_t)4 * kTile * tile_stride(D) * 2 + 2 * kTile * 4;
  static bool configured[kMaxDevices] = {};
  if (int rc = raise_lds_limit(configured, reinterpret_cast<const void*>(kern), smem); rc != TPA_OK) return rc;
  hipLaunchKernelGGL(kern, dim3((unsigned)nwg), dim3(NW * 64), smem, stream, p);
  return hipGetLastError() == hipSuccess ? TPA_OK : TPA_ERR_LAUNCH;
}

template <int D, int NW, int NB, bool SEG>
int launch_dkv(const BwdParams& base, hipStream_t stream) {
  BwdParams p = base;
  p.nblk = (p.lk + NW * NB * 32 - 1) / (NW * NB * 32);
  p.npairs = p.nblk * p.B;
  const int per_xcd = (p.B * p.H + 7) / 8;
  p.pair_group = pair_group_of(per_xcd, p.nblk);
  const int64_t nwg = (int64_t)((per_xcd + p.pair_group - 1) / p.pair_group) * p.pair_group * p.nblk * 8;
  if (nwg > 2147483647LL) return TPA_ERR_SHAPE;
  auto kern = bwd_dkv_kernel<D, NW, NB, SEG>;
  const size_t smem = (size_t)4 * kTile * tile_stride(D) * 2 + 6 * kTile * 4 + (dkv_v_in_lds(D) ? (size_t)NW * NB * (D / 16) * 64 * 16 : 0);
  static bool configured[kMaxDevices] = {};
  if (int rc = raise_lds_limit(configured, reinterpret_cast<const void*>(kern), smem); rc != TPA_OK) return rc;
  hipLaunchKernelGGL(kern, dim3((unsigned)nwg), dim3(NW * 64), smem, stream, p);
  return hipGetLastError() == hipSuccess ? TPA_OK : TPA_ERR_LAUNCH;
}

template <int D>
int launch_both(const BwdParams& p, hipStream_t stream) {
  // dK/dV: 8 waves of 32 keys.  (64 keys per wave would halve the LDS reads per MFMA, but its 384
  // stationary registers at D = 128 leave the compiler spilling.)
  // (measured at D = 128: the dQ kernel with 4 waves of 64 rows, one wave per SIMD and 512 registers, takes
  // 922 us where 8 waves of 32 rows take 401 us)
  constexpr int NW = 8, NB = 1;
  constexpr int QNW = 8, QNB = 1;
  int rc;
  if (p.qseg) {
    rc = launch_dq<D, QNW, QNB, true>(p, stream);
    if (rc == TPA_OK) rc = launch_dkv<D, NW, NB, true>(p, stream);
  } else {
    rc = launch_dq<D, QNW, QNB, false>(p, stream);
    if (rc == TPA_OK) rc = launch_dkv<D, NW, NB, false>(p, stream);
  }
  return rc;
}

}  // namespace
}  // namespace tpa

// dense bf16 q, k, v, d_o [B, l, H, D] with D in {64, 128}; every batch entry below 2 GiB
int dense_bwd_mfma_supported(int dtype, int dk, int dv, int64_t lq, int64_t lk, int64_t H, float sm_scale, const void* bias) {
  if (dtype != TPA_DTYPE_BF16 || dk != dv || (dk != 64 && dk != 128) || bias) return 0;
  if (!(sm_scale > 0.f)) return 0;
  const int64_t big = lq > lk ? lq : lk;
  if (big * H * dk * 2 >= (int64_t(1) << 31)) return 0;
  return 1;
}

int dense_bwd_mfma_launch(const void* q, const void* k, const void* v, const void* d_o, const float* lse, const float* delta,
                          const int32_t* qseg, const int32_t* kvseg, float* dq, float* dk, float* dv, int B, int lq, int lk,
                          int H, int D, float sm_scale, int causal, int coff, hipStream_t stream) {
  tpa::BwdParams p{};
  p.q = static_cast<const uint16_t*>(q); p.k = static_cast<const uint16_t*>(k); p.v = static_cast<const uint16_t*>(v);
  p.d_o = static_cast<const uint16_t*>(d_o); p.lse = lse; p.delta = delta; p.qseg = qseg; p.kvseg = kvseg;
  p.dq = dq; p.dk = dk; p.dv = dv; p.B = B; p.lq = lq; p.lk = lk; p.H = H; p.sm_scale = sm_scale; p.causal = causal; p.coff = causal ? coff : 0;
  if (D == 128) return tpa::launch_both<128>(p, stream);
  return tpa::launch_both<64>(p, stream);
}
