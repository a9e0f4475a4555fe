// Flash-style prefill for gfx950: bf16 MFMA contractions, fp32 online softmax.
//
// One workgroup = one (batch, head, block of 256 query rows), i.e. eight blocks of 32 rows, held
// either by eight waves (two per SIMD) of one row block each (RB = 1) or by four waves (one per
// SIMD, 512 registers) of two row blocks each (RB = 2): a wave then feeds every K / V fragment it
// reads from LDS to two MFMAs, which halves the LDS traffic per MFMA - with one row block per wave
// the LDS read port (128 B/clk, 76 for transposed reads) is as busy as the matrix pipe.  A wave's
// two row blocks are w and 7 - w, so that the waves do equal work on the causal diagonal.
// Per tile of 64 keys the workgroup rebuilds the head's K and V
// tile from the rank factors (K = (1/R) sum_r a_r (x) b_r, tpa/tpa.py:364,417) straight out of
// coalesced 16-byte factor loads and stores it once, as bf16, in LDS.  Each wave then computes
//     S^T = K Q^T        (v_mfma_f32_32x32x16_bf16, A = K rows from LDS, B = Q kept in registers,
//                         Q pre-scaled by sm_scale*log2(e) and the accumulator started at minus
//                         the running reference, so the result is the exponent itself)
//     online softmax     (each lane holds 32 logits of ONE query row, so the row max and sum
//                         are in-lane apart from one exchange with lane ^ 32)
//     O^T += V^T P^T     (A = V^T read with ds_read_b64_tr_b16 from row-major V, B = P^T, which
//                         is the S^T accumulator converted in place: no LDS round trip for P)
// with the deferred normalisation of flash attention (a reference m and a sum l per row), which
// is the normalise-every-step recurrence of tpa/tpa.py:389-424 in another order of operations.
// There is one workgroup barrier per tile (K, V and the head factors are double buffered in
// LDS).  On tiles that need no mask a wave runs everything as ONE instruction stream in which
// each MFMA is followed by a short slice of independent vector work: the softmax of a 32-key
// block runs in the shadow of the MFMAs of the next block, the rebuild of the next K/V tile in
// the shadow of the first S^T and the last O^T MFMAs.  (A vector instruction issued while a
// matrix instruction of the same wave executes is nearly free on this hardware, whereas two
// waves of a SIMD that are both in a vector-only or both in a matrix-only phase just queue up;
// the dot instruction is the exception: it occupies the matrix pipe.)
// The dense flash baseline (tpa/mha.py:23-37) is the same kernel with a plain K/V loader.
#include <stdlib.h>

#include <type_traits>
#include <utility>

#include "tpa_common.h"

namespace tpa {
namespace {

constexpr int kTK = 64;   // keys per tile
constexpr int kBQ = 256;  // query rows per workgroup: 8 blocks of 32, RB of them per wave

enum { LOAD_TPA_R2 = 0, LOAD_TPA_ANY = 1, LOAD_DENSE = 2 };

struct PrefillParams {
  TpaFactor qa, qb, ka, kb, va, vb;  // dense: qb/kb/vb hold q/k/v with stride_l = H*D, ptr at head 0
  const int32_t* qseg;   // [B, lq] or null
  const int32_t* kvseg;  // [B, lk] or null (both or neither)
  const int32_t* kvlen;  // [B] keys per batch entry, or null (= lk)
  uint16_t* o;
  float* lse;
  int B, lq, lk, H, rq, rk;
  float sm_scale;
  int causal;
  int coff;         // with causal: row i sees keys <= i + coff (0 = top-left aligned)
  int nqb;     // query blocks per (batch, head)
  int npairs;  // nqb * B
  int q_scaled;   // dense loader only: 1 = q already holds sm_scale * log2(e) * Q (it was reconstructed with that factor)
};

// LDS: three buffers of a K tile (tile j is read while tile j+1 is already there for waves that run
// a tile ahead with their logits, and tile j+2 is being written), two of a V tile, two slots of head
// factors and two of key segment ids: [K0][K1][K2][V0][V1][A0][A1][seg0][seg1], offsets in uint16 units.
template <int D>
struct Lds {
  static constexpr int KS = D + 8;   // K row stride (elements): 16-byte reads of 16 rows hit distinct banks
  static constexpr int VS = D + 32;  // V row stride: 4 consecutive rows of a transposed read hit distinct banks
  static constexpr int kK = kTK * KS;  // elements of one K buffer
  static constexpr int kV = kTK * VS;  // elements of one V buffer
  static constexpr int kA = 2 * kTK * 2;  // one slot of head factors: [K|V][token][rank 0|1]
  static constexpr int kSeg = 2 * kTK;    // one slot of key segment ids (int32), in uint16 units
  static constexpr int k_off(int buf) { return buf * kK; }
  static constexpr int v_off(int buf) { return 3 * kK + buf * kV; }
  static constexpr int a_off(int buf) { return 3 * kK + 2 * kV + buf * kA; }
  static constexpr int seg_off(int buf) { return 3 * kK + 2 * kV + 2 * kA + buf * kSeg; }
  static constexpr size_t kBytes = (3 * kK + 2 * (kV + kA + kSeg)) * sizeof(uint16_t);
};

// a0*b0 + a1*b1 on packed bf16 pairs, fp32 result.  Through the builtin on purpose: the dot
// instructions need software wait states before a dependent VALU instruction, which the compiler
// only inserts for instructions it selected itself (not for inline assembly).
__device__ __forceinline__ float dot2_bf16(uint32_t pair, uint32_t aa) {
  return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, pair), __builtin_bit_cast(bf16x2, aa), 0.f, false);
}

__device__ __forceinline__ float dot2_bf16_acc(uint32_t pair, uint32_t aa, float c) {
  return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, pair), __builtin_bit_cast(bf16x2, aa), c, false);
}

// Workgroup barrier that waits for this wave's LDS traffic only.  __syncthreads() would also
// wait for the global loads of the next tile's factors, which are meant to stay in flight.
__device__ __forceinline__ void lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

// compile-time loop: f(std::integral_constant<int, 0>{}), ..., f(std::integral_constant<int, N-1>{})
template <typename F, int... I>
__device__ __forceinline__ void static_for_impl(F&& f, std::integer_sequence<int, I...>) {
  (f(std::integral_constant<int, I>{}), ...);
}
template <int N, typename F>
__device__ __forceinline__ void static_for(F&& f) {
  static_for_impl(f, std::make_integer_sequence<int, N>{});
}
template <int V>
using IC = std::integral_constant<int, V>;

template <int D, int LOADER, bool SEG, int RB>
__global__ __launch_bounds__((8 / RB) * 64) void prefill_kernel(PrefillParams pp) {
  static_assert(RB == 1, "one block of 32 query rows per wave");
  constexpr int kNW = 8 / RB;  // waves per workgroup
  constexpr int NT = kNW * 64;
  using L = Lds<D>;
  constexpr int KS = L::KS, VS = L::VS;
  constexpr int CPR = D / 8;             // 16-byte chunks per row
  constexpr int TPP = NT / CPR;          // tokens per loader pass
  constexpr int NPASS = kTK / TPP;       // loader passes per tile and matrix
  static_assert(kTK % TPP == 0 && NPASS >= 1, "loader shape");
  constexpr int NKS = D / 16;            // k-steps of the QK^T contraction
  constexpr int NDB = D / 32;            // 32-row blocks of O^T
  constexpr float kSlack = 8.f;          // the reference only moves when a tile max exceeds it by 2^8

  // scalars out of the argument block (never take the address of the block itself)
  struct Fac { const uint16_t* ptr; int64_t stride_b; int stride_l, stride_r; };
  auto fac = [](const TpaFactor& f) { return Fac{static_cast<const uint16_t*>(f.ptr), f.stride_b, (int)f.stride_l, (int)f.stride_r}; };
  struct { Fac qa, qb, ka, kb, va, vb; const int32_t* qseg; const int32_t* kvseg; const int32_t* kvlen; uint16_t* o; float* lse; int B, lq, lk, H, rq, rk; float sm_scale; int causal, coff, nqb, npairs, q_scaled; } const p = {
      fac(pp.qa), fac(pp.qb), fac(pp.ka), fac(pp.kb), fac(pp.va), fac(pp.vb), pp.qseg, pp.kvseg, pp.kvlen, pp.o, pp.lse, pp.B, pp.lq, pp.lk, pp.H, pp.rq, pp.rk,
      pp.sm_scale, pp.causal, pp.causal ? pp.coff : 0, pp.nqb, pp.npairs, pp.q_scaled};

  extern __shared__ __attribute__((aligned(16))) uint16_t smem[];
  auto lds_k = [&](int buf) __attribute__((always_inline)) { return smem + L::k_off(buf); };    // [kTK][KS]
  auto lds_v = [&](int buf) __attribute__((always_inline)) { return smem + L::v_off(buf); };    // [kTK][VS]
  auto lds_a = [&](int buf) __attribute__((always_inline)) { return smem + L::a_off(buf); };    // [K|V][kTK][2]
  auto lds_seg = [&](int buf) __attribute__((always_inline)) { return reinterpret_cast<int32_t*>(smem + L::seg_off(buf)); };  // [kTK]

  // ---- which (query block, batch, head): heads of one (block, batch) pair sit on one XCD
  // (workgroup ids are dealt round-robin to the 8 XCDs) so they share the B-factor tiles in
  // that XCD's L2; pairs are ordered heaviest (last causal block) first.
  const int id = blockIdx.x;
  const int xcd = id & 7, slot = id >> 3;
  int h, b, qblk;
  if constexpr (LOADER == LOAD_DENSE) {
    // Dense K and V belong to one (batch, head): what workgroups can share is the K/V stream of
    // their head.  An XCD therefore owns whole (batch, head) pairs and runs their query blocks
    // heaviest first, the same block of all its pairs side by side: the 32 workgroups that are
    // resident together are neighbouring query blocks of a few pairs, which walk the same tiles
    // at about the same time and find them in that XCD's L2.
    const int per_xcd = (p.B * p.H + 7) / 8;
    const int bh = (slot % per_xcd) * 8 + xcd;
    if (bh >= p.B * p.H) return;
    qblk = p.nqb - 1 - slot / per_xcd;
    b = bh / p.H;
    h = bh % p.H;
  } else {
    const int round = slot / p.H;
    const int pair = round * 8 + xcd_pair_slot(round, xcd, p.B);
    h = slot % p.H;
    if (pair >= p.npairs) return;
    qblk = p.nqb - 1 - pair / p.B;
    b = pair % p.B;
  }

  const int tid = threadIdx.x;
  const int w = tid >> 6, l = tid & 63, i = l & 31, g = l >> 5;
  const int q0 = qblk * kBQ;
  // row block r of this wave within the workgroup's eight: w, and (RB = 2) 7 - w
  int rblk[RB], wrow0[RB], qrow[RB], qrow_ld[RB];
#pragma unroll
  for (int r = 0; r < RB; ++r) {
    rblk[r] = r == 0 ? w : 7 - w;
    wrow0[r] = q0 + 32 * rblk[r];  // first query row of the block
    qrow[r] = wrow0[r] + i;        // this lane's row in it
    qrow_ld[r] = min(qrow[r], p.lq - 1);
  }
  const float c = (LOADER == LOAD_DENSE && p.q_scaled) ? 1.f : p.sm_scale * kLog2e;

  // ---- Q fragments (B operand of S^T = K Q^T), scaled by c: lane (i, g) holds
  // c * Q[qrow[r]][16ks + 8g + 0..7]
  bf16x8 qf[RB][NKS];
  auto build_q = [&]() __attribute__((always_inline)) {
    // the dense loader serves dense attention and factored attention whose Q, K and V were
    // reconstructed beforehand (Q with its scale factor, so that it is rounded to bf16 once)
    if constexpr (LOADER == LOAD_DENSE) {
#pragma unroll
      for (int r = 0; r < RB; ++r) {
        const uint16_t* qp = p.qb.ptr + b * p.qb.stride_b + (int64_t)qrow_ld[r] * p.qb.stride_l + (int64_t)h * D;
#pragma unroll
        for (int ks = 0; ks < NKS; ++ks) {
          const u32x4 raw = *reinterpret_cast<const u32x4*>(qp + 16 * ks + 8 * g);
          u32x4 sc;
#pragma unroll
          for (int j = 0; j < 4; ++j) sc[j] = pack_bf16(bf16lo_to_f32(raw[j]) * c, bf16hi_to_f32(raw[j]) * c);
          qf[r][ks] = __builtin_bit_cast(bf16x8, sc);
        }
      }
    } else {
      // One rank at a time through LDS: the workgroup copies the 256 x D slab qb[q0.., r, :] with
      // coalesced 16-byte loads (each row is read once, not once per lane pair), then every lane
      // picks up its own row's fragments.  The next rank's loads are in flight meanwhile.
      constexpr int QS = D + 8;                  // row stride in LDS (elements)
      constexpr int CH = kBQ * CPR / NT;         // 16-byte chunks per thread and rank
      uint16_t* const qs = smem;                 // [kBQ][QS]
      uint16_t* const qas = smem + kBQ * QS;     // [kBQ] head factors of this rank
      static_assert((kBQ * QS + kBQ) * sizeof(uint16_t) <= L::kBytes, "Q staging fits the K/V buffers");
      const uint16_t* qb_b = p.qb.ptr + b * p.qb.stride_b;
      const uint16_t* qa_b = p.qa.ptr + b * p.qa.stride_b + h;
      u32x4 nxt[CH];
      uint32_t a_nxt = 0;
      auto load_rank = [&](int r) __attribute__((always_inline)) {
#pragma unroll
        for (int q = 0; q < CH; ++q) {
          const int chunk = q * NT + tid, row = chunk / CPR, cc = chunk % CPR;
          const int grow = min(q0 + row, p.lq - 1);
          nxt[q] = *reinterpret_cast<const u32x4*>(qb_b + (int64_t)grow * p.qb.stride_l + r * p.qb.stride_r + 8 * cc);
        }
        if (tid < kBQ) a_nxt = qa_b[(int64_t)min(q0 + tid, p.lq - 1) * p.qa.stride_l + r * p.qa.stride_r];
      };
      float acc[RB][NKS][8];
#pragma unroll
      for (int rb = 0; rb < RB; ++rb)
#pragma unroll
        for (int ks = 0; ks < NKS; ++ks)
#pragma unroll
          for (int j = 0; j < 8; ++j) acc[rb][ks][j] = 0.f;
      load_rank(0);
      for (int r = 0; r < p.rq; ++r) {
#pragma unroll
        for (int q = 0; q < CH; ++q) {
          const int chunk = q * NT + tid, row = chunk / CPR, cc = chunk % CPR;
          *reinterpret_cast<u32x4*>(qs + row * QS + 8 * cc) = nxt[q];
        }
        if (tid < kBQ) qas[tid] = (uint16_t)a_nxt;
        if (r + 1 < p.rq) load_rank(r + 1);
        lds_barrier();
        // a * b[d] for a packed pair (b[d], b[d+1]) is one dot instruction with (a, 0) or (0, a):
        // no unpacking, and the dot unit is idle here anyway
#pragma unroll
        for (int rb = 0; rb < RB; ++rb) {
          const int row = 32 * rblk[rb] + i;
          const uint32_t a_lo = qas[row], a_hi = a_lo << 16;
#pragma unroll
          for (int ks = 0; ks < NKS; ++ks) {
            const u32x4 bv = *reinterpret_cast<const u32x4*>(qs + row * QS + 16 * ks + 8 * g);
#pragma unroll
            for (int j = 0; j < 4; ++j) {
              uint32_t pair = bv[j];
              asm volatile("" : "+v"(pair));  // keeps the compiler from taking element 0 of the vector for every j
              acc[rb][ks][2 * j] = dot2_bf16_acc(pair, a_lo, acc[rb][ks][2 * j]);
              acc[rb][ks][2 * j + 1] = dot2_bf16_acc(pair, a_hi, acc[rb][ks][2 * j + 1]);
            }
          }
        }
        lds_barrier();  // everyone has read this rank before the next one overwrites it
      }
      const float scale = c / (float)p.rq;
#pragma unroll
      for (int rb = 0; rb < RB; ++rb)
#pragma unroll
        for (int ks = 0; ks < NKS; ++ks) {
          u32x4 packed;
#pragma unroll
          for (int j = 0; j < 4; ++j) packed[j] = pack_bf16(acc[rb][ks][2 * j] * scale, acc[rb][ks][2 * j + 1] * scale);
          qf[rb][ks] = __builtin_bit_cast(bf16x8, packed);
        }
    }
  };

  // ---- key range [kpos0, kend) this workgroup visits; tiles are counted from kpos0
  int kpos0 = 0;
  const int len_b = p.kvlen ? max(0, min(p.kvlen[b], p.lk)) : p.lk;  // keys of this batch entry
  // causal offset of this batch entry: counted from the end of its keys where the caller aligns the last
  // query with the last key
  const int coff = p.coff + (p.causal == TPA_CAUSAL_BOTTOM_RIGHT ? len_b - p.lq : 0);
  int kend = p.causal ? min(len_b, min(q0 + kBQ, p.lq) + coff) : len_b;
  if (kend <= 0) {  // no key at all: the rows end as NaN / -inf (tpa/tpa.py:437-439)
#pragma unroll
    for (int r = 0; r < RB; ++r)
      if (qrow[r] < p.lq) {
        uint16_t* op = p.o + (((int64_t)b * p.lq + qrow[r]) * p.H + h) * D;
        const u32x4 nan4 = {0x7fc07fc0u, 0x7fc07fc0u, 0x7fc07fc0u, 0x7fc07fc0u};
#pragma unroll
        for (int cch = 0; cch < D / 16; ++cch) *reinterpret_cast<u32x4*>(op + 16 * cch + 8 * g) = nan4;
        if (p.lse && g == 0) p.lse[((int64_t)b * p.H + h) * p.lq + qrow[r]] = -INFINITY;
      }
    return;
  }
  bool seg_pure = false;  // every visited key from the second tile on carries the rows' one segment id
  if constexpr (SEG) {
    // Packed sequences: a key can only be visible to this block if its id lies within the
    // [min, max] of the block's query ids.  The workgroup scans the key ids once, keeps the first
    // and the last such key, and visits only the tiles between them (exact for ids that do not
    // decrease along the sequence; any other id pattern just visits more tiles, the mask itself
    // is applied per key as before).  If the rows share one id and the keys with that id form one
    // contiguous run, the tiles inside the run need no segment mask at all.
    int32_t* const red = reinterpret_cast<int32_t*>(smem);
    if (tid == 0) { red[0] = INT32_MAX; red[1] = INT32_MIN; red[2] = INT32_MAX; red[3] = -1; red[4] = 0; }
    __syncthreads();
    if (tid < kBQ && q0 + tid < p.lq) {
      const int32_t sid = p.qseg[(int64_t)b * p.lq + q0 + tid];
      __hip_atomic_fetch_min(&red[0], sid, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
      __hip_atomic_fetch_max(&red[1], sid, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    }
    __syncthreads();
    const int32_t qmin = red[0], qmax = red[1];
    int lo = INT32_MAX, hi = -1, cnt = 0;
    auto visit = [&](int t, int32_t sid) __attribute__((always_inline)) {
      if (sid >= qmin && sid <= qmax) { lo = min(lo, t); hi = max(hi, t); ++cnt; }
    };
    const int32_t* const kid = p.kvseg + (int64_t)b * p.lk;
    // four ids per load and four loads in flight per thread where the row of ids is 16-byte aligned
    const int kv4 = (reinterpret_cast<uintptr_t>(kid) & 15) == 0 ? (kend & ~3) : 0;
    constexpr int U = 4;
    for (int base = 4 * tid; base < kv4; base += 4 * NT * U) {
      int4 ids[U];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int t = base + 4 * NT * u;
        ids[u] = *reinterpret_cast<const int4*>(kid + (t < kv4 ? t : 0));
      }
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int t = base + 4 * NT * u;
        if (t < kv4) { visit(t, ids[u].x); visit(t + 1, ids[u].y); visit(t + 2, ids[u].z); visit(t + 3, ids[u].w); }
      }
    }
    for (int t = kv4 + tid; t < kend; t += NT) visit(t, kid[t]);
    if (cnt) {
      __hip_atomic_fetch_min(&red[2], lo, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
      __hip_atomic_fetch_max(&red[3], hi, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
      __hip_atomic_fetch_add(&red[4], cnt, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    }
    __syncthreads();
    lo = red[2]; hi = red[3]; cnt = red[4];
    __syncthreads();  // the staging below reuses this memory
    if (hi >= 0) {
      kpos0 = lo / kTK * kTK;
      kend = hi + 1;
      seg_pure = qmin == qmax && cnt == hi - lo + 1;
    } else {
      kend = min(kend, kTK);  // nothing visible: one (fully masked) tile, the rows end as NaN / -inf
    }
  }
  const int lk_r = kend - kpos0;          // keys counted from kpos0
  const int ntiles = (lk_r + kTK - 1) / kTK;
  const int last = ntiles - 1;
  // first row of each of this wave's row blocks and this lane's row in it on that scale, shifted by
  // the causal offset: row x sees keys up to x_r, which is negative for a row that sees none;
  // last tile the block needs under the causal mask (its rows: wrow0 .. wrow0 + 31)
  int wrow_r[RB], qrow_r[RB], wave_last_tile[RB];
#pragma unroll
  for (int r = 0; r < RB; ++r) {
    wrow_r[r] = wrow0[r] + coff - kpos0;
    qrow_r[r] = qrow[r] + coff - kpos0;
    wave_last_tile[r] = p.causal ? min(last, max(wrow_r[r] + 31, 0) / kTK) : last;
  }

  // ---- loader: this thread rebuilds chunk lc (8 elements) of token lt (+ TPP per pass).
  // Addresses are a uniform (scalar) tile base plus a per-thread 32-bit element offset.
  const int lt = tid / CPR, lc = tid % CPR;
  u32x4 kreg[NPASS][2], vreg[NPASS][2];  // LOAD_TPA_R2: two ranks; LOAD_DENSE: [0] only

  // all key-side bases point at key kpos0
  const uint16_t* const kb_b = p.kb.ptr + b * p.kb.stride_b + (int64_t)kpos0 * p.kb.stride_l + (LOADER == LOAD_DENSE ? (int64_t)h * D : 0);
  const uint16_t* const vb_b = p.vb.ptr + b * p.vb.stride_b + (int64_t)kpos0 * p.vb.stride_l + (LOADER == LOAD_DENSE ? (int64_t)h * D : 0);
  const uint16_t* const ka_b = p.ka.ptr + b * p.ka.stride_b + (int64_t)kpos0 * p.ka.stride_l + h;
  const uint16_t* const va_b = p.va.ptr + b * p.va.stride_b + (int64_t)kpos0 * p.va.stride_l + h;

  // B-factor loads of one matrix (K or V) for one tile into registers.  They are raw buffer
  // loads: resource = this batch entry's matrix (in scalar registers), scalar offset = (tile,
  // pass, rank), vector offset = this thread's fixed place inside a pass - no vector instruction
  // is spent on addresses, and rows past the end of the sequence read as zero (the range check
  // of the resource), so a ragged last tile needs no clamping.
  constexpr int kRsrcFlags = 0x00020000;  // raw 32-bit data format
  const int k_rows_bytes = ((lk_r - 1) * p.kb.stride_l + (LOADER == LOAD_TPA_R2 ? p.kb.stride_r : 0) + D) * 2;
  const int v_rows_bytes = ((lk_r - 1) * p.vb.stride_l + (LOADER == LOAD_TPA_R2 ? p.vb.stride_r : 0) + D) * 2;
  const __amdgpu_buffer_rsrc_t kb_rs = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint16_t*>(kb_b), 0, k_rows_bytes, kRsrcFlags);
  const __amdgpu_buffer_rsrc_t vb_rs = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint16_t*>(vb_b), 0, v_rows_bytes, kRsrcFlags);
  const int kvoff = (lt * p.kb.stride_l + 8 * lc) * 2, vvoff = (lt * p.vb.stride_l + 8 * lc) * 2;
  auto issue_into = [&](u32x4 (&regs)[NPASS][2], auto is_v_c, int tile) __attribute__((always_inline)) {
    constexpr bool is_v = decltype(is_v_c)::value;
    if constexpr (LOADER == LOAD_TPA_ANY) return;
    const int sl = is_v ? p.vb.stride_l : p.kb.stride_l, sr = is_v ? p.vb.stride_r : p.kb.stride_r;
#pragma unroll
    for (int ps = 0; ps < NPASS; ++ps) {
      const int soff = (tile * kTK + ps * TPP) * sl * 2;  // uniform
      regs[ps][0] = __builtin_amdgcn_raw_buffer_load_b128(is_v ? vb_rs : kb_rs, is_v ? vvoff : kvoff, soff, 0);
      if constexpr (LOADER == LOAD_TPA_R2) regs[ps][1] = __builtin_amdgcn_raw_buffer_load_b128(is_v ? vb_rs : kb_rs, is_v ? vvoff : kvoff, soff + 2 * sr, 0);
    }
  };
  auto issue = [&](auto is_v_c, int tile) __attribute__((always_inline)) {
    if constexpr (decltype(is_v_c)::value) issue_into(vreg, is_v_c, tile); else issue_into(kreg, is_v_c, tile);
  };
  using IsK = std::integral_constant<bool, false>;
  using IsV = std::integral_constant<bool, true>;

  // Head factors (LOAD_TPA_R2): a thread fetches one value a[matrix][token][rank], matrix = (tid % 256) / 128
  // (0: K of tile kt, 1: V of tile vt), token = (tid / 2) % 64, rank = tid % 2, and parks it in a register
  // until it is stored into an LDS slot one iteration later.  Waves 4-7 repeat what waves 0-3 do (same
  // values to the same addresses), so that the eight waves run one instruction stream.
  uint32_t a_pending = 0;
  const int a_idx = tid & (4 * kTK - 1);
  const int a_mat = a_idx / (2 * kTK), a_tok = (a_idx >> 1) % kTK, a_rank = a_idx & 1;
  const int ka_bytes = ((lk_r - 1) * p.ka.stride_l + p.ka.stride_r + 1) * 2, va_bytes = ((lk_r - 1) * p.va.stride_l + p.va.stride_r + 1) * 2;
  const __amdgpu_buffer_rsrc_t ka_rs = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint16_t*>(ka_b), 0, ka_bytes, kRsrcFlags);
  const __amdgpu_buffer_rsrc_t va_rs = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint16_t*>(va_b), 0, va_bytes, kRsrcFlags);
  const int ka_voff = (a_tok * p.ka.stride_l + a_rank * p.ka.stride_r) * 2, va_voff = (a_tok * p.va.stride_l + a_rank * p.va.stride_r) * 2;
  auto issue_a = [&](int kt, int vt) __attribute__((always_inline)) {
    if constexpr (LOADER != LOAD_TPA_R2) return;
    // waves 0, 1 (4, 5) fetch K's head factors, waves 2, 3 (6, 7) V's (uniform per wave); tokens past the end read as 0
    if (a_mat == 0) a_pending = __builtin_amdgcn_raw_buffer_load_b16(ka_rs, ka_voff, kt * kTK * p.ka.stride_l * 2, 0);
    else a_pending = __builtin_amdgcn_raw_buffer_load_b16(va_rs, va_voff, vt * kTK * p.va.stride_l * 2, 0);
  };
  auto store_a = [&](int slot_idx) __attribute__((always_inline)) {
    if constexpr (LOADER != LOAD_TPA_R2) return;
    // stored halved (exact in bf16): the 1/R of the reconstruction with R = 2
    lds_a(slot_idx)[a_idx] = (uint16_t)(pack_bf16(bf16lo_to_f32(a_pending) * 0.5f, 0.f));
  };

  // Key segment ids (packed sequences, tpa/tpa.py:369-375): the threads of one wave (wave 4 where
  // there are eight, else wave 0) fetch one id of a tile each, park it in a register and store it
  // into an LDS slot one iteration later, like the head factors; slot j&1 holds the ids of tile j
  // during iteration j.
  constexpr bool has_seg = SEG;  // a kernel of its own: the mask code slows the others down even when skipped
  constexpr int kSegWave = kNW > 4 ? 4 : 0;
  int32_t seg_pending = 0;
  auto issue_seg = [&](int tile) __attribute__((always_inline)) {
    if constexpr (has_seg)
      if (w == kSegWave) seg_pending = p.kvseg[(int64_t)b * p.lk + kpos0 + min(tile * kTK + l, lk_r - 1)];
  };
  auto store_seg = [&](int slot_idx) __attribute__((always_inline)) {
    if constexpr (has_seg)
      if (w == kSegWave) lds_seg(slot_idx)[l] = seg_pending;
  };
  int32_t qseg[RB] = {};
  if constexpr (has_seg) {
#pragma unroll
    for (int r = 0; r < RB; ++r) qseg[r] = p.qseg[(int64_t)b * p.lq + qrow_ld[r]];
  }

  // (a0/2)*b0[d] + (a1/2)*b1[d] for 8 consecutive d; aa = packed (a0/2, a1/2): fetch_aa hands out
  // halved head factors.
  // Three short assembly pieces, so that they can sit between MFMAs: 8 v_perm_b32 (pair b0[d]
  // with b1[d]), 8 v_dot2_f32_bf16 (the VOP3P form with a zero addend, so no accumulator has to
  // be cleared first) and 4 v_cvt_pk_bf16_f32.  A dot result may only be read by another
  // vector-ALU instruction three wait states later and the hardware does not interlock; the
  // s_nop at the head of the last piece guarantees them whatever was scheduled in between.
  struct Chunk { uint32_t t0, t1, t2, t3, t4, t5, t6, t7; };
  auto rebuild_perm = [&](Chunk& c_, const u32x4& b0, const u32x4& b1) __attribute__((always_inline)) {
    const uint32_t sel_lo = 0x05040100u, sel_hi = 0x07060302u;
    asm volatile(
        "v_perm_b32 %0, %9, %8, %16\n\t"   // (b0[0], b1[0])
        "v_perm_b32 %1, %9, %8, %17\n\t"   // (b0[1], b1[1])
        "v_perm_b32 %2, %11, %10, %16\n\t"
        "v_perm_b32 %3, %11, %10, %17\n\t"
        "v_perm_b32 %4, %13, %12, %16\n\t"
        "v_perm_b32 %5, %13, %12, %17\n\t"
        "v_perm_b32 %6, %15, %14, %16\n\t"
        "v_perm_b32 %7, %15, %14, %17"
        : "=&v"(c_.t0), "=&v"(c_.t1), "=&v"(c_.t2), "=&v"(c_.t3), "=&v"(c_.t4), "=&v"(c_.t5), "=&v"(c_.t6), "=&v"(c_.t7)
        : "v"(b0[0]), "v"(b1[0]), "v"(b0[1]), "v"(b1[1]), "v"(b0[2]), "v"(b1[2]), "v"(b0[3]), "v"(b1[3]), "s"(sel_lo), "s"(sel_hi));
  };
  auto rebuild_dot = [&](Chunk& c_, uint32_t aa) __attribute__((always_inline)) {
    asm volatile(
        "v_dot2_f32_bf16 %0, %0, %8, 0\n\t"
        "v_dot2_f32_bf16 %1, %1, %8, 0\n\t"
        "v_dot2_f32_bf16 %2, %2, %8, 0\n\t"
        "v_dot2_f32_bf16 %3, %3, %8, 0\n\t"
        "v_dot2_f32_bf16 %4, %4, %8, 0\n\t"
        "v_dot2_f32_bf16 %5, %5, %8, 0\n\t"
        "v_dot2_f32_bf16 %6, %6, %8, 0\n\t"
        "v_dot2_f32_bf16 %7, %7, %8, 0"
        : "+v"(c_.t0), "+v"(c_.t1), "+v"(c_.t2), "+v"(c_.t3), "+v"(c_.t4), "+v"(c_.t5), "+v"(c_.t6), "+v"(c_.t7)
        : "v"(aa));
  };
  auto rebuild_cvt = [&](Chunk& c_) __attribute__((always_inline)) -> u32x4 {
    asm volatile(
        "s_nop 2\n\t"
        "v_cvt_pk_bf16_f32 %0, %0, %1\n\t"
        "v_cvt_pk_bf16_f32 %2, %2, %3\n\t"
        "v_cvt_pk_bf16_f32 %4, %4, %5\n\t"
        "v_cvt_pk_bf16_f32 %6, %6, %7"
        : "+v"(c_.t0), "+v"(c_.t1), "+v"(c_.t2), "+v"(c_.t3), "+v"(c_.t4), "+v"(c_.t5), "+v"(c_.t6), "+v"(c_.t7));
    return u32x4{c_.t0, c_.t2, c_.t4, c_.t6};
  };
  // halve a packed (a0, a1) pair (exact in bf16): 1/R with R = 2
  auto halve_pair = [&](uint32_t aa_bits) __attribute__((always_inline)) -> uint32_t {
    return pack_bf16(bf16lo_to_f32(aa_bits) * 0.5f, bf16hi_to_f32(aa_bits) * 0.5f);
  };
  auto rebuild_r2 = [&](const u32x4& b0, const u32x4& b1, uint32_t aa_bits) __attribute__((always_inline)) -> u32x4 {
    Chunk c_;
    rebuild_perm(c_, b0, b1);
    rebuild_dot(c_, aa_bits);
    return rebuild_cvt(c_);
  };

  auto rebuild_any = [&](const uint16_t* bptr, const uint16_t* aptr, int b_stride_r, int a_stride_r) __attribute__((always_inline)) -> u32x4 {
    float acc[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) acc[j] = 0.f;
    for (int r = 0; r < p.rk; ++r) {
      const float a = bf16bits_to_f32(aptr[r * a_stride_r]);
      const u32x4 bv = *reinterpret_cast<const u32x4*>(bptr + r * b_stride_r);
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        acc[2 * j] += a * bf16lo_to_f32(bv[j]);
        acc[2 * j + 1] += a * bf16hi_to_f32(bv[j]);
      }
    }
    const float inv = 1.f / (float)p.rk;
    u32x4 out;
#pragma unroll
    for (int j = 0; j < 4; ++j) out[j] = pack_bf16(acc[2 * j] * inv, acc[2 * j + 1] * inv);
    return out;
  };

  // Head factors of this thread's tokens for one matrix of tile `tile`, as packed (a0, a1) pairs:
  // from the LDS slot ([K|V][token][rank]) or, with a_slot == nullptr, from global memory.
  auto fetch_aa = [&](auto is_v_c, int tile, const uint16_t* a_slot, uint32_t (&aa)[NPASS]) __attribute__((always_inline)) {
    constexpr bool is_v = decltype(is_v_c)::value;
    if constexpr (LOADER != LOAD_TPA_R2) return;
    const uint16_t* ab = is_v ? va_b : ka_b;
    const int a_sl = is_v ? p.va.stride_l : p.ka.stride_l, a_sr = is_v ? p.va.stride_r : p.ka.stride_r;
#pragma unroll
    for (int ps = 0; ps < NPASS; ++ps) {
      const int t = ps * TPP + lt;
      if (a_slot) {
        aa[ps] = *reinterpret_cast<const uint32_t*>(a_slot + (is_v ? 2 * kTK : 0) + 2 * t);
      } else {
        const int tok = min(tile * kTK + t, lk_r - 1);
        const uint32_t a0 = ab[(int64_t)tok * a_sl], a1 = ab[(int64_t)tok * a_sl + a_sr];
        aa[ps] = halve_pair(a0 | (a1 << 16));
      }
    }
  };

  // Rebuild one matrix of tile `tile` from the registers `issue` filled and store it in LDS.
  auto commit_from = [&](const u32x4 (&regs)[NPASS][2], auto is_v_c, int tile, const uint32_t (&aa)[NPASS]) __attribute__((always_inline)) {
    constexpr bool is_v = decltype(is_v_c)::value;
    const uint16_t* bb = is_v ? vb_b : kb_b;
    const uint16_t* ab = is_v ? va_b : ka_b;
    const int b_sl = is_v ? p.vb.stride_l : p.kb.stride_l, b_sr = is_v ? p.vb.stride_r : p.kb.stride_r;
    const int a_sl = is_v ? p.va.stride_l : p.ka.stride_l, a_sr = is_v ? p.va.stride_r : p.ka.stride_r;
    uint16_t* dst = is_v ? lds_v(tile & 1) : lds_k(tile % 3);
    constexpr int row_stride = is_v ? VS : KS;
#pragma unroll
    for (int ps = 0; ps < NPASS; ++ps) {
      const int t = ps * TPP + lt;
      u32x4 val;
      if constexpr (LOADER == LOAD_TPA_R2) {
        val = rebuild_r2(regs[ps][0], regs[ps][1], aa[ps]);
      } else if constexpr (LOADER == LOAD_TPA_ANY) {
        const int tok = min(tile * kTK + t, lk_r - 1);
        val = rebuild_any(bb + (int64_t)tok * b_sl + 8 * lc, ab + (int64_t)tok * a_sl, b_sr, a_sr);
      } else {
        val = regs[ps][0];
      }
      *reinterpret_cast<u32x4*>(dst + t * row_stride + 8 * lc) = val;
    }
  };
  auto commit = [&](auto is_v_c, int tile, const uint32_t (&aa)[NPASS]) __attribute__((always_inline)) {
    if constexpr (decltype(is_v_c)::value) commit_from(vreg, is_v_c, tile, aa); else commit_from(kreg, is_v_c, tile, aa);
  };

  // ---- per-wave state, one set per row block r (always indexed with compile-time constants)
  f32x16 o[RB][NDB];
#pragma unroll
  for (int r = 0; r < RB; ++r)
#pragma unroll
    for (int db = 0; db < NDB; ++db)
#pragma unroll
      for (int v = 0; v < 16; ++v) o[r][db][v] = 0.f;
  f32x16 s[RB][2];      // exponents x*c - mref of the tile in flight: two 32-key blocks per row block
  // P^T of the tile (packed bf16 pairs, the B operands of the four 16-key steps of O^T) is kept
  // in the registers of the logits it was made from: fragment k = s[r][k / 2][4 (k % 2) .. + 3]
  auto pf_set = [&](auto r_c, auto mb_c, auto idx_c, uint32_t bits) __attribute__((always_inline)) {
    s[decltype(r_c)::value][decltype(mb_c)::value][decltype(idx_c)::value] = __uint_as_float(bits);
  };
  auto pf_get = [&](auto r_c, auto kk_c) __attribute__((always_inline)) -> bf16x8 {
    constexpr int r = decltype(r_c)::value, kk = decltype(kk_c)::value, mb = kk / 2, h4 = 4 * (kk % 2);
    const u32x4 w4 = {__float_as_uint(s[r][mb][h4]), __float_as_uint(s[r][mb][h4 + 1]), __float_as_uint(s[r][mb][h4 + 2]), __float_as_uint(s[r][mb][h4 + 3])};
    return __builtin_bit_cast(bf16x8, w4);
  };
  float mref[RB];       // reference (log2 domain, includes c) of row qrow[r]
  // -mref in all 16 registers of an accumulator tuple: the addend of the first S^T MFMA of a
  // block, so the contraction lands on x*c - mref.  Rewritten only when the reference moves.
  f32x16 nmref[RB];
  float lsum[RB];       // this lane's share of sum exp2(x*c - mref)
  bool seen[RB];        // the row has met a visible key (its reference is set)
#pragma unroll
  for (int r = 0; r < RB; ++r) {
    mref[r] = 0.f;
    lsum[r] = 0.f;
    seen[r] = false;
#pragma unroll
    for (int v = 0; v < 16; ++v) nmref[r][v] = 0.f;
  }
  auto refresh_nmref = [&](auto r_c) __attribute__((always_inline)) {
    constexpr int r = decltype(r_c)::value;
#pragma unroll
    for (int v = 0; v < 16; ++v) nmref[r][v] = -mref[r];
  };
  const int lp = l & 15, dhalf = (l >> 4) & 1;

  // masks + online softmax of tile `tile` for row block r (32 of the 64 logits of row qrow[r] live in this lane)
  auto do_softmax = [&](int tile, auto r_c) __attribute__((always_inline)) {
    constexpr int r = decltype(r_c)::value;
    const int k0 = tile * kTK;
    // keys beyond lk, and keys after the query under the causal mask
    const bool need_mask = (k0 + kTK > lk_r) || (p.causal && (k0 + kTK - 1 > wrow_r[r]));
    if (need_mask) {
      const int limit = p.causal ? min(qrow_r[r], lk_r - 1) : lk_r - 1;  // largest visible key index
#pragma unroll
      for (int mb = 0; mb < 2; ++mb)
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          const int t = k0 + 32 * mb + 8 * (v >> 2) + 4 * g + (v & 3);
          if (t > limit) s[r][mb][v] = -INFINITY;
        }
    }
    if constexpr (has_seg) {  // keys of another segment (tpa/tpa.py:369-375)
      const int32_t* slot = lds_seg(tile & 1);
#pragma unroll
      for (int mb = 0; mb < 2; ++mb)
#pragma unroll
        for (int vq = 0; vq < 4; ++vq) {
          const int4 ids = *reinterpret_cast<const int4*>(slot + 32 * mb + 8 * vq + 4 * g);
          if (ids.x != qseg[r]) s[r][mb][4 * vq] = -INFINITY;
          if (ids.y != qseg[r]) s[r][mb][4 * vq + 1] = -INFINITY;
          if (ids.z != qseg[r]) s[r][mb][4 * vq + 2] = -INFINITY;
          if (ids.w != qseg[r]) s[r][mb][4 * vq + 3] = -INFINITY;
        }
    }
    float tmax = s[r][0][0];
#pragma unroll
    for (int mb = 0; mb < 2; ++mb)
#pragma unroll
      for (int v = 0; v < 16; ++v) tmax = fmaxf(tmax, s[r][mb][v]);
    tmax = halves_max(tmax);
    const bool first = !seen[r] && tmax > -INFINITY;  // first tile with a visible key for this row
    const bool up = seen[r] && tmax > kSlack;         // rare: the row's max left the slack
    if (__any(first || up)) {
      // a first tile sets the reference (nothing accumulated yet, so nothing to rescale); later
      // the references move up and O and the row sums are rescaled.  The reference is always a whole
      // number: every exponent 2^(x - mref) then has the mantissa of 2^x itself, so which tile set or
      // moved the reference changes no rounding of P (and all rescaling is by exact powers of two)
      const float delta = (first || up) ? __builtin_ceilf(tmax) : 0.f;
      const float alpha = first ? 1.f : __builtin_amdgcn_exp2f(-delta);
      mref[r] += delta;
      refresh_nmref(r_c);
      lsum[r] *= alpha;
      if (__any(up)) {
#pragma unroll
        for (int db = 0; db < NDB; ++db) {
#pragma unroll
          for (int v = 0; v < 16; ++v) o[r][db][v] *= alpha;
        }
      }
#pragma unroll
      for (int mb = 0; mb < 2; ++mb)
#pragma unroll
        for (int v = 0; v < 16; ++v) s[r][mb][v] -= delta;
      seen[r] = seen[r] || first;
    }
    static_for<4>([&](auto k_c) __attribute__((always_inline)) {
      constexpr int k = decltype(k_c)::value, mb = k / 2, half = k % 2;
      u32x4 pk;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const float p0 = __builtin_amdgcn_exp2f(s[r][mb][8 * half + 2 * j]);
        const float p1 = __builtin_amdgcn_exp2f(s[r][mb][8 * half + 2 * j + 1]);
        lsum[r] += p0 + p1;
        pk[j] = pack_bf16(p0, p1);
      }
      static_for<4>([&](auto j_c) __attribute__((always_inline)) {
        pf_set(r_c, IC<mb>{}, IC<4 * half + decltype(j_c)::value>{}, pk[decltype(j_c)::value]);
      });
    });
  };

  // ---------------------------------------------------------------------------------------
  // Main loop.  K runs one tile ahead of V, so that a wave may compute the logits of tile j+1
  // while it is still busy with the softmax of tile j.  Invariant at entry of iteration j: K tiles
  // j and j+1 are in LDS buffers j%3 and (j+1)%3, V tile j in buffer j&1; kreg holds the B factors
  // of K tile j+2 and vreg those of V tile j+1; head-factor slot j&1 holds those of K tile j+2 and
  // V tile j+1, a_pending (waves 0-3) those of K tile j+3 / V tile j+2 (tile indices clamped to
  // the last tile).  An iteration computes S^T = K Q^T, the softmax and O^T += V^T P^T of tile j,
  // rebuilds K tile j+2 and V tile j+1 into the free buffers and refills the registers with K
  // tile j+3 and V tile j+2; one barrier ends it.
  constexpr int N_QK = 2 * NKS, N_PV = 4 * NDB, N_MFMA = N_QK + N_PV;
  // operand fragment n from LDS, shared by the wave's row blocks: fragments 0..N_QK-1 are rows of K
  // (32-key block mb = n / NKS), the rest columns of V (k-step kk covers keys 16kk .. 16kk+15 of the
  // tile in the slot order the S^T accumulator already has: slot (g, j) = key 16kk + 8(j/4) + 4g + j%4)
  auto load_frag = [&](auto n_c, const uint16_t* ks, const uint16_t* vs) __attribute__((always_inline)) -> bf16x8 {
    constexpr int n = decltype(n_c)::value;
    if constexpr (n < N_QK) {
      constexpr int mb = n / NKS, kk = n % NKS;
      return *reinterpret_cast<const bf16x8*>(ks + (32 * mb + i) * KS + 16 * kk + 8 * g);
    } else {
      constexpr int m = n - N_QK, kk = m / NDB, db = m % NDB;
      const uint16_t* vrow = vs + (16 * kk + 4 * g + (lp >> 2)) * VS + 16 * dhalf + 4 * (lp & 3);
      const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3)))*)(vrow + 32 * db));
      const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3)))*)(vrow + 8 * VS + 32 * db));
      return __builtin_bit_cast(bf16x8, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
    }
  };
  // the MFMA of fragment n for row block r
  auto mfma_with = [&](auto n_c, auto r_c, const bf16x8& f) __attribute__((always_inline)) {
    constexpr int n = decltype(n_c)::value, r = decltype(r_c)::value;
    if constexpr (n < N_QK) {
      constexpr int mb = n / NKS, kk = n % NKS;
      if constexpr (kk == 0) s[r][mb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(f, qf[r][kk], nmref[r], 0, 0, 0);
      else s[r][mb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(f, qf[r][kk], s[r][mb], 0, 0, 0);
    } else {
      constexpr int m = n - N_QK, kk = m / NDB, db = m % NDB;
      o[r][db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(f, pf_get(r_c, IC<kk>{}), o[r][db], 0, 0, 0);
    }
  };
  // ---- pieces of the softmax of one 32-key block, for the interleaved (unmasked) path
  // Move the reference up where this block's row max left the slack (rare).  delta is a whole
  // number, so the scale factors are exact powers of two.  `pf_done` = number of already packed
  // P fragments of this tile, which are rescaled too; s[r][1] is adjusted with s[r][0] because its
  // accumulation (still running when block 0 is inspected) started from the old reference.
  auto move_reference = [&](auto r_c, float tmax, int pf_done) __attribute__((always_inline)) {
    constexpr int r = decltype(r_c)::value;
    const float delta = tmax > 0.f ? __builtin_ceilf(tmax) : 0.f;
    const float alpha = __builtin_amdgcn_exp2f(-delta);
    mref[r] += delta;
    refresh_nmref(r_c);
    lsum[r] *= alpha;
#pragma unroll
    for (int db = 0; db < NDB; ++db) {
#pragma unroll
      for (int v = 0; v < 16; ++v) o[r][db][v] *= alpha;
    }
    // pf_done = 0: block 0 is being inspected, nothing of this tile is packed yet, both blocks move;
    // pf_done = 2: block 0 has become fragments 0 and 1 (s[r][0][0..7]), block 1 moves
    if (pf_done == 0) {
#pragma unroll
      for (int v = 0; v < 16; ++v) s[r][0][v] -= delta;
    } else {
#pragma unroll
      for (int v = 0; v < 8; ++v) {
        const uint32_t w1 = __float_as_uint(s[r][0][v]);
        s[r][0][v] = __uint_as_float(pack_bf16(bf16lo_to_f32(w1) * alpha, bf16hi_to_f32(w1) * alpha));
      }
    }
#pragma unroll
    for (int v = 0; v < 16; ++v) s[r][1][v] -= delta;
  };
  auto sm_max = [&](auto r_c, auto mb_c) __attribute__((always_inline)) {
    constexpr int r = decltype(r_c)::value, mb = decltype(mb_c)::value;
    float t = s[r][mb][0];
#pragma unroll
    for (int v = 1; v < 16; ++v) t = fmaxf(t, s[r][mb][v]);
    t = halves_max(t);
    if (__any(t > kSlack)) move_reference(r_c, t, 2 * mb);
  };
  auto sm_exp = [&](auto r_c, auto mb_c, auto q_c) __attribute__((always_inline)) {  // 4 of the block's 16 logits
    constexpr int r = decltype(r_c)::value, mb = decltype(mb_c)::value, q = decltype(q_c)::value;
    const float p0 = __builtin_amdgcn_exp2f(s[r][mb][4 * q]);
    const float p1 = __builtin_amdgcn_exp2f(s[r][mb][4 * q + 1]);
    const float p2 = __builtin_amdgcn_exp2f(s[r][mb][4 * q + 2]);
    const float p3 = __builtin_amdgcn_exp2f(s[r][mb][4 * q + 3]);
    lsum[r] += (p0 + p1) + (p2 + p3);
    pf_set(r_c, mb_c, IC<2 * q>{}, pack_bf16(p0, p1));
    pf_set(r_c, mb_c, IC<2 * q + 1>{}, pack_bf16(p2, p3));
  };

  // ---- interleaved iteration (tiles that need no mask, with a next tile to rebuild): every
  // MFMA is followed by a short slice of independent vector work of the same wave, so that the
  // vector ALU runs in the shadow of the matrix pipe.  A fragment read from LDS feeds one MFMA
  // per row block; with G = fragments per group:
  //   S^T block 0   | rebuild K tile j+2, refill kreg
  //   S^T block 1   | softmax of block 0 (all row blocks)
  //   O^T, keys 0-31  | softmax of block 1
  //   O^T, keys 32-63 | rebuild V tile j+1, refill vreg
  // LDS operands are read LA fragments ahead of the MFMAs that consume them.
  auto hot_iteration = [&](int j) __attribute__((always_inline)) {
    constexpr int LA = 2;
    const uint16_t* ks = lds_k(j % 3);
    const uint16_t* vs = lds_v(j & 1);
    const uint16_t* a_slot = lds_a(j & 1);
    uint16_t* k_dst = lds_k((j + 2) % 3);
    uint16_t* v_dst = lds_v((j + 1) & 1);
    uint32_t aa_k[NPASS], aa_v[NPASS];
    fetch_aa(IsK{}, j + 2, a_slot, aa_k);
    fetch_aa(IsV{}, j + 1, a_slot, aa_v);
    Chunk ch;
    // one rebuild piece: 3 per loader pass (pair up the ranks, dot with the head factors, pack + store)
    auto piece = [&](auto is_v_c, auto q_c) __attribute__((always_inline)) {
      constexpr bool is_v = decltype(is_v_c)::value;
      constexpr int q = decltype(q_c)::value, ps = q / 3, part = q % 3;
      if constexpr (LOADER == LOAD_DENSE) {  // nothing to rebuild: the loaded rows are the tile
        if constexpr (part == 2) {
          const int t = ps * TPP + lt;
          uint16_t* dst = is_v ? v_dst + t * VS : k_dst + t * KS;
          *reinterpret_cast<u32x4*>(dst + 8 * lc) = is_v ? vreg[ps][0] : kreg[ps][0];
        }
      } else if constexpr (part == 0) {
        if constexpr (is_v) rebuild_perm(ch, vreg[ps][0], vreg[ps][1]); else rebuild_perm(ch, kreg[ps][0], kreg[ps][1]);
      } else if constexpr (part == 1) {
        rebuild_dot(ch, is_v ? aa_v[ps] : aa_k[ps]);
      } else {
        const u32x4 val = rebuild_cvt(ch);
        const int t = ps * TPP + lt;
        uint16_t* dst = is_v ? v_dst + t * VS : k_dst + t * KS;
        *reinterpret_cast<u32x4*>(dst + 8 * lc) = val;
      }
    };
    constexpr int NP = 3 * NPASS;       // rebuild pieces per matrix
    // slots (one per MFMA) of the four groups; slot = fragment * RB + row block
    constexpr int G1 = NKS * RB, G2 = NKS * RB, G3 = 2 * NDB * RB, G4 = 2 * NDB * RB;
    static_assert(G1 > NP && G4 >= 1, "slices fit their groups");
    // the softmax of 32-key block mb as items: with one row block {max (block 0 only), exp 0..3},
    // with two {max r0, max r1, exp (r0, 0), exp (r1, 0), ..., exp (r1, 3)}; item k of NI goes
    // behind MFMA slot k * G / NI of its group.  (With one row block the maximum of block 1 is
    // taken before the group starts, see below.)
    auto softmax_items = [&](auto mb_c, auto q_c, auto g_c) __attribute__((always_inline)) {
      constexpr int mb = decltype(mb_c)::value, q = decltype(q_c)::value, G = decltype(g_c)::value;
      constexpr int NMAX = (RB == 1 && mb == 1) ? 0 : RB, NI = NMAX + 4 * RB;
      static_for<NI>([&](auto k_c) __attribute__((always_inline)) {
        constexpr int k = decltype(k_c)::value;
        if constexpr (k * G / NI == q) {
          if constexpr (k < NMAX) sm_max(IC<k>{}, mb_c);
          else sm_exp(IC<(k - NMAX) % RB>{}, mb_c, IC<(k - NMAX) / RB>{});
        }
      });
    };
    auto slice = [&](auto n_c) __attribute__((always_inline)) {
      constexpr int n = decltype(n_c)::value;
      if constexpr (n < G1) {
        constexpr int NI = NP + 1;  // items: NP rebuild pieces of K, refill kreg
        static_for<NI>([&](auto k_c) __attribute__((always_inline)) {
          constexpr int k = decltype(k_c)::value;
          if constexpr (k * G1 / NI == n) {
            if constexpr (k < NP) piece(IsK{}, k_c);
            else issue(IsK{}, min(j + 3, last));
          }
        });
      } else if constexpr (n < G1 + G2) {
        softmax_items(IC<0>{}, IC<n - G1>{}, IC<G2>{});
      } else if constexpr (n < G1 + G2 + G3) {
        softmax_items(IC<1>{}, IC<n - G1 - G2>{}, IC<G3>{});
      } else {
        constexpr int q = n - G1 - G2 - G3;  // items: NP rebuild pieces of V, refill vreg
        constexpr int NI = NP + 1;
        static_for<NI>([&](auto k_c) __attribute__((always_inline)) {
          constexpr int k = decltype(k_c)::value;
          if constexpr (k * G4 / NI == q) {
            if constexpr (k < NP) piece(IsV{}, k_c);
            else issue(IsV{}, min(j + 2, last));
          }
        });
      }
    };
    bf16x8 fr[N_MFMA];
    static_for<LA>([&](auto n_c) __attribute__((always_inline)) { fr[decltype(n_c)::value] = load_frag(n_c, ks, vs); });
    static_for<N_MFMA>([&](auto n_c) __attribute__((always_inline)) {
      constexpr int n = decltype(n_c)::value;
      if constexpr (RB == 1 && n == N_QK) {
        sm_max(IC<0>{}, IC<1>{});  // before any O^T MFMA of this tile is issued
        __builtin_amdgcn_sched_barrier(0);
      }
      if constexpr (n + LA < N_MFMA) fr[n + LA] = load_frag(IC<n + LA>{}, ks, vs);
      static_for<RB>([&](auto r_c) __attribute__((always_inline)) {
        mfma_with(n_c, r_c, fr[n]);
        slice(IC<n * RB + decltype(r_c)::value>{});
      });
    });
  };

  // ---- plain iteration: first tile, masked tiles, tiles a row block skips, last tile.
  // `mask_c` = the row blocks of this wave that take part (bit r); `part_c` = 0: the whole tile, 1: its
  // logits only (they stay in s), 2: the rest of a tile whose logits are in s already, 3: the logits of
  // its first 32 keys only, 4: the rest of a tile whose first 32 logits are in s already.
  auto cold_compute = [&](int j, auto mask_c, auto part_c) __attribute__((always_inline)) {
    constexpr int M = decltype(mask_c)::value, PART = decltype(part_c)::value;
    const uint16_t* ks = lds_k(j % 3);
    const uint16_t* vs = lds_v(j & 1);
    // operands are read three fragments ahead here too (the V fragments of the first O^T steps
    // while the softmax runs); not with the any-rank loader, whose kernel got slower with it
    constexpr int LA = LOADER == LOAD_TPA_ANY ? 0 : 3;
    bf16x8 fr[N_MFMA];
    // fragments this call uses (0 .. N_QK - 1: K rows, the first NKS of them those of keys 0-31), and which of
    // them belong to the logits
    constexpr int FIRST = PART == 2 ? N_QK : PART == 4 ? NKS : 0, END = PART == 1 ? N_QK : PART == 3 ? NKS : N_MFMA;
    constexpr int QK_END = PART == 3 ? NKS : N_QK;
    static_for<LA>([&](auto n_c) __attribute__((always_inline)) {
      constexpr int n = FIRST + decltype(n_c)::value;
      if constexpr (n < END) fr[n] = load_frag(IC<n>{}, ks, vs);
    });
    if constexpr (PART != 2) {
      static_for<QK_END - FIRST>([&](auto n_c) __attribute__((always_inline)) {
        constexpr int n = FIRST + decltype(n_c)::value;
        if constexpr (n + LA < END) fr[n + LA] = load_frag(IC<n + LA>{}, ks, vs);
        static_for<RB>([&](auto r_c) __attribute__((always_inline)) {
          if constexpr ((M >> decltype(r_c)::value) & 1) mfma_with(IC<n>{}, r_c, fr[n]);
        });
      });
    }
    if constexpr (PART != 1 && PART != 3) {
      static_for<RB>([&](auto r_c) __attribute__((always_inline)) {
        if constexpr ((M >> decltype(r_c)::value) & 1) do_softmax(j, r_c);
      });
      static_for<N_PV>([&](auto n_c) __attribute__((always_inline)) {
        constexpr int n = N_QK + decltype(n_c)::value;
        if constexpr (n + LA < END) fr[n + LA] = load_frag(IC<n + LA>{}, ks, vs);
        static_for<RB>([&](auto r_c) __attribute__((always_inline)) {
          if constexpr ((M >> decltype(r_c)::value) & 1) mfma_with(IC<n>{}, r_c, fr[n]);
        });
      });
    }
  };
  // the loader's share of iteration j: K tile j+2 and V tile j+1 into LDS, K tile j+3 and V tile j+2 on their way
  auto advance_tiles = [&](int j) __attribute__((always_inline)) {
    const uint16_t* a_slot = LOADER == LOAD_TPA_R2 ? lds_a(j & 1) : nullptr;
    if (j + 2 < ntiles) {
      uint32_t aa_k[NPASS];
      fetch_aa(IsK{}, j + 2, a_slot, aa_k);
      commit(IsK{}, j + 2, aa_k);
      issue(IsK{}, min(j + 3, last));
    }
    if (j + 1 < ntiles) {
      uint32_t aa_v[NPASS];
      fetch_aa(IsV{}, j + 1, a_slot, aa_v);
      commit(IsV{}, j + 1, aa_v);
      issue(IsV{}, min(j + 2, last));
    }
  };
  auto cold_iteration = [&](int j) __attribute__((always_inline)) {
    if (j <= wave_last_tile[0]) cold_compute(j, IC<1>{}, IC<0>{});
    advance_tiles(j);
  };

  // ---- prologue: K tiles 0 and 1 and V tile 0 into LDS (head factors straight from global memory),
  // the head factors of K tile 2 / V tile 1 in slot 0, those of K tile 3 / V tile 2 pending, the B
  // factors of K tile 2 and V tile 1 in registers
  {
    u32x4 kreg1[NPASS][2];  // K tile 1, on its way during the Q build like tile 0
    issue(IsK{}, 0);
    issue(IsV{}, 0);
    issue_into(kreg1, IsK{}, min(1, last));
    issue_a(min(2, last), min(1, last));
    build_q();
    uint32_t aa0[NPASS], aa1[NPASS], aa2[NPASS];
    fetch_aa(IsK{}, 0, nullptr, aa0);
    fetch_aa(IsV{}, 0, nullptr, aa1);
    commit(IsK{}, 0, aa0);
    commit(IsV{}, 0, aa1);
    if (last >= 1) {
      fetch_aa(IsK{}, 1, nullptr, aa2);
      commit_from(kreg1, IsK{}, 1, aa2);
    }
  }
  issue(IsK{}, min(2, last));
  issue(IsV{}, min(1, last));
  store_a(0);
  issue_a(min(3, last), min(2, last));
  issue_seg(0);
  store_seg(0);
  issue_seg(min(1, last));
  lds_barrier();

  // Per wave: tile 0 plain, then the run of unmasked tiles interleaved, then plain again (masked
  // tiles, tiles past this wave's causal range, the last tile).  Three separate loops rather than
  // a branch inside one: every wave passes the same number of barriers either way.
  auto tail = [&](int j) __attribute__((always_inline)) {
    // head factors: publish those of K tile j+3 / V tile j+2, fetch those of K tile j+4 / V tile j+3
    store_a((j + 1) & 1);
    issue_a(min(j + 4, last), min(j + 3, last));
    // key segment ids (one wave): publish those of tile j+1, fetch those of tile j+2
    store_seg((j + 1) & 1);
    issue_seg(min(j + 2, last));
    lds_barrier();
  };
  int hot_end = 1;
  if constexpr (LOADER != LOAD_TPA_ANY) {
    int first_masked = lk_r / kTK;                                   // ragged last tile
    int needed = last;                                               // last tile every row block of the wave needs
#pragma unroll
    for (int r = 0; r < RB; ++r) {
      if (p.causal) first_masked = min(first_masked, max(wrow_r[r] + 1, 0) / kTK);  // first tile with a key past the block's first row
      needed = min(needed, wave_last_tile[r]);
    }
    hot_end = max(1, min(min(ntiles - 1, first_masked), needed + 1));
    // segment masks are applied by the plain iteration only: the interleaved one runs where no
    // key of another segment can turn up (tile 0, which may start before the run, is plain anyway)
    if constexpr (has_seg) if (!seg_pure) hot_end = 1;
  }
  int j = 0;
  for (; j < 1; ++j) { cold_iteration(j); tail(j); }
  if constexpr (LOADER == LOAD_DENSE && !SEG) {
    // Unmasked tiles 1 .. hot_end - 1 pipelined: tile j's softmax and O^T run beside the logits of
    // tile j+1 (K is a tile ahead in LDS for this).  The logits of tile 1 are computed here, the
    // loop (generated by gen_prefill_loop.py, which documents the register assignment) then runs
    // iterations 1 .. hot_end - 2 and leaves the logits of tile hot_end - 1, which is finished
    // here.  The state goes in and comes back in operands pinned to the loop's registers.
    if (hot_end >= 3) {
      cold_compute(1, IC<1>{}, IC<1>{});
      auto cat4 = [](const u32x4& a0, const u32x4& a1, const u32x4& a2, const u32x4& a3) __attribute__((always_inline)) -> f32x16 {
        const u32x8 lo = __builtin_shufflevector(a0, a1, 0, 1, 2, 3, 4, 5, 6, 7);
        const u32x8 hi = __builtin_shufflevector(a2, a3, 0, 1, 2, 3, 4, 5, 6, 7);
        return __builtin_bit_cast(f32x16, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7, 8, 9, 10, 11, 12, 13, 14, 15));
      };
      auto qv = [&](int ks) __attribute__((always_inline)) { return __builtin_bit_cast(u32x4, qf[0][ks]); };
      const u32x4 z4 = {0, 0, 0, 0};
      const f32x16 qp0 = cat4(qv(0), qv(1), qv(2), qv(3));
      const f32x16 qp1 = NKS > 4 ? cat4(qv(NKS > 4 ? 4 : 0), qv(NKS > 4 ? 5 : 0), qv(NKS > 4 ? 6 : 0), qv(NKS > 4 ? 7 : 0)) : qp0;
      u32x8 kv_k = __builtin_shufflevector(kreg[0][0], NPASS > 1 ? kreg[NPASS - 1][0] : z4, 0, 1, 2, 3, 4, 5, 6, 7);
      u32x8 kv_v = __builtin_shufflevector(vreg[0][0], NPASS > 1 ? vreg[NPASS - 1][0] : z4, 0, 1, 2, 3, 4, 5, 6, 7);
      f32x16 sa0 = {}, sa1 = {}, sb0 = s[0][0], sb1 = s[0][1];  // tile 1 is odd: its logits sit in the second set
      const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint16_t*)smem;
      u32x16 st16 = {};
      st16[0] = __float_as_uint(mref[0]); st16[1] = __float_as_uint(lsum[0]);
      st16[2] = lds0 + 2 * (L::k_off(0) + i * KS + 8 * g);                                                   // K fragment rows
      st16[3] = lds0 + 2 * (L::v_off(0) + (4 * g + (lp >> 2)) * VS + 16 * dhalf + 4 * (lp & 3));             // V fragment columns
      st16[4] = lds0 + 2 * (L::k_off(0) + lt * KS + 8 * lc);                                                 // this thread's chunk of a K tile
      st16[5] = lds0 + 2 * (L::v_off(0) + lt * VS + 8 * lc);                                                 // ... of a V tile
      st16[6] = kvoff; st16[7] = vvoff;
      auto uni = [](uint32_t x) __attribute__((always_inline)) { return (uint32_t)__builtin_amdgcn_readfirstlane((int)x); };
      u32x16 sc16 = {};
      sc16[0] = 1; sc16[1] = uni(hot_end - 1); sc16[2] = uni(last);
      sc16[3] = uni(kTK * p.kb.stride_l * 2); sc16[4] = uni(kTK * p.vb.stride_l * 2);
      sc16[5] = uni(TPP * p.kb.stride_l * 2); sc16[6] = uni(TPP * p.vb.stride_l * 2);
      sc16[7] = 2 * L::kK * 2; sc16[8] = 0;  // K buffers: iteration 1 reads tile 2 in buffer 2 and writes tile 3 into buffer 0
      auto rsrc_words = [&](const uint16_t* base, int bytes) __attribute__((always_inline)) -> u32x4 {
        const uint64_t a64 = reinterpret_cast<uint64_t>(base);
        return u32x4{uni((uint32_t)a64), uni((uint32_t)(a64 >> 32) & 0xffffu), uni((uint32_t)bytes), (uint32_t)kRsrcFlags};
      };
      const u32x4 kbr = rsrc_words(kb_b, k_rows_bytes), vbr = rsrc_words(vb_b, v_rows_bytes);
      if constexpr (D == 128) {
        asm volatile(
#include "gen/prefill_loop_128_dense.inc"
            : "+{v[0:15]}"(sa0), "+{v[16:31]}"(sa1), "+{v[32:47]}"(sb0), "+{v[48:63]}"(sb1), "+{v[64:79]}"(nmref[0]),
              "+{v[80:95]}"(o[0][0]), "+{v[96:111]}"(o[0][1]), "+{v[112:127]}"(o[0][NDB > 2 ? 2 : 0]), "+{v[128:143]}"(o[0][NDB > 2 ? 3 : 0]),
              "+{v[176:183]}"(kv_k), "+{v[184:191]}"(kv_v), "+{v[204:219]}"(st16), "+{s[32:47]}"(sc16)
            : "{v[144:159]}"(qp0), "{v[160:175]}"(qp1), "{s[48:51]}"(kbr), "{s[52:55]}"(vbr)
            :
#include "gen/prefill_loop_128_dense_clobbers.inc"
        );
      } else {
        asm volatile(
#include "gen/prefill_loop_64_dense.inc"
            : "+{v[0:15]}"(sa0), "+{v[16:31]}"(sa1), "+{v[32:47]}"(sb0), "+{v[48:63]}"(sb1), "+{v[64:79]}"(nmref[0]),
              "+{v[80:95]}"(o[0][0]), "+{v[96:111]}"(o[0][1]),
              "+{v[176:183]}"(kv_k), "+{v[184:191]}"(kv_v), "+{v[204:219]}"(st16), "+{s[32:47]}"(sc16)
            : "{v[144:159]}"(qp0), "{s[48:51]}"(kbr), "{s[52:55]}"(vbr)
            :
#include "gen/prefill_loop_64_dense_clobbers.inc"
        );
      }
      kreg[0][0] = __builtin_shufflevector(kv_k, kv_k, 0, 1, 2, 3);
      vreg[0][0] = __builtin_shufflevector(kv_v, kv_v, 0, 1, 2, 3);
      if constexpr (NPASS > 1) {
        kreg[NPASS - 1][0] = __builtin_shufflevector(kv_k, kv_k, 4, 5, 6, 7);
        vreg[NPASS - 1][0] = __builtin_shufflevector(kv_v, kv_v, 4, 5, 6, 7);
      }
      mref[0] = __uint_as_float(st16[0]); lsum[0] = __uint_as_float(st16[1]);
      j = hot_end - 1;
      const bool odd = j & 1;  // uniform
      s[0][0] = odd ? sb0 : sa0;
      s[0][1] = odd ? sb1 : sa1;
      cold_compute(j, IC<1>{}, IC<2>{});
      advance_tiles(j);
      tail(j);
      ++j;
    }
  } else if constexpr (LOADER == LOAD_TPA_R2 && !SEG) {
    // Unmasked tiles 1 .. hot_end - 1 pipelined in blocks of 32 keys: a block's softmax runs beside the
    // logits of the next block, its O^T beside the rebuild of the tiles ahead.  The logits of the first 32
    // keys of tile 1 are computed here; the loop (generated by gen_prefill_loop.py, which documents the
    // register assignment) runs iterations 1 .. hot_end - 2 - everything advance_tiles() and tail() do
    // included - and leaves the logits of the first 32 keys of tile hot_end - 1, which is finished here.
    if (hot_end >= 3) {
      cold_compute(1, IC<1>{}, IC<3>{});
      auto cat4 = [](const u32x4& a0, const u32x4& a1, const u32x4& a2, const u32x4& a3) __attribute__((always_inline)) -> u32x16 {
        const u32x8 lo = __builtin_shufflevector(a0, a1, 0, 1, 2, 3, 4, 5, 6, 7);
        const u32x8 hi = __builtin_shufflevector(a2, a3, 0, 1, 2, 3, 4, 5, 6, 7);
        return __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7, 8, 9, 10, 11, 12, 13, 14, 15);
      };
      auto qv = [&](int ks) __attribute__((always_inline)) { return __builtin_bit_cast(u32x4, qf[0][ks]); };
      const u32x16 qp0 = cat4(qv(0), qv(1), qv(2), qv(3));
      const u32x16 qp1 = NKS > 4 ? cat4(qv(NKS > 4 ? 4 : 0), qv(NKS > 4 ? 5 : 0), qv(NKS > 4 ? 6 : 0), qv(NKS > 4 ? 7 : 0)) : qp0;
      // rows in flight: (pass, rank) tuples of four registers
      u32x16 kv_k = cat4(kreg[0][0], kreg[0][1], kreg[NPASS - 1][0], kreg[NPASS - 1][1]);
      u32x16 kv_v = cat4(vreg[0][0], vreg[0][1], vreg[NPASS - 1][0], vreg[NPASS - 1][1]);
      f32x16 set0 = s[0][0], set1 = {};
      const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint16_t*)smem;
      u32x16 st16 = {};
      st16[0] = __float_as_uint(mref[0]); st16[1] = __float_as_uint(lsum[0]);
      st16[2] = lds0 + 2 * (L::k_off(0) + i * KS + 8 * g);                                                   // K fragment rows
      st16[3] = lds0 + 2 * (L::v_off(0) + (4 * g + (lp >> 2)) * VS + 16 * dhalf + 4 * (lp & 3));             // V fragment columns
      st16[4] = lds0 + 2 * (L::k_off(0) + lt * KS + 8 * lc);                                                 // this thread's chunk of a K tile
      st16[5] = lds0 + 2 * (L::v_off(0) + lt * VS + 8 * lc);                                                 // ... of a V tile
      st16[6] = kvoff; st16[7] = vvoff;
      st16[8] = lds0 + 2 * L::a_off(0) + 4 * lt;                                                             // head factor pairs of this thread's tokens
      st16[9] = lds0 + 2 * (L::a_off(0) + a_idx);                                                            // where this thread's head factor goes
      st16[10] = a_mat ? va_voff : ka_voff;
      st16[11] = a_pending;
      auto uni = [](uint32_t x) __attribute__((always_inline)) { return (uint32_t)__builtin_amdgcn_readfirstlane((int)x); };
      u32x16 sc16 = {};
      sc16[0] = 1; sc16[1] = uni(hot_end - 1); sc16[2] = uni(last);
      sc16[3] = uni(kTK * p.kb.stride_l * 2); sc16[4] = uni(kTK * p.vb.stride_l * 2);
      sc16[5] = uni(TPP * p.kb.stride_l * 2); sc16[6] = uni(TPP * p.vb.stride_l * 2);
      sc16[7] = 1 * L::kK * 2; sc16[8] = 2 * L::kK * 2; sc16[9] = 0;  // K buffers of tiles 1 and 2, and the one tile 3 goes to
      sc16[10] = uni(p.kb.stride_r * 2); sc16[11] = uni(p.vb.stride_r * 2);
      sc16[12] = uni(kTK * (a_mat ? p.va.stride_l : p.ka.stride_l) * 2);
      sc16[13] = uni(a_mat ? 3 : 4);
      auto rsrc_words = [&](const uint16_t* base, int bytes) __attribute__((always_inline)) -> u32x4 {
        const uint64_t a64 = reinterpret_cast<uint64_t>(base);
        return u32x4{uni((uint32_t)a64), uni((uint32_t)(a64 >> 32) & 0xffffu), uni((uint32_t)bytes), (uint32_t)kRsrcFlags};
      };
      const u32x4 kbr = rsrc_words(kb_b, k_rows_bytes), vbr = rsrc_words(vb_b, v_rows_bytes);
      const u32x4 abr = rsrc_words(a_mat ? va_b : ka_b, a_mat ? va_bytes : ka_bytes);
      if constexpr (D == 128) {
        asm volatile(
#include "gen/prefill_loop_128_r2.inc"
            : "+{v[0:15]}"(set0), "+{v[16:31]}"(set1), "+{v[32:47]}"(nmref[0]),
              "+{v[48:63]}"(o[0][0]), "+{v[64:79]}"(o[0][1]), "+{v[80:95]}"(o[0][NDB > 2 ? 2 : 0]), "+{v[96:111]}"(o[0][NDB > 2 ? 3 : 0]),
              "+{v[144:159]}"(kv_k), "+{v[160:175]}"(kv_v), "+{v[188:203]}"(st16), "+{s[32:47]}"(sc16)
            : "{v[112:127]}"(qp0), "{v[128:143]}"(qp1), "{s[48:51]}"(kbr), "{s[52:55]}"(vbr), "{s[56:59]}"(abr)
            :
#include "gen/prefill_loop_128_r2_clobbers.inc"
        );
      } else {
        u32x8 kv_k8 = __builtin_shufflevector(kv_k, kv_k, 0, 1, 2, 3, 4, 5, 6, 7);
        u32x8 kv_v8 = __builtin_shufflevector(kv_v, kv_v, 0, 1, 2, 3, 4, 5, 6, 7);
        asm volatile(
#include "gen/prefill_loop_64_r2.inc"
            : "+{v[0:15]}"(set0), "+{v[16:31]}"(set1), "+{v[32:47]}"(nmref[0]),
              "+{v[48:63]}"(o[0][0]), "+{v[64:79]}"(o[0][1]),
              "+{v[144:151]}"(kv_k8), "+{v[160:167]}"(kv_v8), "+{v[188:203]}"(st16), "+{s[32:47]}"(sc16)
            : "{v[112:127]}"(qp0), "{s[48:51]}"(kbr), "{s[52:55]}"(vbr), "{s[56:59]}"(abr)
            :
#include "gen/prefill_loop_64_r2_clobbers.inc"
        );
        kv_k = __builtin_shufflevector(kv_k8, kv_k8, 0, 1, 2, 3, 4, 5, 6, 7, 0, 1, 2, 3, 4, 5, 6, 7);
        kv_v = __builtin_shufflevector(kv_v8, kv_v8, 0, 1, 2, 3, 4, 5, 6, 7, 0, 1, 2, 3, 4, 5, 6, 7);
      }
      kreg[0][0] = __builtin_shufflevector(kv_k, kv_k, 0, 1, 2, 3);
      kreg[0][1] = __builtin_shufflevector(kv_k, kv_k, 4, 5, 6, 7);
      vreg[0][0] = __builtin_shufflevector(kv_v, kv_v, 0, 1, 2, 3);
      vreg[0][1] = __builtin_shufflevector(kv_v, kv_v, 4, 5, 6, 7);
      if constexpr (NPASS > 1) {
        kreg[NPASS - 1][0] = __builtin_shufflevector(kv_k, kv_k, 8, 9, 10, 11);
        kreg[NPASS - 1][1] = __builtin_shufflevector(kv_k, kv_k, 12, 13, 14, 15);
        vreg[NPASS - 1][0] = __builtin_shufflevector(kv_v, kv_v, 8, 9, 10, 11);
        vreg[NPASS - 1][1] = __builtin_shufflevector(kv_v, kv_v, 12, 13, 14, 15);
      }
      mref[0] = __uint_as_float(st16[0]); lsum[0] = __uint_as_float(st16[1]);
      a_pending = st16[11];
      j = hot_end - 1;
      s[0][0] = set0;
      cold_compute(j, IC<1>{}, IC<4>{});
      advance_tiles(j);
      tail(j);
      ++j;
    }
  } else if constexpr (LOADER != LOAD_TPA_ANY) {
    for (; j < hot_end; ++j) { hot_iteration(j); tail(j); }
  }
  for (; j < ntiles; ++j) { cold_iteration(j); tail(j); }

  // ---- epilogue: normalise, store O[b, qrow, h, :] and LSE[b, h, qrow]
  // A row block's 32 output rows go through the wave's own slice of LDS (free after the last
  // barrier), so that they leave as whole 16-byte chunks of whole rows instead of 8-byte pieces
  // of 32 rows.  (LDS operations of one wave complete in order: the next row block's writes
  // cannot overtake the reads of this one.)
  static_for<RB>([&](auto r_c) __attribute__((always_inline)) {
    constexpr int r = decltype(r_c)::value;
    const float ltot = halves_sum(lsum[r]);
    const float inv = 1.f / ltot;
    constexpr int OS = D + 8;  // row stride (elements)
    uint16_t* const ot = smem + w * 32 * OS;
    static_assert(kNW * 32 * OS * sizeof(uint16_t) <= L::kBytes, "output staging fits");
#pragma unroll
    for (int db = 0; db < NDB; ++db)
#pragma unroll
      for (int vq = 0; vq < 4; ++vq) {
        u32x2 pk;
        pk[0] = pack_bf16(o[r][db][4 * vq] * inv, o[r][db][4 * vq + 1] * inv);
        pk[1] = pack_bf16(o[r][db][4 * vq + 2] * inv, o[r][db][4 * vq + 3] * inv);
        *reinterpret_cast<u32x2*>(ot + i * OS + 32 * db + 8 * vq + 4 * g) = pk;
      }
    __builtin_amdgcn_wave_barrier();
    constexpr int CPRO = D / 8, RPI = 64 / CPRO;  // 16-byte chunks per row, rows per store instruction
    const int orow_l = l / CPRO, ochunk = l % CPRO;
#pragma unroll
    for (int n = 0; n < 32 / RPI; ++n) {
      const int rr = n * RPI + orow_l;
      const u32x4 val = *reinterpret_cast<const u32x4*>(ot + rr * OS + 8 * ochunk);
      if (wrow0[r] + rr < p.lq)
        *reinterpret_cast<u32x4*>(p.o + (((int64_t)b * p.lq + wrow0[r] + rr) * p.H + h) * D + 8 * ochunk) = val;
    }
    __builtin_amdgcn_wave_barrier();
    if (qrow[r] < p.lq && p.lse && g == 0)
      p.lse[((int64_t)b * p.H + h) * p.lq + qrow[r]] = (mref[r] + __builtin_amdgcn_logf(ltot)) * kLn2;
  });
}

template <int D, int LOADER, bool SEG = false>
int launch_prefill(const PrefillParams& p, hipStream_t stream) {
  auto kern = prefill_kernel<D, LOADER, SEG, 1>;
  constexpr size_t lds_bytes = Lds<D>::kBytes;
  static bool configured[kMaxDevices] = {};
  if (int rc = raise_lds_limit(configured, reinterpret_cast<const void*>(kern), lds_bytes); rc != TPA_OK) return rc;
  // one workgroup per (query block, batch, head): see the kernel for how ids map to them
  const int64_t n = LOADER == LOAD_DENSE ? (int64_t)((p.B * p.H + 7) / 8) * 8 * p.nqb : (int64_t)((p.npairs + 7) / 8) * 8 * p.H;
  if (n > 2147483647LL) return TPA_ERR_SHAPE;
  dim3 grid((unsigned)n);
  hipLaunchKernelGGL(kern, grid, dim3(512), lds_bytes, stream, p);
  return hipGetLastError() == hipSuccess ? TPA_OK : TPA_ERR_LAUNCH;
}

bool aligned16(const void* ptr) { return (reinterpret_cast<uintptr_t>(ptr) & 15) == 0; }
bool factor_ok(const TpaFactor& f) {
  return aligned16(f.ptr) && f.stride_b % 8 == 0 && f.stride_l % 8 == 0 && f.stride_r % 8 == 0;
}
// one batch entry of a K/V-side array is addressed through a buffer resource with 32-bit byte
// offsets: its extent must stay below 2 GiB and its strides must not be negative
bool range_ok(const TpaFactor& f, int64_t tokens, int64_t ranks, int64_t width) {
  if (f.stride_l < 0 || f.stride_r < 0) return false;
  return ((tokens - 1) * f.stride_l + (ranks - 1) * f.stride_r + width) * 2 < (int64_t(1) << 31);
}

}  // namespace
}  // namespace tpa


int tpa_prefill_mfma_supported(const TpaFwdArgs* a) {
  if (a->dtype != TPA_DTYPE_BF16) return 0;
  if (a->dk != a->dv || (a->dk != 64 && a->dk != 128)) return 0;
  if (!(a->sm_scale > 0.f)) return 0;
  if (!tpa::factor_ok(a->qb) || !tpa::factor_ok(a->kb) || !tpa::factor_ok(a->vb)) return 0;
  if (!tpa::range_ok(a->kb, a->lk, a->rk, a->dk) || !tpa::range_ok(a->vb, a->lk, a->rk, a->dv) ||
      !tpa::range_ok(a->ka, a->lk, a->rk, 1) || !tpa::range_ok(a->va, a->lk, a->rk, 1))
    return 0;
  if (!tpa::aligned16(a->o)) return 0;
  return 1;
}

// bytes of workspace that let the prefill kernel run on dense Q [B, lq, H, D], K and V [B, lk, H, D]
// (bf16, each rounded up to 256 bytes); 0 if a batch entry would not fit the kernel's 32-bit tile offsets
size_t tpa_prefill_dense_bytes(int64_t B, int64_t lq, int64_t lk, int64_t H, int64_t D) {
  if (lk * H * D * 2 >= (int64_t(1) << 31)) return 0;
  const auto slot = [](int64_t n) { return (size_t)((n * 2 + 255) / 256 * 256); };
  return slot(B * lq * H * D) + 2 * slot(B * lk * H * D);
}

// Whether reconstructing dense Q, K and V once (one HBM-bound launch) and running the plain tile
// loader beats rebuilding every tile in the flash loop.  The loop over dense tiles overlaps the
// logits of one tile with the softmax of the one before and has no rebuild in it; the
// reconstruction grows with the length only.  Rank 2 has a tuned rebuild in the fused kernel:
// measured at B * H = 64, D = 128 the two routes meet at 1024 rows (51 against 52 us) and the dense
// one wins from 2048 on (105 against 115 us; 4096: 0.32 against 0.38 ms).  Other ranks loop over
// the ranks per tile in the fused kernel: dense from the second query block on.
int tpa_prefill_wants_dense(int64_t lq, int64_t rk) {
  if (rk != 2) return lq > tpa::kBQ;
  return lq >= 2048;
}

int tpa_prefill_mfma_launch(const TpaFwdArgs* a, hipStream_t stream) {
  using namespace tpa;
  PrefillParams p{};
  p.qa = a->qa; p.qb = a->qb; p.ka = a->ka; p.kb = a->kb; p.va = a->va; p.vb = a->vb;
  p.qseg = a->q_segment_ids; p.kvseg = a->kv_segment_ids; p.kvlen = a->kv_lengths;
  p.o = static_cast<uint16_t*>(a->o); p.lse = a->lse;
  p.B = a->B; p.lq = a->lq; p.lk = a->lk; p.H = a->H; p.rq = a->rq; p.rk = a->rk;
  p.sm_scale = a->sm_scale; p.causal = a->causal; p.coff = tpa::causal_offset_of(a);
  p.nqb = (a->lq + kBQ - 1) / kBQ;
  p.npairs = p.nqb * a->B;
  // With a workspace Q (times sm_scale * log2 e), K and V are reconstructed once as dense bf16 and
  // the kernel runs with its plain tile loader: no workgroup rebuilds tiles from the rank factors
  // (the fused kernel does that once per 256 query rows and head).
  const size_t dense_bytes = tpa_prefill_dense_bytes(a->B, a->lq, a->lk, a->H, a->dk);
  if (tpa_prefill_wants_dense(a->lq, a->rk) && a->workspace && dense_bytes && a->workspace_bytes >= dense_bytes &&
      !(reinterpret_cast<uintptr_t>(a->workspace) & 255)) {
    const int64_t hd = (int64_t)a->H * a->dk;
    const size_t kv_slot = ((size_t)a->B * a->lk * hd * 2 + 255) / 256 * 256;
    uint16_t* kd = static_cast<uint16_t*>(a->workspace);
    uint16_t* vd = kd + kv_slot / 2;
    uint16_t* qd = vd + kv_slot / 2;
    int rc = tpa_recon_dense_qkv_bf16(a, qd, kd, vd, a->sm_scale * kLog2e, stream);
    if (rc == TPA_ERR_UNSUPPORTED) {
      rc = tpa_recon_dense_bf16(&a->ka, &a->kb, kd, a->B, a->lk, a->H, a->dk, a->rk, 1.f, stream);
      if (rc == TPA_OK) rc = tpa_recon_dense_bf16(&a->va, &a->vb, vd, a->B, a->lk, a->H, a->dv, a->rk, 1.f, stream);
      if (rc == TPA_OK) rc = tpa_recon_dense_bf16(&a->qa, &a->qb, qd, a->B, a->lq, a->H, a->dk, a->rq, a->sm_scale * kLog2e, stream);
    }
    if (rc != TPA_OK) return rc;
    p.qb = TpaFactor{qd, a->lq * hd, hd, 0};
    p.kb = TpaFactor{kd, a->lk * hd, hd, 0};
    p.vb = TpaFactor{vd, a->lk * hd, hd, 0};
    p.q_scaled = 1;
    if (p.kvseg) {
      if (a->dk == 128) return launch_prefill<128, LOAD_DENSE, true>(p, stream);
      return launch_prefill<64, LOAD_DENSE, true>(p, stream);
    }
    if (a->dk == 128) return launch_prefill<128, LOAD_DENSE>(p, stream);
    return launch_prefill<64, LOAD_DENSE>(p, stream);
  }
  if (p.kvseg) {
    if (a->dk == 128) {
      if (a->rk == 2) return launch_prefill<128, LOAD_TPA_R2, true>(p, stream);
      return launch_prefill<128, LOAD_TPA_ANY, true>(p, stream);
    }
    if (a->rk == 2) return launch_prefill<64, LOAD_TPA_R2, true>(p, stream);
    return launch_prefill<64, LOAD_TPA_ANY, true>(p, stream);
  }
  if (a->dk == 128) {
    if (a->rk == 2) return launch_prefill<128, LOAD_TPA_R2>(p, stream);
    return launch_prefill<128, LOAD_TPA_ANY>(p, stream);
  }
  if (a->rk == 2) return launch_prefill<64, LOAD_TPA_R2>(p, stream);
  return launch_prefill<64, LOAD_TPA_ANY>(p, stream);
}

int mha_prefill_mfma_supported(const MhaFwdArgs* a) {
  if (a->dtype != TPA_DTYPE_BF16) return 0;
  if (a->dk != a->dv || (a->dk != 64 && a->dk != 128)) return 0;
  if (a->bias) return 0;
  if (!(a->sm_scale > 0.f)) return 0;
  if (!tpa::aligned16(a->q) || !tpa::aligned16(a->k) || !tpa::aligned16(a->v) || !tpa::aligned16(a->o)) return 0;
  if ((int64_t)a->lk * a->H * (a->dk > a->dv ? a->dk : a->dv) * 2 >= (int64_t(1) << 31)) return 0;  // 32-bit buffer offsets per batch entry
  return 1;
}

int mha_prefill_mfma_launch(const MhaFwdArgs* a, hipStream_t stream) {
  using namespace tpa;
  PrefillParams p{};
  const int64_t hd = (int64_t)a->H * a->dk;
  p.qb = TpaFactor{a->q, a->lq * hd, hd, 0};
  p.kb = TpaFactor{a->k, a->lk * hd, hd, 0};
  p.vb = TpaFactor{a->v, a->lk * hd, hd, 0};
  p.qa = p.ka = p.va = TpaFactor{nullptr, 0, 0, 0};
  p.o = static_cast<uint16_t*>(a->o); p.lse = a->lse;
  p.B = a->B; p.lq = a->lq; p.lk = a->lk; p.H = a->H; p.rq = 1; p.rk = 1;
  p.sm_scale = a->sm_scale; p.causal = a->causal ? TPA_CAUSAL_TOP_LEFT : TPA_CAUSAL_NONE; p.coff = 0;
  p.nqb = (a->lq + kBQ - 1) / kBQ;
  p.npairs = p.nqb * a->B;
  if (a->dk == 128) return launch_prefill<128, LOAD_DENSE>(p, stream);
  return launch_prefill<64, LOAD_DENSE>(p, stream);
}
