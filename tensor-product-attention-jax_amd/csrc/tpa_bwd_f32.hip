// Backward of dense attention in fp32 on gfx950: fp32 MFMA contractions (v_mfma_f32_32x32x2_f32).
//
// Inputs are dense fp32 Q, K, V, dO [B, l, H, D], LSE [B, H, lq] (natural log) and
// delta = rowsum(O * dO) [B, H, lq]; outputs dense fp32 dQ, dK, dV.  With p = exp(x - lse):
//     dV = p^T dO,  dP = dO V^T,  dS = sm_scale * p * (dP - delta),  dQ = dS K,  dK = dS^T Q
// (tpa/tpa.py:546-995 computes the same quantities per block pair).  Two kernels, each of which
// owns its output rows and therefore needs no atomics:
//   bwd_f32_dq_kernel   workgroup = 128 query rows (4 waves x 32) of one head, loops over key tiles
//   bwd_f32_dkv_kernel  workgroup = 128 keys (4 waves x 32) of one head, loops over query tiles
// The operand placement is that of the fp32 forward kernel: the wave's own 32 rows (queries or
// keys) stay in registers as B operands, so a lane holds the logits of ONE of its rows; the
// streamed tile (64 rows, double buffered in LDS) supplies the A operands with 16-byte reads in
// both roles - as rows (contraction over d: wave half g takes d = 8m + 4g + e) and transposed
// (contraction over the tile's rows: half g takes the row its accumulator register belongs to,
// and the 32 output rows of block db are d = (D/32) i + db) - and the p / dS accumulators are used
// in place as the B operands of the second contraction.
// One wave per SIMD (the register budget of 512 is what holds the wave's rows, two accumulators
// and the next tile in flight); the matrix pipe is the bound by a wide margin.
#include "tpa_common.h"

namespace tpa {
namespace {

constexpr int kTile = 64;    // rows of the streamed tile
constexpr int kWaves = 4;    // waves per workgroup
constexpr int kBlock = 128;  // rows a workgroup owns (32 per wave)
constexpr int kThreads = kWaves * 64;

struct BwdF32Params {
  const float *q, *k, *v, *d_o, *lse, *delta;
  const int32_t *qseg, *kvseg;
  float *dq, *dk, *dv;
  int B, lq, lk, H;
  float sm_scale;
  int causal, coff, nblk, npairs;  // coff: with causal, row i sees keys <= i + coff
};

template <int D>
struct BwdLds {
  static constexpr int RS = D + 4;          // row stride (floats)
  static constexpr int kMat = kTile * RS;   // floats of one tile of one matrix
  // two matrices double buffered, then per buffer: lse2[64], delta[64], segment ids[64]
  static constexpr size_t kBytes = (size_t)(4 * kMat + 2 * 3 * kTile) * 4;
};

// which (block, batch, head): heads of one (block, batch) pair on one XCD, pairs in launch order
__device__ __forceinline__ bool decode_block(int npairs, int H, int B, int& pair, int& h) {
  const int id = blockIdx.x, xcd = id & 7, slot = id >> 3;
  const int round = slot / H;
  pair = round * 8 + xcd_pair_slot(round, xcd, B);
  h = slot % H;
  return pair < npairs;
}

// The 64 x D tile of dense X[b, row0 .., h, :] that `issue` fetched, into LDS; rows >= nrows as zeros.
template <int D>
struct TileRegs {
  static constexpr int CPR = D / 4, CH = kTile * CPR / kThreads;
  f32x4 r[CH];
  __device__ __forceinline__ void issue(const float* base, int64_t row_stride, int row0, int nrows, bool scrub_nan) {
#pragma unroll
    for (int c = 0; c < CH; ++c) {
      const int chunk = c * kThreads + threadIdx.x, t = chunk / CPR, cc = chunk % CPR;
      f32x4 x = {0.f, 0.f, 0.f, 0.f};
      if (row0 + t < nrows) x = *reinterpret_cast<const f32x4*>(base + (int64_t)(row0 + t) * row_stride + 4 * cc);
      if (scrub_nan) {
#pragma unroll
        for (int e = 0; e < 4; ++e) x[e] = x[e] == x[e] ? x[e] : 0.f;
      }
      r[c] = x;
    }
  }
  __device__ __forceinline__ void store(float* dst) const {
#pragma unroll
    for (int c = 0; c < CH; ++c) {
      const int chunk = c * kThreads + threadIdx.x, t = chunk / CPR, cc = chunk % CPR;
      *reinterpret_cast<f32x4*>(dst + t * BwdLds<D>::RS + 4 * cc) = r[c];
    }
  }
};

// the wave's own row (B operand of the row-wise contractions): out[4m + e] = scale * X[row][8m + 4g + e]
template <int D>
__device__ __forceinline__ void load_own_row(const float* rowp, int g, float scale, bool scrub_nan, float (&out)[D / 2]) {
#pragma unroll
  for (int m = 0; m < D / 8; ++m) {
    const f32x4 x = *reinterpret_cast<const f32x4*>(rowp + 8 * m + 4 * g);
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      float y = x[e];
      if (scrub_nan) y = y == y ? y : 0.f;
      out[4 * m + e] = y * scale;
    }
  }
}

// acc0 / acc1 (rows 0-31 / 32-63 of the tile, lane = own row) = tile rows . own row, over d
template <int D>
__device__ __forceinline__ void rows_dot(const float* tile, int i, int g, const float (&own)[D / 2], f32x16& acc0, f32x16& acc1) {
  constexpr int RS = BwdLds<D>::RS;
#pragma unroll
  for (int v = 0; v < 16; ++v) { acc0[v] = 0.f; acc1[v] = 0.f; }
#pragma unroll
  for (int m = 0; m < D / 8; ++m) {
    const f32x4 a0 = *reinterpret_cast<const f32x4*>(tile + i * RS + 8 * m + 4 * g);
    const f32x4 a1 = *reinterpret_cast<const f32x4*>(tile + (32 + i) * RS + 8 * m + 4 * g);
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      acc0 = __builtin_amdgcn_mfma_f32_32x32x2f32(a0[e], own[4 * m + e], acc0, 0, 0, 0);
      acc1 = __builtin_amdgcn_mfma_f32_32x32x2f32(a1[e], own[4 * m + e], acc1, 0, 0, 0);
    }
  }
}

// out[db] (rows d = (D/32) i + db, lane = own row) += tile^T . w, over the tile's rows; w0 / w1 are
// accumulators of rows_dot's layout (register v, half g <-> tile row 32 mb + 8 (v/4) + 4 g + v%4)
template <int D>
__device__ __forceinline__ void cols_accumulate(const float* tile, int i, int g, const f32x16& w0, const f32x16& w1, f32x16 (&out)[D / 32]) {
  constexpr int RS = BwdLds<D>::RS, NDB = D / 32;
  typedef __attribute__((ext_vector_type(NDB))) float f32xN;
#pragma unroll
  for (int mb = 0; mb < 2; ++mb)
#pragma unroll
    for (int v = 0; v < 16; ++v) {
      const int row = 32 * mb + 8 * (v >> 2) + 4 * g + (v & 3);
      const f32xN a = *reinterpret_cast<const f32xN*>(tile + row * RS + NDB * i);
      const float wv = mb == 0 ? w0[v] : w1[v];
#pragma unroll
      for (int db = 0; db < NDB; ++db) out[db] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[db], wv, out[db], 0, 0, 0);
    }
}

template <int D>
__device__ __forceinline__ void store_own_row(float* rowp, int g, const f32x16 (&acc)[D / 32]) {
  constexpr int NDB = D / 32;
  typedef __attribute__((ext_vector_type(NDB))) float f32xN;
#pragma unroll
  for (int v = 0; v < 16; ++v) {
    const int row = 8 * (v >> 2) + 4 * g + (v & 3);
    f32xN out;
#pragma unroll
    for (int db = 0; db < NDB; ++db) out[db] = acc[db][v];
    *reinterpret_cast<f32xN*>(rowp + NDB * row) = out;
  }
}

// ------------------------------------------------------------------------------------- dQ
template <int D, bool SEG>
__global__ __launch_bounds__(kThreads) void bwd_f32_dq_kernel(BwdF32Params p) {
  constexpr int kMat = BwdLds<D>::kMat, NDB = D / 32;
  extern __shared__ __attribute__((aligned(16))) float smem_bwd_f32[];
  float* const lds_k = smem_bwd_f32;             // [2][kTile][RS]
  float* const lds_v = smem_bwd_f32 + 2 * kMat;  // [2][kTile][RS]
  int32_t* const lds_seg = reinterpret_cast<int32_t*>(smem_bwd_f32 + 4 * kMat);  // [2][kTile] key segment ids

  int pair, h;
  if (!decode_block(p.npairs, p.H, p.B, pair, h)) return;
  const int blk = p.nblk - 1 - pair / p.B;  // heaviest causal blocks first
  const int b = pair % p.B;
  const int tid = threadIdx.x, w = tid >> 6, l = tid & 63, i = l & 31, g = l >> 5;
  const int q0 = blk * kBlock, wrow0 = q0 + 32 * w, qrow = wrow0 + i, qrow_ld = min(qrow, p.lq - 1);
  const int64_t hd = (int64_t)p.H * D;

  const int kend = p.causal ? max(1, min(p.lk, q0 + kBlock + p.coff)) : p.lk;  // at least one (then fully masked) tile
  const int ntiles = (kend + kTile - 1) / kTile;
  const int wave_last_tile = p.causal ? min(ntiles - 1, max(wrow0 + p.coff + 31, 0) / kTile) : ntiles - 1;

  float qf[D / 2], gf[D / 2];
  load_own_row<D>(p.q + ((int64_t)b * p.lq + qrow_ld) * hd + (int64_t)h * D, g, p.sm_scale * kLog2e, false, qf);
  load_own_row<D>(p.d_o + ((int64_t)b * p.lq + qrow_ld) * hd + (int64_t)h * D, g, 1.f, true, gf);
  const float lse = p.lse[((int64_t)b * p.H + h) * p.lq + qrow_ld];
  // a row without a visible key (lse = -inf) has no gradient: +inf makes every p of the row zero
  const float lse2 = (qrow < p.lq && lse > -INFINITY) ? lse * kLog2e : INFINITY;
  const float delta = p.delta[((int64_t)b * p.H + h) * p.lq + qrow_ld];
  int32_t qseg = 0;
  if constexpr (SEG) qseg = p.qseg[(int64_t)b * p.lq + qrow_ld];

  f32x16 dq[NDB];
#pragma unroll
  for (int db = 0; db < NDB; ++db)
#pragma unroll
    for (int v = 0; v < 16; ++v) dq[db][v] = 0.f;

  const float* const kbase = p.k + (int64_t)b * p.lk * hd + (int64_t)h * D;
  const float* const vbase = p.v + (int64_t)b * p.lk * hd + (int64_t)h * D;
  TileRegs<D> kreg, vreg;
  int32_t seg_reg = 0;
  auto issue = [&](int tile) __attribute__((always_inline)) {
    kreg.issue(kbase, hd, tile * kTile, kend, false);
    vreg.issue(vbase, hd, tile * kTile, kend, false);
    if constexpr (SEG)
      if (tid < kTile) seg_reg = p.kvseg[(int64_t)b * p.lk + min(tile * kTile + tid, p.lk - 1)];
  };
  auto commit = [&](int tile) __attribute__((always_inline)) {
    kreg.store(lds_k + (tile & 1) * kMat);
    vreg.store(lds_v + (tile & 1) * kMat);
    if constexpr (SEG)
      if (tid < kTile) lds_seg[(tile & 1) * kTile + tid] = seg_reg;
  };

  auto compute = [&](int tile) __attribute__((always_inline)) {
    const float* const ks = lds_k + (tile & 1) * kMat;
    const float* const vs = lds_v + (tile & 1) * kMat;
    const int k0 = tile * kTile;
    f32x16 s[2], dp[2];
    rows_dot<D>(ks, i, g, qf, s[0], s[1]);    // x * log2(e)
    rows_dot<D>(vs, i, g, gf, dp[0], dp[1]);  // dP
    const int limit = p.causal ? min(qrow + p.coff, kend - 1) : kend - 1;  // largest visible key index
#pragma unroll
    for (int mb = 0; mb < 2; ++mb)
#pragma unroll
      for (int vq = 0; vq < 4; ++vq) {
        int4 ids = {0, 0, 0, 0};
        if constexpr (SEG) ids = *reinterpret_cast<const int4*>(lds_seg + (tile & 1) * kTile + 32 * mb + 8 * vq + 4 * g);
        const int idv[4] = {ids.x, ids.y, ids.z, ids.w};
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const int v = 4 * vq + e, t = k0 + 32 * mb + 8 * vq + 4 * g + e;
          bool keep = t <= limit;
          if constexpr (SEG) keep = keep && idv[e] == qseg;
          const float pt = keep ? __builtin_amdgcn_exp2f(s[mb][v] - lse2) : 0.f;
          s[mb][v] = p.sm_scale * pt * (dp[mb][v] - delta);  // dS
        }
      }
    cols_accumulate<D>(ks, i, g, s[0], s[1], dq);
  };

  issue(0);
  commit(0);
  __syncthreads();
  for (int j = 0; j < ntiles; ++j) {
    const bool more = j + 1 < ntiles;
    if (more) issue(j + 1);
    if (j <= wave_last_tile) compute(j);
    if (more) commit(j + 1);
    __syncthreads();
  }
  if (qrow < p.lq) store_own_row<D>(p.dq + ((int64_t)b * p.lq + qrow) * hd + (int64_t)h * D, g, dq);
}

// ------------------------------------------------------------------------------------- dK, dV
template <int D, bool SEG>
__global__ __launch_bounds__(kThreads) void bwd_f32_dkv_kernel(BwdF32Params p) {
  constexpr int kMat = BwdLds<D>::kMat, NDB = D / 32;
  extern __shared__ __attribute__((aligned(16))) float smem_bwd_f32[];
  float* const lds_q = smem_bwd_f32;             // [2][kTile][RS]
  float* const lds_g = smem_bwd_f32 + 2 * kMat;  // [2][kTile][RS]  upstream gradient rows
  float* const lds_row = smem_bwd_f32 + 4 * kMat;  // [2][lse2 | delta | segment id][kTile]

  int pair, h;
  if (!decode_block(p.npairs, p.H, p.B, pair, h)) return;
  const int blk = pair / p.B;  // under the causal mask the first key blocks see the most rows: heaviest first
  const int b = pair % p.B;
  const int tid = threadIdx.x, w = tid >> 6, l = tid & 63, i = l & 31, g = l >> 5;
  const int k0 = blk * kBlock, wkey0 = k0 + 32 * w, key = wkey0 + i, key_ld = min(key, p.lk - 1);
  const int64_t hd = (int64_t)p.H * D;

  // under the causal mask only rows at or after a key see it
  const int first_tile = p.causal ? max(k0 - p.coff, 0) / kTile : 0;
  const int ntiles = (p.lq + kTile - 1) / kTile;
  const int wave_first_tile = p.causal ? max(wkey0 - p.coff, 0) / kTile : 0;

  float kf[D / 2], vf[D / 2];
  load_own_row<D>(p.k + ((int64_t)b * p.lk + key_ld) * hd + (int64_t)h * D, g, p.sm_scale * kLog2e, false, kf);
  load_own_row<D>(p.v + ((int64_t)b * p.lk + key_ld) * hd + (int64_t)h * D, g, 1.f, false, vf);
  int32_t kseg = 0;
  if constexpr (SEG) kseg = p.kvseg[(int64_t)b * p.lk + key_ld];

  f32x16 dk[NDB], dv[NDB];
#pragma unroll
  for (int db = 0; db < NDB; ++db)
#pragma unroll
    for (int v = 0; v < 16; ++v) { dk[db][v] = 0.f; dv[db][v] = 0.f; }

  const float* const qbase = p.q + (int64_t)b * p.lq * hd + (int64_t)h * D;
  const float* const gbase = p.d_o + (int64_t)b * p.lq * hd + (int64_t)h * D;
  const float* const lse_b = p.lse + ((int64_t)b * p.H + h) * p.lq;
  const float* const delta_b = p.delta + ((int64_t)b * p.H + h) * p.lq;
  TileRegs<D> qreg, greg;
  float row_reg = 0.f;  // threads 0-63: lse2, 64-127: delta, 128-191: segment id of one row of the tile
  auto issue = [&](int tile) __attribute__((always_inline)) {
    qreg.issue(qbase, hd, tile * kTile, p.lq, false);
    greg.issue(gbase, hd, tile * kTile, p.lq, true);
    const int r = tile * kTile + (tid & (kTile - 1)), what = tid / kTile;
    if (what == 0) {
      const float lse = r < p.lq ? lse_b[r] : -INFINITY;
      row_reg = lse > -INFINITY ? lse * kLog2e : INFINITY;  // +inf: every p of the row is zero
    } else if (what == 1) {
      row_reg = r < p.lq ? delta_b[r] : 0.f;
    } else if (what == 2) {
      if constexpr (SEG) row_reg = __int_as_float(p.qseg[(int64_t)b * p.lq + min(r, p.lq - 1)]);
    }
  };
  auto commit = [&](int tile) __attribute__((always_inline)) {
    qreg.store(lds_q + (tile & 1) * kMat);
    greg.store(lds_g + (tile & 1) * kMat);
    if (tid < 3 * kTile) lds_row[(tile & 1) * 3 * kTile + tid] = row_reg;
  };

  auto compute = [&](int tile) __attribute__((always_inline)) {
    const float* const qs = lds_q + (tile & 1) * kMat;
    const float* const gs = lds_g + (tile & 1) * kMat;
    const float* const rows = lds_row + (tile & 1) * 3 * kTile;
    const int r0 = tile * kTile;
    f32x16 s[2], dp[2];
    rows_dot<D>(qs, i, g, kf, s[0], s[1]);    // x * log2(e); lane = key, registers = rows of the tile
    rows_dot<D>(gs, i, g, vf, dp[0], dp[1]);  // dP
#pragma unroll
    for (int mb = 0; mb < 2; ++mb)
#pragma unroll
      for (int vq = 0; vq < 4; ++vq) {
        const int off = 32 * mb + 8 * vq + 4 * g;
        const f32x4 lse2 = *reinterpret_cast<const f32x4*>(rows + off);
        const f32x4 dl = *reinterpret_cast<const f32x4*>(rows + kTile + off);
        f32x4 idf = {0.f, 0.f, 0.f, 0.f};
        if constexpr (SEG) idf = *reinterpret_cast<const f32x4*>(rows + 2 * kTile + off);
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const int v = 4 * vq + e, r = r0 + off + e;
          bool keep = !p.causal || key - p.coff <= r;
          if constexpr (SEG) keep = keep && __float_as_int(idf[e]) == kseg;
          const float pt = keep ? __builtin_amdgcn_exp2f(s[mb][v] - lse2[e]) : 0.f;
          s[mb][v] = pt;                                            // p
          dp[mb][v] = p.sm_scale * pt * (dp[mb][v] - dl[e]);        // dS
        }
      }
    cols_accumulate<D>(gs, i, g, s[0], s[1], dv);
    cols_accumulate<D>(qs, i, g, dp[0], dp[1], dk);
  };

  if (first_tile < ntiles) {
    issue(first_tile);
    commit(first_tile);
  }
  __syncthreads();
  for (int j = first_tile; j < ntiles; ++j) {
    const bool more = j + 1 < ntiles;
    if (more) issue(j + 1);
    if (j >= wave_first_tile) compute(j);
    if (more) commit(j + 1);
    __syncthreads();
  }
  if (key < p.lk) {
    store_own_row<D>(p.dk + ((int64_t)b * p.lk + key) * hd + (int64_t)h * D, g, dk);
    store_own_row<D>(p.dv + ((int64_t)b * p.lk + key) * hd + (int64_t)h * D, g, dv);
  }
}

template <int D, bool SEG>
int launch_pair(const BwdF32Params& base, hipStream_t stream) {
  static bool configured_q[kMaxDevices] = {}, configured_kv[kMaxDevices] = {};
  const size_t smem = BwdLds<D>::kBytes;
  {
    BwdF32Params p = base;
    p.nblk = (p.lq + kBlock - 1) / kBlock;
    p.npairs = p.nblk * p.B;
    auto kern = bwd_f32_dq_kernel<D, SEG>;
    if (int rc = raise_lds_limit(configured_q, reinterpret_cast<const void*>(kern), smem); rc != TPA_OK) return rc;
    hipLaunchKernelGGL(kern, dim3(((p.npairs + 7) / 8) * 8 * p.H), dim3(kThreads), smem, stream, p);
    if (hipGetLastError() != hipSuccess) return TPA_ERR_LAUNCH;
  }
  {
    BwdF32Params p = base;
    p.nblk = (p.lk + kBlock - 1) / kBlock;
    p.npairs = p.nblk * p.B;
    auto kern = bwd_f32_dkv_kernel<D, SEG>;
    if (int rc = raise_lds_limit(configured_kv, reinterpret_cast<const void*>(kern), smem); rc != TPA_OK) return rc;
    hipLaunchKernelGGL(kern, dim3(((p.npairs + 7) / 8) * 8 * p.H), dim3(kThreads), smem, stream, p);
    if (hipGetLastError() != hipSuccess) return TPA_ERR_LAUNCH;
  }
  return TPA_OK;
}

}  // namespace
}  // namespace tpa

// dense fp32 q, k, v, d_o [B, l, H, D] with D in {64, 128}, rows 16-byte aligned, no bias
int dense_bwd_f32_supported(int dtype, int dk, int dv, int64_t lq, int64_t lk, const void* bias) {
  if (dtype != TPA_DTYPE_F32 || dk != dv || (dk != 64 && dk != 128) || bias) return 0;
  // both kernels spend a 128-row block on every head however few rows there are
  if (lq < 64 || lk < 64) return 0;
  return 1;
}

int dense_bwd_f32_launch(const float* q, const float* k, const float* v, const float* d_o, const float* lse, const float* delta,
                         const int32_t* qseg, const int32_t* kvseg, float* dq, float* dk, float* dv, int B, int lq, int lk,
                         int H, int D, float sm_scale, int causal, int coff, hipStream_t stream) {
  tpa::BwdF32Params p{};
  p.q = q; p.k = k; p.v = v; p.d_o = d_o; p.lse = lse; p.delta = delta; p.qseg = qseg; p.kvseg = kvseg;
  p.dq = dq; p.dk = dk; p.dv = dv; p.B = B; p.lq = lq; p.lk = lk; p.H = H; p.sm_scale = sm_scale; p.causal = causal; p.coff = causal ? coff : 0;
  if (qseg) return D == 128 ? tpa::launch_pair<128, true>(p, stream) : tpa::launch_pair<64, true>(p, stream);
  return D == 128 ? tpa::launch_pair<128, false>(p, stream) : tpa::launch_pair<64, false>(p, stream);
}
