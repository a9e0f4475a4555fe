// Any-shape forward kernel: fp32 arithmetic on the vector ALUs, no MFMA.
//
// It serves the problems the MFMA kernels do not take: fp32 inputs, head dimensions other than
// 64 and 128, unaligned operands and dense biases.  One thread owns one query row of one
// head and keeps q and the output accumulator in registers; the workgroup rebuilds the head's
// K and V tile from the rank factors in LDS (tpa/tpa.py:364,417) and every thread walks the
// tile with an online softmax (tpa/tpa.py:389-424, in the deferred-normalisation form).
#include "tpa_common.h"

namespace tpa {
namespace {

constexpr int kRows = 128;  // query rows (= threads) per workgroup
constexpr int kTile = 32;   // keys per LDS tile

struct GenericParams {
  // TPA factors (dense == 0) or dense q/k/v (dense == 1: *a unused, *b = dense tensors with
  // stride_r unused, stride_l = H*d, and the head offset added per workgroup)
  TpaFactor qa, qb, ka, kb, va, vb;
  const int32_t* qseg;
  const int32_t* kvseg;
  const float* bias;  // [B, lq, lk] or null
  const int32_t* kvlen;  // [B] keys per batch entry, or null (= lk)
  void* o;
  float* lse;
  int B, lq, lk, H, dk, dv, rq, rk;
  float sm_scale;
  int causal;
  int coff;  // with causal: row i sees keys <= i + coff
  int dense;
};

template <typename T, int DMAX>
__global__ __launch_bounds__(kRows) void generic_fwd_kernel(GenericParams p) {
  const int b = blockIdx.z;
  const int h = blockIdx.y;
  const int row = blockIdx.x * kRows + threadIdx.x;
  const bool row_ok = row < p.lq;
  const int dk = p.dk, dv = p.dv;

  extern __shared__ float smem[];
  float* ks = smem;               // [kTile][dk]
  float* vs = smem + kTile * dk;  // [kTile][dv]
  int* segs = reinterpret_cast<int*>(vs + kTile * dv);  // [kTile]

  // ---- this thread's query row
  float q[DMAX];
#pragma unroll
  for (int d = 0; d < DMAX; ++d) q[d] = 0.f;
  if (row_ok) {
    if (p.dense) {
      const T* qp = static_cast<const T*>(p.qb.ptr) + b * p.qb.stride_b + row * p.qb.stride_l + (int64_t)h * dk;
#pragma unroll
      for (int d = 0; d < DMAX; ++d)
        if (d < dk) q[d] = load_as_f32(qp + d);
    } else {
      const T* ap = static_cast<const T*>(p.qa.ptr) + b * p.qa.stride_b + row * p.qa.stride_l + h;
      const T* bp = static_cast<const T*>(p.qb.ptr) + b * p.qb.stride_b + row * p.qb.stride_l;
      for (int r = 0; r < p.rq; ++r) {
        const float a = load_as_f32(ap + r * p.qa.stride_r);
#pragma unroll
        for (int d = 0; d < DMAX; ++d)
          if (d < dk) q[d] += a * load_as_f32(bp + r * p.qb.stride_r + d);
      }
      const float inv = 1.f / (float)p.rq;
#pragma unroll
      for (int d = 0; d < DMAX; ++d) q[d] *= inv;
    }
  }
  const int qseg = (row_ok && p.qseg) ? p.qseg[(int64_t)b * p.lq + row] : 0;

  float acc[DMAX];
#pragma unroll
  for (int d = 0; d < DMAX; ++d) acc[d] = 0.f;
  float m = -INFINITY;  // running max of the scaled logits
  float l = 0.f;        // running sum of exp(x - m)

  // keys this workgroup has to visit
  int k_end = p.kvlen ? max(0, min(p.kvlen[b], p.lk)) : p.lk;
  const int coff = p.coff + (p.causal == TPA_CAUSAL_BOTTOM_RIGHT ? k_end - p.lq : 0);  // counted from the end of this entry's keys
  if (p.causal) {
    const int last_row = min(p.lq, (int)(blockIdx.x + 1) * kRows) - 1;
    k_end = min(k_end, last_row + 1 + coff);
  }

  for (int k0 = 0; k0 < k_end; k0 += kTile) {
    const int nk = min(kTile, k_end - k0);
    __syncthreads();
    // ---- rebuild the K and V tile of head h
    for (int idx = threadIdx.x; idx < nk * dk; idx += kRows) {
      const int t = idx / dk, d = idx - t * dk;
      const int tok = k0 + t;
      float val;
      if (p.dense) {
        val = load_as_f32(static_cast<const T*>(p.kb.ptr) + b * p.kb.stride_b + tok * p.kb.stride_l + (int64_t)h * dk + d);
      } else {
        const T* ap = static_cast<const T*>(p.ka.ptr) + b * p.ka.stride_b + tok * p.ka.stride_l + h;
        const T* bp = static_cast<const T*>(p.kb.ptr) + b * p.kb.stride_b + tok * p.kb.stride_l + d;
        val = 0.f;
        for (int r = 0; r < p.rk; ++r) val += load_as_f32(ap + r * p.ka.stride_r) * load_as_f32(bp + r * p.kb.stride_r);
        val *= 1.f / (float)p.rk;
      }
      ks[t * dk + d] = val;
    }
    for (int idx = threadIdx.x; idx < nk * dv; idx += kRows) {
      const int t = idx / dv, d = idx - t * dv;
      const int tok = k0 + t;
      float val;
      if (p.dense) {
        val = load_as_f32(static_cast<const T*>(p.vb.ptr) + b * p.vb.stride_b + tok * p.vb.stride_l + (int64_t)h * dv + d);
      } else {
        const T* ap = static_cast<const T*>(p.va.ptr) + b * p.va.stride_b + tok * p.va.stride_l + h;
        const T* bp = static_cast<const T*>(p.vb.ptr) + b * p.vb.stride_b + tok * p.vb.stride_l + d;
        val = 0.f;
        for (int r = 0; r < p.rk; ++r) val += load_as_f32(ap + r * p.va.stride_r) * load_as_f32(bp + r * p.vb.stride_r);
        val *= 1.f / (float)p.rk;
      }
      vs[t * dv + d] = val;
    }
    if (p.kvseg)
      for (int t = threadIdx.x; t < nk; t += kRows) segs[t] = p.kvseg[(int64_t)b * p.lk + k0 + t];
    __syncthreads();

    if (!row_ok) continue;
    // ---- logits of this row against the tile
    float s[kTile];
    float tile_max = -INFINITY;
#pragma unroll
    for (int t = 0; t < kTile; ++t) {
      float x = -INFINITY;
      if (t < nk) {
        float dot = 0.f;
#pragma unroll
        for (int d = 0; d < DMAX; ++d)
          if (d < dk) dot += q[d] * ks[t * dk + d];
        x = dot * p.sm_scale;
        if (p.bias) x += p.bias[((int64_t)b * p.lq + row) * p.lk + k0 + t];
        bool keep = true;
        if (p.kvseg) keep = segs[t] == qseg;
        if (p.causal) keep = keep && (k0 + t <= row + coff);
        if (!keep) x = -INFINITY;
      }
      s[t] = x;
      tile_max = fmaxf(tile_max, x);
    }
    if (tile_max == -INFINITY) continue;  // nothing visible in this tile
    const float m_new = fmaxf(m, tile_max);
    const float alpha = expf(m - m_new);  // m = -inf -> 0
    l *= alpha;
#pragma unroll
    for (int d = 0; d < DMAX; ++d) acc[d] *= alpha;
#pragma unroll
    for (int t = 0; t < kTile; ++t) {
      if (t < nk) {
        const float pt = expf(s[t] - m_new);  // -inf -> 0
        l += pt;
#pragma unroll
        for (int d = 0; d < DMAX; ++d)
          if (d < dv) acc[d] += pt * vs[t * dv + d];
      }
    }
    m = m_new;
  }

  if (!row_ok) return;
  // ---- finish: normalise, NaN for rows with no visible key (tpa/tpa.py:437-439)
  const bool empty = (m == -INFINITY);
  const float inv_l = empty ? 0.f : 1.f / l;
  T* op = static_cast<T*>(p.o) + (((int64_t)b * p.lq + row) * p.H + h) * dv;
#pragma unroll
  for (int d = 0; d < DMAX; ++d)
    if (d < dv) store_from_f32(op + d, empty ? NAN : acc[d] * inv_l);
  if (p.lse) p.lse[((int64_t)b * p.H + h) * p.lq + row] = empty ? -INFINITY : m + logf(l);
}

// A few query rows over many keys (a decode that the split-key kernels do not take: odd head sizes,
// masks, ranks that are no power of two).  One thread per row would leave a workgroup with one busy
// thread, so here a workgroup owns ONE (batch, head, query row) and spreads the keys: per chunk of
// keys the four waves take keys in turn, lanes over d, for the logits (the non-materialising form
// s = (1/R) sum_r a_r (q . b_r), tpa/tpa.py:333-359); the chunk's maximum and sum are block
// reductions; then thread d accumulates o[d] over the chunk's keys.  Same recurrence as above.
constexpr int kChunk = 1024;    // keys per pass
constexpr int kFewThreads = 256;

__device__ __forceinline__ float wave_sum(float x) {
#pragma unroll
  for (int m = 32; m >= 1; m >>= 1) x += __shfl_xor(x, m, 64);
  return x;
}
__device__ __forceinline__ float wave_max(float x) {
#pragma unroll
  for (int m = 32; m >= 1; m >>= 1) x = fmaxf(x, __shfl_xor(x, m, 64));
  return x;
}

template <typename T>
__global__ __launch_bounds__(kFewThreads) void generic_fewrows_kernel(GenericParams p) {
  const int b = blockIdx.z, h = blockIdx.y, row = blockIdx.x;
  const int dk = p.dk, dv = p.dv;
  const int tid = threadIdx.x, w = tid >> 6, lane = tid & 63;
  extern __shared__ float smem[];
  float* qs = smem;            // [dk] the query row, scaled
  float* xs = smem + dk;       // [kChunk] logits, then probabilities
  float* red = xs + kChunk;    // [8] block reductions

  for (int d = tid; d < dk; d += kFewThreads) {
    float q = 0.f;
    if (p.dense) {
      q = load_as_f32(static_cast<const T*>(p.qb.ptr) + b * p.qb.stride_b + row * p.qb.stride_l + (int64_t)h * dk + d);
    } else {
      const T* ap = static_cast<const T*>(p.qa.ptr) + b * p.qa.stride_b + row * p.qa.stride_l + h;
      const T* bp = static_cast<const T*>(p.qb.ptr) + b * p.qb.stride_b + row * p.qb.stride_l + d;
      for (int r = 0; r < p.rq; ++r) q += load_as_f32(ap + r * p.qa.stride_r) * load_as_f32(bp + r * p.qb.stride_r);
      q *= 1.f / (float)p.rq;
    }
    qs[d] = q * p.sm_scale;
  }
  const int qseg = p.qseg ? p.qseg[(int64_t)b * p.lq + row] : 0;
  int k_end = p.kvlen ? max(0, min(p.kvlen[b], p.lk)) : p.lk;
  const int coff = p.coff + (p.causal == TPA_CAUSAL_BOTTOM_RIGHT ? k_end - p.lq : 0);  // counted from the end of this entry's keys
  if (p.causal) k_end = min(k_end, row + 1 + coff);
  const float inv_rk = 1.f / (float)p.rk;

  float m = -INFINITY, l = 0.f, acc = 0.f;  // acc: o[tid] for tid < dv
  for (int c0 = 0; c0 < k_end; c0 += kChunk) {
    const int nk = min(kChunk, k_end - c0);
    __syncthreads();  // qs written / the previous chunk's xs consumed
    // ---- logits: wave w takes keys 4w .. 4w + 3, then 16 further on, ... (four keys' loads in flight together)
    for (int t0 = 4 * w; t0 < nk; t0 += 4 * (kFewThreads / 64)) {
      float x[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int tok = c0 + min(t0 + u, nk - 1);
        float xu = 0.f;
        if (p.dense) {
          const T* kp = static_cast<const T*>(p.kb.ptr) + b * p.kb.stride_b + tok * p.kb.stride_l + (int64_t)h * dk;
          for (int d = lane; d < dk; d += 64) xu += qs[d] * load_as_f32(kp + d);
        } else {
          const T* ap = static_cast<const T*>(p.ka.ptr) + b * p.ka.stride_b + tok * p.ka.stride_l + h;
          const T* bp = static_cast<const T*>(p.kb.ptr) + b * p.kb.stride_b + tok * p.kb.stride_l;
          for (int r = 0; r < p.rk; ++r) {
            float part = 0.f;
            for (int d = lane; d < dk; d += 64) part += qs[d] * load_as_f32(bp + r * p.kb.stride_r + d);
            xu += load_as_f32(ap + r * p.ka.stride_r) * part;  // the same a for every lane: the sum over lanes can wait
          }
          xu *= inv_rk;
        }
        x[u] = xu;
      }
#pragma unroll
      for (int u = 0; u < 4; ++u) x[u] = wave_sum(x[u]);
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int t = t0 + u;
        if (t < nk) {
          const int tok = c0 + t;
          float xu = x[u];
          if (p.bias) xu += p.bias[((int64_t)b * p.lq + row) * p.lk + tok];
          if (p.kvseg && p.kvseg[(int64_t)b * p.lk + tok] != qseg) xu = -INFINITY;
          if (lane == 0) xs[t] = xu;
        }
      }
    }
    __syncthreads();
    // ---- the chunk's maximum
    float cm = -INFINITY;
    for (int t = tid; t < nk; t += kFewThreads) cm = fmaxf(cm, xs[t]);
    cm = wave_max(cm);
    if (lane == 0) red[w] = cm;
    __syncthreads();
    cm = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
    if (cm == -INFINITY) continue;  // nothing visible in this chunk (uniform over the workgroup)
    const float m_new = fmaxf(m, cm);
    const float alpha = expf(m - m_new);  // m = -inf -> 0
    float ls = 0.f;
    for (int t = tid; t < nk; t += kFewThreads) {
      const float pt = expf(xs[t] - m_new);  // -inf -> 0
      xs[t] = pt;
      ls += pt;
    }
    ls = wave_sum(ls);
    if (lane == 0) red[4 + w] = ls;
    __syncthreads();
    l = l * alpha + (red[4] + red[5]) + (red[6] + red[7]);
    m = m_new;
    // ---- o[d] += sum_t p_t V[t][d], thread = d
    if (tid < dv) {
      acc *= alpha;
      constexpr int U = 16;  // keys whose loads are in flight together
      for (int t0 = 0; t0 < nk; t0 += U) {
        float pv[U], vv[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
          const int t = min(t0 + u, nk - 1);
          const int tok = c0 + t;
          pv[u] = t0 + u < nk ? xs[t] : 0.f;
          if (p.dense) {
            vv[u] = load_as_f32(static_cast<const T*>(p.vb.ptr) + b * p.vb.stride_b + tok * p.vb.stride_l + (int64_t)h * dv + tid);
          } else {
            const T* ap = static_cast<const T*>(p.va.ptr) + b * p.va.stride_b + tok * p.va.stride_l + h;
            const T* bp = static_cast<const T*>(p.vb.ptr) + b * p.vb.stride_b + tok * p.vb.stride_l + tid;
            float v = 0.f;
            for (int r = 0; r < p.rk; ++r) v += load_as_f32(ap + r * p.va.stride_r) * load_as_f32(bp + r * p.vb.stride_r);
            vv[u] = v * inv_rk;
          }
        }
#pragma unroll
        for (int u = 0; u < U; ++u) acc += pv[u] == 0.f ? 0.f : pv[u] * vv[u];  // a masked key contributes nothing, whatever its value
      }
    }
  }
  // ---- finish: normalise, NaN for a row with no visible key (tpa/tpa.py:437-439)
  const bool empty = (m == -INFINITY);
  if (tid < dv) {
    T* op = static_cast<T*>(p.o) + (((int64_t)b * p.lq + row) * p.H + h) * dv;
    store_from_f32(op + tid, empty ? NAN : acc / l);
  }
  if (p.lse && tid == 0) p.lse[((int64_t)b * p.H + h) * p.lq + row] = empty ? -INFINITY : m + logf(l);
}

template <typename T>
int launch_generic(const GenericParams& p, hipStream_t stream) {
  const int dmax = p.dk > p.dv ? p.dk : p.dv;
  if (p.lq <= 16 && p.lk >= 256 && dmax <= kFewThreads && p.lq <= 65535) {
    const size_t smem_few = (size_t)(p.dk + kChunk + 8) * sizeof(float);
    hipLaunchKernelGGL((generic_fewrows_kernel<T>), dim3(p.lq, p.H, p.B), dim3(kFewThreads), smem_few, stream, p);
    return hipGetLastError() == hipSuccess ? TPA_OK : TPA_ERR_LAUNCH;
  }
  dim3 grid((p.lq + kRows - 1) / kRows, p.H, p.B);
  dim3 block(kRows);
  const size_t smem = (size_t)kTile * (p.dk + p.dv) * sizeof(float) + kTile * sizeof(int);
  if (dmax <= 8)
    hipLaunchKernelGGL((generic_fwd_kernel<T, 8>), grid, block, smem, stream, p);
  else if (dmax <= 32)
    hipLaunchKernelGGL((generic_fwd_kernel<T, 32>), grid, block, smem, stream, p);
  else if (dmax <= 64)
    hipLaunchKernelGGL((generic_fwd_kernel<T, 64>), grid, block, smem, stream, p);
  else if (dmax <= 128)
    hipLaunchKernelGGL((generic_fwd_kernel<T, 128>), grid, block, smem, stream, p);
  else if (dmax <= 256) {
    // two 256-wide tiles are a few bytes over the 64 KB a kernel gets without asking
    if (smem > 64 * 1024 &&
        hipFuncSetAttribute(reinterpret_cast<const void*>(generic_fwd_kernel<T, 256>), hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem) != hipSuccess)
      return TPA_ERR_LAUNCH;
    hipLaunchKernelGGL((generic_fwd_kernel<T, 256>), grid, block, smem, stream, p);
  }
  else
    return TPA_ERR_SHAPE;
  return hipGetLastError() == hipSuccess ? TPA_OK : TPA_ERR_LAUNCH;
}

}  // namespace
}  // namespace tpa

int tpa_generic_launch(const TpaFwdArgs* a, hipStream_t stream) {
  tpa::GenericParams p{};
  p.qa = a->qa; p.qb = a->qb; p.ka = a->ka; p.kb = a->kb; p.va = a->va; p.vb = a->vb;
  p.qseg = a->q_segment_ids; p.kvseg = a->kv_segment_ids; p.bias = nullptr; p.kvlen = a->kv_lengths;
  p.o = a->o; p.lse = a->lse;
  p.B = a->B; p.lq = a->lq; p.lk = a->lk; p.H = a->H; p.dk = a->dk; p.dv = a->dv; p.rq = a->rq; p.rk = a->rk;
  p.sm_scale = a->sm_scale; p.causal = a->causal; p.coff = tpa::causal_offset_of(a); p.dense = 0;
  if (a->B > 65535 || a->H > 65535) return TPA_ERR_SHAPE;
  if (a->dtype == TPA_DTYPE_F32) return tpa::launch_generic<float>(p, stream);
  if (a->dtype == TPA_DTYPE_BF16) return tpa::launch_generic<uint16_t>(p, stream);
  return TPA_ERR_DTYPE;
}

int mha_generic_launch(const MhaFwdArgs* a, hipStream_t stream) {
  tpa::GenericParams p{};
  p.qb = TpaFactor{a->q, (int64_t)a->lq * a->H * a->dk, (int64_t)a->H * a->dk, 0};
  p.kb = TpaFactor{a->k, (int64_t)a->lk * a->H * a->dk, (int64_t)a->H * a->dk, 0};
  p.vb = TpaFactor{a->v, (int64_t)a->lk * a->H * a->dv, (int64_t)a->H * a->dv, 0};
  p.qseg = nullptr; p.kvseg = nullptr; p.bias = a->bias;
  p.o = a->o; p.lse = a->lse;
  p.B = a->B; p.lq = a->lq; p.lk = a->lk; p.H = a->H; p.dk = a->dk; p.dv = a->dv; p.rq = 1; p.rk = 1;
  p.sm_scale = a->sm_scale; p.causal = a->causal ? TPA_CAUSAL_TOP_LEFT : TPA_CAUSAL_NONE; p.dense = 1;
  if (a->B > 65535 || a->H > 65535) return TPA_ERR_SHAPE;
  if (a->dtype == TPA_DTYPE_F32) return tpa::launch_generic<float>(p, stream);
  if (a->dtype == TPA_DTYPE_BF16) return tpa::launch_generic<uint16_t>(p, stream);
  return TPA_ERR_DTYPE;
}
