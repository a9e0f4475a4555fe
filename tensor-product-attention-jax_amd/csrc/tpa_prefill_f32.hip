// Flash-style prefill for fp32 inputs on gfx950: fp32 MFMA contractions, fp32 online softmax.
//
// Same decomposition as the bf16 kernel: one workgroup = one (batch, head, block of 256 query
// rows), eight waves of 32 rows; per tile of 64 keys the workgroup rebuilds the head's K and V
// tile from the rank factors (K = (1/R) sum_r a_r (x) b_r, tpa/tpa.py:364,417) into LDS, as fp32,
// and each wave computes
//     S^T = K Q^T      v_mfma_f32_32x32x2_f32; Q stays in registers, pre-scaled by
//                      sm_scale*log2(e); each lane ends up with 32 logits of ONE query row
//     online softmax   the recurrence of tpa/tpa.py:389-424 with the normalisation deferred
//     O^T += V^T P^T   the S^T accumulator, turned into P in place, is the B operand
// A 32x32x2 step takes two contraction indices, one per half of the wave.  Neither contraction
// cares about the order of its index, so the halves walk it in the order that makes every LDS
// operand read a 16-byte one: over d, half g takes d = 8m + 4g + e (m outer, e = 0..3 from one
// read); over keys, half g takes the key its S^T register already belongs to; and the rows of a
// 32-row block of O^T are d = (D/32) i + block, so one read of V[key][(D/32) i ...] feeds all
// blocks and the epilogue stores whole vectors.
// The matrix pipe is the bound by a wide margin (256 MFMAs of 64 cycles per wave and tile against
// a few hundred vector instructions), so the loop is plain: rebuild the next tile, compute this
// one, one barrier.  The dense baseline (tpa/mha.py:23-37) is the same kernel with rank 1 and
// weight 1.
#include "tpa_common.h"

namespace tpa {
namespace {

constexpr int kTK = 64;   // keys per tile
constexpr int kNW = 8;    // waves per workgroup
constexpr int kBQ = 256;  // query rows per workgroup (32 per wave)

struct F32Params {
  TpaFactor qa, qb, ka, kb, va, vb;  // dense: a pointers null, b = q/k/v with stride_l = H*D
  const int32_t* qseg;
  const int32_t* kvseg;
  const int32_t* kvlen;
  float* o;
  float* lse;
  int B, lq, lk, H, rq, rk;
  float sm_scale;
  int causal, coff, nqb, npairs;  // coff: with causal, row i sees keys <= i + coff
};

template <int D>
struct LdsF32 {
  static constexpr int RS = D + 4;        // row stride (floats): 16-byte reads of 16 rows hit distinct banks
  static constexpr int kTile = kTK * RS;  // floats of one tile
  static constexpr size_t kBytes = (size_t)(4 * kTile + 2 * kTK) * 4;  // K and V double buffered + key segment ids
};

template <int D, bool SEG>
__global__ __launch_bounds__(kNW * 64) void prefill_f32_kernel(F32Params pp) {
  constexpr int NT = kNW * 64;
  constexpr int RS = LdsF32<D>::RS, kTile = LdsF32<D>::kTile;
  constexpr int NDB = D / 32;         // 32-row blocks of O^T
  constexpr int NQ = D / 2;           // Q values per lane
  constexpr int CPR = D / 4;          // 16-byte chunks per row
  constexpr int CH = kTK * CPR / NT;  // chunks per thread, tile and matrix
  static_assert(CH >= 1 && kTK * CPR % NT == 0, "loader shape");
  typedef __attribute__((ext_vector_type(NDB))) float f32xN;

  struct Fac { const float* ptr; int64_t stride_b, stride_l, stride_r; };
  auto fac = [](const TpaFactor& f) { return Fac{static_cast<const float*>(f.ptr), f.stride_b, f.stride_l, f.stride_r}; };
  struct { Fac qa, qb, ka, kb, va, vb; const int32_t* qseg; const int32_t* kvseg; const int32_t* kvlen; float* o; float* lse; int B, lq, lk, H, rq, rk; float sm_scale; int causal, coff, nqb, npairs; } const p = {
      fac(pp.qa), fac(pp.qb), fac(pp.ka), fac(pp.kb), fac(pp.va), fac(pp.vb), pp.qseg, pp.kvseg, pp.kvlen, pp.o, pp.lse,
      pp.B, pp.lq, pp.lk, pp.H, pp.rq, pp.rk, pp.sm_scale, pp.causal, pp.causal ? pp.coff : 0, pp.nqb, pp.npairs};

  extern __shared__ __attribute__((aligned(16))) float smem_f32[];
  float* const lds_k = smem_f32;                                         // [2][kTK][RS]
  float* const lds_v = smem_f32 + 2 * kTile;                             // [2][kTK][RS]
  int32_t* const lds_seg = reinterpret_cast<int32_t*>(smem_f32 + 4 * kTile);  // [2][kTK]

  // heads of one (query block, batch) pair on one XCD (they share the B factors in its L2),
  // heaviest causal blocks first
  const int id = blockIdx.x;
  const int xcd = id & 7, slot = id >> 3;
  const int round = slot / p.H;
  const int pair = round * 8 + xcd_pair_slot(round, xcd, p.B);
  const int h = slot % p.H;
  if (pair >= p.npairs) return;
  const int qblk = p.nqb - 1 - pair / p.B;
  const int b = pair % p.B;

  const int tid = threadIdx.x;
  const int w = tid >> 6, l = tid & 63, i = l & 31, g = l >> 5;
  const int q0 = qblk * kBQ;
  const int wrow0 = q0 + 32 * w;
  const int qrow = wrow0 + i;
  const int qrow_ld = min(qrow, p.lq - 1);
  const bool dense = p.ka.ptr == nullptr;  // dense q, k, v: weight 1, the head's slice of the row

  // ---- key range
  const int len_b = p.kvlen ? max(0, min(p.kvlen[b], p.lk)) : p.lk;
  const int coff = p.coff + (p.causal == TPA_CAUSAL_BOTTOM_RIGHT ? len_b - p.lq : 0);  // bottom-right alignment counts from the end of this entry's keys
  const int kend = p.causal ? min(len_b, min(q0 + kBQ, p.lq) + coff) : len_b;
  float* const orow = p.o + (((int64_t)b * p.lq + qrow) * p.H + h) * D;
  if (kend <= 0) {  // no key at all: the rows end as NaN / -inf (tpa/tpa.py:437-439)
    if (qrow < p.lq) {
      const f32x4 nan4 = {__builtin_nanf(""), __builtin_nanf(""), __builtin_nanf(""), __builtin_nanf("")};
#pragma unroll
      for (int cch = 0; cch < D / 8; ++cch) *reinterpret_cast<f32x4*>(orow + 8 * cch + 4 * g) = nan4;
      if (p.lse && g == 0) p.lse[((int64_t)b * p.H + h) * p.lq + qrow] = -INFINITY;
    }
    return;
  }
  const int ntiles = (kend + kTK - 1) / kTK;
  const int wave_last_tile = p.causal ? min(ntiles - 1, max(wrow0 + coff + 31, 0) / kTK) : ntiles - 1;

  // ---- Q (B operand of S^T = K Q^T), scaled: qf[4m + e] = c * Q[qrow][8m + 4g + e]
  float qf[NQ];
#pragma unroll
  for (int j = 0; j < NQ; ++j) qf[j] = 0.f;
  {
    const float* qb = p.qb.ptr + b * p.qb.stride_b + (int64_t)qrow_ld * p.qb.stride_l + (dense ? (int64_t)h * D : 0) + 4 * g;
    const float* qa = dense ? nullptr : p.qa.ptr + b * p.qa.stride_b + (int64_t)qrow_ld * p.qa.stride_l + h;
    for (int r = 0; r < p.rq; ++r) {
      const float a = dense ? 1.f : qa[r * p.qa.stride_r];
#pragma unroll
      for (int m = 0; m < D / 8; ++m) {
        const f32x4 bv = *reinterpret_cast<const f32x4*>(qb + r * p.qb.stride_r + 8 * m);
#pragma unroll
        for (int e = 0; e < 4; ++e) qf[4 * m + e] += a * bv[e];
      }
    }
    const float scale = p.sm_scale * kLog2e / (float)p.rq;
#pragma unroll
    for (int j = 0; j < NQ; ++j) qf[j] *= scale;
  }

  // ---- tile rebuild: thread -> CH chunks of 4 floats per matrix
  const float* const kb_b = p.kb.ptr + b * p.kb.stride_b + (dense ? (int64_t)h * D : 0);
  const float* const vb_b = p.vb.ptr + b * p.vb.stride_b + (dense ? (int64_t)h * D : 0);
  const float* const ka_b = dense ? nullptr : p.ka.ptr + b * p.ka.stride_b + h;
  const float* const va_b = dense ? nullptr : p.va.ptr + b * p.va.stride_b + h;
  const float inv_r = 1.f / (float)p.rk;
  auto rebuild = [&](int tile) __attribute__((always_inline)) {
    float* const kd = lds_k + (tile & 1) * kTile;
    float* const vd = lds_v + (tile & 1) * kTile;
#pragma unroll
    for (int q = 0; q < CH; ++q) {
      const int chunk = q * NT + tid, t = chunk / CPR, cc = chunk % CPR;
      const int tok = tile * kTK + t;
      f32x4 ak = {0.f, 0.f, 0.f, 0.f}, av = {0.f, 0.f, 0.f, 0.f};
      if (tok < kend) {  // rows past the end stay zero: they are masked, and 0 * padding must not make NaN
        for (int r = 0; r < p.rk; ++r) {
          const float wk = dense ? 1.f : ka_b[(int64_t)tok * p.ka.stride_l + r * p.ka.stride_r];
          const float wv = dense ? 1.f : va_b[(int64_t)tok * p.va.stride_l + r * p.va.stride_r];
          const f32x4 bk = *reinterpret_cast<const f32x4*>(kb_b + (int64_t)tok * p.kb.stride_l + r * p.kb.stride_r + 4 * cc);
          const f32x4 bv = *reinterpret_cast<const f32x4*>(vb_b + (int64_t)tok * p.vb.stride_l + r * p.vb.stride_r + 4 * cc);
          ak += wk * bk;
          av += wv * bv;
        }
      }
      *reinterpret_cast<f32x4*>(kd + t * RS + 4 * cc) = ak * inv_r;
      *reinterpret_cast<f32x4*>(vd + t * RS + 4 * cc) = av * inv_r;
    }
    if constexpr (SEG)
      if (tid < kTK) lds_seg[(tile & 1) * kTK + tid] = p.kvseg[(int64_t)b * p.lk + min(tile * kTK + tid, p.lk - 1)];
  };

  // ---- per-wave state
  f32x16 o[NDB];
#pragma unroll
  for (int db = 0; db < NDB; ++db)
#pragma unroll
    for (int v = 0; v < 16; ++v) o[db][v] = 0.f;
  float m_run = -INFINITY;  // running max of row qrow (log2 domain, scale included)
  float lsum = 0.f;         // this lane's share of sum exp2(x - m_run)
  int32_t qseg = 0;
  if constexpr (SEG) qseg = p.qseg[(int64_t)b * p.lq + qrow_ld];

  f32x16 s[2];  // logits, then probabilities, of the tile in flight: two 32-key blocks
  auto logits_softmax = [&](int tile) __attribute__((always_inline)) {
    const float* const ks = lds_k + (tile & 1) * kTile;
    const int k0 = tile * kTK;
#pragma unroll
    for (int mb = 0; mb < 2; ++mb)
#pragma unroll
      for (int v = 0; v < 16; ++v) s[mb][v] = 0.f;
    // the two blocks' accumulation chains alternate, so no MFMA waits for the one just issued
#pragma unroll
    for (int m = 0; m < D / 8; ++m) {
      const f32x4 kf0 = *reinterpret_cast<const f32x4*>(ks + i * RS + 8 * m + 4 * g);
      const f32x4 kf1 = *reinterpret_cast<const f32x4*>(ks + (32 + i) * RS + 8 * m + 4 * g);
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        s[0] = __builtin_amdgcn_mfma_f32_32x32x2f32(kf0[e], qf[4 * m + e], s[0], 0, 0, 0);
        s[1] = __builtin_amdgcn_mfma_f32_32x32x2f32(kf1[e], qf[4 * m + e], s[1], 0, 0, 0);
      }
    }
    // register v of block mb, wave half g  <->  key k0 + 32 mb + 8 (v / 4) + 4 g + v % 4
    const bool need_mask = (k0 + kTK > kend) || (p.causal && (k0 + kTK - 1 > wrow0 + coff));
    if (need_mask) {
      const int limit = p.causal ? min(qrow + coff, kend - 1) : kend - 1;  // largest visible key index
#pragma unroll
      for (int mb = 0; mb < 2; ++mb)
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          const int t = k0 + 32 * mb + 8 * (v >> 2) + 4 * g + (v & 3);
          if (t > limit) s[mb][v] = -INFINITY;
        }
    }
    if constexpr (SEG) {  // keys of another segment (tpa/tpa.py:369-375)
      const int32_t* idslot = lds_seg + (tile & 1) * kTK;
#pragma unroll
      for (int mb = 0; mb < 2; ++mb)
#pragma unroll
        for (int vq = 0; vq < 4; ++vq) {
          const int4 ids = *reinterpret_cast<const int4*>(idslot + 32 * mb + 8 * vq + 4 * g);
          if (ids.x != qseg) s[mb][4 * vq] = -INFINITY;
          if (ids.y != qseg) s[mb][4 * vq + 1] = -INFINITY;
          if (ids.z != qseg) s[mb][4 * vq + 2] = -INFINITY;
          if (ids.w != qseg) s[mb][4 * vq + 3] = -INFINITY;
        }
    }
    float tmax = s[0][0];
#pragma unroll
    for (int mb = 0; mb < 2; ++mb)
#pragma unroll
      for (int v = 0; v < 16; ++v) tmax = fmaxf(tmax, s[mb][v]);
    tmax = halves_max(tmax);
    const float m_new = fmaxf(m_run, tmax);
    const float m_use = m_new == -INFINITY ? 0.f : m_new;  // a row that has met no visible key yet
    const float alpha = __builtin_amdgcn_exp2f(m_run - m_use);  // 0 while m_run is -inf (nothing accumulated)
    m_run = m_new;
    if (__any(alpha != 1.f)) {
      lsum *= alpha;
#pragma unroll
      for (int db = 0; db < NDB; ++db)
#pragma unroll
        for (int v = 0; v < 16; ++v) o[db][v] *= alpha;
    }
#pragma unroll
    for (int mb = 0; mb < 2; ++mb)
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const float pv = __builtin_amdgcn_exp2f(s[mb][v] - m_use);
        lsum += pv;
        s[mb][v] = pv;
      }
  };
  // O^T += V^T P^T: the step of register v takes, in wave half g, the key that register belongs to
  auto accumulate = [&](int tile) __attribute__((always_inline)) {
    const float* const vs = lds_v + (tile & 1) * kTile;
#pragma unroll
    for (int mb = 0; mb < 2; ++mb)
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int kr = 32 * mb + 8 * (v >> 2) + 4 * g + (v & 3);
        const f32xN vf = *reinterpret_cast<const f32xN*>(vs + kr * RS + NDB * i);
#pragma unroll
        for (int db = 0; db < NDB; ++db) o[db] = __builtin_amdgcn_mfma_f32_32x32x2f32(vf[db], s[mb][v], o[db], 0, 0, 0);
      }
  };

  rebuild(0);
  __syncthreads();
  // The next tile may be rebuilt anywhere between two barriers.  Waves w and w + 4 share a SIMD:
  // one of them rebuilds (waiting for its factor loads) before its matrix work, the other in the
  // middle of it, so the SIMD always has a wave with matrix work and both end the tile together.
  const bool rebuild_first = w < kNW / 2;
  for (int j = 0; j < ntiles; ++j) {
    const bool more = j + 1 < ntiles, mine = j <= wave_last_tile && wrow0 < p.lq;  // waves past the last row only help rebuild
    if (rebuild_first && more) rebuild(j + 1);
    if (mine) logits_softmax(j);
    if (!rebuild_first && more) rebuild(j + 1);
    if (mine) accumulate(j);
    __syncthreads();
  }

  // ---- epilogue: row 8 (v / 4) + 4 g + v % 4 of block db is d = NDB * row + db
  const float ltot = halves_sum(lsum);
  const float inv = 1.f / ltot;  // no visible key: 0 * inf = NaN, as in tpa/tpa.py:437-439
  if (qrow < p.lq) {
#pragma unroll
    for (int v = 0; v < 16; ++v) {
      const int row = 8 * (v >> 2) + 4 * g + (v & 3);
      f32xN out;
#pragma unroll
      for (int db = 0; db < NDB; ++db) out[db] = o[db][v] * inv;
      *reinterpret_cast<f32xN*>(orow + NDB * row) = out;
    }
    if (p.lse && g == 0) p.lse[((int64_t)b * p.H + h) * p.lq + qrow] = (m_run + __builtin_amdgcn_logf(ltot)) * kLn2;
  }
}

template <int D, bool SEG>
int launch_f32(const F32Params& p, hipStream_t stream) {
  auto kern = prefill_f32_kernel<D, SEG>;
  static bool configured[kMaxDevices] = {};
  if (int rc = raise_lds_limit(configured, reinterpret_cast<const void*>(kern), LdsF32<D>::kBytes); rc != TPA_OK) return rc;
  const int groups = (p.npairs + 7) / 8;
  hipLaunchKernelGGL(kern, dim3(groups * 8 * p.H), dim3(kNW * 64), LdsF32<D>::kBytes, stream, p);
  return hipGetLastError() == hipSuccess ? TPA_OK : TPA_ERR_LAUNCH;
}

int launch_any(const F32Params& p, int d, hipStream_t stream) {
  if (p.kvseg) return d == 128 ? launch_f32<128, true>(p, stream) : launch_f32<64, true>(p, stream);
  return d == 128 ? launch_f32<128, false>(p, stream) : launch_f32<64, false>(p, stream);
}

bool aligned16(const void* ptr) { return (reinterpret_cast<uintptr_t>(ptr) & 15) == 0; }
bool rows_ok(const TpaFactor& f) {  // rows of 4-float vectors
  return aligned16(f.ptr) && f.stride_b % 4 == 0 && f.stride_l % 4 == 0 && f.stride_r % 4 == 0;
}
}  // namespace
}  // namespace tpa

int tpa_prefill_f32_supported(const TpaFwdArgs* a) {
  if (a->dtype != TPA_DTYPE_F32) return 0;
  if (a->dk != a->dv || (a->dk != 64 && a->dk != 128)) return 0;
  if (!tpa::rows_ok(a->qb) || !tpa::rows_ok(a->kb) || !tpa::rows_ok(a->vb) || !tpa::aligned16(a->o)) return 0;
  return 1;
}

int tpa_prefill_f32_launch(const TpaFwdArgs* a, hipStream_t stream) {
  using namespace tpa;
  F32Params p{};
  p.qa = a->qa; p.qb = a->qb; p.ka = a->ka; p.kb = a->kb; p.va = a->va; p.vb = a->vb;
  p.qseg = a->q_segment_ids; p.kvseg = a->kv_segment_ids; p.kvlen = a->kv_lengths;
  p.o = static_cast<float*>(a->o); p.lse = a->lse;
  p.B = a->B; p.lq = a->lq; p.lk = a->lk; p.H = a->H; p.rq = a->rq; p.rk = a->rk;
  p.sm_scale = a->sm_scale; p.causal = a->causal; p.coff = causal_offset_of(a);
  p.nqb = (a->lq + kBQ - 1) / kBQ;
  p.npairs = p.nqb * a->B;
  return launch_any(p, a->dk, stream);
}

int mha_prefill_f32_supported(const MhaFwdArgs* a) {
  if (a->dtype != TPA_DTYPE_F32) return 0;
  if (a->dk != a->dv || (a->dk != 64 && a->dk != 128)) return 0;
  if (a->bias) return 0;
  if (!tpa::aligned16(a->q) || !tpa::aligned16(a->k) || !tpa::aligned16(a->v) || !tpa::aligned16(a->o)) return 0;
  return 1;
}

int mha_prefill_f32_launch(const MhaFwdArgs* a, hipStream_t stream) {
  using namespace tpa;
  F32Params p{};
  const int64_t hd = (int64_t)a->H * a->dk;
  p.qb = TpaFactor{a->q, a->lq * hd, hd, 0};
  p.kb = TpaFactor{a->k, a->lk * hd, hd, 0};
  p.vb = TpaFactor{a->v, a->lk * hd, hd, 0};
  p.qa = p.ka = p.va = TpaFactor{nullptr, 0, 0, 0};
  p.o = static_cast<float*>(a->o); p.lse = a->lse;
  p.B = a->B; p.lq = a->lq; p.lk = a->lk; p.H = a->H; p.rq = 1; p.rk = 1;
  p.sm_scale = a->sm_scale; p.causal = a->causal ? TPA_CAUSAL_TOP_LEFT : TPA_CAUSAL_NONE;
  p.nqb = (a->lq + kBQ - 1) / kBQ;
  p.npairs = p.nqb * a->B;
  return launch_any(p, a->dk, stream);
}
