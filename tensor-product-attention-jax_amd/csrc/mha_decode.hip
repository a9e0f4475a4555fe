// Dense multi-head attention for few query tokens over a long dense K/V cache (tpa/mha.py:23-37
// at lq = 1): the HBM-bound baseline the factored decode is compared with.  Per cached token
// it reads H*(dk+dv) elements, 16 384 B at H = 32, D = 128, against 1 280 B of rank-2 factors.
//
// A token's K row for all heads is one contiguous run of H*D elements, so a wave reads it with
// 16-byte loads, D/8 lanes per head; the lanes of a head reduce their partial dot products with
// DPP adds, every lane keeps the running max / sum of its heads and 8 output columns per head.
// Keys are split into ranges (grid.x) and token pairs are dealt round-robin to the 4 waves of a
// workgroup; the waves are merged through LDS, the ranges by a second small kernel with the
// rule of _lse_accum (tpa/tpa.py:228-242).
#include "tpa_common.h"

namespace tpa {
namespace {

constexpr int kWaves = 4;
constexpr int kNL = 4;   // 16-byte loads per token and lane for K (and for V)
constexpr int kTok = 2;  // tokens per wave iteration

struct MhaDecodeParams {
  const uint16_t* q;
  const uint16_t* k;
  const uint16_t* v;
  float* part_o;  // [B*lq, S, H, D]
  float* part_m;  // [B*lq, S, H]  running max (log2 domain)
  float* part_l;  // [B*lq, S, H]  sum of 2^(x - m)
  int B, lq, lk, H, S;
  float c;  // sm_scale * log2(e)
};

// sum over the LPH lanes that share a head (LPH = 8 or 16, aligned groups)
template <int LPH>
__device__ __forceinline__ float head_sum(float x) {
  x += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0xB1, 0xf, 0xf, false));   // quad_perm [1,0,3,2]
  x += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0x4E, 0xf, 0xf, false));   // quad_perm [2,3,0,1]
  x += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0x141, 0xf, 0xf, false));  // row_half_mirror
  if (LPH == 16)
    x += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0x140, 0xf, 0xf, false));  // row_mirror
  return x;
}

template <int D>
__global__ __launch_bounds__(kWaves * 64) void mha_decode_kernel(MhaDecodeParams p) {
  constexpr int LPH = D / 8;      // lanes per head
  constexpr int HPL = 64 / LPH;   // heads per load instruction
  constexpr int HW = kNL * HPL;   // heads per wave
  const int l = threadIdx.x & 63, w = threadIdx.x >> 6;
  const int b = blockIdx.x / p.S, s = blockIdx.x % p.S;
  const int qi = blockIdx.y;
  const int hbase = blockIdx.z * HW;
  const int H = p.H;
  const int sub = l / LPH, col = (l % LPH) * 8;

  // key range of this workgroup
  const int per = (p.lk + p.S - 1) / p.S;
  const int t_begin = s * per, t_end = min(p.lk, t_begin + per);

  // heads of slot i: hbase + i*HPL + sub; slots past H are skipped (uniform per wave)
  bool slot_ok[kNL];
  u32x4 qv[kNL];
#pragma unroll
  for (int i = 0; i < kNL; ++i) {
    slot_ok[i] = hbase + i * HPL < H;
    qv[i] = u32x4{0, 0, 0, 0};
    if (slot_ok[i])
      qv[i] = *reinterpret_cast<const u32x4*>(p.q + (((int64_t)b * p.lq + qi) * H + hbase + i * HPL + sub) * D + col);
  }

  float m[kNL], lsum[kNL], acc[kNL][8];
#pragma unroll
  for (int i = 0; i < kNL; ++i) {
    m[i] = -INFINITY;
    lsum[i] = 0.f;
#pragma unroll
    for (int j = 0; j < 8; ++j) acc[i][j] = 0.f;
  }

  const int64_t row = (int64_t)H * D;  // elements per token
  const uint16_t* kb = p.k + (int64_t)b * p.lk * row + (int64_t)(hbase + sub) * D + col;
  const uint16_t* vb = p.v + (int64_t)b * p.lk * row + (int64_t)(hbase + sub) * D + col;

  u32x4 kr[kTok][kNL], vr[kTok][kNL];
  auto issue = [&](int t0) __attribute__((always_inline)) {
#pragma unroll
    for (int u = 0; u < kTok; ++u) {
      const int t = min(t0 + u, t_end - 1);  // reads past the range repeat its last token; their weight is 0
#pragma unroll
      for (int i = 0; i < kNL; ++i)
        if (slot_ok[i]) {
          kr[u][i] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(kb + t * row + i * HPL * D));
          vr[u][i] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(vb + t * row + i * HPL * D));
        }
    }
  };

  const int stride = kWaves * kTok;
  int t0 = t_begin + w * kTok;
  if (t0 < t_end) issue(t0);
  for (; t0 < t_end; t0 += stride) {
    u32x4 kc[kTok][kNL], vc[kTok][kNL];
#pragma unroll
    for (int u = 0; u < kTok; ++u)
#pragma unroll
      for (int i = 0; i < kNL; ++i) {
        kc[u][i] = kr[u][i];
        vc[u][i] = vr[u][i];
      }
    if (t0 + stride < t_end) issue(t0 + stride);
#pragma unroll
    for (int i = 0; i < kNL; ++i) {
      if (!slot_ok[i]) continue;
      float x[kTok];
#pragma unroll
      for (int u = 0; u < kTok; ++u) {
        // Each dword goes through an empty asm statement first: without it the compiler turns
        // "element j of the 4-dword vector, viewed as two bf16" into a sub-vector extract that it
        // then selects as element 0 for every j (seen in the generated code: all four dot
        // products of a load read the same registers).
        float d[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          uint32_t kw = kc[u][i][j], qw = qv[i][j];
          asm volatile("" : "+v"(kw), "+v"(qw));
          d[j] = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, kw), __builtin_bit_cast(bf16x2, qw), 0.f, false);
        }
        x[u] = head_sum<LPH>((d[0] + d[1]) + (d[2] + d[3])) * p.c;
        if (t0 + u >= t_end) x[u] = -INFINITY;
      }
      float mnew = m[i];
#pragma unroll
      for (int u = 0; u < kTok; ++u) mnew = fmaxf(mnew, x[u]);
      const float alpha = __builtin_amdgcn_exp2f(m[i] - mnew);  // first tile: 2^(-inf) = 0; token t0 is always valid
      m[i] = mnew;
      float pw[kTok];
      lsum[i] *= alpha;
#pragma unroll
      for (int u = 0; u < kTok; ++u) {
        pw[u] = __builtin_amdgcn_exp2f(x[u] - mnew);
        lsum[i] += pw[u];
      }
#pragma unroll
      for (int j = 0; j < 8; ++j) acc[i][j] *= alpha;
#pragma unroll
      for (int u = 0; u < kTok; ++u)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          acc[i][2 * j] += pw[u] * bf16lo_to_f32(vc[u][i][j]);
          acc[i][2 * j + 1] += pw[u] * bf16hi_to_f32(vc[u][i][j]);
        }
    }
  }

  // ---- merge the waves: every wave publishes (m, l, acc) per head, then each thread finishes
  // a few (head, column) outputs
  __shared__ float s_acc[kWaves][HW][D];
  __shared__ float s_m[kWaves][HW];
  __shared__ float s_l[kWaves][HW];
#pragma unroll
  for (int i = 0; i < kNL; ++i) {
    const int hs = i * HPL + sub;
#pragma unroll
    for (int j = 0; j < 8; ++j) s_acc[w][hs][col + j] = acc[i][j];
    if (l % LPH == 0) {
      s_m[w][hs] = m[i];
      s_l[w][hs] = lsum[i];
    }
  }
  __syncthreads();
  const int64_t pbase = (((int64_t)b * p.lq + qi) * p.S + s) * H;
  for (int idx = threadIdx.x; idx < HW * D; idx += kWaves * 64) {
    const int hs = idx / D, d = idx % D;
    const int h = hbase + hs;
    if (h >= H) continue;
    float mm = -INFINITY;
#pragma unroll
    for (int ww = 0; ww < kWaves; ++ww) mm = fmaxf(mm, s_m[ww][hs]);
    float o = 0.f, ls = 0.f;
#pragma unroll
    for (int ww = 0; ww < kWaves; ++ww) {
      const float mw = s_m[ww][hs];
      const float f = mw == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(mw - mm);  // waves that saw no token
      o += f * s_acc[ww][hs][d];
      ls += f * s_l[ww][hs];
    }
    p.part_o[(pbase + h) * D + d] = o;
    if (d == 0) {
      p.part_m[pbase + h] = mm;
      p.part_l[pbase + h] = ls;
    }
  }
}

// o = sum_s f_s O_s / sum_s f_s l_s with f_s = 2^(m_s - max m); lse = ln of the total
template <int D>
__global__ __launch_bounds__(D) void mha_decode_merge_kernel(const float* part_o, const float* part_m, const float* part_l,
                                                             uint16_t* o, float* lse, int S, int H, int lq) {
  const int bq = blockIdx.x, h = blockIdx.y, d = threadIdx.x;
  float mmax = -INFINITY;
  for (int s = 0; s < S; ++s) mmax = fmaxf(mmax, part_m[((int64_t)bq * S + s) * H + h]);
  float acc = 0.f, lacc = 0.f;
  for (int s = 0; s < S; ++s) {
    const int64_t idx = ((int64_t)bq * S + s) * H + h;
    const float ms = part_m[idx];
    const float f = ms == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(ms - mmax);
    acc += f * part_o[idx * D + d];
    lacc += f * part_l[idx];
  }
  store_from_f32(o + ((int64_t)bq * H + h) * D + d, acc / lacc);
  if (lse && d == 0) {
    const int b = bq / lq, qi = bq % lq;
    lse[((int64_t)b * H + h) * lq + qi] = (mmax + __builtin_amdgcn_logf(lacc)) * kLn2;
  }
}

int heads_per_wave(int D) { return kNL * (64 / (D / 8)); }

int default_splits(int B, int lq, int lk, int H, int D) {
  // 4 workgroups fit a CU: aim for 1024 workgroups, and at least 64 tokens per wave
  const int hw = heads_per_wave(D);
  const int groups = B * lq * ((H + hw - 1) / hw);
  int S = (1024 + groups - 1) / groups;
  const int max_s = (lk + kWaves * 64 - 1) / (kWaves * 64);
  if (S > max_s) S = max_s;
  if (S < 1) S = 1;
  return S;
}

size_t workspace_bytes(int B, int lq, int H, int D, int S) { return (size_t)B * lq * S * H * (D + 2) * sizeof(float); }

template <int D>
int launch(const MhaFwdArgs* a, int S, hipStream_t stream) {
  MhaDecodeParams p{};
  p.q = static_cast<const uint16_t*>(a->q);
  p.k = static_cast<const uint16_t*>(a->k);
  p.v = static_cast<const uint16_t*>(a->v);
  float* ws = static_cast<float*>(a->workspace);
  const size_t no = (size_t)a->B * a->lq * S * a->H * D, nm = (size_t)a->B * a->lq * S * a->H;
  p.part_o = ws; p.part_m = ws + no; p.part_l = ws + no + nm;
  p.B = a->B; p.lq = a->lq; p.lk = a->lk; p.H = a->H; p.S = S;
  p.c = a->sm_scale * kLog2e;
  const int hw = heads_per_wave(D);
  dim3 grid(a->B * S, a->lq, (a->H + hw - 1) / hw);
  hipLaunchKernelGGL(mha_decode_kernel<D>, grid, dim3(kWaves * 64), 0, stream, p);
  if (hipGetLastError() != hipSuccess) return TPA_ERR_LAUNCH;
  hipLaunchKernelGGL(mha_decode_merge_kernel<D>, dim3(a->B * a->lq, a->H), dim3(D), 0, stream, p.part_o, p.part_m, p.part_l,
                     static_cast<uint16_t*>(a->o), a->lse, S, a->H, a->lq);
  return hipGetLastError() == hipSuccess ? TPA_OK : TPA_ERR_LAUNCH;
}

}  // namespace
}  // namespace tpa

// The split-key kernel takes: bf16, dk == dv in {64, 128}, at most 8 query tokens, no mask or
// bias, heads a multiple of the heads one 16-byte-per-lane load covers, 16-byte aligned arrays.
int mha_decode_supported(const MhaFwdArgs* a) {
  if (a->dtype != TPA_DTYPE_BF16) return 0;
  if (a->dk != a->dv || (a->dk != 64 && a->dk != 128)) return 0;
  if (a->lq > 8 || a->causal || a->bias) return 0;
  if (a->H % (64 / (a->dk / 8)) != 0) return 0;
  if (a->lk < 256) return 0;  // short caches: the one-launch kernels do as well
  const void* ptrs[3] = {a->q, a->k, a->v};
  for (const void* ptr : ptrs)
    if ((reinterpret_cast<uintptr_t>(ptr) & 15) != 0) return 0;
  return 1;
}

int mha_decode_launch(const MhaFwdArgs* a, hipStream_t stream) {
  using namespace tpa;
  const int S = a->num_splits > 0 ? a->num_splits : default_splits(a->B, a->lq, a->lk, a->H, a->dk);
  if (S > a->lk) return TPA_ERR_SHAPE;
  if ((int64_t)a->B * S > 2147483647LL || a->lq > 65535) return TPA_ERR_SHAPE;
  if (!a->workspace || a->workspace_bytes < workspace_bytes(a->B, a->lq, a->H, a->dv, S)) return TPA_ERR_WORKSPACE;
  if ((reinterpret_cast<uintptr_t>(a->workspace) & 15) != 0) return TPA_ERR_ALIGN;
  return a->dk == 128 ? launch<128>(a, S, stream) : launch<64>(a, S, stream);
}

extern "C" size_t mha_fwd_workspace_bytes(int32_t B, int32_t lq, int32_t lk, int32_t H, int32_t dv, int32_t num_splits) {
  if (B <= 0 || lq <= 0 || lk <= 0 || H <= 0 || (dv != 64 && dv != 128) || lq > 8 || lk < 256) return 0;
  const int S = num_splits > 0 ? num_splits : tpa::default_splits(B, lq, lk, H, dv);
  return tpa::workspace_bytes(B, lq, H, dv, S);
}
