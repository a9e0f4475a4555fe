// Producer step of a TPA layer for gfx950: the six rank factors of n new tokens per sequence as
// one matrix product y = x W^T, rotary position embedding on the B factors of Q and K, and the K / V
// factors written straight into the factored cache (contiguous or paged) that the decode and
// prefill kernels read.  The reference has no such step (its tests draw the factors at random,
// tpa/tpa_test.py:86-91); the arithmetic follows arXiv 2501.06425, section 3.
//
// bf16: one workgroup computes a 64-token x 64-column tile of y with v_mfma_f32_32x32x16_bf16 (four
// waves, one 32 x 32 block each; x and W tiles of 64 x 64 double buffered in LDS, the next tiles in
// registers while the current ones are multiplied), stages the fp32 tile in LDS, and every thread
// then finishes whole 16-byte chunks of eight columns: a chunk lies inside one rank row of one
// factor (H and D are multiples of 8), so the rotation partners (2j, 2j+1) are inside it.
// Any other dtype / shape: one thread per chunk of eight columns, fp32 arithmetic.
#include "tpa_common.h"

namespace tpa {
namespace {

constexpr int kBM = 64, kBN = 64, kBK = 64;
constexpr int kXS = kBK + 8;   // LDS row stride of the x / W tiles (elements): 16-byte reads of 32 rows are conflict free
constexpr int kCS = kBN + 4;   // LDS row stride of the staged fp32 tile

struct AppendParams {
  const void* x;
  const void* w;
  const float* cosv;
  const float* sinv;
  const int32_t* positions;
  const int32_t* kvlen;
  int32_t* new_kvlen;
  TpaFactor qa, qb, ka, kb, va, vb;
  const int32_t* page_table;
  int page_size, pages_per_seq;
  int B, n, K, H, D, rq, rk, cache_len, rope_len;
  int M, N;          // tokens (B * n), output columns
  int seg[7];        // first column of qa, qb, ka, kb, va, vb, and N
  float* partial;    // decode-step kernel with the contraction split over workgroups: [slabs][kFewTokens][N] fp32
  int slabs;
};

// Where chunk (token m, columns c0 .. c0 + 7) of y goes: the factor it belongs to, and the address
// of its first element (nullptr = dropped).  `rotate` = the chunk is part of a rotated B factor;
// `j0` = index of its first rotation pair.
template <typename T>
__device__ __forceinline__ T* chunk_destination(const AppendParams& p, int m, int c0, bool& rotate, int& j0, int& pos) {
  int f = 0;
#pragma unroll
  for (int k = 1; k < 6; ++k) f += c0 >= p.seg[k];
  const int width = (f & 1) ? p.D : p.H;         // qa, ka, va have H columns per rank; qb, kb, vb have D
  const int local = c0 - p.seg[f], r = local / width, e = local % width;
  const int b = m / p.n, i = m % p.n;
  const int base_len = p.kvlen ? max(0, min(p.kvlen[b], p.cache_len)) : 0;
  pos = p.positions ? p.positions[(int64_t)b * p.n + i] : base_len + i;
  pos = max(0, min(pos, p.rope_len - 1));
  rotate = f == 1 || f == 3;
  j0 = e >> 1;
  // (selected member by member: a reference into the argument block would force it into memory)
  auto pick = [&](auto get) __attribute__((always_inline)) {
    return f == 0 ? get(p.qa) : f == 1 ? get(p.qb) : f == 2 ? get(p.ka) : f == 3 ? get(p.kb) : f == 4 ? get(p.va) : get(p.vb);
  };
  T* base = static_cast<T*>(const_cast<void*>(pick([](const TpaFactor& x) { return x.ptr; })));
  const int64_t sb = pick([](const TpaFactor& x) { return x.stride_b; });
  const int64_t sl = pick([](const TpaFactor& x) { return x.stride_l; });
  const int64_t sr = pick([](const TpaFactor& x) { return x.stride_r; });
  if (f < 2) return base + b * sb + (int64_t)i * sl + (int64_t)r * sr + e;
  const int t = base_len + i;                    // token index in the sequence's cache
  if (t >= p.cache_len) return nullptr;
  if (p.page_table) {
    const int64_t page = p.page_table[(int64_t)b * p.pages_per_seq + t / p.page_size];
    return base + page * sb + (int64_t)(t % p.page_size) * sl + (int64_t)r * sr + e;
  }
  return base + b * sb + (int64_t)t * sl + (int64_t)r * sr + e;
}

// rotate the four pairs of a chunk in place: (y[2j], y[2j+1]) by the angle (pos, j0 + j)
__device__ __forceinline__ void rotate_chunk(const AppendParams& p, float (&y)[8], int pos, int j0) {
  const int half = p.D / 2;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const float c = p.cosv[(int64_t)pos * half + j0 + j], s = p.sinv[(int64_t)pos * half + j0 + j];
    const float a = y[2 * j], bb = y[2 * j + 1];
    y[2 * j] = a * c - bb * s;
    y[2 * j + 1] = bb * c + a * s;
  }
}

__device__ __forceinline__ void store_chunk(uint16_t* dst, const float (&y)[8]) {
  u32x4 v;
#pragma unroll
  for (int j = 0; j < 4; ++j) v[j] = pack_bf16(y[2 * j], y[2 * j + 1]);
  *reinterpret_cast<u32x4*>(dst) = v;
}
__device__ __forceinline__ void store_chunk(float* dst, const float (&y)[8]) {
#pragma unroll
  for (int j = 0; j < 8; ++j) dst[j] = y[j];
}

__device__ __forceinline__ void write_new_lengths(const AppendParams& p) {
  if (p.new_kvlen && blockIdx.x == 0 && blockIdx.y == 0)
    for (int b = threadIdx.x; b < p.B; b += blockDim.x) {
      const int base_len = p.kvlen ? max(0, min(p.kvlen[b], p.cache_len)) : 0;
      p.new_kvlen[b] = min(base_len + p.n, p.cache_len);
    }
}

// ---- bf16 on the matrix cores
__global__ __launch_bounds__(256) void append_mfma_kernel(AppendParams p) {
  __shared__ __attribute__((aligned(16))) uint16_t xs[2][kBM * kXS];
  __shared__ __attribute__((aligned(16))) uint16_t ws[2][kBN * kXS];
  const int tid = threadIdx.x, w = tid >> 6, l = tid & 63, i = l & 31, g = l >> 5;
  const int m0 = blockIdx.y * kBM, n0 = blockIdx.x * kBN;
  const int wm = w >> 1, wn = w & 1;       // this wave's 32 x 32 block of the tile
  const uint16_t* x = static_cast<const uint16_t*>(p.x);
  const uint16_t* wt = static_cast<const uint16_t*>(p.w);

  // loader: a 64 x 64 tile is 512 chunks of 16 bytes, two per thread (rows past the end repeat the last)
  u32x4 xr[2], wr[2];
  auto load = [&](int k0) {
#pragma unroll
    for (int q = 0; q < 2; ++q) {
      const int c = q * 256 + tid, row = c >> 3, cc = c & 7;
      xr[q] = *reinterpret_cast<const u32x4*>(x + (int64_t)min(m0 + row, p.M - 1) * p.K + k0 + 8 * cc);
      wr[q] = *reinterpret_cast<const u32x4*>(wt + (int64_t)min(n0 + row, p.N - 1) * p.K + k0 + 8 * cc);
    }
  };
  auto stage = [&](int buf) {
#pragma unroll
    for (int q = 0; q < 2; ++q) {
      const int c = q * 256 + tid, row = c >> 3, cc = c & 7;
      *reinterpret_cast<u32x4*>(&xs[buf][row * kXS + 8 * cc]) = xr[q];
      *reinterpret_cast<u32x4*>(&ws[buf][row * kXS + 8 * cc]) = wr[q];
    }
  };
  f32x16 acc;
#pragma unroll
  for (int v = 0; v < 16; ++v) acc[v] = 0.f;
  const int nk = p.K / kBK;
  load(0);
  stage(0);
  __syncthreads();
  for (int kt = 0; kt < nk; ++kt) {
    if (kt + 1 < nk) load((kt + 1) * kBK);
    const uint16_t* xb = xs[kt & 1] + (32 * wm + i) * kXS + 8 * g;
    const uint16_t* wb = ws[kt & 1] + (32 * wn + i) * kXS + 8 * g;
#pragma unroll
    for (int ks = 0; ks < kBK / 16; ++ks) {
      // A = 32 tokens x 16, B = 16 x 32 output columns (rows of W): acc[v] = y[token 8(v/4) + 4g + v%4][column i]
      const bf16x8 a = *reinterpret_cast<const bf16x8*>(xb + 16 * ks);
      const bf16x8 bq = *reinterpret_cast<const bf16x8*>(wb + 16 * ks);
      acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, bq, acc, 0, 0, 0);
    }
    if (kt + 1 < nk) stage((kt + 1) & 1);
    __syncthreads();
  }
  // ---- stage the fp32 tile (it reuses the x / W buffers, which every wave has finished reading)
  float* cs = reinterpret_cast<float*>(&xs[0][0]);
  static_assert(sizeof(xs) >= kBM * kCS * sizeof(float), "the staged tile fits the x buffers");
#pragma unroll
  for (int v = 0; v < 16; ++v) cs[(32 * wm + 8 * (v >> 2) + 4 * g + (v & 3)) * kCS + 32 * wn + i] = acc[v];
  __syncthreads();
#pragma unroll
  for (int q = 0; q < 2; ++q) {
    const int c = q * 256 + tid, row = c >> 3, cc = c & 7;
    const int m = m0 + row, c0 = n0 + 8 * cc;
    if (m >= p.M || c0 >= p.N) continue;
    float y[8];
    const f32x4 lo = *reinterpret_cast<const f32x4*>(cs + row * kCS + 8 * cc), hi = *reinterpret_cast<const f32x4*>(cs + row * kCS + 8 * cc + 4);
#pragma unroll
    for (int j = 0; j < 4; ++j) { y[j] = lo[j]; y[4 + j] = hi[j]; }
    bool rotate; int j0, pos;
    uint16_t* dst = chunk_destination<uint16_t>(p, m, c0, rotate, j0, pos);
    if (!dst) continue;
    if (rotate) rotate_chunk(p, y, pos, j0);
    store_chunk(dst, y);
  }
  write_new_lengths(p);
}

// ---- bf16, at most 64 new tokens in all (a decode step): the call is one read of W, and 64 x 64 tiles
// would leave most of the chip idle.  Operands go from global memory straight into
// v_mfma_f32_16x16x32_bf16 fragments (a lane holds 8 consecutive k of one token / one row of W, which
// is how both arrays lie in memory); the eight waves of a workgroup split its share of k, their partial
// tiles meet in LDS and one thread per chunk of eight columns finishes.
// What bounds it: a wave ingests fragments as half cache lines (16 rows x 64 bytes per load
// instruction), about 18 bytes per clock and CU, and every workgroup needs all 64 tokens of x for its
// share of k.  Without a workspace a workgroup owns 16 columns and all of k (100 workgroups at 1600
// columns; x alone is 512 KB per workgroup, 14 of the kernel's 22 us at d_model = 4096).  With a
// workspace the contraction is also split over `slabs` workgroups (blockIdx.y) that own 64 columns
// each: x is then read once per 64 columns and slab, the fp32 partial tiles go to the workspace and
// append_finish_kernel adds them up and finishes.
// U = k steps of 32 whose loads are in flight together, NCB = blocks of 16 columns per workgroup.
constexpr int kFewTokens = 64, kFewWaves = 8;
template <int U, int NCB>
__global__ __launch_bounds__(kFewWaves * 64) void append_fewrows_kernel(AppendParams p) {
  constexpr int kCols = 16 * NCB;
  extern __shared__ __attribute__((aligned(16))) float part_mem[];  // [kFewWaves][kFewTokens][kCols + 4]
  auto part = [&](int ww, int m, int c) -> float& { return part_mem[(ww * kFewTokens + m) * (kCols + 4) + c]; };
  const int tid = threadIdx.x, w = tid >> 6, l = tid & 63, r16 = l & 15, kg = l >> 4;
  const int n0 = blockIdx.x * kCols;
  const uint16_t* x = static_cast<const uint16_t*>(p.x);
  const uint16_t* wt = static_cast<const uint16_t*>(p.w);
  const int kw = p.K / (kFewWaves * p.slabs), k_begin = (blockIdx.y * kFewWaves + w) * kw;  // this wave's share of the contraction
  const uint16_t* wrow[NCB];
#pragma unroll
  for (int cb = 0; cb < NCB; ++cb) wrow[cb] = wt + (int64_t)min(n0 + 16 * cb + r16, p.N - 1) * p.K + k_begin + 8 * kg;
  const uint16_t* xrow[4];
#pragma unroll
  for (int mb = 0; mb < 4; ++mb) xrow[mb] = x + (int64_t)min(16 * mb + r16, p.M - 1) * p.K + k_begin + 8 * kg;
  // (all four blocks of 16 tokens are always computed: rows past the last token repeat it and are dropped
  // at the end - branches around the loads would keep them from being in flight together)
  f32x4 acc[4][NCB];
#pragma unroll
  for (int mb = 0; mb < 4; ++mb)
#pragma unroll
    for (int cb = 0; cb < NCB; ++cb) acc[mb][cb] = f32x4{0.f, 0.f, 0.f, 0.f};
  for (int k0 = 0; k0 < kw; k0 += 32 * U) {
    bf16x8 bq[U][NCB], a[U][4];
#pragma unroll
    for (int u = 0; u < U; ++u) {
#pragma unroll
      for (int cb = 0; cb < NCB; ++cb) bq[u][cb] = __builtin_nontemporal_load(reinterpret_cast<const bf16x8*>(wrow[cb] + k0 + 32 * u));
#pragma unroll
      for (int mb = 0; mb < 4; ++mb) a[u][mb] = *reinterpret_cast<const bf16x8*>(xrow[mb] + k0 + 32 * u);
    }
    __builtin_amdgcn_sched_barrier(0);  // every load of the group is issued before the first matrix instruction waits
#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
      for (int mb = 0; mb < 4; ++mb)
#pragma unroll
        for (int cb = 0; cb < NCB; ++cb) acc[mb][cb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[u][mb], bq[u][cb], acc[mb][cb], 0, 0, 0);
  }
  // acc[mb][cb][v] = partial y[token 16 mb + 4 kg + v][column n0 + 16 cb + r16]
#pragma unroll
  for (int mb = 0; mb < 4; ++mb)
#pragma unroll
    for (int cb = 0; cb < NCB; ++cb)
#pragma unroll
      for (int v = 0; v < 4; ++v) part(w, 16 * mb + 4 * kg + v, 16 * cb + r16) = acc[mb][cb][v];
  __syncthreads();
  for (int idx = tid; idx < kFewTokens * (kCols / 8); idx += kFewWaves * 64) {
    const int m = idx / (kCols / 8), cc = idx % (kCols / 8), c0 = n0 + 8 * cc;
    if (m >= p.M || c0 >= p.N) continue;
    float y[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) y[j] = 0.f;
#pragma unroll
    for (int ww = 0; ww < kFewWaves; ++ww) {
      const f32x4 lo = *reinterpret_cast<const f32x4*>(&part(ww, m, 8 * cc)), hi = *reinterpret_cast<const f32x4*>(&part(ww, m, 8 * cc + 4));
#pragma unroll
      for (int j = 0; j < 4; ++j) { y[j] += lo[j]; y[4 + j] += hi[j]; }
    }
    if (p.partial) {  // this slab's share of the chunk; append_finish_kernel takes it from there
      float* dst = p.partial + ((int64_t)blockIdx.y * kFewTokens + m) * p.N + c0;
      *reinterpret_cast<f32x4*>(dst) = f32x4{y[0], y[1], y[2], y[3]};
      *reinterpret_cast<f32x4*>(dst + 4) = f32x4{y[4], y[5], y[6], y[7]};
      continue;
    }
    bool rotate; int j0, pos;
    uint16_t* dst = chunk_destination<uint16_t>(p, m, c0, rotate, j0, pos);
    if (dst) {
      if (rotate) rotate_chunk(p, y, pos, j0);
      store_chunk(dst, y);
    }
  }
  if (!p.partial) write_new_lengths(p);  // (with partial sums the finishing kernel writes them)
}

// second kernel of the split decode step: eight lanes per chunk of eight columns, one per slab of k; they add
// their partial sums with three exchanges and the first of them finishes the chunk
__global__ __launch_bounds__(256) void append_finish_kernel(AppendParams p) {
  const int idx = (blockIdx.x * 256 + threadIdx.x) >> 3, sl = threadIdx.x & 7, nchunks = p.N / 8;
  const bool live = idx < p.M * nchunks;
  const int m = live ? idx / nchunks : 0, c0 = live ? 8 * (idx % nchunks) : 0;
  float y[8];
#pragma unroll
  for (int j = 0; j < 8; ++j) y[j] = 0.f;
  if (live && sl < p.slabs) {
    const float* src = p.partial + ((int64_t)sl * kFewTokens + m) * p.N + c0;
    const f32x4 lo = *reinterpret_cast<const f32x4*>(src), hi = *reinterpret_cast<const f32x4*>(src + 4);
#pragma unroll
    for (int j = 0; j < 4; ++j) { y[j] = lo[j]; y[4 + j] = hi[j]; }
  }
#pragma unroll
  for (int off = 1; off < 8; off <<= 1)
#pragma unroll
    for (int j = 0; j < 8; ++j) y[j] += __shfl_xor(y[j], off);
  if (live && sl == 0) {
    bool rotate; int j0, pos;
    uint16_t* dst = chunk_destination<uint16_t>(p, m, c0, rotate, j0, pos);
    if (dst) {
      if (rotate) rotate_chunk(p, y, pos, j0);
      store_chunk(dst, y);
    }
  }
  write_new_lengths(p);
}

// ---- any dtype and shape: one thread per chunk of eight columns
template <typename T>
__global__ __launch_bounds__(256) void append_generic_kernel(AppendParams p) {
  const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int nchunks = p.N / 8;
  if (idx < (int64_t)p.M * nchunks) {
    const int m = (int)(idx / nchunks), c0 = 8 * (int)(idx % nchunks);
    const T* xr = static_cast<const T*>(p.x) + (int64_t)m * p.K;
    const T* wr = static_cast<const T*>(p.w) + (int64_t)c0 * p.K;
    float y[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) y[j] = 0.f;
    for (int k = 0; k < p.K; ++k) {
      const float xv = load_as_f32(xr + k);
#pragma unroll
      for (int j = 0; j < 8; ++j) y[j] += xv * load_as_f32(wr + (int64_t)j * p.K + k);
    }
    bool rotate; int j0, pos;
    T* dst = chunk_destination<T>(p, m, c0, rotate, j0, pos);
    if (dst) {
      if (rotate) rotate_chunk(p, y, pos, j0);
#pragma unroll
      for (int j = 0; j < 8; ++j) store_from_f32(dst + j, y[j]);
    }
  }
  write_new_lengths(p);
}

bool aligned16(const void* ptr) { return (reinterpret_cast<uintptr_t>(ptr) & 15) == 0; }

// slabs of k that a split decode step uses: as many as 8, each a whole number of k steps per wave
int few_slabs(int d_model) {
  for (int sl = 8; sl > 1; sl >>= 1)
    if (d_model % (32 * kFewWaves * sl) == 0) return sl;
  return 1;
}

template <int U, int NCB>
int launch_fewrows(const AppendParams& p, hipStream_t s) {
  auto kern = append_fewrows_kernel<U, NCB>;
  const size_t lds = (size_t)kFewWaves * kFewTokens * (16 * NCB + 4) * sizeof(float);
  static bool configured[kMaxDevices] = {};
  if (int rc = raise_lds_limit(configured, reinterpret_cast<const void*>(kern), lds); rc != TPA_OK) return rc;
  hipLaunchKernelGGL(kern, dim3((p.N + 16 * NCB - 1) / (16 * NCB), p.slabs), dim3(kFewWaves * 64), lds, s, p);
  return hipGetLastError() == hipSuccess ? TPA_OK : TPA_ERR_LAUNCH;
}
bool chunk_ok(const TpaFactor& f) { return aligned16(f.ptr) && f.stride_b % 8 == 0 && f.stride_l % 8 == 0 && f.stride_r % 8 == 0; }

}  // namespace
}  // namespace tpa

extern "C" size_t tpa_cache_append_workspace_bytes(int32_t B, int32_t n, int32_t d_model, int32_t H, int32_t D, int32_t rq, int32_t rk, int32_t dtype) {
  using namespace tpa;
  if (B <= 0 || n <= 0 || d_model <= 0 || H <= 0 || D <= 0 || rq <= 0 || rk <= 0 || dtype != TPA_DTYPE_BF16) return 0;
  if ((int64_t)B * n > kFewTokens || H % 8 != 0 || D % 8 != 0) return 0;
  const int slabs = few_slabs(d_model);
  if (slabs == 1) return 0;
  const int64_t n_out = (int64_t)(rq + 2 * rk) * (H + D);
  return (size_t)slabs * kFewTokens * n_out * sizeof(float);
}

extern "C" int tpa_cache_append(const TpaAppendArgs* a, void* stream) {
  using namespace tpa;
  if (!a) return TPA_ERR_NULL;
  if (a->dtype != TPA_DTYPE_F32 && a->dtype != TPA_DTYPE_BF16) return TPA_ERR_DTYPE;
  if (a->B <= 0 || a->n <= 0 || a->d_model <= 0 || a->H <= 0 || a->D <= 0 || a->rq <= 0 || a->rk <= 0 || a->cache_len <= 0 ||
      a->rope_len <= 0)
    return TPA_ERR_SHAPE;
  // a chunk of eight columns must lie inside one rank row, and rotation pairs must not straddle rows
  if (a->H % 8 != 0 || a->D % 8 != 0) return TPA_ERR_SHAPE;
  if ((int64_t)a->B * a->n > 2147483647LL) return TPA_ERR_SHAPE;
  if (!a->x || !a->w || !a->rope_cos || !a->rope_sin) return TPA_ERR_NULL;
  const TpaFactor* fs[6] = {&a->qa, &a->qb, &a->ka, &a->kb, &a->va, &a->vb};
  for (const TpaFactor* f : fs)
    if (!f->ptr) return TPA_ERR_NULL;
  if (a->new_kv_lengths && a->new_kv_lengths == a->kv_lengths) return TPA_ERR_UNSUPPORTED;
  if (a->page_table && (a->page_size <= 0 || (int64_t)a->pages_per_seq * a->page_size < a->cache_len)) return TPA_ERR_SHAPE;
  if (a->kernel != TPA_KERNEL_AUTO && a->kernel != TPA_KERNEL_GENERIC && a->kernel != TPA_KERNEL_MFMA) return TPA_ERR_UNSUPPORTED;

  AppendParams p{};
  p.x = a->x; p.w = a->w; p.cosv = a->rope_cos; p.sinv = a->rope_sin;
  p.positions = a->positions; p.kvlen = a->kv_lengths; p.new_kvlen = a->new_kv_lengths;
  p.qa = a->qa; p.qb = a->qb; p.ka = a->ka; p.kb = a->kb; p.va = a->va; p.vb = a->vb;
  p.page_table = a->page_table; p.page_size = a->page_size; p.pages_per_seq = a->pages_per_seq;
  p.B = a->B; p.n = a->n; p.K = a->d_model; p.H = a->H; p.D = a->D; p.rq = a->rq; p.rk = a->rk;
  p.cache_len = a->cache_len; p.rope_len = a->rope_len;
  p.M = a->B * a->n;
  const int widths[6] = {a->rq * a->H, a->rq * a->D, a->rk * a->H, a->rk * a->D, a->rk * a->H, a->rk * a->D};
  p.seg[0] = 0;
  for (int k = 0; k < 6; ++k) p.seg[k + 1] = p.seg[k] + widths[k];
  p.N = p.seg[6];

  hipStream_t s = static_cast<hipStream_t>(stream);
  bool mfma = a->kernel != TPA_KERNEL_GENERIC && a->dtype == TPA_DTYPE_BF16 && a->d_model % kBK == 0 && aligned16(a->x) && aligned16(a->w);
  for (const TpaFactor* f : fs) mfma = mfma && chunk_ok(*f);
  if (a->kernel == TPA_KERNEL_MFMA && !mfma) return TPA_ERR_UNSUPPORTED;
  if (mfma && p.M <= kFewTokens && a->d_model % (32 * kFewWaves) == 0) {
    const size_t need = tpa_cache_append_workspace_bytes(a->B, a->n, a->d_model, a->H, a->D, a->rq, a->rk, a->dtype);
    const bool split = need && a->workspace && a->workspace_bytes >= need && aligned16(a->workspace);
    p.slabs = split ? few_slabs(a->d_model) : 1;
    p.partial = split ? static_cast<float*>(a->workspace) : nullptr;
    const int steps = a->d_model / (32 * kFewWaves * p.slabs);  // k steps of 32 per wave
    int rc;
    if (split) rc = steps % 4 == 0 ? launch_fewrows<4, 4>(p, s) : steps % 2 == 0 ? launch_fewrows<2, 4>(p, s) : launch_fewrows<1, 4>(p, s);
    else rc = steps % 4 == 0 ? launch_fewrows<4, 1>(p, s) : launch_fewrows<1, 1>(p, s);
    if (rc != TPA_OK) return rc;
    if (split) hipLaunchKernelGGL(append_finish_kernel, dim3((p.M * (p.N / 8) * 8 + 255) / 256), dim3(256), 0, s, p);
  } else if (mfma) {
    dim3 grid((p.N + kBN - 1) / kBN, (p.M + kBM - 1) / kBM);
    if (grid.y > 65535) return TPA_ERR_SHAPE;
    hipLaunchKernelGGL(append_mfma_kernel, grid, dim3(256), 0, s, p);
  } else {
    const int64_t chunks = (int64_t)p.M * (p.N / 8);
    const int64_t blocks = (chunks + 255) / 256;
    if (blocks > 2147483647LL) return TPA_ERR_SHAPE;
    if (a->dtype == TPA_DTYPE_BF16) hipLaunchKernelGGL(append_generic_kernel<uint16_t>, dim3((unsigned)blocks), dim3(256), 0, s, p);
    else hipLaunchKernelGGL(append_generic_kernel<float>, dim3((unsigned)blocks), dim3(256), 0, s, p);
  }
  return hipGetLastError() == hipSuccess ? TPA_OK : TPA_ERR_LAUNCH;
}
