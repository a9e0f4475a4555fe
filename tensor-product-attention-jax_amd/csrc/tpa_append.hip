// Producer step of a TPA layer for gfx950: the six rank factors of n new tokens per sequence as
// one matrix product y = x W^T, rotary position embedding on the B factors of Q and K, and the K / V
// factors written straight into the factored cache (contiguous or paged) that the decode and
// prefill kernels read.  The reference has no such step (its tests draw the factors at random,
// tpa/tpa_test.py:86-91); the arithmetic follows arXiv 2501.06425, section 3.
//
// bf16, three kernels by the number of new tokens: 256 x 256 tiles once they fill the chip (a prefill
// chunk), 64 x 64 tiles below that, and for a decode step (at most 64 tokens in all) a kernel that
// splits the contraction instead of the tokens.  All of them compute with v_mfma_f32_*_bf16, stage the
// fp32 results in LDS, and finish whole 16-byte chunks of eight columns: a chunk lies inside one rank
// row of one factor (H and D are multiples of 8), so the rotation partners (2j, 2j+1) are inside it.
// Any other dtype / shape: one thread per chunk of eight columns, fp32 arithmetic.
#include <type_traits>
#include <utility>

#include "tpa_common.h"

namespace tpa {
namespace {

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

// ---- bf16, 64 x 64 tiles: four waves, one 32 x 32 block each; x and W tiles of 64 x 64 double buffered in LDS,
// the next tiles in registers while the current ones are multiplied
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

// ---- bf16, many new tokens (a prefill chunk): 256 tokens x 256 columns of y per workgroup, four waves
// (one per SIMD, 512 registers each: the 256 accumulators sit in AGPRs).  A wave owns 128 tokens x 128
// columns = 4 x 4 blocks of v_mfma_f32_32x32x16_bf16, computed transposed (A = rows of W, B = tokens), so
// that a lane ends up with runs of four consecutive columns of one token.  A k step reads 8 fragments for
// 16 MFMAs (the 64 x 64 tiles above read 2 for 1, which is what bounds them; eight waves of 64 x 128 read
// 6 for 8 and measured the same time as this form).  x and W tiles of 256 rows x 64 k are double buffered
// in LDS (row stride 72 elements), raw buffer loads over the tile's rows only (rows past the end read as
// zeros and are never stored).
// One wave per SIMD has nobody to hide behind, so the order inside an iteration is fixed by hand:
//   k step 0, 1: fragments of the next step requested, 16 MFMAs
//   k step 2:    fragments of step 3 requested, 16 MFMAs with the stores of the next tile between them
//   barrier
//   k step 3:    fragments of the next tile's step 0 requested, 16 MFMAs with the loads of the tile after next
// Epilogue: each wave stages its fp32 tile through its own quarter of the (now free) buffers, 64 tokens x 64
// columns at a time, and finishes 16-byte chunks; everything that depends on the token alone (sequence,
// position, cache row or page) is worked out once per workgroup into a small LDS table, everything that
// depends on the column alone once per lane and piece.
// Grid: linear ids are dealt to the 8 XCDs round robin, so the column tiles of one token tile get ids
// that are 8 apart (same XCD: its L2 serves their x tiles).
// WB = blocks of 32 per wave and dimension: 4 (the tile described above) or 2 (128 x 128 tiles, a wave owns
// 64 x 64, 4 fragment reads per 4 MFMAs, two workgroups per CU) for chunks too small to fill the chip with the large tiles.
constexpr int kGK = 64, kGS = kGK + 8;
constexpr int kGCS = 64 + 4;                          // row stride of a wave's staged fp32 piece
template <int WB>
struct GemmTile {
  static constexpr int kM = 64 * WB, kN = 64 * WB;    // tokens, columns per workgroup
  static constexpr int kStage = (kM + kN) * kGS;      // elements per buffer
  static constexpr size_t kLds = 2 * kStage * sizeof(uint16_t) + kM * 5 * sizeof(int32_t);
  static_assert(64 * kGCS <= kStage / 4 && kStage % 16 == 0, "a wave's staged piece fits its slice");
};
template <int WB>
__global__ __launch_bounds__(256) void append_gemm_kernel(AppendParams p) {
  constexpr int kGM = GemmTile<WB>::kM, kGN = GemmTile<WB>::kN, kGStage = GemmTile<WB>::kStage;
  constexpr int kWT = 32 * WB;                        // tokens / columns per wave
  extern __shared__ __attribute__((aligned(16))) uint16_t gsm[];
  int32_t* const table = reinterpret_cast<int32_t*>(gsm + 2 * kGStage);  // [5][kGM]: pos, b, i, cache row coordinates
  const int tid = threadIdx.x, w = tid >> 6, l = tid & 63, i = l & 31, g = l >> 5;
  const int wm = w >> 1, wn = w & 1;
  const int ntn = (p.N + kGN - 1) / kGN, ntm = (p.M + kGM - 1) / kGM;
  const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
  const int tm = (slot / ntn) * 8 + xcd, tn = slot % ntn;
  if (tm >= ntm) return;  // the grid is rounded up to whole groups of 8 token tiles
  const int m0 = tm * kGM, n0 = tn * kGN;
  const uint16_t* x = static_cast<const uint16_t*>(p.x);
  const uint16_t* wt = static_cast<const uint16_t*>(p.w);

  if (tid < kGM) {  // what the epilogue needs to know about a token (one per thread)
    const int m = min(m0 + tid, p.M - 1);
    const int b = m / p.n, ii = m % p.n;
    const int base_len = p.kvlen ? max(0, min(p.kvlen[b], p.cache_len)) : 0;
    int pos = p.positions ? p.positions[(int64_t)b * p.n + ii] : base_len + ii;
    pos = max(0, min(pos, p.rope_len - 1));
    const int t = base_len + ii;
    int ra = b, rb = t;
    if (t >= p.cache_len) { ra = 0; rb = -1; }  // dropped
    else if (p.page_table) { ra = p.page_table[(int64_t)b * p.pages_per_seq + t / p.page_size]; rb = t % p.page_size; }
    table[tid] = pos; table[kGM + tid] = b; table[2 * kGM + tid] = ii; table[3 * kGM + tid] = ra; table[4 * kGM + tid] = rb;
  }

  // loader: thread -> chunk tid & 7 of rows (tid >> 3) + 32 q of x and of W
  const int lrow = tid >> 3, lc = tid & 7;
  constexpr int kRsrcFlags = 0x00020000;  // raw 32-bit data format
  const __amdgpu_buffer_rsrc_t x_rs = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint16_t*>(x + (int64_t)m0 * p.K), 0, min(kGM, p.M - m0) * p.K * 2, kRsrcFlags);
  const __amdgpu_buffer_rsrc_t w_rs = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint16_t*>(wt + (int64_t)n0 * p.K), 0, min(kGN, p.N - n0) * p.K * 2, kRsrcFlags);
  const int voff = (lrow * p.K + 8 * lc) * 2;
  const int nk = p.K / kGK;
  constexpr int NLD = 2 * WB;  // 16-byte chunks of x and of W per thread and tile
  u32x4 xr[NLD], wr[NLD];
  auto load = [&](int kt) __attribute__((always_inline)) {  // (tiles past the last repeat it: loaded, stored, never read)
    const int k0 = min(kt, nk - 1) * kGK;
#pragma unroll
    for (int q = 0; q < NLD; ++q) {
      xr[q] = __builtin_amdgcn_raw_buffer_load_b128(x_rs, voff, (32 * q * p.K + k0) * 2, 0);
      wr[q] = __builtin_amdgcn_raw_buffer_load_b128(w_rs, voff, (32 * q * p.K + k0) * 2, 0);
    }
  };
  auto stage = [&](int buf) __attribute__((always_inline)) {
    uint16_t* xs = gsm + buf * kGStage + lrow * kGS + 8 * lc;
#pragma unroll
    for (int q = 0; q < NLD; ++q) {
      *reinterpret_cast<u32x4*>(xs + 32 * q * kGS) = xr[q];
      *reinterpret_cast<u32x4*>(xs + (kGM + 32 * q) * kGS) = wr[q];
    }
  };
  f32x16 acc[WB][WB];
#pragma unroll
  for (int cb = 0; cb < WB; ++cb)
#pragma unroll
    for (int tb = 0; tb < WB; ++tb)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[cb][tb][v] = 0.f;
  // (a wave whose columns all lie past the end multiplies zeros: with one wave per SIMD nobody would use the time)
  bf16x8 fa[2][WB], fb[2][WB];
  const int frag_x = (kWT * wm + i) * kGS + 8 * g, frag_w = (kGM + kWT * wn + i) * kGS + 8 * g;
  auto read_frags = [&](auto slot_c, int buf, auto ks_c) __attribute__((always_inline)) {
    constexpr int sl = decltype(slot_c)::value, ks = decltype(ks_c)::value;
    const uint16_t* base = gsm + buf * kGStage + 16 * ks;
#pragma unroll
    for (int cb = 0; cb < WB; ++cb) fa[sl][cb] = *reinterpret_cast<const bf16x8*>(base + frag_w + 32 * cb * kGS);
#pragma unroll
    for (int tb = 0; tb < WB; ++tb) fb[sl][tb] = *reinterpret_cast<const bf16x8*>(base + frag_x + 32 * tb * kGS);
  };
  // acc[cb][tb][v] = y[token kWT wm + 32 tb + i][column kWT wn + 32 cb + 8 (v / 4) + 4 g + v % 4]
  auto mfmas = [&](auto slot_c) __attribute__((always_inline)) {
    constexpr int sl = decltype(slot_c)::value;
#pragma unroll
    for (int cb = 0; cb < WB; ++cb)
#pragma unroll
      for (int tb = 0; tb < WB; ++tb) acc[cb][tb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[sl][cb], fb[sl][tb], acc[cb][tb], 0, 0, 0);
  };
  load(0);
  stage(0);
  load(1);
  __syncthreads();
  read_frags(IC<0>{}, 0, IC<0>{});
  for (int kt = 0; kt < nk; ++kt) {
    const int cur = kt & 1, nxt = cur ^ 1;
    read_frags(IC<1>{}, cur, IC<1>{});
    __builtin_amdgcn_sched_barrier(0);
    mfmas(IC<0>{});
    __builtin_amdgcn_sched_barrier(0);
    read_frags(IC<0>{}, cur, IC<2>{});
    __builtin_amdgcn_sched_barrier(0);
    mfmas(IC<1>{});
    __builtin_amdgcn_sched_barrier(0);
    read_frags(IC<1>{}, cur, IC<3>{});
    __builtin_amdgcn_sched_barrier(0);
    mfmas(IC<0>{});
    stage(nxt);
#pragma unroll
    for (int n = 0; n < WB * WB; ++n) {  // the tile stores spread behind the MFMAs
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x200, 2 * NLD / (WB * WB), 0);
    }
    __builtin_amdgcn_sched_barrier(0);
    __syncthreads();
    read_frags(IC<0>{}, nxt, IC<0>{});
    __builtin_amdgcn_sched_barrier(0);
    mfmas(IC<1>{});
    load(kt + 2);
#pragma unroll
    for (int n = 0; n < WB * WB; ++n) {  // the tile loads spread behind the MFMAs
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x020, 2 * NLD / (WB * WB), 0);
    }
    __builtin_amdgcn_sched_barrier(0);
  }
  __syncthreads();  // every wave has left the loop: the buffers are free

  // ---- epilogue: pieces of 64 tokens x 64 columns through this wave's quarter of the buffers
  float* const cs = reinterpret_cast<float*>(gsm) + w * (kGStage / 4);
  const int cc = l & 7, trow = l >> 3;
#pragma unroll
  for (int ch = 0; ch < WB / 2; ++ch) {
    const int c0 = n0 + kWT * wn + 64 * ch + 8 * cc;
    const bool col_ok = c0 < p.N;
    // the column's side of the address: factor, rank row, element
    int f = 0;
#pragma unroll
    for (int k = 1; k < 6; ++k) f += c0 >= p.seg[k];
    const int width = (f & 1) ? p.D : p.H;
    const int local = c0 - p.seg[f], r = local / width, e = local % width;
    const bool rotate = f == 1 || f == 3;
    auto pick = [&](auto get) __attribute__((always_inline)) {
      return f == 0 ? get(p.qa) : f == 1 ? get(p.qb) : f == 2 ? get(p.ka) : f == 3 ? get(p.kb) : f == 4 ? get(p.va) : get(p.vb);
    };
    uint16_t* const base = static_cast<uint16_t*>(const_cast<void*>(pick([](const TpaFactor& t) { return t.ptr; }))) +
                           (int64_t)r * pick([](const TpaFactor& t) { return t.stride_r; }) + e;
    const int64_t sb = pick([](const TpaFactor& t) { return t.stride_b; });
    const int64_t sl = pick([](const TpaFactor& t) { return t.stride_l; });
    const int half_d = p.D / 2;
#pragma unroll
    for (int th = 0; th < WB / 2; ++th) {
      __builtin_amdgcn_wave_barrier();
#pragma unroll
      for (int cq = 0; cq < 2; ++cq)
#pragma unroll
        for (int tq = 0; tq < 2; ++tq)
#pragma unroll
          for (int vq = 0; vq < 4; ++vq) {
            const f32x16& t = acc[2 * ch + cq][2 * th + tq];
            *reinterpret_cast<f32x4*>(cs + (32 * tq + i) * kGCS + 32 * cq + 8 * vq + 4 * g) = f32x4{t[4 * vq], t[4 * vq + 1], t[4 * vq + 2], t[4 * vq + 3]};
          }
      __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0): the wave's own writes have landed
      __builtin_amdgcn_wave_barrier();
      if (!col_ok) continue;
      // everything a pass fetches from memory first (row coordinates, angles), then the arithmetic and the stores
      int64_t off[8];
      f32x4 c4[8], s4[8];
#pragma unroll
      for (int pass = 0; pass < 8; ++pass) {
        const int tl = kWT * wm + 64 * th + 8 * pass + trow;  // token within the workgroup's tile
        const int ra = f < 2 ? table[kGM + tl] : table[3 * kGM + tl], rb = f < 2 ? table[2 * kGM + tl] : table[4 * kGM + tl];
        off[pass] = m0 + tl < p.M && rb >= 0 ? ra * sb + rb * sl : -1;
        if (rotate) {
          const int64_t at = (int64_t)table[tl] * half_d + (e >> 1);
          c4[pass] = *reinterpret_cast<const f32x4*>(p.cosv + at);
          s4[pass] = *reinterpret_cast<const f32x4*>(p.sinv + at);
        }
      }
#pragma unroll
      for (int pass = 0; pass < 8; ++pass) {
        if (off[pass] < 0) continue;
        const float* src = cs + (8 * pass + trow) * kGCS + 8 * cc;
        const f32x4 lo = *reinterpret_cast<const f32x4*>(src), hi = *reinterpret_cast<const f32x4*>(src + 4);
        float y[8] = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
        if (rotate) {
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            const float a0 = y[2 * j], b0 = y[2 * j + 1];
            y[2 * j] = a0 * c4[pass][j] - b0 * s4[pass][j];
            y[2 * j + 1] = b0 * c4[pass][j] + a0 * s4[pass][j];
          }
        }
        store_chunk(base + off[pass], y);
      }
    }
  }
  if (blockIdx.x == 0) write_new_lengths(p);
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

// 256 x 256 tiles (WB = 4) pay once they fill three quarters of the chip (256 CUs, one workgroup each), 128 x 128
// tiles (WB = 2) from half of it; the rotation tables must allow 16-byte reads of four angles
template <int WB>
bool gemm_tiles_pay(const AppendParams& p, const TpaAppendArgs* a) {
  constexpr int kM = GemmTile<WB>::kM, kN = GemmTile<WB>::kN;
  const int64_t tiles = (int64_t)((p.M + kM - 1) / kM) * ((p.N + kN - 1) / kN);
  return tiles >= (WB == 4 ? 192 : 128) && tiles < (1 << 28) && p.D % 8 == 0 && aligned16(a->rope_cos) && aligned16(a->rope_sin);
}

template <int WB>
int launch_gemm(const AppendParams& p, hipStream_t s) {
  constexpr int kM = GemmTile<WB>::kM, kN = GemmTile<WB>::kN;
  const int ntn = (p.N + kN - 1) / kN, ntm = (p.M + kM - 1) / kM;
  auto kern = append_gemm_kernel<WB>;
  static bool configured[kMaxDevices] = {};
  if (int rc = raise_lds_limit(configured, reinterpret_cast<const void*>(kern), GemmTile<WB>::kLds); rc != TPA_OK) return rc;
  hipLaunchKernelGGL(kern, dim3((ntm + 7) / 8 * 8 * ntn), dim3(256), GemmTile<WB>::kLds, s, p);
  return hipGetLastError() == hipSuccess ? TPA_OK : TPA_ERR_LAUNCH;
}

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
  } else if (mfma && gemm_tiles_pay<4>(p, a)) {
    if (int rc = launch_gemm<4>(p, s); rc != TPA_OK) return rc;
  } else if (mfma && gemm_tiles_pay<2>(p, a)) {
    if (int rc = launch_gemm<2>(p, s); rc != TPA_OK) return rc;
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
