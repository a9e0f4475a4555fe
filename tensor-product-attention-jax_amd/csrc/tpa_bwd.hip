// Backward pass: gradients of the attention output with respect to the rank factors
// (tpa/tpa.py:168-214,546-995) and, for the dense baseline, with respect to q, k, v
// (tpa/mha.py:40-65).  Any-shape fp32 arithmetic on the vector ALUs, except stages 3 and 4, which
// run on the matrix cores for bf16 inputs with a head size of 64 or 128.
//
// The factored problem is taken through dense intermediates that live in the caller's
// workspace, so that every stage is a plain, separately checkable kernel:
//   1. recon:    Q, K, V [B, l, H, d] = (1/R) sum_r a_r (x) b_r               (tpa/tpa.py:605-606,623)
//   2. delta:    delta[b, h, i] = sum_d o * do, NaN products skipped          (tpa/tpa.py:965-995)
//   3. dq:       one thread per query row walks the keys:  p = exp(x - lse),
//                dp = do . v, ds = scale * p * (dp - delta), dQ += ds * k      (tpa/tpa.py:779-781)
//   4. dkv:      one thread per key walks the query rows: dV += p * do,
//                dK += ds * q                                                  (tpa/tpa.py:765-777)
//   5. project:  da[r, h] = (1/R) sum_d dX[h, d] b[r, d],  db[r, d] = (1/R) sum_h dX[h, d] a[r, h]
//                for X in {Q, K, V}                                            (tpa/tpa.py:767-768,776-777,782-783)
// Rows without a visible key (lse = -inf) contribute nothing (tpa/tpa.py:675-676).
// Gradients are written as fp32 whatever the input type is.
#include "tpa_common.h"

namespace tpa {
namespace {

constexpr int kThreads = 128;  // rows (dq) or keys (dkv) per workgroup
// keys (dq) or rows (dkv) per LDS tile: the tiles of the widest heads stay below 64 KB
constexpr int tile_of(int dmax) { return dmax > 128 ? 16 : 32; }

// ------------------------------------------------------------------------------------ stage 1
template <typename T, typename TO>
__global__ void recon_kernel(TpaFactor fa, TpaFactor fb, TO* out, int L, int H, int D, int R) {
  const int t = blockIdx.x, b = blockIdx.y;
  const T* ap = static_cast<const T*>(fa.ptr) + b * fa.stride_b + t * fa.stride_l;
  const T* bp = static_cast<const T*>(fb.ptr) + b * fb.stride_b + t * fb.stride_l;
  TO* op = out + ((int64_t)b * L + t) * H * D;
  const float inv = 1.f / (float)R;
  for (int idx = threadIdx.x; idx < H * D; idx += blockDim.x) {
    const int h = idx / D, d = idx - h * D;
    float acc = 0.f;
    for (int r = 0; r < R; ++r) acc += load_as_f32(ap + r * fa.stride_r + h) * load_as_f32(bp + r * fb.stride_r + d);
    store_from_f32(op + idx, acc * inv);
  }
}

// bf16 factors -> dense bf16, 8 elements per thread and token.  A workgroup takes kReconTokens
// consecutive tokens and every thread works on the same (head, 16-byte piece) of all of them at
// once, so that several independent load chains are in flight (one token per workgroup left the
// kernel waiting for one small load after the other).  Needs D % 8 == 0 and 16-byte aligned b rows.
constexpr int kReconTokens = 4;
__global__ __launch_bounds__(256) void recon_bf16_kernel(TpaFactor fa, TpaFactor fb, uint16_t* out, int L, int H, int D, int R, float scale) {
  const int t0 = blockIdx.x * kReconTokens, b = blockIdx.y;
  const uint16_t* ap = static_cast<const uint16_t*>(fa.ptr) + b * fa.stride_b;
  const uint16_t* bp = static_cast<const uint16_t*>(fb.ptr) + b * fb.stride_b;
  const float inv = scale / (float)R;
  const int cpr = D / 8;
  for (int idx = threadIdx.x; idx < H * cpr; idx += blockDim.x) {
    const int h = idx / cpr, cc = idx - h * cpr;
    float acc[kReconTokens][8];
#pragma unroll
    for (int u = 0; u < kReconTokens; ++u)
#pragma unroll
      for (int j = 0; j < 8; ++j) acc[u][j] = 0.f;
    for (int r = 0; r < R; ++r) {
      float av[kReconTokens];
      u32x4 bv[kReconTokens];
#pragma unroll
      for (int u = 0; u < kReconTokens; ++u) {
        const int64_t t = min(t0 + u, L - 1);
        av[u] = bf16bits_to_f32(ap[t * fa.stride_l + r * fa.stride_r + h]);
        bv[u] = *reinterpret_cast<const u32x4*>(bp + t * fb.stride_l + r * fb.stride_r + 8 * cc);
      }
#pragma unroll
      for (int u = 0; u < kReconTokens; ++u)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          acc[u][2 * j] += av[u] * bf16lo_to_f32(bv[u][j]);
          acc[u][2 * j + 1] += av[u] * bf16hi_to_f32(bv[u][j]);
        }
    }
#pragma unroll
    for (int u = 0; u < kReconTokens; ++u) {
      if (t0 + u >= L) break;
      u32x4 pk;
#pragma unroll
      for (int j = 0; j < 4; ++j) pk[j] = pack_bf16(acc[u][2 * j] * inv, acc[u][2 * j + 1] * inv);
      *reinterpret_cast<u32x4*>(out + (((int64_t)b * L + t0 + u) * H + h) * D + 8 * cc) = pk;
    }
  }
}

// The same for head counts that are multiples of 8 with 16-byte aligned a rows: a thread owns one
// (token, 16-byte piece of D, group of 8 heads) and reads, per rank, one 16-byte piece of b and
// the 8 head factors as one 16-byte piece of a - 64 multiply-adds per two loads.  Pieces are the
// fastest thread index, so the 16 threads of a (token, head group) store whole rows of D.
struct ReconJob { TpaFactor fa, fb; uint16_t* out; int L, R; float scale; };
struct ReconJobs { ReconJob job[3]; };  // blockIdx.z picks one: several arrays in one launch
__global__ __launch_bounds__(256) void recon_bf16_h8_kernel(ReconJobs jobs, int H, int D) {
  const TpaFactor fa = blockIdx.z == 0 ? jobs.job[0].fa : blockIdx.z == 1 ? jobs.job[1].fa : jobs.job[2].fa;
  const TpaFactor fb = blockIdx.z == 0 ? jobs.job[0].fb : blockIdx.z == 1 ? jobs.job[1].fb : jobs.job[2].fb;
  uint16_t* const out = blockIdx.z == 0 ? jobs.job[0].out : blockIdx.z == 1 ? jobs.job[1].out : jobs.job[2].out;
  const int L = blockIdx.z == 0 ? jobs.job[0].L : blockIdx.z == 1 ? jobs.job[1].L : jobs.job[2].L;
  const int R = blockIdx.z == 0 ? jobs.job[0].R : blockIdx.z == 1 ? jobs.job[1].R : jobs.job[2].R;
  const float scale = blockIdx.z == 0 ? jobs.job[0].scale : blockIdx.z == 1 ? jobs.job[1].scale : jobs.job[2].scale;
  const int cpr = D / 8, hg = H / 8;
  const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
  const int cc = (int)(idx % cpr);
  const int g = (int)(idx / cpr % hg);
  const int64_t t = idx / ((int64_t)cpr * hg);
  const int b = blockIdx.y;
  if (t >= L) return;
  const uint16_t* ap = static_cast<const uint16_t*>(fa.ptr) + b * fa.stride_b + t * fa.stride_l + 8 * g;
  const uint16_t* bp = static_cast<const uint16_t*>(fb.ptr) + b * fb.stride_b + t * fb.stride_l + 8 * cc;
  float acc[8][8];
#pragma unroll
  for (int i = 0; i < 8; ++i)
#pragma unroll
    for (int j = 0; j < 8; ++j) acc[i][j] = 0.f;
  // Two ranks per step of the inner product: the head factors of ranks (r, r + 1) and the b elements of the
  // same two ranks are paired into packed bf16 words (16 byte permutes per pair of ranks), and one dot
  // instruction then adds a_r[h] b_r[d] + a_r+1[h] b_r+1[d] to the accumulator - half the instructions of
  // unpacking both and multiplying in fp32, which is what bounds this kernel from rank 8 on.
  constexpr int G = 4;  // ranks whose loads are in flight together (at low ranks the kernel is bound by their latency)
  for (int r0 = 0; r0 < R; r0 += G) {
    u32x4 av[G], bv[G];
#pragma unroll
    for (int u = 0; u < G; ++u) {
      const int r = min(r0 + u, R - 1);
      av[u] = *reinterpret_cast<const u32x4*>(ap + (int64_t)r * fa.stride_r);
      bv[u] = *reinterpret_cast<const u32x4*>(bp + (int64_t)r * fb.stride_r);
      if (r0 + u >= R) av[u] = u32x4{0u, 0u, 0u, 0u};  // past the last rank: weight zero
    }
#pragma unroll
    for (int u = 0; u < G; u += 2) {
      if (r0 + u >= R) break;
      uint32_t apair[8], bpair[8];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        apair[2 * j] = __builtin_amdgcn_perm(av[u + 1][j], av[u][j], 0x05040100u);      // (a_r[2j], a_r+1[2j])
        apair[2 * j + 1] = __builtin_amdgcn_perm(av[u + 1][j], av[u][j], 0x07060302u);  // (a_r[2j+1], a_r+1[2j+1])
        bpair[2 * j] = __builtin_amdgcn_perm(bv[u + 1][j], bv[u][j], 0x05040100u);
        bpair[2 * j + 1] = __builtin_amdgcn_perm(bv[u + 1][j], bv[u][j], 0x07060302u);
      }
#pragma unroll
      for (int i = 0; i < 8; ++i)
#pragma unroll
        for (int j = 0; j < 8; ++j)
          acc[i][j] = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, apair[i]), __builtin_bit_cast(bf16x2, bpair[j]), acc[i][j], false);
    }
  }
  const float inv = scale / (float)R;
  uint16_t* op = out + (((int64_t)b * L + t) * H + 8 * g) * D + 8 * cc;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    u32x4 pk;
#pragma unroll
    for (int j = 0; j < 4; ++j) pk[j] = pack_bf16(acc[i][2 * j] * inv, acc[i][2 * j + 1] * inv);
    *reinterpret_cast<u32x4*>(op + (int64_t)i * D) = pk;
  }
}

template <typename T>
__global__ void to_f32_kernel(const T* in, float* out, int64_t n) {
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x)
    out[i] = load_as_f32(in + i);
}

// ------------------------------------------------------------------------------------ stage 2
// delta[b, h, i] = sum_d o[b, i, h, d] * do[b, i, h, d], skipping NaN products (an empty row's o).
// Sixteen lanes share a row; with bf16 rows of a multiple of 8 elements each lane takes 16 bytes
// per step, so a wave reads four rows with fully coalesced loads.
template <typename T>
__global__ void delta_kernel(const T* o, const T* d_o, float* delta, int B, int lq, int H, int dv, int vec) {
  const int64_t row = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) >> 4;  // over (b, i, h)
  const int sub = threadIdx.x & 15;
  const bool ok = row < (int64_t)B * lq * H;
  float acc = 0.f;
  if (ok) {
    const T* op = o + row * dv;
    const T* gp = d_o + row * dv;
    if constexpr (sizeof(T) == 2) {
      if (vec) {
        for (int d = 8 * sub; d < dv; d += 128) {
          const u32x4 a = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(op + d));
          const u32x4 g = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(gp + d));
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            const float x0 = bf16lo_to_f32(a[j]) * bf16lo_to_f32(g[j]), x1 = bf16hi_to_f32(a[j]) * bf16hi_to_f32(g[j]);
            if (x0 == x0) acc += x0;
            if (x1 == x1) acc += x1;
          }
        }
      }
    }
    if (!(sizeof(T) == 2 && vec)) {
      for (int d = sub; d < dv; d += 16) {
        const float x = load_as_f32(op + d) * load_as_f32(gp + d);
        if (x == x) acc += x;
      }
    }
  }
#pragma unroll
  for (int m = 8; m >= 1; m >>= 1) acc += __shfl_xor(acc, m, 16);
  if (ok && sub == 0) {
    const int h = row % H;
    const int64_t bi = row / H;
    const int i = bi % lq, b = bi / lq;
    delta[((int64_t)b * H + h) * lq + i] = acc;
  }
}

struct DenseParams {
  const float* q;  // [B, lq, H, dk]
  const float* k;  // [B, lk, H, dk]
  const float* v;  // [B, lk, H, dv]
  const void* d_o;  // [B, lq, H, dv], element type T
  const float* lse;    // [B, H, lq]
  const float* delta;  // [B, H, lq]
  const int32_t* qseg;
  const int32_t* kvseg;
  const float* bias;  // [B, lq, lk] or null
  float* dq;          // [B, lq, H, dk]
  float* dk_out;      // [B, lk, H, dk]
  float* dv_out;      // [B, lk, H, dv]
  int B, lq, lk, H, dk, dv;
  float sm_scale;
  int causal;
  int coff;  // with causal: row i sees keys <= i + coff
};

// ------------------------------------------------------------------------------------ stage 3
template <typename T, int DMAX>
__global__ __launch_bounds__(kThreads) void bwd_dq_kernel(DenseParams p) {
  constexpr int kTile = tile_of(DMAX);
  const int b = blockIdx.z, h = blockIdx.y;
  const int row = blockIdx.x * kThreads + threadIdx.x;
  const int dk = p.dk, dv = p.dv;
  extern __shared__ float smem[];
  float* ks = smem;               // [kTile][dk]
  float* vs = smem + kTile * dk;  // [kTile][dv]
  int* segs = reinterpret_cast<int*>(vs + kTile * dv);

  float lse = -INFINITY, delta = 0.f;
  float q[DMAX], g[DMAX], acc[DMAX];
#pragma unroll
  for (int d = 0; d < DMAX; ++d) { q[d] = 0.f; g[d] = 0.f; acc[d] = 0.f; }
  const bool row_ok = row < p.lq;
  if (row_ok) {
    lse = p.lse[((int64_t)b * p.H + h) * p.lq + row];
    delta = p.delta[((int64_t)b * p.H + h) * p.lq + row];
    const float* qp = p.q + (((int64_t)b * p.lq + row) * p.H + h) * dk;
    const T* gp = static_cast<const T*>(p.d_o) + (((int64_t)b * p.lq + row) * p.H + h) * dv;
#pragma unroll
    for (int d = 0; d < DMAX; ++d) {
      if (d < dk) q[d] = qp[d];
      if (d < dv) {
        const float x = load_as_f32(gp + d);
        g[d] = x == x ? x : 0.f;
      }
    }
  }
  const bool live = row_ok && lse > -INFINITY;  // a row without a visible key has no gradient
  const int qseg = (row_ok && p.qseg) ? p.qseg[(int64_t)b * p.lq + row] : 0;

  int k_end = p.lk;
  if (p.causal) k_end = min(p.lk, min(p.lq, (int)(blockIdx.x + 1) * kThreads) + p.coff);
  for (int k0 = 0; k0 < k_end; k0 += kTile) {
    const int nk = min(kTile, k_end - k0);
    __syncthreads();
    for (int idx = threadIdx.x; idx < nk * dk; idx += kThreads) {
      const int t = idx / dk, d = idx - t * dk;
      ks[idx] = p.k[(((int64_t)b * p.lk + k0 + t) * p.H + h) * dk + d];
    }
    for (int idx = threadIdx.x; idx < nk * dv; idx += kThreads) {
      const int t = idx / dv, d = idx - t * dv;
      vs[idx] = p.v[(((int64_t)b * p.lk + k0 + t) * p.H + h) * dv + d];
    }
    if (p.kvseg)
      for (int t = threadIdx.x; t < nk; t += kThreads) segs[t] = p.kvseg[(int64_t)b * p.lk + k0 + t];
    __syncthreads();
    if (!live) continue;
    for (int t = 0; t < nk; ++t) {
      bool keep = true;
      if (p.kvseg) keep = segs[t] == qseg;
      if (p.causal) keep = keep && (k0 + t <= row + p.coff);
      if (!keep) continue;
      float dot = 0.f;
#pragma unroll
      for (int d = 0; d < DMAX; ++d)
        if (d < dk) dot += q[d] * ks[t * dk + d];
      float x = dot * p.sm_scale;
      if (p.bias) x += p.bias[((int64_t)b * p.lq + row) * p.lk + k0 + t];
      const float pt = expf(x - lse);
      float dp = 0.f;
#pragma unroll
      for (int d = 0; d < DMAX; ++d)
        if (d < dv) dp += g[d] * vs[t * dv + d];
      const float ds = p.sm_scale * pt * (dp - delta);
#pragma unroll
      for (int d = 0; d < DMAX; ++d)
        if (d < dk) acc[d] += ds * ks[t * dk + d];
    }
  }
  if (!row_ok) return;
  float* op = p.dq + (((int64_t)b * p.lq + row) * p.H + h) * dk;
#pragma unroll
  for (int d = 0; d < DMAX; ++d)
    if (d < dk) op[d] = acc[d];
}

// ------------------------------------------------------------------------------------ stage 4
template <typename T, int DMAX>
__global__ __launch_bounds__(kThreads) void bwd_dkv_kernel(DenseParams p) {
  constexpr int kTile = tile_of(DMAX);
  const int b = blockIdx.z, h = blockIdx.y;
  const int key = blockIdx.x * kThreads + threadIdx.x;
  const int dk = p.dk, dv = p.dv;
  extern __shared__ float smem[];
  float* qs = smem;                   // [kTile][dk]
  float* gs = smem + kTile * dk;      // [kTile][dv]  upstream gradient rows
  float* ls = gs + kTile * dv;        // [kTile] lse
  float* des = ls + kTile;            // [kTile] delta
  int* segs = reinterpret_cast<int*>(des + kTile);

  float kr[DMAX], vr[DMAX], dkr[DMAX], dvr[DMAX];
#pragma unroll
  for (int d = 0; d < DMAX; ++d) { kr[d] = 0.f; vr[d] = 0.f; dkr[d] = 0.f; dvr[d] = 0.f; }
  const bool key_ok = key < p.lk;
  if (key_ok) {
    const float* kp = p.k + (((int64_t)b * p.lk + key) * p.H + h) * dk;
    const float* vp = p.v + (((int64_t)b * p.lk + key) * p.H + h) * dv;
#pragma unroll
    for (int d = 0; d < DMAX; ++d) {
      if (d < dk) kr[d] = kp[d];
      if (d < dv) vr[d] = vp[d];
    }
  }
  const int kseg = (key_ok && p.kvseg) ? p.kvseg[(int64_t)b * p.lk + key] : 0;

  // under the causal mask only rows at or after this workgroup's first key can see its keys
  const int q_begin = p.causal ? min(p.lq, max((int)blockIdx.x * kThreads - p.coff, 0)) / kTile * kTile : 0;
  for (int q0 = q_begin; q0 < p.lq; q0 += kTile) {
    const int nq = min(kTile, p.lq - q0);
    __syncthreads();
    for (int idx = threadIdx.x; idx < nq * dk; idx += kThreads) {
      const int i = idx / dk, d = idx - i * dk;
      qs[idx] = p.q[(((int64_t)b * p.lq + q0 + i) * p.H + h) * dk + d];
    }
    for (int idx = threadIdx.x; idx < nq * dv; idx += kThreads) {
      const int i = idx / dv, d = idx - i * dv;
      const float x = load_as_f32(static_cast<const T*>(p.d_o) + (((int64_t)b * p.lq + q0 + i) * p.H + h) * dv + d);
      gs[idx] = x == x ? x : 0.f;
    }
    for (int i = threadIdx.x; i < nq; i += kThreads) {
      ls[i] = p.lse[((int64_t)b * p.H + h) * p.lq + q0 + i];
      des[i] = p.delta[((int64_t)b * p.H + h) * p.lq + q0 + i];
      if (p.qseg) segs[i] = p.qseg[(int64_t)b * p.lq + q0 + i];
    }
    __syncthreads();
    if (!key_ok) continue;
    for (int i = 0; i < nq; ++i) {
      const float lse = ls[i];
      bool keep = lse > -INFINITY;
      if (p.qseg) keep = keep && segs[i] == kseg;
      if (p.causal) keep = keep && (key <= q0 + i + p.coff);
      if (!keep) continue;
      float dot = 0.f;
#pragma unroll
      for (int d = 0; d < DMAX; ++d)
        if (d < dk) dot += kr[d] * qs[i * dk + d];
      float x = dot * p.sm_scale;
      if (p.bias) x += p.bias[((int64_t)b * p.lq + q0 + i) * p.lk + key];
      const float pt = expf(x - lse);
      float dp = 0.f;
#pragma unroll
      for (int d = 0; d < DMAX; ++d)
        if (d < dv) {
          const float gd = gs[i * dv + d];
          dp += gd * vr[d];
          dvr[d] += pt * gd;
        }
      const float ds = p.sm_scale * pt * (dp - des[i]);
#pragma unroll
      for (int d = 0; d < DMAX; ++d)
        if (d < dk) dkr[d] += ds * qs[i * dk + d];
    }
  }
  if (!key_ok) return;
  float* okp = p.dk_out + (((int64_t)b * p.lk + key) * p.H + h) * dk;
  float* ovp = p.dv_out + (((int64_t)b * p.lk + key) * p.H + h) * dv;
#pragma unroll
  for (int d = 0; d < DMAX; ++d) {
    if (d < dk) okp[d] = dkr[d];
    if (d < dv) ovp[d] = dvr[d];
  }
}

// ------------------------------------------------------------------------------------ stage 5
// One workgroup (256 threads) per token: da[r, h] and db[r, d] from the token's dense gradient
// dX[h, d].  With STAGE the token's dX (row stride D + 1), a and b sit in LDS; each da output is
// shared by `ns` neighbouring lanes that split the sum over d and combine with lane shuffles.
template <typename T, bool STAGE>
__global__ __launch_bounds__(256) void project_kernel(const float* dx, TpaFactor fa, TpaFactor fb, TpaGrad ga, TpaGrad gb, int L, int H,
                                                       int D, int R, int dsh, int nsh) {
  const int t = blockIdx.x, b = blockIdx.y;
  const float* xp = dx + ((int64_t)b * L + t) * H * D;
  const T* ap = static_cast<const T*>(fa.ptr) + b * fa.stride_b + t * fa.stride_l;
  const T* bp = static_cast<const T*>(fb.ptr) + b * fb.stride_b + t * fb.stride_l;
  float* oa = ga.ptr + b * ga.stride_b + t * ga.stride_l;
  float* ob = gb.ptr + b * gb.stride_b + t * gb.stride_l;
  const float inv = 1.f / (float)R;
  extern __shared__ __attribute__((aligned(16))) float xs[];  // [H][XS], then b[R][D], then a[R][H]
  if constexpr (STAGE) {
    // D = 1 << dsh here (indices by shifts, not divisions); rows 16 bytes apart in the banks, so
    // that lanes that read 16 bytes of different rows (the da part) spread over the banks
    const int XS = D + 4, d4sh = dsh - 2, d4mask = (D >> 2) - 1;
    float* bs = xs + H * XS;
    float* as = bs + R * D;
    for (int idx = threadIdx.x; idx < (H << d4sh); idx += 256) {
      const int h = idx >> d4sh, d4 = idx & d4mask;
      *reinterpret_cast<f32x4*>(xs + h * XS + 4 * d4) = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(xp + 4 * idx));
    }
    for (int idx = threadIdx.x; idx < (R << dsh); idx += 256) {
      const int r = idx >> dsh, d = idx & (D - 1);
      bs[idx] = load_as_f32(bp + r * fb.stride_r + d);
    }
    for (int idx = threadIdx.x; idx < R * H; idx += 256) {
      const int r = idx / H, h = idx - r * H;
      as[idx] = load_as_f32(ap + r * fa.stride_r + h);
    }
    __syncthreads();
    // db: four neighbouring d per thread
    for (int idx = threadIdx.x; idx < (R << d4sh); idx += 256) {
      const int r = idx >> d4sh, d4 = idx & d4mask;
      f32x4 acc = {0.f, 0.f, 0.f, 0.f};
      for (int h = 0; h < H; ++h) {
        const f32x4 xv = *reinterpret_cast<const f32x4*>(xs + h * XS + 4 * d4);
        const float av = as[r * H + h];
#pragma unroll
        for (int e = 0; e < 4; ++e) acc[e] += xv[e] * av;
      }
#pragma unroll
      for (int e = 0; e < 4; ++e) ob[r * gb.stride_r + 4 * d4 + e] = acc[e] * inv;
    }
    // da: ns = 1 << nsh neighbouring lanes share an output
    const int per_pass = 256 >> nsh, sub = threadIdx.x & ((1 << nsh) - 1);
    for (int base = 0; base < R * H; base += per_pass) {  // uniform trip count: the shuffles below need every lane
      const int idx = base + (threadIdx.x >> nsh);
      const bool ok = idx < R * H;
      const int r = ok ? idx / H : 0, h = ok ? idx - r * H : 0;
      float acc = 0.f;
      for (int d = 4 * sub; d < D; d += 4 << nsh) {
        const f32x4 xv = *reinterpret_cast<const f32x4*>(xs + h * XS + d);
        const f32x4 bv = *reinterpret_cast<const f32x4*>(bs + r * D + d);
        acc += xv[0] * bv[0] + xv[1] * bv[1] + xv[2] * bv[2] + xv[3] * bv[3];
      }
      for (int m = (1 << nsh) >> 1; m >= 1; m >>= 1) acc += __shfl_xor(acc, m, 64);
      if (ok && sub == 0) oa[r * ga.stride_r + h] = acc * inv;
    }
  } else {
    for (int idx = threadIdx.x; idx < R * D; idx += 256) {
      const int r = idx / D, d = idx - r * D;
      float acc = 0.f;
      for (int h = 0; h < H; ++h) acc += xp[h * D + d] * load_as_f32(ap + r * fa.stride_r + h);
      ob[r * gb.stride_r + d] = acc * inv;
    }
    for (int idx = threadIdx.x; idx < R * H; idx += 256) {
      const int r = idx / H, h = idx - r * H;
      float acc = 0.f;
      for (int d = 0; d < D; ++d) acc += xp[h * D + d] * load_as_f32(bp + r * fb.stride_r + d);
      oa[r * ga.stride_r + h] = acc * inv;
    }
  }
}

// The same projections for bf16 factors with H % 8 == 0 and (D / 8) (H / 8) a power of two up to 64,
// without LDS: a thread owns an 8 x 8 piece of one token's dX, rows 8 hg .. 8 hg + 7, columns 4 cc .. 4 cc + 3 of
// the lower and of the upper half of D (pieces of D are the fastest thread index, so each of the 16 loads of a
// piece reads whole contiguous half rows across the lanes: 12 % faster than 8 consecutive columns per thread,
// where one load instruction touched every other 16 bytes), multiplies it
// with its 8 values of b (for da) and of a (for db) rank by rank, and the sums over d and over h are
// reductions across the lanes that share a token: over the D / 8 neighbouring lanes with DPP adds,
// over the H / 8 groups above them with lane exchanges.  Several tokens share a wave.
template <int CTRL>
__device__ __forceinline__ float dpp_add(float v) {
  return v + __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, false));
}
__global__ __launch_bounds__(256) void project_h8_kernel(const float* dx, TpaFactor fa, TpaFactor fb, TpaGrad ga, TpaGrad gb, int L, int H,
                                                         int D, int R) {
  const int cpr = D / 8, hgs = H / 8, tt = cpr * hgs;  // threads per token
  const int64_t gtid = (int64_t)blockIdx.x * 256 + threadIdx.x;
  const int cc = (int)(gtid % cpr), hg = (int)(gtid / cpr % hgs);
  const int64_t tok = gtid / tt;
  const bool live = tok < L;
  const int64_t t = live ? tok : L - 1;  // lanes past the end idle along: the reductions need whole waves
  const int b = blockIdx.y;
  const int dh = D / 2;  // a thread's eight columns: 4 cc .. 4 cc + 3 and the same in the upper half of the row
  const float* xp = dx + (((int64_t)b * L + t) * H + 8 * hg) * D + 4 * cc;
  const uint16_t* ap = static_cast<const uint16_t*>(fa.ptr) + b * fa.stride_b + t * fa.stride_l + 8 * hg;
  const uint16_t* bp = static_cast<const uint16_t*>(fb.ptr) + b * fb.stride_b + t * fb.stride_l + 4 * cc;
  float x[8][8];
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const f32x4 lo = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(xp + (int64_t)i * D));
    const f32x4 hi = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(xp + (int64_t)i * D + dh));
#pragma unroll
    for (int j = 0; j < 4; ++j) { x[i][j] = lo[j]; x[i][4 + j] = hi[j]; }
  }
  const float inv = 1.f / (float)R;
  float* oa = ga.ptr + b * ga.stride_b + t * ga.stride_l + 8 * hg;
  float* ob = gb.ptr + b * gb.stride_b + t * gb.stride_l + 4 * cc;
  for (int r = 0; r < R; ++r) {
    const u32x4 av = *reinterpret_cast<const u32x4*>(ap + (int64_t)r * fa.stride_r);
    const u32x2 bl = *reinterpret_cast<const u32x2*>(bp + (int64_t)r * fb.stride_r);
    const u32x2 bh = *reinterpret_cast<const u32x2*>(bp + (int64_t)r * fb.stride_r + dh);
    const u32x4 bv = u32x4{bl[0], bl[1], bh[0], bh[1]};
    float af[8], bf[8];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      af[2 * j] = bf16lo_to_f32(av[j]); af[2 * j + 1] = bf16hi_to_f32(av[j]);
      bf[2 * j] = bf16lo_to_f32(bv[j]); bf[2 * j + 1] = bf16hi_to_f32(bv[j]);
    }
    float da[8], db[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      float acc = 0.f;
#pragma unroll
      for (int j = 0; j < 8; ++j) acc += x[i][j] * bf[j];
      da[i] = acc;
    }
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      float acc = 0.f;
#pragma unroll
      for (int i = 0; i < 8; ++i) acc += x[i][j] * af[i];
      db[j] = acc;
    }
    // da: sum over the cpr (8 or 16) neighbouring lanes of this (token, head group)
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      float v = da[i];
      v = dpp_add<0xB1>(v);   // quad_perm [1, 0, 3, 2]
      v = dpp_add<0x4E>(v);   // quad_perm [2, 3, 0, 1]
      v = dpp_add<0x141>(v);  // row_half_mirror: the other quad of the same eight lanes
      if (cpr == 16) v = dpp_add<0x140>(v);  // row_mirror: the other eight lanes of the row
      da[i] = v;
    }
    // db: sum over the head groups, which lie cpr lanes apart
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      float v = db[j];
      for (int m = cpr; m < tt; m <<= 1) v += __shfl_xor(v, m, 64);
      db[j] = v;
    }
    if (live && cc == 0) {
      *reinterpret_cast<f32x4*>(oa + (int64_t)r * ga.stride_r) = f32x4{da[0] * inv, da[1] * inv, da[2] * inv, da[3] * inv};
      *reinterpret_cast<f32x4*>(oa + (int64_t)r * ga.stride_r + 4) = f32x4{da[4] * inv, da[5] * inv, da[6] * inv, da[7] * inv};
    }
    if (live && hg == 0) {
      *reinterpret_cast<f32x4*>(ob + (int64_t)r * gb.stride_r) = f32x4{db[0] * inv, db[1] * inv, db[2] * inv, db[3] * inv};
      *reinterpret_cast<f32x4*>(ob + (int64_t)r * gb.stride_r + dh) = f32x4{db[4] * inv, db[5] * inv, db[6] * inv, db[7] * inv};
    }
  }
}

template <typename T>
void launch_project(const float* dx, const TpaFactor& fa, const TpaFactor& fb, const TpaGrad& ga, const TpaGrad& gb, int B, int L,
                    int H, int D, int R, hipStream_t stream) {
  if constexpr (sizeof(T) == 2) {
    const int cpr = D / 8, hgs = H / 8, tt = cpr * hgs;
    auto al16 = [](const void* ptr) { return (reinterpret_cast<uintptr_t>(ptr) & 15) == 0; };
    const bool fast = D % 8 == 0 && H % 8 == 0 && (cpr == 8 || cpr == 16) && tt <= 64 && (tt & (tt - 1)) == 0 && al16(dx) && al16(fa.ptr) &&
                      al16(fb.ptr) && al16(ga.ptr) && al16(gb.ptr) && fa.stride_b % 8 == 0 && fa.stride_l % 8 == 0 && fa.stride_r % 8 == 0 &&
                      fb.stride_b % 8 == 0 && fb.stride_l % 8 == 0 && fb.stride_r % 8 == 0 && ga.stride_b % 4 == 0 && ga.stride_l % 4 == 0 &&
                      ga.stride_r % 4 == 0 && gb.stride_b % 4 == 0 && gb.stride_l % 4 == 0 && gb.stride_r % 4 == 0;
    const int64_t blocks = ((int64_t)L * tt + 255) / 256;
    if (fast && blocks <= 2147483647LL) {
      hipLaunchKernelGGL(project_h8_kernel, dim3((unsigned)blocks, B), dim3(256), 0, stream, dx, fa, fb, ga, gb, L, H, D, R);
      return;
    }
  }
  const size_t smem = ((size_t)H * (D + 4) + (size_t)R * D + (size_t)R * H) * sizeof(float);
  int dsh = 0;
  while ((1 << dsh) < D) ++dsh;
  int nsh = 0;  // lanes per da output: a power of two, at most a wave, so that one pass covers the outputs if it can
  while (nsh < 6 && (4 << nsh) * R * H <= 512 && (16 << nsh) <= D) ++nsh;
  if (smem <= 60 * 1024 && (1 << dsh) == D && D >= 4)
    hipLaunchKernelGGL((project_kernel<T, true>), dim3(L, B), dim3(256), smem, stream, dx, fa, fb, ga, gb, L, H, D, R, dsh, nsh);
  else
    hipLaunchKernelGGL((project_kernel<T, false>), dim3(L, B), dim3(256), 0, stream, dx, fa, fb, ga, gb, L, H, D, R, dsh, nsh);
}

template <typename T, int DMAX>
int launch_dense_t(const DenseParams& p, hipStream_t stream) {
  constexpr int kTile = tile_of(DMAX);
  const size_t smem_q = (size_t)kTile * (p.dk + p.dv) * sizeof(float) + kTile * sizeof(int);
  const size_t smem_kv = (size_t)kTile * (p.dk + p.dv + 2) * sizeof(float) + kTile * sizeof(int);
  hipLaunchKernelGGL((bwd_dq_kernel<T, DMAX>), dim3((p.lq + kThreads - 1) / kThreads, p.H, p.B), dim3(kThreads), smem_q, stream, p);
  if (hipGetLastError() != hipSuccess) return TPA_ERR_LAUNCH;
  hipLaunchKernelGGL((bwd_dkv_kernel<T, DMAX>), dim3((p.lk + kThreads - 1) / kThreads, p.H, p.B), dim3(kThreads), smem_kv, stream, p);
  return hipGetLastError() == hipSuccess ? TPA_OK : TPA_ERR_LAUNCH;
}

template <typename T>
int launch_dense(const DenseParams& p, hipStream_t stream) {
  const int dmax = p.dk > p.dv ? p.dk : p.dv;
  if (dmax <= 8) return launch_dense_t<T, 8>(p, stream);
  if (dmax <= 32) return launch_dense_t<T, 32>(p, stream);
  if (dmax <= 64) return launch_dense_t<T, 64>(p, stream);
  if (dmax <= 128) return launch_dense_t<T, 128>(p, stream);
  if (dmax <= 256) return launch_dense_t<T, 256>(p, stream);
  return TPA_ERR_SHAPE;
}

inline size_t align256(size_t n) { return (n + 255) & ~size_t(255); }

template <typename T>
int tpa_bwd_t(const TpaBwdArgs* a, hipStream_t stream, bool mfma) {
  const size_t nq = (size_t)a->B * a->lq * a->H * a->dk, nk = (size_t)a->B * a->lk * a->H * a->dk,
               nv = (size_t)a->B * a->lk * a->H * a->dv, nd = (size_t)a->B * a->H * a->lq;
  char* w = static_cast<char*>(a->workspace);
  auto take = [&](size_t floats) { float* ptr = reinterpret_cast<float*>(w); w += align256(floats * sizeof(float)); return ptr; };
  // dense Q, K, V (fp32, or bf16 for the MFMA kernels: then only half of each slot is used)
  float *qd = take(nq), *kd = take(nk), *vd = take(nv), *dqd = take(nq), *dkd = take(nk), *dvd = take(nv), *delta = take(nd);

  const int threads = 256;
  // the matrix-core kernels: bf16 ones on bf16 copies of Q, K, V; fp32 ones on the fp32 copies
  const bool mfma32 = mfma && sizeof(T) == sizeof(float);
  mfma = mfma && !mfma32;
  if (mfma) {
    uint16_t *q16 = reinterpret_cast<uint16_t*>(qd), *k16 = reinterpret_cast<uint16_t*>(kd), *v16 = reinterpret_cast<uint16_t*>(vd);
    auto recon16 = [&](const TpaFactor& fa, const TpaFactor& fb, uint16_t* out, int L, int D, int R) {
      const bool vec = sizeof(T) == 2 && !(reinterpret_cast<uintptr_t>(fb.ptr) & 15) && fb.stride_b % 8 == 0 && fb.stride_l % 8 == 0 &&
                       fb.stride_r % 8 == 0;
      if (vec)
        hipLaunchKernelGGL(recon_bf16_kernel, dim3((L + kReconTokens - 1) / kReconTokens, a->B), dim3(threads), 0, stream, fa, fb, out, L, a->H, D, R, 1.f);
      else
        hipLaunchKernelGGL((recon_kernel<T, uint16_t>), dim3(L, a->B), dim3(threads), 0, stream, fa, fb, out, L, a->H, D, R);
    };
    // all three in one launch where the vectorised kernel applies (16-byte aligned factors, H % 8 == 0)
    bool one_launch = sizeof(T) == 2 && a->H % 8 == 0 && a->dk % 8 == 0 && a->dk == a->dv;
    const TpaFactor* fs[6] = {&a->qa, &a->qb, &a->ka, &a->kb, &a->va, &a->vb};
    for (const TpaFactor* f : fs)
      one_launch = one_launch && !(reinterpret_cast<uintptr_t>(f->ptr) & 15) && f->stride_b % 8 == 0 && f->stride_l % 8 == 0 && f->stride_r % 8 == 0;
    const int lmax = a->lq > a->lk ? a->lq : a->lk;
    const int64_t blocks = ((int64_t)lmax * (a->dk / 8) * (a->H / 8) + 255) / 256;
    if (one_launch && blocks <= 2147483647LL) {
      ReconJobs jobs{};
      jobs.job[0] = ReconJob{a->qa, a->qb, q16, a->lq, a->rq, 1.f};
      jobs.job[1] = ReconJob{a->ka, a->kb, k16, a->lk, a->rk, 1.f};
      jobs.job[2] = ReconJob{a->va, a->vb, v16, a->lk, a->rk, 1.f};
      hipLaunchKernelGGL(recon_bf16_h8_kernel, dim3((unsigned)blocks, a->B, 3), dim3(256), 0, stream, jobs, a->H, a->dk);
    } else {
      recon16(a->qa, a->qb, q16, a->lq, a->dk, a->rq);
      recon16(a->ka, a->kb, k16, a->lk, a->dk, a->rk);
      recon16(a->va, a->vb, v16, a->lk, a->dv, a->rk);
    }
  } else {
    hipLaunchKernelGGL((recon_kernel<T, float>), dim3(a->lq, a->B), dim3(threads), 0, stream, a->qa, a->qb, qd, a->lq, a->H, a->dk, a->rq);
    hipLaunchKernelGGL((recon_kernel<T, float>), dim3(a->lk, a->B), dim3(threads), 0, stream, a->ka, a->kb, kd, a->lk, a->H, a->dk, a->rk);
    hipLaunchKernelGGL((recon_kernel<T, float>), dim3(a->lk, a->B), dim3(threads), 0, stream, a->va, a->vb, vd, a->lk, a->H, a->dv, a->rk);
  }
  {
    const int vec = a->dv % 8 == 0 && !(reinterpret_cast<uintptr_t>(a->o) & 15) && !(reinterpret_cast<uintptr_t>(a->d_o) & 15);
    hipLaunchKernelGGL((delta_kernel<T>), dim3((unsigned)((nd * 16 + threads - 1) / threads)), dim3(threads), 0, stream,
                       static_cast<const T*>(a->o), static_cast<const T*>(a->d_o), delta, a->B, a->lq, a->H, a->dv, vec);
  }
  if (hipGetLastError() != hipSuccess) return TPA_ERR_LAUNCH;

  int rc;
  if (mfma) {
    rc = dense_bwd_mfma_launch(qd, kd, vd, a->d_o, a->lse, delta, a->q_segment_ids, a->kv_segment_ids, dqd, dkd, dvd,
                               a->B, a->lq, a->lk, a->H, a->dk, a->sm_scale, a->causal, causal_offset_of(a), stream);
  } else if (mfma32) {
    rc = dense_bwd_f32_launch(qd, kd, vd, static_cast<const float*>(a->d_o), a->lse, delta, a->q_segment_ids, a->kv_segment_ids,
                              dqd, dkd, dvd, a->B, a->lq, a->lk, a->H, a->dk, a->sm_scale, a->causal, causal_offset_of(a), stream);
  } else {
    DenseParams p{};
    p.q = qd; p.k = kd; p.v = vd; p.d_o = a->d_o; p.lse = a->lse; p.delta = delta;
    p.qseg = a->q_segment_ids; p.kvseg = a->kv_segment_ids; p.bias = nullptr;
    p.dq = dqd; p.dk_out = dkd; p.dv_out = dvd;
    p.B = a->B; p.lq = a->lq; p.lk = a->lk; p.H = a->H; p.dk = a->dk; p.dv = a->dv;
    p.sm_scale = a->sm_scale; p.causal = a->causal; p.coff = causal_offset_of(a);
    rc = launch_dense<T>(p, stream);
  }
  if (rc != TPA_OK) return rc;

  launch_project<T>(dqd, a->qa, a->qb, a->dqa, a->dqb, a->B, a->lq, a->H, a->dk, a->rq, stream);
  launch_project<T>(dkd, a->ka, a->kb, a->dka, a->dkb, a->B, a->lk, a->H, a->dk, a->rk, stream);
  launch_project<T>(dvd, a->va, a->vb, a->dva, a->dvb, a->B, a->lk, a->H, a->dv, a->rk, stream);
  return hipGetLastError() == hipSuccess ? TPA_OK : TPA_ERR_LAUNCH;
}

template <typename T>
int mha_bwd_t(const MhaBwdArgs* a, hipStream_t stream, bool mfma) {
  const size_t nq = (size_t)a->B * a->lq * a->H * a->dk, nk = (size_t)a->B * a->lk * a->H * a->dk,
               nv = (size_t)a->B * a->lk * a->H * a->dv, nd = (size_t)a->B * a->H * a->lq;
  char* w = static_cast<char*>(a->workspace);
  auto take = [&](size_t floats) { float* ptr = reinterpret_cast<float*>(w); w += align256(floats * sizeof(float)); return ptr; };
  float* delta = take(nd);
  const int threads = 256;
  {
    const int vec = a->dv % 8 == 0 && !(reinterpret_cast<uintptr_t>(a->o) & 15) && !(reinterpret_cast<uintptr_t>(a->d_o) & 15);
    hipLaunchKernelGGL((delta_kernel<T>), dim3((unsigned)((nd * 16 + threads - 1) / threads)), dim3(threads), 0, stream,
                       static_cast<const T*>(a->o), static_cast<const T*>(a->d_o), delta, a->B, a->lq, a->H, a->dv, vec);
  }
  if (hipGetLastError() != hipSuccess) return TPA_ERR_LAUNCH;
  if (mfma && sizeof(T) == sizeof(float))
    return dense_bwd_f32_launch(static_cast<const float*>(a->q), static_cast<const float*>(a->k), static_cast<const float*>(a->v),
                                static_cast<const float*>(a->d_o), a->lse, delta, nullptr, nullptr, a->dq, a->dk_out, a->dv_out,
                                a->B, a->lq, a->lk, a->H, a->dk, a->sm_scale, a->causal, 0, stream);
  if (mfma)
    return dense_bwd_mfma_launch(a->q, a->k, a->v, a->d_o, a->lse, delta, nullptr, nullptr, a->dq, a->dk_out, a->dv_out,
                                 a->B, a->lq, a->lk, a->H, a->dk, a->sm_scale, a->causal, 0, stream);
  const float *qd, *kd, *vd;
  if constexpr (sizeof(T) == sizeof(float)) {
    qd = static_cast<const float*>(a->q); kd = static_cast<const float*>(a->k); vd = static_cast<const float*>(a->v);
  } else {
    float *q32 = take(nq), *k32 = take(nk), *v32 = take(nv);
    auto blocks = [&](size_t n) { return dim3((unsigned)((n + threads - 1) / threads < 65535 * 16 ? (n + threads - 1) / threads : 65535 * 16)); };
    hipLaunchKernelGGL((to_f32_kernel<T>), blocks(nq), dim3(threads), 0, stream, static_cast<const T*>(a->q), q32, (int64_t)nq);
    hipLaunchKernelGGL((to_f32_kernel<T>), blocks(nk), dim3(threads), 0, stream, static_cast<const T*>(a->k), k32, (int64_t)nk);
    hipLaunchKernelGGL((to_f32_kernel<T>), blocks(nv), dim3(threads), 0, stream, static_cast<const T*>(a->v), v32, (int64_t)nv);
    qd = q32; kd = k32; vd = v32;
  }
  if (hipGetLastError() != hipSuccess) return TPA_ERR_LAUNCH;
  DenseParams p{};
  p.q = qd; p.k = kd; p.v = vd; p.d_o = a->d_o; p.lse = a->lse; p.delta = delta;
  p.qseg = nullptr; p.kvseg = nullptr; p.bias = a->bias;
  p.dq = a->dq; p.dk_out = a->dk_out; p.dv_out = a->dv_out;
  p.B = a->B; p.lq = a->lq; p.lk = a->lk; p.H = a->H; p.dk = a->dk; p.dv = a->dv;
  p.sm_scale = a->sm_scale; p.causal = a->causal;
  return launch_dense<T>(p, stream);
}

}  // namespace
}  // namespace tpa

int tpa_recon_dense_bf16(const TpaFactor* fa, const TpaFactor* fb, uint16_t* out, int B, int L, int H, int D, int R, float scale, hipStream_t stream) {
  if (B > 65535) return TPA_ERR_SHAPE;
  const bool vec = D % 8 == 0 && !(reinterpret_cast<uintptr_t>(fb->ptr) & 15) && fb->stride_b % 8 == 0 && fb->stride_l % 8 == 0 &&
                   fb->stride_r % 8 == 0;
  const bool vec_a = vec && H % 8 == 0 && !(reinterpret_cast<uintptr_t>(fa->ptr) & 15) && fa->stride_b % 8 == 0 && fa->stride_l % 8 == 0 &&
                     fa->stride_r % 8 == 0;
  const int64_t threads = (int64_t)L * (D / 8) * (H / 8);
  if (vec_a && (threads + 255) / 256 <= 2147483647LL) {
    tpa::ReconJobs jobs{};
    jobs.job[0] = tpa::ReconJob{*fa, *fb, out, L, R, scale};
    hipLaunchKernelGGL(tpa::recon_bf16_h8_kernel, dim3((unsigned)((threads + 255) / 256), B, 1), dim3(256), 0, stream, jobs, H, D);
  } else if (vec)
    hipLaunchKernelGGL(tpa::recon_bf16_kernel, dim3((L + tpa::kReconTokens - 1) / tpa::kReconTokens, B), dim3(256), 0, stream, *fa, *fb, out, L, H, D, R, scale);
  else if (scale != 1.f)
    return TPA_ERR_ALIGN;  // the scaled form exists for 16-byte aligned factors only
  else
    hipLaunchKernelGGL((tpa::recon_kernel<uint16_t, uint16_t>), dim3(L, B), dim3(256), 0, stream, *fa, *fb, out, L, H, D, R);
  return hipGetLastError() == hipSuccess ? TPA_OK : TPA_ERR_LAUNCH;
}

// Q (with its scale), K and V in one launch where every factor is 16-byte aligned and H % 8 == 0;
// TPA_ERR_UNSUPPORTED otherwise (the caller then reconstructs them one by one).
int tpa_recon_dense_qkv_bf16(const TpaFwdArgs* a, uint16_t* qd, uint16_t* kd, uint16_t* vd, float q_scale, hipStream_t stream) {
  if (a->B > 65535 || a->H % 8 != 0 || a->dk % 8 != 0 || a->dk != a->dv) return TPA_ERR_UNSUPPORTED;
  const TpaFactor* fs[6] = {&a->qa, &a->qb, &a->ka, &a->kb, &a->va, &a->vb};
  for (const TpaFactor* f : fs)
    if ((reinterpret_cast<uintptr_t>(f->ptr) & 15) || f->stride_b % 8 != 0 || f->stride_l % 8 != 0 || f->stride_r % 8 != 0) return TPA_ERR_UNSUPPORTED;
  const int lmax = a->lq > a->lk ? a->lq : a->lk;
  const int64_t blocks = ((int64_t)lmax * (a->dk / 8) * (a->H / 8) + 255) / 256;
  if (blocks > 2147483647LL) return TPA_ERR_UNSUPPORTED;
  tpa::ReconJobs jobs{};
  jobs.job[0] = tpa::ReconJob{a->qa, a->qb, qd, a->lq, a->rq, q_scale};
  jobs.job[1] = tpa::ReconJob{a->ka, a->kb, kd, a->lk, a->rk, 1.f};
  jobs.job[2] = tpa::ReconJob{a->va, a->vb, vd, a->lk, a->rk, 1.f};
  hipLaunchKernelGGL(tpa::recon_bf16_h8_kernel, dim3((unsigned)blocks, a->B, 3), dim3(256), 0, stream, jobs, a->H, a->dk);
  return hipGetLastError() == hipSuccess ? TPA_OK : TPA_ERR_LAUNCH;
}

size_t tpa_bwd_workspace_size(int64_t B, int64_t lq, int64_t lk, int64_t H, int64_t dk, int64_t dv) {
  using tpa::align256;
  const size_t nq = (size_t)(B * lq * H * dk), nk = (size_t)(B * lk * H * dk), nv = (size_t)(B * lk * H * dv), nd = (size_t)(B * H * lq);
  return 2 * (align256(nq * 4) + align256(nk * 4) + align256(nv * 4)) + align256(nd * 4);
}

size_t mha_bwd_workspace_size(int64_t B, int64_t lq, int64_t lk, int64_t H, int64_t dk, int64_t dv, int dtype) {
  using tpa::align256;
  const size_t nq = (size_t)(B * lq * H * dk), nk = (size_t)(B * lk * H * dk), nv = (size_t)(B * lk * H * dv), nd = (size_t)(B * H * lq);
  size_t bytes = align256(nd * 4);
  if (dtype != TPA_DTYPE_F32) bytes += align256(nq * 4) + align256(nk * 4) + align256(nv * 4);
  return bytes;
}

int tpa_bwd_launch(const TpaBwdArgs* a, hipStream_t stream, int mfma) {
  if (a->B > 65535 || a->H > 65535) return TPA_ERR_SHAPE;
  if (a->dtype == TPA_DTYPE_F32) return tpa::tpa_bwd_t<float>(a, stream, mfma != 0);
  if (a->dtype == TPA_DTYPE_BF16) return tpa::tpa_bwd_t<uint16_t>(a, stream, mfma != 0);
  return TPA_ERR_DTYPE;
}

int mha_bwd_launch(const MhaBwdArgs* a, hipStream_t stream, int mfma) {
  if (a->B > 65535 || a->H > 65535) return TPA_ERR_SHAPE;
  if (a->dtype == TPA_DTYPE_F32) return tpa::mha_bwd_t<float>(a, stream, mfma != 0);
  if (a->dtype == TPA_DTYPE_BF16) return tpa::mha_bwd_t<uint16_t>(a, stream, mfma != 0);
  return TPA_ERR_DTYPE;
}
