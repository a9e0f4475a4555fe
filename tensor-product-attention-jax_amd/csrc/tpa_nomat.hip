// The reference's `nomat` evaluation order on the matrix cores of gfx950 (tpa/tpa.py:333-359, 398-413):
// K and V are never formed, and neither is Q.  Per block of keys the logits are
//
//     bb[r, s][k, q] = kb_s[k, :] . qb_r[q, :]                          one table per rank pair, shared by
//                                                                       every head of the workgroup (MFMA)
//     x[h][k, q]     = c sum_r qa_r[q, h] (sum_s ka_s[k, h] bb[r, s][k, q])   the head factors, on the vector ALU
//
// with c = sm_scale log2(e) / (rq rk), and the output
//
//     o[h][q, :]     = (1 / rk) sum_s sum_k (p[h][k, q] va_s[k, h]) vb_s[k, :]       (MFMA, one product per rank)
//
// - the double scan over the rank pairs of tpa/tpa.py:349-357 and the scan over the value ranks of
// tpa/tpa.py:405-412.  A workgroup is eight waves of 32 query rows and a block of kHB heads (the reference's
// block_h); everything is computed transposed (keys along the registers of a lane, one query row per lane), as in
// the materialising kernel, so the online softmax is in-lane.
//
// This order is never chosen by the library: per logit and head it spends rq (rk + 1) vector instructions on the
// combination where the materialising kernel spends none, and rk times the matrix instructions on the output.
// It exists so that the reference's switch can select the reference's arithmetic, and to measure it.
#include "tpa_common.h"

namespace tpa {
namespace {

constexpr int kHB = 2;      // heads per workgroup that share the rank-pair tables
constexpr int kTK = 32;     // keys per block
constexpr int kNW = 8;      // waves per workgroup, 32 query rows each
constexpr int kBQ = 32 * kNW;

struct NomatParams {
  TpaFactor qa, qb, ka, kb, va, vb;
  const int32_t* kvlen;
  uint16_t* o;
  float* lse;
  int B, lq, lk, H;
  float sm_scale;
  int causal, coff;
};

template <int D, int RK>
struct NomatLds {
  static constexpr int KS = D + 8;    // row stride of a kb tile (elements): conflict-free 16-byte row reads
  static constexpr int VS = D + 32;   // row stride of a vb tile: conflict-free transposed reads
  static constexpr int kKb = RK * kTK * KS;
  static constexpr int kVb = RK * kTK * VS;
  static constexpr int kA = 2 * RK * kHB * kTK * 2;  // ka and va of the block as fp32 [K|V][s][head][key], in uint16 units
  static constexpr size_t kBytes = (kKb + kVb + kA) * sizeof(uint16_t);
};

template <int D, int RQ, int RK>
__global__ __launch_bounds__(kNW * 64) void nomat_pairs_kernel(NomatParams p) {
  using L = NomatLds<D, RK>;
  constexpr int KS = L::KS, VS = L::VS, NKS = D / 16, NDB = D / 32, CPR = D / 8, NT = kNW * 64;
  extern __shared__ __attribute__((aligned(16))) uint16_t smem[];
  uint16_t* const kbs = smem;                                  // [RK][kTK][KS]
  uint16_t* const vbs = smem + L::kKb;                         // [RK][kTK][VS]
  float* const kas = reinterpret_cast<float*>(smem + L::kKb + L::kVb);   // [RK][kHB][kTK]
  float* const vas = kas + RK * kHB * kTK;                     // [RK][kHB][kTK], already divided by rk

  const int tid = threadIdx.x, w = tid >> 6, l = tid & 63, i = l & 31, g = l >> 5;
  const int lp = l & 15, dhalf = (l >> 4) & 1;
  const int q0 = blockIdx.x * kBQ, h0 = blockIdx.y * kHB, b = blockIdx.z;
  const int qrow = q0 + 32 * w + i, qrow_ld = min(qrow, p.lq - 1);
  const int nh = min(kHB, p.H - h0);

  const int len_b = p.kvlen ? max(0, min(p.kvlen[b], p.lk)) : p.lk;
  const int coff = p.causal ? p.coff + (p.causal == TPA_CAUSAL_BOTTOM_RIGHT ? len_b - p.lq : 0) : 0;
  const int kend = p.causal ? max(0, min(len_b, min(q0 + kBQ, p.lq) + coff)) : len_b;  // keys any row of the workgroup sees
  const int limit = p.causal ? min(qrow + coff, len_b - 1) : len_b - 1;               // last key this lane's row sees

  const uint16_t* const qb_row = static_cast<const uint16_t*>(p.qb.ptr) + b * p.qb.stride_b + (int64_t)qrow_ld * p.qb.stride_l + 8 * g;
  const uint16_t* const qa_row = static_cast<const uint16_t*>(p.qa.ptr) + b * p.qa.stride_b + (int64_t)qrow_ld * p.qa.stride_l + h0;
  const uint16_t* const kb_b = static_cast<const uint16_t*>(p.kb.ptr) + b * p.kb.stride_b;
  const uint16_t* const vb_b = static_cast<const uint16_t*>(p.vb.ptr) + b * p.vb.stride_b;
  const uint16_t* const ka_b = static_cast<const uint16_t*>(p.ka.ptr) + b * p.ka.stride_b + h0;
  const uint16_t* const va_b = static_cast<const uint16_t*>(p.va.ptr) + b * p.va.stride_b + h0;

  const float c = p.sm_scale * kLog2e / (float)(RQ * RK);  // the constant of the logits, folded into qa below

  f32x16 o[kHB][NDB];
  float m[kHB], lsum[kHB];
#pragma unroll
  for (int hh = 0; hh < kHB; ++hh) {
    m[hh] = -INFINITY;
    lsum[hh] = 0.f;
#pragma unroll
    for (int db = 0; db < NDB; ++db)
#pragma unroll
      for (int v = 0; v < 16; ++v) o[hh][db][v] = 0.f;
  }

  for (int k0 = 0; k0 < kend; k0 += kTK) {
    __syncthreads();  // the previous block has been consumed
    // ---- the block's rows of kb_s and vb_s, and its head factors, into LDS (keys past the end repeat the last key)
    for (int ch = tid; ch < RK * kTK * CPR; ch += NT) {
      const int s = ch / (kTK * CPR), t = (ch / CPR) % kTK, cc = ch % CPR;
      const int64_t tok = min(k0 + t, len_b - 1);
      *reinterpret_cast<u32x4*>(kbs + (s * kTK + t) * KS + 8 * cc) = *reinterpret_cast<const u32x4*>(kb_b + tok * p.kb.stride_l + s * p.kb.stride_r + 8 * cc);
      *reinterpret_cast<u32x4*>(vbs + (s * kTK + t) * VS + 8 * cc) = *reinterpret_cast<const u32x4*>(vb_b + tok * p.vb.stride_l + s * p.vb.stride_r + 8 * cc);
    }
    for (int e = tid; e < 2 * RK * kHB * kTK; e += NT) {
      const int mat = e / (RK * kHB * kTK), s = (e / (kHB * kTK)) % RK, hh = (e / kTK) % kHB, t = e % kTK;
      const int64_t tok = min(k0 + t, len_b - 1);
      float val = 0.f;
      if (hh < nh) val = mat ? bf16bits_to_f32(va_b[tok * p.va.stride_l + s * p.va.stride_r + hh]) * (1.f / (float)RK)
                             : bf16bits_to_f32(ka_b[tok * p.ka.stride_l + s * p.ka.stride_r + hh]);
      (mat ? vas : kas)[(s * kHB + hh) * kTK + t] = val;
    }
    __syncthreads();

    // ---- logits of every head of the block: x[hh][v] belongs to key k0 + 8 (v / 4) + 4 g + v % 4
    f32x16 x[kHB];
#pragma unroll
    for (int hh = 0; hh < kHB; ++hh)
#pragma unroll
      for (int v = 0; v < 16; ++v) x[hh][v] = 0.f;
    // one query rank at a time (a loop, not unrolled: six ranks' tables and fragments do not fit the registers)
#pragma clang loop unroll(disable)
    for (int r = 0; r < RQ; ++r) {
      // c qa_r[q, h] of this lane's row, and the qb_r fragments of the row: lane (row, g) holds
      // qb_r[row][16 ks + 8 g + 0..7]
      float qa[kHB];
#pragma unroll
      for (int hh = 0; hh < kHB; ++hh) qa[hh] = hh < nh ? c * bf16bits_to_f32(qa_row[r * p.qa.stride_r + hh]) : 0.f;
      bf16x8 qf[NKS];
#pragma unroll
      for (int ks = 0; ks < NKS; ++ks) qf[ks] = *reinterpret_cast<const bf16x8*>(qb_row + r * p.qb.stride_r + 16 * ks);
      // one key / value rank at a time: bb[v] = kb_s[key(v)] . qb_r[row], then every head of the block adds
      // (c qa_r[row, h] ka_s[key(v), h]) bb[v] to its logits
#pragma clang loop unroll(disable)
      for (int s = 0; s < RK; ++s) {
        f32x16 bb;
#pragma unroll
        for (int v = 0; v < 16; ++v) bb[v] = 0.f;
#pragma unroll
        for (int ks = 0; ks < NKS; ++ks) {
          const bf16x8 kf = *reinterpret_cast<const bf16x8*>(kbs + (s * kTK + i) * KS + 16 * ks + 8 * g);
          bb = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf, qf[ks], bb, 0, 0, 0);
        }
#pragma unroll
        for (int hh = 0; hh < kHB; ++hh)
#pragma unroll
          for (int vq = 0; vq < 4; ++vq) {
            const f32x4 a4 = *reinterpret_cast<const f32x4*>(kas + (s * kHB + hh) * kTK + 8 * vq + 4 * g);
#pragma unroll
            for (int j = 0; j < 4; ++j) x[hh][4 * vq + j] += (qa[hh] * a4[j]) * bb[4 * vq + j];
          }
        __builtin_amdgcn_sched_barrier(0);  // the next table's operands are not fetched before this one is folded in
      }
    }

    // ---- per head: mask, online softmax (tpa/tpa.py:389-393), o += sum_s (p * va_s) vb_s (tpa/tpa.py:398-413)
#pragma unroll
    for (int hh = 0; hh < kHB; ++hh) {
      __builtin_amdgcn_sched_barrier(0);  // one head at a time: interleaved, the heads' temporaries do not fit the registers
      float tmax = -INFINITY;
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int t = k0 + 8 * (v >> 2) + 4 * g + (v & 3);
        if (t > limit) x[hh][v] = -INFINITY;
        tmax = fmaxf(tmax, x[hh][v]);
      }
      tmax = halves_max(tmax);
      const float m_new = fmaxf(m[hh], tmax);
      const float m_use = m_new == -INFINITY ? 0.f : m_new;
      if (__any(m_new > m[hh])) {
        const float alpha = __builtin_amdgcn_exp2f(m[hh] - m_use);  // exp2(-inf) = 0 for a row's first visible key
        lsum[hh] *= alpha;
#pragma unroll
        for (int db = 0; db < NDB; ++db)
#pragma unroll
          for (int v = 0; v < 16; ++v) o[hh][db][v] *= alpha;
        m[hh] = m_new;
      }
      float pr[16];
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        pr[v] = __builtin_amdgcn_exp2f(x[hh][v] - m_use);
        lsum[hh] += pr[v];
      }
#pragma clang loop unroll(disable)
      for (int s = 0; s < RK; ++s) {
        // P'_s^T fragments: slot (g, j) of k-step kk = key 16 kk + 8 (j / 4) + 4 g + j % 4, the accumulator's own order
        bf16x8 pf[2];
#pragma unroll
        for (int kk = 0; kk < 2; ++kk) {
          u32x4 pk;
#pragma unroll
          for (int jq = 0; jq < 2; ++jq) {
            const f32x4 a4 = *reinterpret_cast<const f32x4*>(vas + (s * kHB + hh) * kTK + 16 * kk + 8 * jq + 4 * g);
            pk[2 * jq] = pack_bf16(pr[8 * kk + 4 * jq] * a4[0], pr[8 * kk + 4 * jq + 1] * a4[1]);
            pk[2 * jq + 1] = pack_bf16(pr[8 * kk + 4 * jq + 2] * a4[2], pr[8 * kk + 4 * jq + 3] * a4[3]);
          }
          pf[kk] = __builtin_bit_cast(bf16x8, pk);
        }
#pragma unroll
        for (int kk = 0; kk < 2; ++kk)
#pragma unroll
          for (int db = 0; db < NDB; ++db) {
            const uint16_t* vrow = vbs + (s * kTK + 16 * kk + 4 * g + (lp >> 2)) * VS + 16 * dhalf + 4 * (lp & 3) + 32 * db;
            const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3)))*)(vrow));
            const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3)))*)(vrow + 8 * VS));
            const bf16x8 vf = __builtin_bit_cast(bf16x8, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
            o[hh][db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf, pf[kk], o[hh][db], 0, 0, 0);
          }
      }
    }
  }

  // ---- normalise and store; rows without a visible key end as NaN / -inf (tpa/tpa.py:437-439)
  if (qrow >= p.lq) return;
#pragma unroll
  for (int hh = 0; hh < kHB; ++hh) {
    if (hh >= nh) break;
    const float ltot = halves_sum(lsum[hh]);
    const float inv = 1.f / ltot;  // 1 / 0 = inf, and 0 * inf = NaN: the empty row
    uint16_t* op = p.o + (((int64_t)b * p.lq + qrow) * p.H + h0 + hh) * D;
#pragma unroll
    for (int db = 0; db < NDB; ++db)
#pragma unroll
      for (int vq = 0; vq < 4; ++vq) {
        u32x2 pk;
        pk[0] = pack_bf16(o[hh][db][4 * vq] * inv, o[hh][db][4 * vq + 1] * inv);
        pk[1] = pack_bf16(o[hh][db][4 * vq + 2] * inv, o[hh][db][4 * vq + 3] * inv);
        if (m[hh] == -INFINITY) pk[0] = pk[1] = 0x7fc07fc0u;
        *reinterpret_cast<u32x2*>(op + 32 * db + 8 * vq + 4 * g) = pk;
      }
    if (p.lse && g == 0)
      p.lse[((int64_t)b * p.H + h0 + hh) * p.lq + qrow] = m[hh] == -INFINITY ? -INFINITY : (m[hh] + __builtin_amdgcn_logf(ltot)) * kLn2;
  }
}

template <int D, int RQ, int RK>
int launch(const NomatParams& p, hipStream_t stream) {
  auto kern = nomat_pairs_kernel<D, RQ, RK>;
  constexpr size_t lds_bytes = NomatLds<D, RK>::kBytes;
  static bool configured[kMaxDevices] = {};
  if (lds_bytes > 64 * 1024)
    if (int rc = raise_lds_limit(configured, reinterpret_cast<const void*>(kern), lds_bytes); rc != TPA_OK) return rc;
  dim3 grid((unsigned)((p.lq + kBQ - 1) / kBQ), (unsigned)((p.H + kHB - 1) / kHB), (unsigned)p.B);
  hipLaunchKernelGGL(kern, grid, dim3(kNW * 64), lds_bytes, stream, p);
  return hipGetLastError() == hipSuccess ? TPA_OK : TPA_ERR_LAUNCH;
}

template <int D, int RQ>
int launch_rk(const NomatParams& p, int rk, hipStream_t stream) {
  switch (rk) {
    case 1: return launch<D, RQ, 1>(p, stream);
    case 2: return launch<D, RQ, 2>(p, stream);
    case 4: return launch<D, RQ, 4>(p, stream);
  }
  return TPA_ERR_UNSUPPORTED;
}

bool aligned16(const void* ptr) { return (reinterpret_cast<uintptr_t>(ptr) & 15) == 0; }

}  // namespace
}  // namespace tpa

// The instances: bf16, head size 64 / 128, query ranks 1 and 6, key / value ranks 1, 2 and 4 (the ranks of the
// reference's test grid, tpa/tpa_test.py:62-63, and of the benchmark configurations' 6 / 2).
int tpa_nomat_pairs_supported(const TpaFwdArgs* a) {
  if (a->dtype != TPA_DTYPE_BF16 || a->dk != a->dv || (a->dk != 64 && a->dk != 128)) return 0;
  if (a->rq != 1 && a->rq != 6) return 0;
  if (a->rk != 1 && a->rk != 2 && a->rk != 4) return 0;
  if (a->q_segment_ids || a->page_table) return 0;
  for (const TpaFactor* f : {&a->qb, &a->kb, &a->vb})
    if (!tpa::aligned16(f->ptr) || f->stride_b % 8 || f->stride_l % 8 || f->stride_r % 8) return 0;
  return tpa::aligned16(a->o) ? 1 : 0;
}

int tpa_nomat_pairs_launch(const TpaFwdArgs* a, hipStream_t stream) {
  using namespace tpa;
  NomatParams p{};
  p.qa = a->qa; p.qb = a->qb; p.ka = a->ka; p.kb = a->kb; p.va = a->va; p.vb = a->vb;
  p.kvlen = a->kv_lengths;
  p.o = static_cast<uint16_t*>(a->o); p.lse = a->lse;
  p.B = a->B; p.lq = a->lq; p.lk = a->lk; p.H = a->H;
  p.sm_scale = a->sm_scale; p.causal = a->causal; p.coff = causal_offset_of(a);
  if (a->dk == 128) return a->rq == 1 ? launch_rk<128, 1>(p, a->rk, stream) : launch_rk<128, 6>(p, a->rk, stream);
  return a->rq == 1 ? launch_rk<64, 1>(p, a->rk, stream) : launch_rk<64, 6>(p, a->rk, stream);
}
