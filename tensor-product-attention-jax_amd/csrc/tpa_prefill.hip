// Flash-style prefill for gfx950: bf16 MFMA contractions, fp32 online softmax.
//
// One workgroup = one (batch, head, block of kBQ query rows); each of its waves owns 32 query
// rows.  Per tile of 64 keys the workgroup rebuilds the head's K and V tile from the rank
// factors (K = (1/R) sum_r a_r (x) b_r, tpa/tpa.py:364,417) straight out of coalesced 16-byte
// factor loads and stores it once, as bf16, in LDS.  The waves then compute
//     S^T = K Q^T        (v_mfma_f32_32x32x16_bf16, A = K rows from LDS, B = Q kept in registers)
//     online softmax     (each lane holds 32 logits of ONE query row, so the row max and sum
//                         are in-lane apart from one exchange with lane ^ 32)
//     O^T += V^T P^T     (A = V^T read with ds_read_b64_tr_b16 from row-major V, B = P^T, which
//                         is the S^T accumulator converted in place: no LDS round trip for P)
// and keep the deferred normalisation of flash attention (m, l per row), which is the
// normalise-every-step recurrence of tpa/tpa.py:389-424 in another order of operations.
// The dense flash baseline (tpa/mha.py:23-37) is the same kernel with a plain K/V loader.
#include "tpa_common.h"

namespace tpa {
namespace {

constexpr int kTK = 64;  // keys per tile

enum { LOAD_TPA_R2 = 0, LOAD_TPA_ANY = 1, LOAD_DENSE = 2 };

struct PrefillParams {
  TpaFactor qa, qb, ka, kb, va, vb;  // dense: qb/kb/vb hold q/k/v with stride_l = H*D, ptr at head 0
  uint16_t* o;
  float* lse;
  int B, lq, lk, H, rq, rk;
  float sm_scale;
  int causal;
  int nqb;     // query blocks per (batch, head)
  int npairs;  // nqb * B
};

template <int D>
struct Lds {
  static constexpr int KS = D + 8;   // K row stride (elements): 16-byte reads of 16 rows hit distinct banks
  static constexpr int VS = D + 32;  // V row stride: 4 consecutive rows of a transposed read hit distinct banks
  static constexpr int kStage = kTK * KS + kTK * VS;  // elements per stage
  static constexpr size_t kBytes = 2 * kStage * sizeof(uint16_t);
};

template <int D, int NW, int LOADER>
__global__ __launch_bounds__(NW * 64) void prefill_kernel(PrefillParams p) {
  constexpr int NT = NW * 64;
  constexpr int BQ = NW * 32;
  constexpr int KS = Lds<D>::KS, VS = Lds<D>::VS;
  constexpr int CPR = D / 8;             // 16-byte chunks per row
  constexpr int TPP = NT / CPR;          // tokens per loader pass
  constexpr int NPASS = kTK / TPP;       // loader passes per tile and matrix
  static_assert(kTK % TPP == 0 && NPASS >= 1, "loader shape");
  constexpr int NKS = D / 16;            // k-steps of the QK^T contraction
  constexpr int NDB = D / 32;            // 32-row blocks of O^T

  extern __shared__ __attribute__((aligned(16))) uint16_t smem[];

  // ---- which (query block, batch, head): heads of one (block, batch) pair sit on one XCD
  // (workgroup ids are dealt round-robin to the 8 XCDs) so they share the B-factor tiles in
  // that XCD's L2; pairs are ordered heaviest (last causal block) first.
  const int id = blockIdx.x;
  const int xcd = id & 7, slot = id >> 3;
  const int pair = (slot / p.H) * 8 + xcd;
  const int h = slot % p.H;
  if (pair >= p.npairs) return;
  const int qblk = p.nqb - 1 - pair / p.B;
  const int b = pair % p.B;

  const int tid = threadIdx.x;
  const int w = tid >> 6, l = tid & 63, i = l & 31, g = l >> 5;
  const int q0 = qblk * BQ;
  const int qrow = q0 + 32 * w + i;
  const int qrow_ld = min(qrow, p.lq - 1);
  const float c = p.sm_scale * kLog2e;

  // ---- Q fragments (B operand of S^T = K Q^T): lane (i, g) holds Q[qrow][16ks + 8g + 0..7].
  // Built after the first K/V factor loads are in flight; per rank all loads are issued together.
  bf16x8 qf[NKS];
  auto build_q = [&]() {
    if constexpr (LOADER == LOAD_DENSE) {
      const uint16_t* qp = static_cast<const uint16_t*>(p.qb.ptr) + b * p.qb.stride_b + (int64_t)qrow_ld * p.qb.stride_l + (int64_t)h * D;
#pragma unroll
      for (int ks = 0; ks < NKS; ++ks) qf[ks] = *reinterpret_cast<const bf16x8*>(qp + 16 * ks + 8 * g);
    } else {
      const uint16_t* ap = static_cast<const uint16_t*>(p.qa.ptr) + b * p.qa.stride_b + (int64_t)qrow_ld * p.qa.stride_l + h;
      const uint16_t* bp = static_cast<const uint16_t*>(p.qb.ptr) + b * p.qb.stride_b + (int64_t)qrow_ld * p.qb.stride_l + 8 * g;
      build_q_fragments<NKS, 3>(ap, p.qa.stride_r, bp, p.qb.stride_r, p.rq, 1.f / (float)p.rq, qf);
    }
  };

  // ---- tile range
  int ntiles = (p.lk + kTK - 1) / kTK;
  if (p.causal) ntiles = min(ntiles, (min(q0 + BQ, p.lq) + kTK - 1) / kTK);
  // last tile this wave needs under the causal mask (rows of the wave: q0+32w .. +31)
  const int wave_last_tile = p.causal ? min(ntiles - 1, (q0 + 32 * w + 31) / kTK) : ntiles - 1;

  // ---- loader state: this thread rebuilds chunk lc (8 elements) of token lt (+ TPP per pass)
  const int lt = tid / CPR, lc = tid % CPR;
  u32x4 kreg[NPASS][2], vreg[NPASS][2];  // LOAD_TPA_R2: two ranks; LOAD_DENSE: [0] only
  uint32_t kaa[NPASS], vaa[NPASS];       // LOAD_TPA_R2: packed (a0/2, a1/2) bf16 pair

  const uint16_t* kbp = static_cast<const uint16_t*>(p.kb.ptr) + b * p.kb.stride_b + 8 * lc;
  const uint16_t* vbp = static_cast<const uint16_t*>(p.vb.ptr) + b * p.vb.stride_b + 8 * lc;
  const uint16_t* kap = static_cast<const uint16_t*>(p.ka.ptr) + b * p.ka.stride_b + h;
  const uint16_t* vap = static_cast<const uint16_t*>(p.va.ptr) + b * p.va.stride_b + h;
  if constexpr (LOADER == LOAD_DENSE) {
    kbp += (int64_t)h * D;
    vbp += (int64_t)h * D;
  }

  auto issue = [&](int tile) {
    if constexpr (LOADER == LOAD_TPA_ANY) return;
#pragma unroll
    for (int ps = 0; ps < NPASS; ++ps) {
      const int tok = min(tile * kTK + ps * TPP + lt, p.lk - 1);
      if constexpr (LOADER == LOAD_TPA_R2) {
        kreg[ps][0] = *reinterpret_cast<const u32x4*>(kbp + (int64_t)tok * p.kb.stride_l);
        kreg[ps][1] = *reinterpret_cast<const u32x4*>(kbp + (int64_t)tok * p.kb.stride_l + p.kb.stride_r);
        vreg[ps][0] = *reinterpret_cast<const u32x4*>(vbp + (int64_t)tok * p.vb.stride_l);
        vreg[ps][1] = *reinterpret_cast<const u32x4*>(vbp + (int64_t)tok * p.vb.stride_l + p.vb.stride_r);
        const uint32_t ka0 = kap[(int64_t)tok * p.ka.stride_l], ka1 = kap[(int64_t)tok * p.ka.stride_l + p.ka.stride_r];
        const uint32_t va0 = vap[(int64_t)tok * p.va.stride_l], va1 = vap[(int64_t)tok * p.va.stride_l + p.va.stride_r];
        kaa[ps] = ka0 | (ka1 << 16);
        vaa[ps] = va0 | (va1 << 16);
      } else {
        kreg[ps][0] = *reinterpret_cast<const u32x4*>(kbp + (int64_t)tok * p.kb.stride_l);
        vreg[ps][0] = *reinterpret_cast<const u32x4*>(vbp + (int64_t)tok * p.vb.stride_l);
      }
    }
  };

  // a0*b0[d] + a1*b1[d] for the two elements of a dword pair, as two bf16 dot products
  auto rebuild_r2 = [&](const u32x4& b0, const u32x4& b1, uint32_t aa_bits) -> u32x4 {
    // halve the a pair (exact in bf16): 1/R with R = 2
    const float a0 = bf16lo_to_f32(aa_bits) * 0.5f, a1 = bf16hi_to_f32(aa_bits) * 0.5f;
    const bf16x2 aa = __builtin_bit_cast(bf16x2, pack_bf16(a0, a1));
    u32x4 out;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const uint32_t lo = __builtin_amdgcn_perm(b1[j], b0[j], 0x05040100u);  // (b0[d],   b1[d])
      const uint32_t hi = __builtin_amdgcn_perm(b1[j], b0[j], 0x07060302u);  // (b0[d+1], b1[d+1])
      const float x0 = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, lo), aa, 0.f, false);
      const float x1 = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, hi), aa, 0.f, false);
      out[j] = pack_bf16(x0, x1);
    }
    return out;
  };

  auto rebuild_any = [&](const uint16_t* bptr, const uint16_t* aptr, int64_t b_stride_r, int64_t a_stride_r) -> u32x4 {
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

  auto commit = [&](int tile, int stage) {
    uint16_t* ks = smem + stage * Lds<D>::kStage;
    uint16_t* vs = ks + kTK * KS;
#pragma unroll
    for (int ps = 0; ps < NPASS; ++ps) {
      const int t = ps * TPP + lt;
      u32x4 kv, vv;
      if constexpr (LOADER == LOAD_TPA_R2) {
        kv = rebuild_r2(kreg[ps][0], kreg[ps][1], kaa[ps]);
        vv = rebuild_r2(vreg[ps][0], vreg[ps][1], vaa[ps]);
      } else if constexpr (LOADER == LOAD_TPA_ANY) {
        const int tok = min(tile * kTK + t, p.lk - 1);
        kv = rebuild_any(kbp + (int64_t)tok * p.kb.stride_l, kap + (int64_t)tok * p.ka.stride_l, p.kb.stride_r, p.ka.stride_r);
        vv = rebuild_any(vbp + (int64_t)tok * p.vb.stride_l, vap + (int64_t)tok * p.va.stride_l, p.vb.stride_r, p.va.stride_r);
      } else {
        kv = kreg[ps][0];
        vv = vreg[ps][0];
      }
      *reinterpret_cast<u32x4*>(ks + t * KS + 8 * lc) = kv;
      *reinterpret_cast<u32x4*>(vs + t * VS + 8 * lc) = vv;
    }
  };

  // ---- accumulators
  f32x16 o[NDB];
#pragma unroll
  for (int db = 0; db < NDB; ++db)
#pragma unroll
    for (int v = 0; v < 16; ++v) o[db][v] = 0.f;
  float m = -INFINITY;  // running max of the raw (unscaled) logits of row qrow
  float lsum = 0.f;     // this lane's share of sum exp2(c*(s - m))

  issue(0);
  build_q();
  commit(0, 0);
  __syncthreads();

  for (int tile = 0; tile < ntiles; ++tile) {
    const int stage = tile & 1;
    if (tile + 1 < ntiles) issue(tile + 1);

    if (tile <= wave_last_tile) {
      const uint16_t* ks = smem + stage * Lds<D>::kStage;
      const uint16_t* vs = ks + kTK * KS;
      const int k0 = tile * kTK;

      // ---- S^T = K Q^T : two 32-key blocks
      f32x16 s[2];
#pragma unroll
      for (int mb = 0; mb < 2; ++mb) {
#pragma unroll
        for (int v = 0; v < 16; ++v) s[mb][v] = 0.f;
#pragma unroll
        for (int kk = 0; kk < NKS; ++kk) {
          const bf16x8 kf = *reinterpret_cast<const bf16x8*>(ks + (32 * mb + i) * KS + 16 * kk + 8 * g);
          s[mb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf, qf[kk], s[mb], 0, 0, 0);
        }
      }

      // ---- masks: keys beyond lk, and keys after the query under the causal mask
      const bool need_mask = (k0 + kTK > p.lk) || (p.causal && (k0 + kTK - 1 > q0 + 32 * w));
      if (need_mask) {
        const int limit = p.causal ? min(qrow, p.lk - 1) : p.lk - 1;  // largest visible key index
#pragma unroll
        for (int mb = 0; mb < 2; ++mb)
#pragma unroll
          for (int v = 0; v < 16; ++v) {
            const int t = k0 + 32 * mb + 8 * (v >> 2) + 4 * g + (v & 3);
            if (t > limit) s[mb][v] = -INFINITY;
          }
      }

      // ---- online softmax for row qrow (32 of its 64 logits live in this lane)
      float tmax = s[0][0];
#pragma unroll
      for (int mb = 0; mb < 2; ++mb)
#pragma unroll
        for (int v = 0; v < 16; ++v) tmax = fmaxf(tmax, s[mb][v]);
      tmax = halves_max(tmax);
      const float m_new = fmaxf(m, tmax);
      const float alpha = __builtin_amdgcn_exp2f((m - m_new) * c);
      const float mc = m_new * c;
      m = m_new;
      float psum = 0.f;
      bf16x8 pf[4];
#pragma unroll
      for (int mb = 0; mb < 2; ++mb) {
        float pv[16];
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          pv[v] = __builtin_amdgcn_exp2f(__builtin_fmaf(s[mb][v], c, -mc));
          psum += pv[v];
        }
#pragma unroll
        for (int half = 0; half < 2; ++half) {
          u32x4 pk;
#pragma unroll
          for (int j = 0; j < 4; ++j) pk[j] = pack_bf16(pv[8 * half + 2 * j], pv[8 * half + 2 * j + 1]);
          pf[2 * mb + half] = __builtin_bit_cast(bf16x8, pk);
        }
      }
      lsum = lsum * alpha + psum;
#pragma unroll
      for (int db = 0; db < NDB; ++db)
#pragma unroll
        for (int v = 0; v < 16; ++v) o[db][v] *= alpha;

      // ---- O^T += V^T P^T : k-step kk covers keys 16kk .. 16kk+15 of the tile, in the slot
      // order the S^T accumulator already has: slot (g, j) = key 16kk + 8(j/4) + 4g + j%4
      const int lp = l & 15, dhalf = (l >> 4) & 1;
#pragma unroll
      for (int kk = 0; kk < 4; ++kk) {
        const uint16_t* vrow = vs + (16 * kk + 4 * g + (lp >> 2)) * VS + 16 * dhalf + 4 * (lp & 3);
#pragma unroll
        for (int db = 0; db < NDB; ++db) {
          const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
              (s16x4 __attribute__((address_space(3)))*)(vrow + 32 * db));
          const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
              (s16x4 __attribute__((address_space(3)))*)(vrow + 8 * VS + 32 * db));
          const bf16x8 vf = __builtin_bit_cast(bf16x8, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
          o[db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf, pf[kk], o[db], 0, 0, 0);
        }
      }
    }

    if (tile + 1 < ntiles) commit(tile + 1, stage ^ 1);
    __syncthreads();
  }

  // ---- epilogue: normalise, store O[b, qrow, h, :] and LSE[b, h, qrow]
  const float ltot = halves_sum(lsum);
  const float inv = 1.f / ltot;
  if (qrow < p.lq) {
    uint16_t* op = p.o + (((int64_t)b * p.lq + qrow) * p.H + h) * D;
#pragma unroll
    for (int db = 0; db < NDB; ++db)
#pragma unroll
      for (int vq = 0; vq < 4; ++vq) {
        u32x2 pk;
        pk[0] = pack_bf16(o[db][4 * vq] * inv, o[db][4 * vq + 1] * inv);
        pk[1] = pack_bf16(o[db][4 * vq + 2] * inv, o[db][4 * vq + 3] * inv);
        *reinterpret_cast<u32x2*>(op + 32 * db + 8 * vq + 4 * g) = pk;
      }
    if (p.lse && g == 0) p.lse[((int64_t)b * p.H + h) * p.lq + qrow] = (m * c + __builtin_amdgcn_logf(ltot)) * kLn2;
  }
}

template <int D, int NW, int LOADER>
int launch_prefill(const PrefillParams& p, hipStream_t stream) {
  auto kern = prefill_kernel<D, NW, LOADER>;
  static bool configured = false;  // idempotent attribute; a race only repeats the same call
  if (!configured) {
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)Lds<D>::kBytes) != hipSuccess)
      return TPA_ERR_LAUNCH;
    configured = true;
  }
  const int groups = (p.npairs + 7) / 8;
  dim3 grid(groups * 8 * p.H);
  hipLaunchKernelGGL(kern, grid, dim3(NW * 64), Lds<D>::kBytes, stream, p);
  return hipGetLastError() == hipSuccess ? TPA_OK : TPA_ERR_LAUNCH;
}

bool aligned16(const void* ptr) { return (reinterpret_cast<uintptr_t>(ptr) & 15) == 0; }
bool factor_ok(const TpaFactor& f) {
  return aligned16(f.ptr) && f.stride_b % 8 == 0 && f.stride_l % 8 == 0 && f.stride_r % 8 == 0;
}

constexpr int kNW = 8;

}  // namespace
}  // namespace tpa

int tpa_prefill_mfma_supported(const TpaFwdArgs* a) {
  if (a->dtype != TPA_DTYPE_BF16) return 0;
  if (a->dk != a->dv || (a->dk != 64 && a->dk != 128)) return 0;
  if (a->q_segment_ids || a->kv_segment_ids) return 0;
  if (!(a->sm_scale > 0.f)) return 0;
  if (!tpa::factor_ok(a->qb) || !tpa::factor_ok(a->kb) || !tpa::factor_ok(a->vb)) return 0;
  if (!tpa::aligned16(a->o)) return 0;
  return 1;
}

int tpa_prefill_mfma_launch(const TpaFwdArgs* a, hipStream_t stream) {
  using namespace tpa;
  PrefillParams p{};
  p.qa = a->qa; p.qb = a->qb; p.ka = a->ka; p.kb = a->kb; p.va = a->va; p.vb = a->vb;
  p.o = static_cast<uint16_t*>(a->o); p.lse = a->lse;
  p.B = a->B; p.lq = a->lq; p.lk = a->lk; p.H = a->H; p.rq = a->rq; p.rk = a->rk;
  p.sm_scale = a->sm_scale; p.causal = a->causal;
  p.nqb = (a->lq + kNW * 32 - 1) / (kNW * 32);
  p.npairs = p.nqb * a->B;
  if (a->dk == 128) {
    if (a->rk == 2) return launch_prefill<128, kNW, LOAD_TPA_R2>(p, stream);
    return launch_prefill<128, kNW, LOAD_TPA_ANY>(p, stream);
  }
  if (a->rk == 2) return launch_prefill<64, kNW, LOAD_TPA_R2>(p, stream);
  return launch_prefill<64, kNW, LOAD_TPA_ANY>(p, stream);
}

int mha_prefill_mfma_supported(const MhaFwdArgs* a) {
  if (a->dtype != TPA_DTYPE_BF16) return 0;
  if (a->dk != a->dv || (a->dk != 64 && a->dk != 128)) return 0;
  if (a->bias) return 0;
  if (!(a->sm_scale > 0.f)) return 0;
  if (!tpa::aligned16(a->q) || !tpa::aligned16(a->k) || !tpa::aligned16(a->v) || !tpa::aligned16(a->o)) return 0;
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
  p.sm_scale = a->sm_scale; p.causal = a->causal;
  p.nqb = (a->lq + kNW * 32 - 1) / (kNW * 32);
  p.npairs = p.nqb * a->B;
  if (a->dk == 128) return launch_prefill<128, kNW, LOAD_DENSE>(p, stream);
  return launch_prefill<64, kNW, LOAD_DENSE>(p, stream);
}
