// extern "C" entry points of libtpa_gfx950.so: argument validation and kernel selection.
#include "tpa_common.h"

namespace {

int check_factor(const TpaFactor& f) { return f.ptr == nullptr ? TPA_ERR_NULL : TPA_OK; }

}  // namespace

int tpa_validate_fwd_args(const TpaFwdArgs* a) {
  if (!a) return TPA_ERR_NULL;
  if (a->dtype != TPA_DTYPE_F32 && a->dtype != TPA_DTYPE_BF16) return TPA_ERR_DTYPE;
  if (a->B <= 0 || a->lq <= 0 || a->lk <= 0 || a->H <= 0 || a->dk <= 0 || a->dv <= 0 || a->rq <= 0 || a->rk <= 0)
    return TPA_ERR_SHAPE;
  if (a->dk > 256 || a->dv > 256) return TPA_ERR_SHAPE;
  const TpaFactor* fs[6] = {&a->qa, &a->qb, &a->ka, &a->kb, &a->va, &a->vb};
  for (const TpaFactor* f : fs)
    if (check_factor(*f) != TPA_OK) return TPA_ERR_NULL;
  if (!a->o) return TPA_ERR_NULL;
  // segment ids come in pairs (tpa/tpa.py:369-371)
  if ((a->q_segment_ids == nullptr) != (a->kv_segment_ids == nullptr)) return TPA_ERR_NULL;
  if (a->causal < TPA_CAUSAL_NONE || a->causal > TPA_CAUSAL_BOTTOM_RIGHT) return TPA_ERR_UNSUPPORTED;
  if (a->kernel != TPA_KERNEL_AUTO && a->kernel != TPA_KERNEL_GENERIC && a->kernel != TPA_KERNEL_MFMA)
    return TPA_ERR_UNSUPPORTED;
  return TPA_OK;
}

namespace {

int validate_mha(const MhaFwdArgs* a) {
  if (!a) return TPA_ERR_NULL;
  if (a->dtype != TPA_DTYPE_F32 && a->dtype != TPA_DTYPE_BF16) return TPA_ERR_DTYPE;
  if (a->B <= 0 || a->lq <= 0 || a->lk <= 0 || a->H <= 0 || a->dk <= 0 || a->dv <= 0) return TPA_ERR_SHAPE;
  if (a->dk > 256 || a->dv > 256) return TPA_ERR_SHAPE;
  if (!a->q || !a->k || !a->v || !a->o) return TPA_ERR_NULL;
  if (a->causal != 0 && a->causal != 1) return TPA_ERR_UNSUPPORTED;  // dense attention knows the top-left mask only
  if (a->kernel != TPA_KERNEL_AUTO && a->kernel != TPA_KERNEL_GENERIC && a->kernel != TPA_KERNEL_MFMA)
    return TPA_ERR_UNSUPPORTED;
  return TPA_OK;
}

}  // namespace

extern "C" {

int tpa_abi_version(void) { return TPA_ABI_VERSION; }

const char* tpa_strerror(int code) {
  switch (code) {
    case TPA_OK: return "ok";
    case TPA_ERR_NULL: return "a required pointer is NULL (or only one of the two segment-id arrays was given)";
    case TPA_ERR_SHAPE: return "a dimension is not positive or exceeds what the kernels support";
    case TPA_ERR_DTYPE: return "unknown dtype";
    case TPA_ERR_ALIGN: return "pointer or stride not aligned for the selected kernel";
    case TPA_ERR_WORKSPACE: return "workspace missing or too small";
    case TPA_ERR_UNSUPPORTED: return "the requested kernel cannot run this problem";
    case TPA_ERR_LAUNCH: return "the HIP runtime refused the launch";
    default: return "unknown error code";
  }
}

namespace {

constexpr int kNomatWindow = 64;  // query rows one pass of the split-key kernels serves

bool nomat_rank_and_heads(int dk, int dv, int rk) {
  return dk == dv && (dk == 64 || dk == 128) && rk >= 1 && rk <= 32 && (rk & (rk - 1)) == 0;
}

// tpa_fwd with nomat: the split-key kernels, which never form K or V, over windows of query rows.  Every window
// shares the workspace; they run one after the other on the stream.
int tpa_fwd_nomat(const TpaFwdArgs* a, hipStream_t s) {
  TpaFwdArgs w = *a;
  w.lq = a->lq < kNomatWindow ? a->lq : kNomatWindow;
  w.nomat = 0;
  const bool bf16 = a->kernel != TPA_KERNEL_GENERIC && tpa_decode_mfma_supported(&w);
  const bool f32 = a->kernel != TPA_KERNEL_GENERIC && !bf16 && tpa_decode_f32_supported(&w);
  if (!bf16 && !f32) {
    if (a->kernel == TPA_KERNEL_MFMA) return TPA_ERR_UNSUPPORTED;
    return tpa_generic_launch(a, s);
  }
  const size_t need = a->num_splits > 0 ? tpa_decode_workspace_bytes(a->B, w.lq, a->lk, a->H, a->dv, a->num_splits)
                                        : tpa_fwd_nomat_workspace_bytes(a->B, a->lq, a->lk, a->H, a->dk, a->dv, a->rq, a->rk);
  if (!a->workspace || a->workspace_bytes < need) return TPA_ERR_WORKSPACE;
  const size_t esz = a->dtype == TPA_DTYPE_BF16 ? 2 : 4;
  for (int row0 = 0; row0 < a->lq; row0 += kNomatWindow) {
    w.lq = a->lq - row0 < kNomatWindow ? a->lq - row0 : kNomatWindow;
    w.qa.ptr = static_cast<const char*>(a->qa.ptr) + (size_t)row0 * a->qa.stride_l * esz;
    w.qb.ptr = static_cast<const char*>(a->qb.ptr) + (size_t)row0 * a->qb.stride_l * esz;
    const int rc = bf16 ? tpa_decode_mfma_launch_rows(&w, s, row0, a->lq) : tpa_decode_f32_launch_rows(&w, s, row0, a->lq);
    if (rc != TPA_OK) return rc;
  }
  return TPA_OK;
}

}  // namespace

size_t tpa_fwd_nomat_workspace_bytes(int32_t B, int32_t lq, int32_t lk, int32_t H, int32_t dk, int32_t dv, int32_t rq, int32_t rk) {
  (void)rq;
  if (B <= 0 || lq <= 0 || lk <= 0 || H <= 0 || !nomat_rank_and_heads(dk, dv, rk)) return 0;
  // full windows and the last, shorter one choose their own number of key ranges
  const int full = lq < kNomatWindow ? lq : kNomatWindow, tail = lq % kNomatWindow;
  size_t need = tpa_decode_workspace_bytes(B, full, lk, H, dv, 0);
  if (lq > kNomatWindow && tail) {
    const size_t t = tpa_decode_workspace_bytes(B, tail, lk, H, dv, 0);
    if (t > need) need = t;
  }
  return need;
}

int tpa_fwd(const TpaFwdArgs* a, void* stream) {
  const int rc = tpa_validate_fwd_args(a);
  if (rc != TPA_OK) return rc;
  if (a->page_table) return TPA_ERR_UNSUPPORTED;  // paged caches are read by tpa_decode only
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (a->nomat == TPA_NOMAT_RANK_PAIRS) {
    if (a->kernel != TPA_KERNEL_GENERIC && tpa_nomat_pairs_supported(a)) return tpa_nomat_pairs_launch(a, s);
    if (a->kernel == TPA_KERNEL_MFMA) return TPA_ERR_UNSUPPORTED;
    return tpa_generic_launch(a, s);
  }
  if (a->nomat) return tpa_fwd_nomat(a, s);
  // few query tokens over a long cache (the reference's decode is this same call with lq = 1,
  // tpa/tpa.py:485): split over keys, if the caller brought the workspace for it
  if (a->kernel != TPA_KERNEL_GENERIC && a->workspace && a->lq <= 16 && a->lk >= 1024 &&
      !a->q_segment_ids && a->workspace_bytes >= tpa_decode_workspace_bytes(a->B, a->lq, a->lk, a->H, a->dv, a->num_splits)) {
    if (tpa_decode_mfma_supported(a)) return tpa_decode_mfma_launch(a, s);
    if (tpa_decode_f32_supported(a)) return tpa_decode_f32_launch(a, s);
  }
  if (a->kernel != TPA_KERNEL_GENERIC && tpa_prefill_mfma_supported(a)) return tpa_prefill_mfma_launch(a, s);
  if (a->kernel != TPA_KERNEL_GENERIC && tpa_prefill_f32_supported(a)) return tpa_prefill_f32_launch(a, s);
  if (a->kernel == TPA_KERNEL_MFMA) return TPA_ERR_UNSUPPORTED;
  return tpa_generic_launch(a, s);
}

size_t tpa_fwd_workspace_bytes(int32_t B, int32_t lq, int32_t lk, int32_t H, int32_t dk, int32_t dv, int32_t rq, int32_t rk) {
  (void)rq;
  if (B <= 0 || lq <= 0 || lk <= 0 || H <= 0 || dk <= 0 || dv <= 0 || rk <= 0) return 0;
  if (dk != dv || (dk != 64 && dk != 128)) return 0;  // the kernels that use a workspace take these head sizes only
  size_t need = 0;
  if (lq <= 16 && lk >= 1024) need = tpa_decode_workspace_bytes(B, lq, lk, H, dv, 0);
  if (tpa_prefill_wants_dense(lq, rk)) {
    const size_t dense = tpa_prefill_dense_bytes(B, lq, lk, H, dk);
    if (dense > need) need = dense;
  }
  return need;
}

int tpa_decode(const TpaFwdArgs* a, void* stream) {
  const int rc = tpa_validate_fwd_args(a);
  if (rc != TPA_OK) return rc;
  if (a->q_segment_ids) return TPA_ERR_UNSUPPORTED;
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (a->kernel != TPA_KERNEL_GENERIC && tpa_decode_mfma_supported(a)) return tpa_decode_mfma_launch(a, s);
  if (a->kernel != TPA_KERNEL_GENERIC && tpa_decode_f32_supported(a)) return tpa_decode_f32_launch(a, s);
  if (a->kernel == TPA_KERNEL_MFMA || a->page_table) return TPA_ERR_UNSUPPORTED;  // only the split-key kernel reads page pools
  return tpa_generic_launch(a, s);
}

int mha_fwd(const MhaFwdArgs* a, void* stream) {
  const int rc = validate_mha(a);
  if (rc != TPA_OK) return rc;
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (a->kernel != TPA_KERNEL_GENERIC) {
    // few query tokens over a long cache: split over keys, if the caller brought the workspace
    if (mha_decode_supported(a) && a->workspace) return mha_decode_launch(a, s);
    if (mha_prefill_mfma_supported(a)) return mha_prefill_mfma_launch(a, s);
    if (mha_prefill_f32_supported(a)) return mha_prefill_f32_launch(a, s);
  }
  if (a->kernel == TPA_KERNEL_MFMA) return TPA_ERR_UNSUPPORTED;
  return mha_generic_launch(a, s);
}

int tpa_bwd(const TpaBwdArgs* a, void* stream) {
  if (!a) return TPA_ERR_NULL;
  if (a->dtype != TPA_DTYPE_F32 && a->dtype != TPA_DTYPE_BF16) return TPA_ERR_DTYPE;
  if (a->B <= 0 || a->lq <= 0 || a->lk <= 0 || a->H <= 0 || a->dk <= 0 || a->dv <= 0 || a->rq <= 0 || a->rk <= 0)
    return TPA_ERR_SHAPE;
  if (a->dk > 256 || a->dv > 256) return TPA_ERR_SHAPE;
  const TpaFactor* fs[6] = {&a->qa, &a->qb, &a->ka, &a->kb, &a->va, &a->vb};
  for (const TpaFactor* f : fs)
    if (check_factor(*f) != TPA_OK) return TPA_ERR_NULL;
  const TpaGrad* gs[6] = {&a->dqa, &a->dqb, &a->dka, &a->dkb, &a->dva, &a->dvb};
  for (const TpaGrad* g : gs)
    if (!g->ptr) return TPA_ERR_NULL;
  if (!a->o || !a->lse || !a->d_o) return TPA_ERR_NULL;
  if ((a->q_segment_ids == nullptr) != (a->kv_segment_ids == nullptr)) return TPA_ERR_NULL;
  if (a->causal < TPA_CAUSAL_NONE || a->causal > TPA_CAUSAL_BOTTOM_RIGHT) return TPA_ERR_UNSUPPORTED;
  if (a->kernel != TPA_KERNEL_AUTO && a->kernel != TPA_KERNEL_GENERIC && a->kernel != TPA_KERNEL_MFMA)
    return TPA_ERR_UNSUPPORTED;
  // matrix-core kernels: bf16 ones for bf16 inputs, fp32 ones for fp32 inputs; both read do with 16-byte loads
  const int mfma = a->kernel != TPA_KERNEL_GENERIC &&
                   (dense_bwd_mfma_supported(a->dtype, a->dk, a->dv, a->lq, a->lk, a->H, a->sm_scale, nullptr) ||
                    dense_bwd_f32_supported(a->dtype, a->dk, a->dv, a->lq, a->lk, nullptr)) &&
                   !(reinterpret_cast<uintptr_t>(a->d_o) & 15);
  if (a->kernel == TPA_KERNEL_MFMA && !mfma) return TPA_ERR_UNSUPPORTED;
  if (!a->workspace || a->workspace_bytes < tpa_bwd_workspace_bytes(a->B, a->lq, a->lk, a->H, a->dk, a->dv))
    return TPA_ERR_WORKSPACE;
  if (reinterpret_cast<uintptr_t>(a->workspace) & 255) return TPA_ERR_ALIGN;
  return tpa_bwd_launch(a, static_cast<hipStream_t>(stream), mfma);
}

size_t tpa_bwd_workspace_bytes(int32_t B, int32_t lq, int32_t lk, int32_t H, int32_t dk, int32_t dv) {
  if (B <= 0 || lq <= 0 || lk <= 0 || H <= 0 || dk <= 0 || dv <= 0) return 0;
  return tpa_bwd_workspace_size(B, lq, lk, H, dk, dv);
}

int mha_bwd(const MhaBwdArgs* a, void* stream) {
  if (!a) return TPA_ERR_NULL;
  if (a->dtype != TPA_DTYPE_F32 && a->dtype != TPA_DTYPE_BF16) return TPA_ERR_DTYPE;
  if (a->B <= 0 || a->lq <= 0 || a->lk <= 0 || a->H <= 0 || a->dk <= 0 || a->dv <= 0) return TPA_ERR_SHAPE;
  if (a->dk > 256 || a->dv > 256) return TPA_ERR_SHAPE;
  if (!a->q || !a->k || !a->v || !a->o || !a->lse || !a->d_o || !a->dq || !a->dk_out || !a->dv_out) return TPA_ERR_NULL;
  if (a->causal != 0 && a->causal != 1) return TPA_ERR_UNSUPPORTED;  // dense attention knows the top-left mask only
  if (a->kernel != TPA_KERNEL_AUTO && a->kernel != TPA_KERNEL_GENERIC && a->kernel != TPA_KERNEL_MFMA)
    return TPA_ERR_UNSUPPORTED;
  const int mfma = a->kernel != TPA_KERNEL_GENERIC &&
                   (dense_bwd_mfma_supported(a->dtype, a->dk, a->dv, a->lq, a->lk, a->H, a->sm_scale, a->bias) ||
                    dense_bwd_f32_supported(a->dtype, a->dk, a->dv, a->lq, a->lk, a->bias)) &&
                   !(reinterpret_cast<uintptr_t>(a->q) & 15) && !(reinterpret_cast<uintptr_t>(a->k) & 15) &&
                   !(reinterpret_cast<uintptr_t>(a->v) & 15) && !(reinterpret_cast<uintptr_t>(a->d_o) & 15) &&
                   !(reinterpret_cast<uintptr_t>(a->dq) & 15) && !(reinterpret_cast<uintptr_t>(a->dk_out) & 15) &&
                   !(reinterpret_cast<uintptr_t>(a->dv_out) & 15);
  if (a->kernel == TPA_KERNEL_MFMA && !mfma) return TPA_ERR_UNSUPPORTED;
  if (!a->workspace || a->workspace_bytes < mha_bwd_workspace_bytes(a->B, a->lq, a->lk, a->H, a->dk, a->dv, a->dtype))
    return TPA_ERR_WORKSPACE;
  if (reinterpret_cast<uintptr_t>(a->workspace) & 255) return TPA_ERR_ALIGN;
  return mha_bwd_launch(a, static_cast<hipStream_t>(stream), mfma);
}

size_t mha_bwd_workspace_bytes(int32_t B, int32_t lq, int32_t lk, int32_t H, int32_t dk, int32_t dv, int32_t dtype) {
  if (B <= 0 || lq <= 0 || lk <= 0 || H <= 0 || dk <= 0 || dv <= 0) return 0;
  return mha_bwd_workspace_size(B, lq, lk, H, dk, dv, dtype);
}

}  // extern "C"
