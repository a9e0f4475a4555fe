// XLA FFI handlers over the C ABI of libtpa_gfx950.so, for use from jax on ROCm:
//   jax.ffi.register_ffi_target("tpa_gfx950_TpaFwd", jax.ffi.pycapsule(lib.TpaFwd), platform="ROCM")
// These replace the pl.pallas_call of _fwd (tpa/tpa.py:492-543) and the jax.vmap around it
// (tpa/tpa.py:144-163): the operands are the reference's concatenated q[b,lq,rq,h+dk],
// k[b,lk,rk,h+dk], v[b,lk,rk,h+dv], read in place through strides.
//
// Not part of `make`: it needs the XLA FFI headers (python -c "import jax; print(jax.ffi.include_dir())").
// SOURCE ONLY: no XLA headers exist where this library is built and tested, so this file has never
// been through a compiler; every tested path binds the C ABI directly.
#include <hip/hip_runtime.h>

#include <cstdint>
#include <string>

#include "tpa_abi.h"
#include "xla/ffi/api/ffi.h"

namespace ffi = xla::ffi;

namespace {

int dtype_code(ffi::DataType t) {
  switch (t) {
    case ffi::DataType::F32: return TPA_DTYPE_F32;
    case ffi::DataType::BF16: return TPA_DTYPE_BF16;
    default: return -1;
  }
}

size_t elem_bytes(int code) { return code == TPA_DTYPE_F32 ? 4 : 2; }

// A / B factor views of a concatenated [b, l, r, h + d] buffer
void split(const ffi::AnyBuffer& x, int h, int code, TpaFactor* a, TpaFactor* b) {
  const auto d = x.dimensions();
  const int64_t sr = d[3], sl = d[2] * sr, sb = d[1] * sl;
  const char* base = static_cast<const char*>(x.untyped_data());
  *a = TpaFactor{base, sb, sl, sr};
  *b = TpaFactor{base + (size_t)h * elem_bytes(code), sb, sl, sr};
}

ffi::Error fail(int rc) { return ffi::Error::InvalidArgument(std::string("libtpa_gfx950: ") + tpa_strerror(rc)); }

ffi::Error fill(TpaFwdArgs* a, const ffi::AnyBuffer& q, const ffi::AnyBuffer& k, const ffi::AnyBuffer& v,
                ffi::Result<ffi::AnyBuffer>& o, ffi::Result<ffi::AnyBuffer>& lse, int32_t num_heads, float sm_scale,
                bool causal) {
  const auto qd = q.dimensions(), kd = k.dimensions(), vd = v.dimensions();
  if (qd.size() != 4 || kd.size() != 4 || vd.size() != 4) return ffi::Error::InvalidArgument("q, k, v must be [b, l, r, h+d]");
  const int code = dtype_code(q.element_type());
  if (code < 0 || k.element_type() != q.element_type() || v.element_type() != q.element_type())
    return ffi::Error::InvalidArgument("q, k, v must share one of f32 / bf16");
  // shape rules of tpa/tpa.py:475
  if (kd[0] != qd[0] || vd[0] != qd[0] || kd[1] != vd[1] || kd[2] != vd[2] || kd[3] != qd[3] || num_heads <= 0 ||
      qd[3] <= num_heads || vd[3] <= num_heads)
    return ffi::Error::InvalidArgument("inconsistent q / k / v shapes");
  // results: o[b, lq, h, dv] in the input type, lse[b, h, lq] fp32 (NOT the reference's l[b, lq, h] in
  // the input type, tpa/tpa.py:530: a caller that declares that shape for bf16 would be written past)
  const auto od = o->dimensions(), ld = lse->dimensions();
  if (o->element_type() != q.element_type() || od.size() != 4 || od[0] != qd[0] || od[1] != qd[1] || od[2] != num_heads ||
      od[3] != vd[3] - num_heads)
    return ffi::Error::InvalidArgument("o must be [b, lq, h, dv] in the type of q");
  if (lse->element_type() != ffi::DataType::F32 || ld.size() != 3 || ld[0] != qd[0] || ld[1] != num_heads || ld[2] != qd[1])
    return ffi::Error::InvalidArgument("lse must be f32 [b, h, lq]");
  *a = TpaFwdArgs{};
  split(q, num_heads, code, &a->qa, &a->qb);
  split(k, num_heads, code, &a->ka, &a->kb);
  split(v, num_heads, code, &a->va, &a->vb);
  a->o = o->untyped_data();
  a->lse = static_cast<float*>(lse->untyped_data());
  a->B = (int32_t)qd[0]; a->lq = (int32_t)qd[1]; a->lk = (int32_t)kd[1]; a->H = num_heads;
  a->dk = (int32_t)qd[3] - num_heads; a->dv = (int32_t)vd[3] - num_heads;
  a->rq = (int32_t)qd[2]; a->rk = (int32_t)kd[2];
  a->dtype = code; a->sm_scale = sm_scale; a->causal = causal ? 1 : 0; a->kernel = TPA_KERNEL_AUTO;
  return ffi::Error::Success();
}

// workspace: an extra u8 result of max(tpa_fwd_workspace_bytes(...), 1) bytes allocated by XLA (256-byte aligned,
// as XLA's buffers are), with which tpa_fwd picks the split-key decode kernel or the dense-K/V route where
// they are faster; a one-byte buffer keeps every call on the fused prefill kernel.  `nomat` is the reference's
// static of that name (tpa/tpa.py:250): the evaluation order that never forms K or V, which needs the
// workspace of tpa_fwd_nomat_workspace_bytes(...) instead.
void attach_workspace(TpaFwdArgs* a, ffi::Result<ffi::AnyBuffer>& workspace, bool nomat) {
  a->nomat = nomat ? 1 : 0;
  const size_t need = nomat ? tpa_fwd_nomat_workspace_bytes(a->B, a->lq, a->lk, a->H, a->dk, a->dv, a->rq, a->rk)
                            : tpa_fwd_workspace_bytes(a->B, a->lq, a->lk, a->H, a->dk, a->dv, a->rq, a->rk);
  if (need && workspace->size_bytes() >= need) {
    a->workspace = workspace->untyped_data();
    a->workspace_bytes = workspace->size_bytes();
  }
}

bool seg_ok(const ffi::Buffer<ffi::DataType::S32>& ids, int64_t b, int64_t l) {
  const auto d = ids.dimensions();
  return d.size() == 2 && d[0] == b && d[1] == l;
}

ffi::Error TpaFwdImpl(hipStream_t stream, ffi::AnyBuffer q, ffi::AnyBuffer k, ffi::AnyBuffer v,
                      ffi::Result<ffi::AnyBuffer> o, ffi::Result<ffi::AnyBuffer> lse,
                      ffi::Result<ffi::AnyBuffer> workspace, int32_t num_heads, float sm_scale, bool causal, bool nomat) {
  TpaFwdArgs a;
  if (ffi::Error e = fill(&a, q, k, v, o, lse, num_heads, sm_scale, causal); e.failure()) return e;
  attach_workspace(&a, workspace, nomat);
  const int rc = tpa_fwd(&a, stream);
  return rc == TPA_OK ? ffi::Error::Success() : fail(rc);
}

ffi::Error TpaFwdSegImpl(hipStream_t stream, ffi::AnyBuffer q, ffi::AnyBuffer k, ffi::AnyBuffer v,
                         ffi::Buffer<ffi::DataType::S32> q_segment_ids, ffi::Buffer<ffi::DataType::S32> kv_segment_ids,
                         ffi::Result<ffi::AnyBuffer> o, ffi::Result<ffi::AnyBuffer> lse,
                         ffi::Result<ffi::AnyBuffer> workspace, int32_t num_heads, float sm_scale, bool causal, bool nomat) {
  TpaFwdArgs a;
  if (ffi::Error e = fill(&a, q, k, v, o, lse, num_heads, sm_scale, causal); e.failure()) return e;
  if (!seg_ok(q_segment_ids, a.B, a.lq) || !seg_ok(kv_segment_ids, a.B, a.lk))
    return ffi::Error::InvalidArgument("segment ids must be s32 [b, lq] and [b, lk]");
  attach_workspace(&a, workspace, nomat);
  a.q_segment_ids = q_segment_ids.typed_data();
  a.kv_segment_ids = kv_segment_ids.typed_data();
  const int rc = tpa_fwd(&a, stream);
  return rc == TPA_OK ? ffi::Error::Success() : fail(rc);
}

// workspace: an extra u8 result of tpa_decode_workspace_bytes(...) bytes, allocated by XLA
ffi::Error TpaDecodeImpl(hipStream_t stream, ffi::AnyBuffer q, ffi::AnyBuffer k, ffi::AnyBuffer v,
                         ffi::Result<ffi::AnyBuffer> o, ffi::Result<ffi::AnyBuffer> lse,
                         ffi::Result<ffi::AnyBuffer> workspace, int32_t num_heads, float sm_scale) {
  TpaFwdArgs a;
  if (ffi::Error e = fill(&a, q, k, v, o, lse, num_heads, sm_scale, false); e.failure()) return e;
  a.workspace = workspace->untyped_data();
  a.workspace_bytes = workspace->size_bytes();
  const int rc = tpa_decode(&a, stream);
  return rc == TPA_OK ? ffi::Error::Success() : fail(rc);
}

// dense q[b,lq,h,dk] k[b,lk,h,dk] v[b,lk,h,dv] (tpa/mha.py:11-17); causal instead of a dense bias
ffi::Error MhaFwdImpl(hipStream_t stream, ffi::AnyBuffer q, ffi::AnyBuffer k, ffi::AnyBuffer v,
                      ffi::Result<ffi::AnyBuffer> o, ffi::Result<ffi::AnyBuffer> lse,
                      ffi::Result<ffi::AnyBuffer> workspace, float sm_scale, bool causal) {
  const auto qd = q.dimensions(), kd = k.dimensions(), vd = v.dimensions();
  if (qd.size() != 4 || kd.size() != 4 || vd.size() != 4) return ffi::Error::InvalidArgument("q, k, v must be [b, l, h, d]");
  const auto od = o->dimensions(), ld = lse->dimensions();
  if (k.element_type() != q.element_type() || v.element_type() != q.element_type() || o->element_type() != q.element_type() ||
      od.size() != 4 || od[0] != qd[0] || od[1] != qd[1] || od[2] != qd[2] || od[3] != vd[3])
    return ffi::Error::InvalidArgument("q, k, v, o must share one type; o is [b, lq, h, dv]");
  if (lse->element_type() != ffi::DataType::F32 || ld.size() != 3 || ld[0] != qd[0] || ld[1] != qd[2] || ld[2] != qd[1])
    return ffi::Error::InvalidArgument("lse must be f32 [b, h, lq]");
  MhaFwdArgs a{};
  a.q = q.untyped_data(); a.k = k.untyped_data(); a.v = v.untyped_data();
  a.o = o->untyped_data(); a.lse = static_cast<float*>(lse->untyped_data());
  a.B = (int32_t)qd[0]; a.lq = (int32_t)qd[1]; a.lk = (int32_t)kd[1]; a.H = (int32_t)qd[2];
  a.dk = (int32_t)qd[3]; a.dv = (int32_t)vd[3];
  a.dtype = dtype_code(q.element_type());
  a.sm_scale = sm_scale; a.causal = causal ? 1 : 0; a.kernel = TPA_KERNEL_AUTO;
  a.workspace = workspace->untyped_data(); a.workspace_bytes = workspace->size_bytes();
  const int rc = mha_fwd(&a, stream);
  return rc == TPA_OK ? ffi::Error::Success() : fail(rc);
}

// Backward (replaces _tpa_bwd, tpa/tpa.py:168-214): operands q, k, v, o, lse[b, h, lq] (fp32, as
// TpaFwd returned it) and do; results dq, dk, dv as fp32 arrays shaped like q, k, v, plus a u8
// workspace of tpa_bwd_workspace_bytes(...) bytes that XLA allocates (256-byte aligned, as XLA's
// buffers are).  Segment ids, when used, are two more operands (TpaBwdSeg).
void split_grad(ffi::Result<ffi::AnyBuffer>& x, int h, TpaGrad* a, TpaGrad* b) {
  const auto d = x->dimensions();
  const int64_t sr = d[3], sl = d[2] * sr, sb = d[1] * sl;
  float* base = static_cast<float*>(x->untyped_data());
  *a = TpaGrad{base, sb, sl, sr};
  *b = TpaGrad{base + h, sb, sl, sr};
}

ffi::Error TpaBwdCommon(hipStream_t stream, const ffi::AnyBuffer& q, const ffi::AnyBuffer& k, const ffi::AnyBuffer& v,
                        const int32_t* qseg, const int32_t* kvseg, const ffi::AnyBuffer& o, const ffi::AnyBuffer& lse,
                        const ffi::AnyBuffer& d_o, ffi::Result<ffi::AnyBuffer>& dq, ffi::Result<ffi::AnyBuffer>& dk,
                        ffi::Result<ffi::AnyBuffer>& dv, ffi::Result<ffi::AnyBuffer>& workspace, int32_t num_heads,
                        float sm_scale, bool causal) {
  const auto qd = q.dimensions(), kd = k.dimensions(), vd = v.dimensions();
  if (qd.size() != 4 || kd.size() != 4 || vd.size() != 4) return ffi::Error::InvalidArgument("q, k, v must be [b, l, r, h+d]");
  const int code = dtype_code(q.element_type());
  if (code < 0 || k.element_type() != q.element_type() || v.element_type() != q.element_type() ||
      o.element_type() != q.element_type() || d_o.element_type() != q.element_type())
    return ffi::Error::InvalidArgument("q, k, v, o, do must share one of f32 / bf16");
  if (lse.element_type() != ffi::DataType::F32 || dq->element_type() != ffi::DataType::F32 ||
      dk->element_type() != ffi::DataType::F32 || dv->element_type() != ffi::DataType::F32)
    return ffi::Error::InvalidArgument("lse and the gradients are f32");
  const auto ld = lse.dimensions();
  if (ld.size() != 3 || ld[0] != qd[0] || ld[1] != num_heads || ld[2] != qd[1]) return ffi::Error::InvalidArgument("lse must be [b, h, lq]");
  if (dq->dimensions() != qd || dk->dimensions() != kd || dv->dimensions() != vd || o.dimensions() != d_o.dimensions())
    return ffi::Error::InvalidArgument("gradients are shaped like q, k, v; do like o");
  TpaBwdArgs a{};
  split(q, num_heads, code, &a.qa, &a.qb);
  split(k, num_heads, code, &a.ka, &a.kb);
  split(v, num_heads, code, &a.va, &a.vb);
  split_grad(dq, num_heads, &a.dqa, &a.dqb);
  split_grad(dk, num_heads, &a.dka, &a.dkb);
  split_grad(dv, num_heads, &a.dva, &a.dvb);
  a.q_segment_ids = qseg; a.kv_segment_ids = kvseg;
  a.o = o.untyped_data(); a.lse = static_cast<const float*>(lse.untyped_data()); a.d_o = d_o.untyped_data();
  a.B = (int32_t)qd[0]; a.lq = (int32_t)qd[1]; a.lk = (int32_t)kd[1]; a.H = num_heads;
  a.dk = (int32_t)qd[3] - num_heads; a.dv = (int32_t)vd[3] - num_heads;
  a.rq = (int32_t)qd[2]; a.rk = (int32_t)kd[2];
  a.dtype = code; a.sm_scale = sm_scale; a.causal = causal ? 1 : 0; a.kernel = TPA_KERNEL_AUTO;
  a.workspace = workspace->untyped_data(); a.workspace_bytes = workspace->size_bytes();
  const int rc = tpa_bwd(&a, stream);
  return rc == TPA_OK ? ffi::Error::Success() : fail(rc);
}

ffi::Error TpaBwdImpl(hipStream_t stream, ffi::AnyBuffer q, ffi::AnyBuffer k, ffi::AnyBuffer v, ffi::AnyBuffer o,
                      ffi::AnyBuffer lse, ffi::AnyBuffer d_o, ffi::Result<ffi::AnyBuffer> dq, ffi::Result<ffi::AnyBuffer> dk,
                      ffi::Result<ffi::AnyBuffer> dv, ffi::Result<ffi::AnyBuffer> workspace, int32_t num_heads,
                      float sm_scale, bool causal) {
  return TpaBwdCommon(stream, q, k, v, nullptr, nullptr, o, lse, d_o, dq, dk, dv, workspace, num_heads, sm_scale, causal);
}

ffi::Error TpaBwdSegImpl(hipStream_t stream, ffi::AnyBuffer q, ffi::AnyBuffer k, ffi::AnyBuffer v,
                         ffi::Buffer<ffi::DataType::S32> q_segment_ids, ffi::Buffer<ffi::DataType::S32> kv_segment_ids,
                         ffi::AnyBuffer o, ffi::AnyBuffer lse, ffi::AnyBuffer d_o, ffi::Result<ffi::AnyBuffer> dq,
                         ffi::Result<ffi::AnyBuffer> dk, ffi::Result<ffi::AnyBuffer> dv,
                         ffi::Result<ffi::AnyBuffer> workspace, int32_t num_heads, float sm_scale, bool causal) {
  const auto qd = q.dimensions(), kd = k.dimensions();
  if (qd.size() != 4 || kd.size() != 4 || !seg_ok(q_segment_ids, qd[0], qd[1]) || !seg_ok(kv_segment_ids, kd[0], kd[1]))
    return ffi::Error::InvalidArgument("segment ids must be s32 [b, lq] and [b, lk]");
  return TpaBwdCommon(stream, q, k, v, q_segment_ids.typed_data(), kv_segment_ids.typed_data(), o, lse, d_o, dq, dk, dv,
                      workspace, num_heads, sm_scale, causal);
}

}  // namespace

XLA_FFI_DEFINE_HANDLER_SYMBOL(TpaBwd, TpaBwdImpl,
                              ffi::Ffi::Bind()
                                  .Ctx<ffi::PlatformStream<hipStream_t>>()
                                  .Arg<ffi::AnyBuffer>().Arg<ffi::AnyBuffer>().Arg<ffi::AnyBuffer>()
                                  .Arg<ffi::AnyBuffer>().Arg<ffi::AnyBuffer>().Arg<ffi::AnyBuffer>()
                                  .Ret<ffi::AnyBuffer>().Ret<ffi::AnyBuffer>().Ret<ffi::AnyBuffer>().Ret<ffi::AnyBuffer>()
                                  .Attr<int32_t>("num_heads").Attr<float>("sm_scale").Attr<bool>("causal"));

XLA_FFI_DEFINE_HANDLER_SYMBOL(TpaBwdSeg, TpaBwdSegImpl,
                              ffi::Ffi::Bind()
                                  .Ctx<ffi::PlatformStream<hipStream_t>>()
                                  .Arg<ffi::AnyBuffer>().Arg<ffi::AnyBuffer>().Arg<ffi::AnyBuffer>()
                                  .Arg<ffi::Buffer<ffi::DataType::S32>>().Arg<ffi::Buffer<ffi::DataType::S32>>()
                                  .Arg<ffi::AnyBuffer>().Arg<ffi::AnyBuffer>().Arg<ffi::AnyBuffer>()
                                  .Ret<ffi::AnyBuffer>().Ret<ffi::AnyBuffer>().Ret<ffi::AnyBuffer>().Ret<ffi::AnyBuffer>()
                                  .Attr<int32_t>("num_heads").Attr<float>("sm_scale").Attr<bool>("causal"));

XLA_FFI_DEFINE_HANDLER_SYMBOL(TpaFwd, TpaFwdImpl,
                              ffi::Ffi::Bind()
                                  .Ctx<ffi::PlatformStream<hipStream_t>>()
                                  .Arg<ffi::AnyBuffer>().Arg<ffi::AnyBuffer>().Arg<ffi::AnyBuffer>()
                                  .Ret<ffi::AnyBuffer>().Ret<ffi::AnyBuffer>().Ret<ffi::AnyBuffer>()
                                  .Attr<int32_t>("num_heads").Attr<float>("sm_scale").Attr<bool>("causal").Attr<bool>("nomat"));

XLA_FFI_DEFINE_HANDLER_SYMBOL(TpaFwdSeg, TpaFwdSegImpl,
                              ffi::Ffi::Bind()
                                  .Ctx<ffi::PlatformStream<hipStream_t>>()
                                  .Arg<ffi::AnyBuffer>().Arg<ffi::AnyBuffer>().Arg<ffi::AnyBuffer>()
                                  .Arg<ffi::Buffer<ffi::DataType::S32>>().Arg<ffi::Buffer<ffi::DataType::S32>>()
                                  .Ret<ffi::AnyBuffer>().Ret<ffi::AnyBuffer>().Ret<ffi::AnyBuffer>()
                                  .Attr<int32_t>("num_heads").Attr<float>("sm_scale").Attr<bool>("causal").Attr<bool>("nomat"));

XLA_FFI_DEFINE_HANDLER_SYMBOL(TpaDecode, TpaDecodeImpl,
                              ffi::Ffi::Bind()
                                  .Ctx<ffi::PlatformStream<hipStream_t>>()
                                  .Arg<ffi::AnyBuffer>().Arg<ffi::AnyBuffer>().Arg<ffi::AnyBuffer>()
                                  .Ret<ffi::AnyBuffer>().Ret<ffi::AnyBuffer>().Ret<ffi::AnyBuffer>()
                                  .Attr<int32_t>("num_heads").Attr<float>("sm_scale"));

XLA_FFI_DEFINE_HANDLER_SYMBOL(MhaFwd, MhaFwdImpl,
                              ffi::Ffi::Bind()
                                  .Ctx<ffi::PlatformStream<hipStream_t>>()
                                  .Arg<ffi::AnyBuffer>().Arg<ffi::AnyBuffer>().Arg<ffi::AnyBuffer>()
                                  .Ret<ffi::AnyBuffer>().Ret<ffi::AnyBuffer>().Ret<ffi::AnyBuffer>()
                                  .Attr<float>("sm_scale").Attr<bool>("causal"));
