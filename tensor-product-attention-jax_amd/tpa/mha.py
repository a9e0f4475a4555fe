"""Dense multi-head attention: the API of the reference's tpa/mha.py, as gfx950 flash kernels."""

from __future__ import annotations

import torch

from . import _dispatch as _d
from .tpa import _as_device_tensor, _pick_device

__all__ = ["mha", "_mha_fwd", "_mha_bwd"]


def _mha_fwd_impl(q, k, v, bias, sm_scale, causal, kernel):
    device = _pick_device(q, k, v)
    q, k, v = (_as_device_tensor(x, device).contiguous() for x in (q, k, v))
    if q.dtype != k.dtype or q.dtype != v.dtype:
        raise TypeError("q, k, v must share a dtype")
    b, lq, h, dk = q.shape
    _, lk, _, dv = v.shape
    assert tuple(k.shape) == (b, lk, h, dk), k.shape
    assert tuple(v.shape) == (b, lk, h, dv), v.shape
    bias_t = None
    if bias is not None:
        bias_t = _as_device_tensor(bias, device).to(torch.float32).contiguous()
        assert tuple(bias_t.shape) == (b, lq, lk), bias_t.shape
    lib = _d.load_library()
    o = torch.empty((b, lq, h, dv), dtype=q.dtype, device=device)
    lse = torch.empty((b, h, lq), dtype=torch.float32, device=device)
    need = lib.mha_fwd_workspace_bytes(b, lq, lk, h, dv, 0)
    ws = torch.empty(max(need, 16), dtype=torch.uint8, device=device)
    args = _d.MhaFwdArgs(
        q=q.data_ptr(), k=k.data_ptr(), v=v.data_ptr(),
        bias=bias_t.data_ptr() if bias_t is not None else None,
        o=o.data_ptr(), lse=lse.data_ptr(),
        B=b, lq=lq, lk=lk, H=h, dk=dk, dv=dv,
        dtype=_d.dtype_code(q.dtype), sm_scale=float(sm_scale), causal=int(bool(causal)), kernel=int(kernel),
        workspace=ws.data_ptr(), workspace_bytes=ws.numel(), num_splits=0,
    )
    with torch.cuda.device(device):
        _d.check("mha_fwd", lib.mha_fwd(args, _d.current_stream_ptr(device)))
    return o, lse, (q, k, v, bias_t)


def _mha_bwd_impl(q, k, v, bias_t, o, lse, do, sm_scale, causal, kernel=_d.KERNEL_AUTO):
    device = q.device
    b, lq, h, dk = q.shape
    _, lk, _, dv = v.shape
    do = _as_device_tensor(do, device).to(q.dtype).contiguous()
    dq = torch.empty(q.shape, dtype=torch.float32, device=device)
    dk_ = torch.empty(k.shape, dtype=torch.float32, device=device)
    dv_ = torch.empty(v.shape, dtype=torch.float32, device=device)
    lib = _d.load_library()
    need = lib.mha_bwd_workspace_bytes(b, lq, lk, h, dk, dv, _d.dtype_code(q.dtype))
    ws = torch.empty(need + 256, dtype=torch.uint8, device=device)
    pad = (-ws.data_ptr()) % 256
    args = _d.MhaBwdArgs(
        q=q.data_ptr(), k=k.data_ptr(), v=v.data_ptr(),
        bias=bias_t.data_ptr() if bias_t is not None else None,
        o=o.data_ptr(), lse=lse.data_ptr(), d_o=do.data_ptr(),
        dq=dq.data_ptr(), dk_out=dk_.data_ptr(), dv_out=dv_.data_ptr(),
        B=b, lq=lq, lk=lk, H=h, dk=dk, dv=dv,
        dtype=_d.dtype_code(q.dtype), sm_scale=float(sm_scale), causal=int(bool(causal)), kernel=int(kernel),
        workspace=ws.data_ptr() + pad, workspace_bytes=ws.numel() - pad,
    )
    with torch.cuda.device(device):
        _d.check("mha_bwd", lib.mha_bwd(args, _d.current_stream_ptr(device)))
    return dq, dk_, dv_


def _mha_fwd(q, k, v, bias, sm_scale, causal: bool = False, kernel: int = _d.KERNEL_AUTO):
    """tpa/mha.py:23-37.  q[b,lq,h,dk] k[b,lk,h,dk] v[b,lk,h,dv] bias[b,lq,lk] -> (o, residuals).

    The reference returns (p, v, q, k, sm_scale) as residuals for its backward; a flash kernel
    never forms p, so the residuals here are (lse[b,h,lq] fp32, o, q, k, v, bias, sm_scale, causal):
    what `_mha_bwd` recomputes p from.
    """
    o, lse, (q, k, v, bias_t) = _mha_fwd_impl(q, k, v, bias, sm_scale, causal, kernel)
    return o, (lse, o, q, k, v, bias_t, float(sm_scale), bool(causal))


def _mha_bwd(res, do, kernel: int = _d.KERNEL_AUTO):
    """tpa/mha.py:40-65: (dq, dk, dv, None, None) in the dtype of q, k, v.  Rows whose logits
    were all -inf contribute nothing (tpa/mha.py:52-56)."""
    lse, o, q, k, v, bias_t, sm_scale, causal = res
    dq, dk, dv = _mha_bwd_impl(q, k, v, bias_t, o, lse, do, sm_scale, causal, kernel)
    return dq.to(q.dtype), dk.to(k.dtype), dv.to(v.dtype), None, None


class _MhaFunction(torch.autograd.Function):
    """mha with its vjp, as mha.defvjp(_mha_fwd, _mha_bwd) registers it (tpa/mha.py:68)."""

    @staticmethod
    def forward(ctx, q, k, v, bias, sm_scale, causal):
        o, lse, (q_, k_, v_, bias_t) = _mha_fwd_impl(q, k, v, bias, sm_scale, causal, _d.KERNEL_AUTO)
        ctx.save_for_backward(q_, k_, v_, o, lse, *([bias_t] if bias_t is not None else []))
        ctx.statics = (float(sm_scale), bool(causal))
        return o

    @staticmethod
    def backward(ctx, do):
        q, k, v, o, lse, *rest = ctx.saved_tensors
        sm_scale, causal = ctx.statics
        dq, dk, dv = _mha_bwd_impl(q, k, v, rest[0] if rest else None, o, lse, do, sm_scale, causal)
        return dq.to(q.dtype), dk.to(k.dtype), dv.to(v.dtype), None, None, None


def mha(q, k, v, bias=None, sm_scale: float = 1, *, causal: bool = False):
    """Multi-head attention (tpa/mha.py:10-20).  `causal` is an addition: the reference passes
    causality as a dense -inf bias (tpa/tpa_test.py:52-54), which cannot exist at long lengths."""
    if isinstance(q, torch.Tensor) and q.is_cuda and torch.is_grad_enabled() and any(
        isinstance(t, torch.Tensor) and t.requires_grad for t in (q, k, v)
    ):
        return _MhaFunction.apply(q, k, v, bias, sm_scale, causal)
    o, _ = _mha_fwd(q, k, v, bias, sm_scale, causal=causal)
    return o
