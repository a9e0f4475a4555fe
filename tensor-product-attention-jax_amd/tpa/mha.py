"""Dense multi-head attention: the API of the reference's tpa/mha.py, as gfx950 flash kernels."""

from __future__ import annotations

import torch

from . import _dispatch as _d
from .tpa import _as_device_tensor, _pick_device

__all__ = ["mha", "_mha_fwd"]


def _mha_fwd(q, k, v, bias, sm_scale, causal: bool = False, kernel: int = _d.KERNEL_AUTO):
    """tpa/mha.py:23-37.  q[b,lq,h,dk] k[b,lk,h,dk] v[b,lk,h,dv] bias[b,lq,lk] -> (o, (lse,)).

    The reference returns (p, v, q, k, sm_scale) as residuals for its backward; a flash kernel
    never forms p, so the residual here is the logsumexp lse[b,h,lq] (fp32).
    """
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
    return o, (lse,)


def mha(q, k, v, bias=None, sm_scale: float = 1, *, causal: bool = False):
    """Multi-head attention (tpa/mha.py:10-20).  `causal` is an addition: the reference passes
    causality as a dense -inf bias (tpa/tpa_test.py:52-54), which cannot exist at long lengths."""
    o, _ = _mha_fwd(q, k, v, bias, sm_scale, causal=causal)
    return o
