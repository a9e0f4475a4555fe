"""tpa_decode_noalloc (the entry point that allocates nothing: split partials in a fixed device
array inside the library) against tpa_decode (partials in a caller workspace), through the C ABI.

Both entry points run the same kernels with the same key ranges, so the outputs must be
bit-identical.  Two calls in a row, the second with a smaller problem: the array keeps the first
call's partials, which the second call must not pick up.  The first call's result is also held
against the CPU oracle (bf16 outputs <= 2e-2, logsumexp <= 1e-3).
"""

import ctypes

import numpy as np
import pytest
import torch

from conftest import make_factors
from oracle import tpa_oracle as orc
from tpa import _dispatch as _d

pytestmark = pytest.mark.gpu

SCRATCH_BYTES = 8 << 20  # TPA_DECODE_NOALLOC_SCRATCH_BYTES in include/tpa_abi.h


def _problem(gpu, seed, b, lq, lk, h, d, rq, rk, dtype):
    q, k, v = make_factors(seed, b, lq, lk, h, d, d, rq, rk, scale_by_rank=True)
    tq, tk, tv = (torch.from_numpy(x).to(dtype).to(gpu) for x in (q, k, v))
    parts = [t[..., :h].contiguous() for t in (tq, tk, tv)] + [t[..., h:].contiguous() for t in (tq, tk, tv)]
    qa, ka, va, qb, kb, vb = parts
    return (tq, tk, tv), (qa, qb, ka, kb, va, vb)


def _args(fs, o, lse, b, lq, lk, h, d, rq, rk, dtype, sm_scale, causal, workspace):
    qa, qb, ka, kb, va, vb = fs
    return _d.TpaFwdArgs(
        qa=_d.factor(qa), qb=_d.factor(qb), ka=_d.factor(ka), kb=_d.factor(kb), va=_d.factor(va), vb=_d.factor(vb),
        q_segment_ids=None, kv_segment_ids=None, o=o.data_ptr(), lse=lse.data_ptr(),
        B=b, lq=lq, lk=lk, H=h, dk=d, dv=d, rq=rq, rk=rk,
        dtype=_d.dtype_code(dtype), sm_scale=float(sm_scale), causal=int(causal), kernel=_d.KERNEL_MFMA,
        workspace=None if workspace is None else workspace.data_ptr(),
        workspace_bytes=0 if workspace is None else workspace.numel(),
        num_splits=0, kv_lengths=None, page_table=None, page_size=0, pages_per_seq=0,
        causal_offset=lk - lq if causal else 0,
    )


def _both(gpu, lib, seed, b, lq, lk, h, d, rq, rk, dtype, causal=False):
    """Run tpa_decode and tpa_decode_noalloc on the same inputs; returns (inputs, o, lse) of the latter."""
    full, fs = _problem(gpu, seed, b, lq, lk, h, d, rq, rk, dtype)
    sm_scale = d**-0.5
    stream = _d.current_stream_ptr(gpu)
    need = lib.tpa_decode_workspace_bytes(b, lq, lk, h, d, 0)
    assert need <= SCRATCH_BYTES
    ws = torch.empty(need, dtype=torch.uint8, device=gpu)
    o_ref = torch.empty((b, lq, h, d), dtype=dtype, device=gpu)
    lse_ref = torch.empty((b, h, lq), dtype=torch.float32, device=gpu)
    a = _args(fs, o_ref, lse_ref, b, lq, lk, h, d, rq, rk, dtype, sm_scale, causal, ws)
    assert lib.tpa_decode(ctypes.byref(a), stream) == 0
    # outputs start as NaN patterns so that an entry the call does not write cannot pass
    o = torch.full((b, lq, h, d), float("nan"), dtype=dtype, device=gpu)
    lse = torch.full((b, h, lq), float("nan"), dtype=torch.float32, device=gpu)
    a2 = _args(fs, o, lse, b, lq, lk, h, d, rq, rk, dtype, sm_scale, causal, None)
    assert lib.tpa_decode_noalloc(ctypes.byref(a2), stream) == 0
    torch.cuda.synchronize()
    assert torch.equal(o.view(torch.int16 if dtype == torch.bfloat16 else torch.int32),
                       o_ref.view(torch.int16 if dtype == torch.bfloat16 else torch.int32))
    assert torch.equal(lse.view(torch.int32), lse_ref.view(torch.int32))
    return full, o, lse, sm_scale


def test_noalloc_decode_matches_workspace_decode_twice_in_a_row(gpu):
    lib = _d.load_library()
    h, d, rq, rk = 32, 128, 6, 2
    # first call: 16 sequences of 4096 cached tokens; second call: fewer, shorter sequences and a
    # different number of key ranges, over the array the first call left behind
    (tq, tk, tv), o, lse, sm_scale = _both(gpu, lib, 1, 16, 1, 4096, h, d, rq, rk, torch.bfloat16)
    f64 = lambda t: t.float().cpu().numpy().astype(np.float64)
    o_want, l_want = orc.tpa_reference(f64(tq), f64(tk), f64(tv), None, None, h, sm_scale=sm_scale)
    assert np.abs(f64(o) - o_want).max() <= 2e-2
    assert np.abs(f64(lse).transpose(0, 2, 1) - l_want).max() <= 1e-3
    (tq, tk, tv), o, lse, sm_scale = _both(gpu, lib, 2, 3, 1, 1100, h, d, rq, rk, torch.bfloat16)
    o_want, l_want = orc.tpa_reference(f64(tq), f64(tk), f64(tv), None, None, h, sm_scale=sm_scale)
    assert np.abs(f64(o) - o_want).max() <= 2e-2
    assert np.abs(f64(lse).transpose(0, 2, 1) - l_want).max() <= 1e-3


def test_noalloc_decode_other_instances(gpu):
    lib = _d.load_library()
    # two appended query tokens masked to their predecessors, head size 64, rank 4; then an fp32 cache
    _both(gpu, lib, 3, 4, 2, 2048, 16, 64, 3, 4, torch.bfloat16, causal=True)
    _both(gpu, lib, 4, 2, 1, 1500, 8, 64, 2, 2, torch.float32)
    _both(gpu, lib, 5, 1, 1, 300, 8, 64, 2, 2, torch.float32)


def test_noalloc_decode_refuses_what_does_not_fit(gpu):
    lib = _d.load_library()
    b, lq, lk, h, d, rq, rk = 64, 8, 8192, 32, 128, 6, 2  # partials of 8 query rows: beyond the fixed array
    assert lib.tpa_decode_workspace_bytes(b, lq, lk, h, d, 0) > SCRATCH_BYTES
    z = lambda *s: torch.zeros(s, dtype=torch.bfloat16, device=gpu)
    fs = (z(b, lq, rq, h), z(b, lq, rq, d), z(b, lk, rk, h), z(b, lk, rk, d), z(b, lk, rk, h), z(b, lk, rk, d))
    o = torch.zeros((b, lq, h, d), dtype=torch.bfloat16, device=gpu)
    lse = torch.zeros((b, h, lq), dtype=torch.float32, device=gpu)
    a = _args(fs, o, lse, b, lq, lk, h, d, rq, rk, torch.bfloat16, 1.0, False, None)
    assert lib.tpa_decode_noalloc(ctypes.byref(a), _d.current_stream_ptr(gpu)) == -5  # TPA_ERR_WORKSPACE
    # a head size the split-key kernels do not take: refused, not served by another kernel
    fs2 = (fs[0][:1, :1], fs[1][:1, :1, :, :48].contiguous(), fs[2][:1, :64], fs[3][:1, :64, :, :48].contiguous(),
           fs[4][:1, :64], fs[5][:1, :64, :, :48].contiguous())
    a = _args(fs2, o, lse, 1, 1, 64, h, 48, rq, rk, torch.bfloat16, 1.0, False, None)
    assert lib.tpa_decode_noalloc(ctypes.byref(a), _d.current_stream_ptr(gpu)) == -6  # TPA_ERR_UNSUPPORTED
    torch.cuda.synchronize()
