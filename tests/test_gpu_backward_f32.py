"""GPU parity of the fp32 MFMA backward kernels (fp32 inputs, head size 64 or 128) against the CPU
oracle, through tpa_bwd / mha_bwd of the C ABI.  kernel=2 makes a fall-back to the vector-ALU
kernels an error.  fp32 gradients are held to 2e-4 of the largest entry, as for the other fp32
backward path (the reference's own test uses atol 1e-3 / rtol 1e-2, tpa/tpa_test.py:128-205).
"""

import numpy as np
import pytest
import torch

from conftest import make_factors, segment_ids
from oracle import tpa_oracle as orc
from test_gpu_backward import rel_err

pytestmark = pytest.mark.gpu


def _f32_case(gpu, seed, b, lq, lk, h, d, rq, rk, seg, causal, kernel, sm_scale=None):
    from tpa import tpa

    q, k, v = make_factors(seed, b, lq, lk, h, d, d, rq, rk)
    do = np.random.default_rng(seed + 1).standard_normal((b, lq, h, d)).astype(np.float32)
    qseg = segment_ids(lq, seg, b) if seg else None
    kvseg = segment_ids(lk, seg, b) if seg else None
    scale = d**-0.5 if sm_scale is None else sm_scale
    tq, tk, tv, tdo = (torch.from_numpy(x).to(gpu) for x in (q, k, v, do))
    sp = lambda t: (t[..., :h], t[..., h:])
    tqs = None if qseg is None else torch.from_numpy(qseg).to(gpu)
    tks = None if kvseg is None else torch.from_numpy(kvseg).to(gpu)
    o, lse = tpa.tpa_factors(*sp(tq), *sp(tk), *sp(tv), tqs, tks, scale, causal)
    grads = tpa.tpa_factors_bwd(*sp(tq), *sp(tk), *sp(tv), tqs, tks, o, lse, tdo, scale, causal, kernel=kernel)
    want = orc.tpa_backward(q, k, v, qseg, kvseg, h, do, sm_scale=scale, causal=causal)
    got = [np.concatenate([g.cpu().numpy() for g in grads[2 * n : 2 * n + 2]], axis=-1) for n in range(3)]
    return got, want


@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize(
    "b,lq,lk,h,d,rq,rk,seg",
    [
        (2, 512, 512, 4, 128, 6, 2, None),
        (1, 300, 300, 2, 128, 2, 2, None),   # ragged last tiles and blocks
        (2, 200, 450, 2, 64, 3, 4, None),    # lq != lk
        (1, 700, 333, 2, 128, 2, 1, None),   # lq > lk, rank 1
        (2, 384, 384, 2, 64, 6, 2, 100),     # packed sequences
        (1, 640, 384, 2, 128, 2, 2, 77),     # rows whose segment has no key: no gradient from them
    ],
)
def test_backward_f32_mfma_kernels(gpu, b, lq, lk, h, d, rq, rk, seg, causal):
    got, want = _f32_case(gpu, 61, b, lq, lk, h, d, rq, rk, seg, causal, kernel=2)
    for name, g, w in zip("qkv", got, want):
        assert rel_err(g, w) <= 2e-4, name


def test_backward_f32_mfma_matches_vector_kernels(gpu):
    """Same inputs through the vector-ALU kernels (kernel=1) and the matrix-core kernels (kernel=2)."""
    a, want = _f32_case(gpu, 63, 2, 320, 448, 2, 64, 4, 2, 90, True, kernel=1)
    b_, _ = _f32_case(gpu, 63, 2, 320, 448, 2, 64, 4, 2, 90, True, kernel=2)
    for x, y, w in zip(a, b_, want):
        assert rel_err(x, w) <= 2e-4 and rel_err(y, w) <= 2e-4 and rel_err(y, x) <= 2e-4


def test_backward_f32_mfma_sharp_softmax(gpu):
    """sm_scale = 1 on N(0,1) factors: logits of order ten, probabilities that span many decades."""
    got, want = _f32_case(gpu, 65, 1, 384, 384, 2, 64, 2, 2, None, False, kernel=2, sm_scale=1.0)
    for name, g, w in zip("qkv", got, want):
        assert rel_err(g, w) <= 2e-4, name


def test_backward_f32_through_autograd_uses_the_same_path(gpu):
    """d nansum(o) through torch.autograd on tpa() with fp32 inputs of head size 64 (default kernel
    choice: the matrix-core kernels forward and backward)."""
    from tpa import tpa

    b, lq, lk, h, d = 2, 256, 320, 4, 64
    q, k, v = make_factors(67, b, lq, lk, h, d, d, 6, 2)
    qseg, kvseg = segment_ids(lq, 100, b), segment_ids(lk, 100, b)
    tq, tk, tv = (torch.from_numpy(x).to(gpu).requires_grad_() for x in (q, k, v))
    o = tpa.tpa(tq, tk, tv, num_heads=h, q_segment_ids=qseg, kv_segment_ids=kvseg, sm_scale=d**-0.5, causal=True)
    torch.nansum(o).backward()
    want = orc.tpa_backward(q, k, v, qseg, kvseg, h, np.ones((b, lq, h, d)), sm_scale=d**-0.5, causal=True)
    for name, t, w in zip("qkv", (tq, tk, tv), want):
        assert rel_err(t.grad.cpu().numpy(), w) <= 2e-4, name


@pytest.mark.parametrize("d,causal", [(64, False), (128, True)])
def test_mha_backward_f32_mfma(gpu, d, causal):
    from tpa import mha

    b, lq, lk, h = 2, 333, 290, 3
    rng = np.random.default_rng(69)
    mk = lambda *s: torch.from_numpy(rng.standard_normal(s).astype(np.float32)).to(gpu)
    q, k, v, do = mk(b, lq, h, d), mk(b, lk, h, d), mk(b, lk, h, d), mk(b, lq, h, d)
    o, res = mha._mha_fwd(q, k, v, None, d**-0.5, causal=causal)
    dq, dk, dv, _, _ = mha._mha_bwd(res, do, kernel=2)
    f64 = lambda t: t.detach().cpu().numpy().astype(np.float64)
    bias = np.where(np.tril(np.ones((lq, lk), bool)), 0.0, -np.inf)[None].repeat(b, 0) if causal else None
    want = orc.mha_backward(f64(q), f64(k), f64(v), bias, d**-0.5, f64(do))
    for t, w in zip((dq, dk, dv), want):
        assert rel_err(f64(t), w) <= 2e-4
