"""Launches in which an XCD owns many (batch, head) pairs and runs them in groups.

The dense-loader prefill kernel and the matrix-core backward kernels deal whole (batch, head) pairs
to the eight XCDs and let an XCD run its pairs a group at a time; the grid is rounded up to whole
groups, so the last group of an XCD can be short and an XCD can own fewer pairs than its neighbours.
These shapes have such remainders: pair counts that are no multiple of 8, pairs per XCD that are no
multiple of the group size.  What a pair receives must not depend on the other pairs of the launch:
a call on a subset of the heads gives the same bits, and sampled rows meet the oracle.
"""

import numpy as np
import pytest
import torch

from conftest import make_factors
from error_model import tpa_bounds
from oracle import tpa_oracle as orc
from test_gpu_parity import as_f64, run_bf16

pytestmark = pytest.mark.gpu


def _randn(gpu, seed, *shape):
    g = torch.Generator(device="cpu")
    g.manual_seed(seed)
    return torch.randn(shape, generator=g).to(gpu).to(torch.bfloat16)


def test_prefill_sampled_rows_with_a_short_last_group(gpu):
    """B=3, H=40 (120 pairs, 15 per XCD), 1536 rows = 6 query blocks: groups of 11 pairs, the second one
    holds 4; sampled rows of every batch entry, all heads, against the oracle within the per-row bounds
    of the kernels' rounding points (tests/error_model.py)."""
    b, t, h, d, scale = 3, 1536, 40, 64, 64**-0.5
    rows = np.array([0, 255, 256, 700, 1279, 1535])
    q, k, v = make_factors(5, b, t, t, h, d, d, 2, 2, scale_by_rank=True)
    (tq, tk, tv), o, lse = run_bf16(gpu, q, k, v, h, scale, True)
    for bi in range(b):
        sl = slice(bi, bi + 1)
        o_ref, l_ref = orc.tpa_reference_rows(
            as_f64(tq[sl]), as_f64(tk[sl]), as_f64(tv[sl]), None, None, h, rows, sm_scale=scale, causal=True, dtype=np.float32
        )
        lse_bound, o_bound = tpa_bounds(as_f64(tq[sl][:, rows]), as_f64(tk[sl]), as_f64(tv[sl]), h, scale)
        got = as_f64(o[sl][:, rows])
        got_l = as_f64(lse[sl][:, :, rows]).transpose(0, 2, 1)
        assert (np.abs(got - o_ref) <= o_bound[..., None]).all(), bi
        assert (np.abs(got_l - l_ref) <= lse_bound).all(), bi
        assert np.abs(got - o_ref).max() <= 2e-2


@pytest.mark.parametrize("d,causal", [(128, True), (64, False)])
def test_dense_attention_with_an_odd_pair_count(gpu, d, causal):
    """B=3, H=5: 15 pairs, the last XCD owns one pair where the others own two; forward and backward
    against the oracle."""
    from tpa import mha

    b, t, h = 3, 1300, 5
    q, k, v, do = (_randn(gpu, 70 + n, b, t, h, d) for n in range(4))
    o, res = mha._mha_fwd(q, k, v, None, d**-0.5, causal=causal)
    dq, dk, dv, _, _ = mha._mha_bwd(res, do, kernel=2)
    f64 = lambda x: x.detach().float().cpu().numpy().astype(np.float64)
    bias = np.where(np.tril(np.ones((t, t), bool)), 0.0, -np.inf)[None].repeat(b, 0) if causal else None
    o_ref, _ = orc.mha_forward(f64(q), f64(k), f64(v), bias, d**-0.5)
    assert np.abs(f64(o) - o_ref).max() <= 2e-2
    want = orc.mha_backward(f64(q), f64(k), f64(v), bias, d**-0.5, f64(do))
    for name, got, w in zip(("dq", "dk", "dv"), (dq, dk, dv), want):
        assert np.abs(f64(got) - w).max() <= 2e-2 * np.abs(w).max(), name


@pytest.mark.parametrize("d,t,causal", [(64, 2048, False), (128, 2304, True)])
def test_a_pair_does_not_depend_on_the_other_pairs_of_the_launch(gpu, d, t, causal):
    """B=3, H=40 at 8 / 9 blocks per pair: the forward runs 15 pairs per XCD in groups of 8, the backward
    kernels too (8 + 7).  The same call on eight of the heads (3 pairs per XCD, one group) must give
    identical bits for those heads: forward output, logsumexp and all three gradients."""
    from tpa import mha

    b, h, hs = 3, 40, slice(16, 24)
    q, k, v, do = (_randn(gpu, 80 + n, b, t, h, d) for n in range(4))
    o, res = mha._mha_fwd(q, k, v, None, d**-0.5, causal=causal)
    grads = mha._mha_bwd(res, do, kernel=2)[:3]
    sub = lambda x: x[:, :, hs].contiguous()
    o_s, res_s = mha._mha_fwd(sub(q), sub(k), sub(v), None, d**-0.5, causal=causal)
    grads_s = mha._mha_bwd(res_s, sub(do), kernel=2)[:3]
    assert torch.equal(o[:, :, hs], o_s)
    for name, g, g_s in zip(("dq", "dk", "dv"), grads, grads_s):
        assert torch.equal(g[:, :, hs], g_s), name
    # and the subset itself is right: a few rows of one batch entry against the oracle
    rows = np.array([0, 300, t - 1])
    f64 = lambda x: x.detach().float().cpu().numpy().astype(np.float64)
    qs, ks, vs = f64(sub(q)[1:2]), f64(sub(k)[1:2]), f64(sub(v)[1:2])
    bias = None
    if causal:
        bias = np.where(np.arange(t)[None, :] <= rows[:, None], 0.0, -np.inf)[None]
    o_ref, _ = orc.mha_forward(qs[:, rows], ks, vs, bias, d**-0.5)
    assert np.abs(f64(o_s[1:2][:, rows]) - o_ref).max() <= 2e-2
