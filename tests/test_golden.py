"""Committed fixtures (tests/golden/, written by tests/golden/make_golden.py).

CPU: the oracle still reproduces them, and the seeded input recipe still yields the inputs they
were computed from.  GPU: the kernels, through the C ABI, reproduce them.
"""

import os

import numpy as np
import pytest

from conftest import bf16_round, make_factors, segment_ids
from oracle import tpa_oracle as orc

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
SMALL = np.load(os.path.join(GOLDEN, "small_cases.npz"))
SAMPLED = np.load(os.path.join(GOLDEN, "sampled_rows.npz"))
SMALL_NAMES = sorted({k.split(".")[0] for k in SMALL.files if not k.startswith("upstream_mha_literal")})
SAMPLED_NAMES = sorted({k.split(".")[0] for k in SAMPLED.files})


def small_case(name):
    h, seg, causal = (int(x) for x in SMALL[f"{name}.meta"])
    q, k, v = SMALL[f"{name}.q"], SMALL[f"{name}.k"], SMALL[f"{name}.v"]
    qs = segment_ids(q.shape[1], seg, q.shape[0]) if seg else None
    ks = segment_ids(k.shape[1], seg, q.shape[0]) if seg else None
    return q, k, v, qs, ks, h, float(SMALL[f"{name}.sm_scale"]), bool(causal)


def sampled_case(name):
    seed, b, lq, lk, h, dk, dv, rq, rk, seg, causal, sbr = (int(x) for x in SAMPLED[f"{name}.recipe"])
    q, k, v = make_factors(seed, b, lq, lk, h, dk, dv, rq, rk, dist=str(SAMPLED[f"{name}.dist"]), scale_by_rank=bool(sbr))
    qs = segment_ids(lq, seg, b) if seg else None
    ks = segment_ids(lk, seg, b) if seg else None
    return q, k, v, qs, ks, h, float(SAMPLED[f"{name}.sm_scale"]), bool(causal), SAMPLED[f"{name}.rows"]


def same(a, b, tol):
    np.testing.assert_array_equal(np.isnan(a), np.isnan(b))
    np.testing.assert_array_equal(np.isneginf(a), np.isneginf(b))
    ok = np.isfinite(b)
    assert np.max(np.abs(a[ok] - b[ok]), initial=0.0) <= tol


# ------------------------------------------------------------------------------------ CPU
@pytest.mark.parametrize("name", SMALL_NAMES)
def test_oracle_reproduces_small_fixture(name):
    q, k, v, qs, ks, h, scale, causal = small_case(name)
    o, lse = orc.tpa_reference(q, k, v, qs, ks, h, sm_scale=scale, causal=causal)
    same(o, SMALL[f"{name}.o"], 1e-13)
    same(lse, SMALL[f"{name}.lse"], 1e-13)


def test_oracle_reproduces_upstream_literal():
    """tpa/mha_test.py:44-118: o = [[1, 1], [1, 1], [nan, nan]]."""
    o, _ = orc.mha_forward(SMALL["upstream_mha_literal.q"], SMALL["upstream_mha_literal.k"],
                           SMALL["upstream_mha_literal.v"], SMALL["upstream_mha_literal.bias"])
    np.testing.assert_array_equal(o, SMALL["upstream_mha_literal.o"])


@pytest.mark.parametrize("name", SAMPLED_NAMES)
def test_seed_recipe_and_oracle_reproduce_sampled_fixture(name):
    q, k, v, qs, ks, h, scale, causal, rows = sampled_case(name)
    s = sum(float(np.sum(a.astype(np.float64))) for a in (q, k, v))
    s2 = sum(float(np.sum(a.astype(np.float64) ** 2)) for a in (q, k, v))
    np.testing.assert_allclose([s, s2], SAMPLED[f"{name}.input_checksum"], rtol=1e-12)
    o, lse = orc.tpa_reference_rows(q, k, v, qs, ks, h, rows, sm_scale=scale, causal=causal)
    same(o, SAMPLED[f"{name}.o"], 1e-12)
    same(lse, SAMPLED[f"{name}.lse"], 1e-12)


# ------------------------------------------------------------------------------------ GPU
@pytest.mark.gpu
@pytest.mark.parametrize("name", SMALL_NAMES)
def test_kernel_reproduces_small_fixture(gpu, name):
    import torch
    from tpa import tpa

    q, k, v, qs, ks, h, scale, causal = small_case(name)
    tq, tk, tv = (torch.from_numpy(x).to(gpu) for x in (q, k, v))
    o, res = tpa._tpa_fwd(tq, tk, tv, h, qs, ks, scale, causal, None, False, False, False)
    same(o.double().cpu().numpy(), SMALL[f"{name}.o"], 1e-4)
    same(res[-1].double().cpu().numpy(), SMALL[f"{name}.lse"], 1e-3)


@pytest.mark.gpu
def test_kernel_reproduces_upstream_literal(gpu):
    import torch
    from tpa import mha

    q, k, v, bias = (torch.from_numpy(SMALL[f"upstream_mha_literal.{n}"]).float().to(gpu) for n in "q k v bias".split())
    o = mha.mha(q, k, v, bias).double().cpu().numpy()
    np.testing.assert_array_equal(o, SMALL["upstream_mha_literal.o"])


@pytest.mark.gpu
@pytest.mark.parametrize("name", SAMPLED_NAMES)
def test_kernel_reproduces_sampled_fixture(gpu, name):
    import torch
    from tpa import tpa

    q, k, v, qs, ks, h, scale, causal, rows = sampled_case(name)
    bf16 = "bf16" in name
    if bf16:
        # the fixture was computed from the fp32 inputs; bf16 kernels see rounded inputs, so compare with
        # the oracle on the rounded inputs as well and require the fixture within the bf16 bound
        dtype, otol, ltol = torch.bfloat16, 2e-2, 1e-3
    else:
        dtype, otol, ltol = torch.float32, 1e-4, 1e-3
    tq, tk, tv = (torch.from_numpy(x).to(dtype).to(gpu) for x in (q, k, v))
    o, res = tpa._tpa_fwd(tq, tk, tv, h, qs, ks, scale, causal, None, False, False, False)
    o = o[:, rows].double().cpu().numpy()
    lse = res[-1][:, rows].double().cpu().numpy()
    if bf16:
        qr, kr, vr = (bf16_round(x) for x in (q, k, v))
        o_ref, l_ref = orc.tpa_reference_rows(qr, kr, vr, qs, ks, h, rows, sm_scale=scale, causal=causal)
        otol = otol * max(1.0, float(np.nanmax(np.abs(o_ref))))
        ltol = ltol * max(1.0, float(np.max(np.abs(l_ref[np.isfinite(l_ref)]))))
        same(o, o_ref, otol)
        same(lse, l_ref, ltol)
    else:
        same(o, SAMPLED[f"{name}.o"], otol)
        same(lse, SAMPLED[f"{name}.lse"], ltol)


# ------------------------------------------------------------------------------------ backward
BACK = np.load(os.path.join(GOLDEN, "backward_cases.npz"))


@pytest.mark.parametrize("name", SMALL_NAMES)
def test_oracle_reproduces_backward_fixture(name):
    q, k, v, qs, ks, h, scale, causal = small_case(name)
    got = orc.tpa_backward(q, k, v, qs, ks, h, BACK[f"{name}.do"], sm_scale=scale, causal=causal)
    for g, key in zip(got, ("dq", "dk", "dv")):
        np.testing.assert_allclose(g, BACK[f"{name}.{key}"], rtol=0, atol=1e-13)


def test_oracle_reproduces_upstream_literal_gradients():
    """tpa/mha_test.py:87-118: dq = dk = 0, dv = [[1, 1], [0, 0], [1, 1]] for nansum(o)."""
    got = orc.mha_backward(SMALL["upstream_mha_literal.q"], SMALL["upstream_mha_literal.k"], SMALL["upstream_mha_literal.v"],
                           SMALL["upstream_mha_literal.bias"], 1.0, np.ones((1, 3, 1, 2)))
    for g, key in zip(got, ("dq", "dk", "dv")):
        np.testing.assert_allclose(g, BACK[f"upstream_mha_literal.{key}"], atol=1e-15)


@pytest.mark.gpu
@pytest.mark.parametrize("name", SMALL_NAMES)
def test_kernel_reproduces_backward_fixture(gpu, name):
    import torch
    from tpa import tpa

    q, k, v, qs, ks, h, scale, causal = small_case(name)
    tq, tk, tv = (torch.from_numpy(x).to(gpu) for x in (q, k, v))
    o, res = tpa._tpa_fwd(tq, tk, tv, h, qs, ks, scale, causal, None, False, False, False)
    grads = tpa._tpa_bwd(h, scale, causal, None, False, False, False, res, torch.from_numpy(BACK[f"{name}.do"]).to(gpu))
    for g, key in zip(grads[:3], ("dq", "dk", "dv")):
        want = BACK[f"{name}.{key}"]
        assert np.max(np.abs(g.double().cpu().numpy() - want)) <= 2e-4 * max(1.0, float(np.max(np.abs(want))))
