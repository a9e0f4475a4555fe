"""Pins the CPU oracle (oracle/tpa_oracle.py) without importing the reference: brute force,
independent library routines, closed forms, invariances and the one literal known-answer the
reference holds."""

import numpy as np
import pytest
import scipy.special
import torch

from conftest import make_factors, segment_ids
from oracle import tpa_oracle as orc


def brute_force(q, k, v, qseg, kvseg, h, sm_scale, causal):
    """Float64 scalar loops straight from the definition (tpa/tpa_test.py:22-57, tpa/mha.py:23-37)."""
    b, lq, rq, _ = q.shape
    _, lk, rk, _ = k.shape
    dk = q.shape[-1] - h
    dv = v.shape[-1] - h
    o = np.zeros((b, lq, h, dv))
    lse = np.zeros((b, lq, h))
    for bi in range(b):
        for hi in range(h):
            for i in range(lq):
                qv = np.zeros(dk)
                for r in range(rq):
                    qv += q[bi, i, r, hi] * q[bi, i, r, h:]
                qv /= rq
                logits = []
                vals = []
                for t in range(lk):
                    kvec = np.zeros(dk)
                    vvec = np.zeros(dv)
                    for r in range(rk):
                        kvec += k[bi, t, r, hi] * k[bi, t, r, h:]
                        vvec += v[bi, t, r, hi] * v[bi, t, r, h:]
                    kvec /= rk
                    vvec /= rk
                    x = sm_scale * float(qv @ kvec)
                    if qseg is not None and qseg[bi, i] != kvseg[bi, t]:
                        x = -np.inf
                    if causal and t > i:
                        x = -np.inf
                    logits.append(x)
                    vals.append(vvec)
                logits = np.array(logits)
                if np.all(np.isneginf(logits)):
                    o[bi, i, hi] = np.nan
                    lse[bi, i, hi] = -np.inf
                    continue
                mx = logits.max()
                w = np.exp(logits - mx)
                o[bi, i, hi] = (w[:, None] * np.array(vals)).sum(0) / w.sum()
                lse[bi, i, hi] = mx + np.log(w.sum())
    return o, lse


@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("seg", [None, 3])
@pytest.mark.parametrize("rq,rk", [(1, 1), (6, 4), (3, 2)])
def test_brute_force_tiny(causal, seg, rq, rk):
    # the reference's smallest shape (1, 8, 8, 1, 4, 6) and a ragged one
    for (b, lq, lk, h, dk, dv) in [(1, 8, 8, 1, 4, 6), (2, 5, 7, 3, 2, 3)]:
        q, k, v = make_factors(7, b, lq, lk, h, dk, dv, rq, rk)
        qseg = segment_ids(lq, seg, b) if seg else None
        kvseg = segment_ids(lk, seg, b) if seg else None
        o, l = orc.tpa_reference(q, k, v, qseg, kvseg, h, sm_scale=0.7, causal=causal)
        o_bf, l_bf = brute_force(q.astype(np.float64), k.astype(np.float64), v.astype(np.float64), qseg, kvseg, h, 0.7, causal)
        np.testing.assert_allclose(o, o_bf, rtol=1e-12, atol=1e-12)
        np.testing.assert_allclose(l, l_bf, rtol=1e-12, atol=1e-12)


def test_known_answer_from_reference_mha_test():
    """tpa/mha_test.py:44-118 (commented out upstream): the only literal expected output."""
    q = np.array([[2, 1], [1, 1], [1, 1]], dtype=float)[None, :, None, :]
    k = np.ones((3, 2))[None, :, None, :]
    v = np.ones((3, 2))[None, :, None, :]
    ninf = -np.inf
    bias = np.array([[0, ninf, 0], [0, ninf, 0], [ninf, ninf, ninf]])[None]
    o, l = orc.mha_forward(q, k, v, bias)
    expect = np.array([[1.0, 1.0], [1.0, 1.0], [np.nan, np.nan]])[None, :, None, :]
    np.testing.assert_array_equal(o, expect)
    assert np.isneginf(l[0, 2, 0])
    # rows 0 and 1: logits (3, -inf, 3) and (2, -inf, 2)
    np.testing.assert_allclose(l[0, :2, 0], [3 + np.log(2), 2 + np.log(2)], rtol=1e-14)


@pytest.mark.parametrize("causal", [False, True])
def test_against_torch_sdpa_and_scipy(causal):
    b, l, h, dk, dv, rq, rk = 2, 33, 4, 16, 16, 6, 2
    q, k, v = make_factors(3, b, l, l, h, dk, dv, rq, rk)
    scale = 0.31
    o, lse = orc.tpa_reference(q, k, v, None, None, h, sm_scale=scale, causal=causal)
    # independent reconstruction with torch, attention with the library routine
    tq, tk, tv = (torch.from_numpy(x).double() for x in (q, k, v))
    Q = torch.einsum("blrh,blrd->bhld", tq[..., :h], tq[..., h:]) / rq
    K = torch.einsum("blrh,blrd->bhld", tk[..., :h], tk[..., h:]) / rk
    V = torch.einsum("blrh,blrd->bhld", tv[..., :h], tv[..., h:]) / rk
    ref = torch.nn.functional.scaled_dot_product_attention(Q, K, V, is_causal=causal, scale=scale)
    np.testing.assert_allclose(o, ref.permute(0, 2, 1, 3).numpy(), rtol=1e-9, atol=1e-11)
    logits = scale * torch.einsum("bhqd,bhkd->bhqk", Q, K).numpy()
    if causal:
        logits = np.where(np.tril(np.ones((l, l), bool)), logits, -np.inf)
    np.testing.assert_allclose(lse, scipy.special.logsumexp(logits, axis=-1).transpose(0, 2, 1), rtol=1e-12)
    p = scipy.special.softmax(logits, axis=-1)
    np.testing.assert_allclose(o, np.einsum("bhqk,bhkd->bqhd", p, V.numpy()), rtol=1e-9, atol=1e-12)


def test_segments_against_sdpa_mask():
    b, lq, lk, h, dk, dv, rq, rk = 2, 40, 24, 2, 8, 8, 2, 4
    q, k, v = make_factors(5, b, lq, lk, h, dk, dv, rq, rk, dist="uniform")
    qseg, kvseg = segment_ids(lq, 7, b), segment_ids(lk, 7, b)
    o, lse = orc.tpa_reference(q, k, v, qseg, kvseg, h)
    tq, tk, tv = (torch.from_numpy(x).double() for x in (q, k, v))
    Q = torch.einsum("blrh,blrd->bhld", tq[..., :h], tq[..., h:]) / rq
    K = torch.einsum("blrh,blrd->bhld", tk[..., :h], tk[..., h:]) / rk
    V = torch.einsum("blrh,blrd->bhld", tv[..., :h], tv[..., h:]) / rk
    mask = torch.from_numpy(qseg[:, :, None] == kvseg[:, None, :])[:, None]
    ref = torch.nn.functional.scaled_dot_product_attention(Q, K, V, attn_mask=mask, scale=1.0).permute(0, 2, 1, 3).numpy()
    has_key = mask[:, 0].any(-1).numpy()  # rows with at least one visible key
    assert not has_key.all() and has_key.any()  # q ids run past the kv ids: some rows are empty
    np.testing.assert_allclose(o[has_key], ref[has_key], rtol=1e-9, atol=1e-12)
    # empty rows: NaN output, -inf logsumexp (tpa/tpa.py:437-439)
    assert np.isnan(o[~has_key]).all()
    assert np.isneginf(lse[~has_key]).all()


def test_reference_shape_with_empty_rows():
    """(2, 1024, 128, 2, 3, 5, 42) of tpa/tpa_test.py:67: q ids reach 24, kv ids stop at 3,
    so rows >= 168 see no key."""
    q, k, v = make_factors(0, 2, 1024, 128, 2, 3, 5, 1, 1, dist="uniform")
    o, lse = orc.tpa_reference(q, k, v, segment_ids(1024, 42, 2), segment_ids(128, 42, 2), 2)
    assert np.isfinite(o[:, :168]).all() and np.isnan(o[:, 168:]).all()
    assert np.isfinite(lse[:, :168]).all() and np.isneginf(lse[:, 168:]).all()


def test_closed_forms():
    b, l, h, dk, dv, rq, rk = 1, 17, 3, 4, 5, 2, 3
    q, k, v = make_factors(11, b, l, l, h, dk, dv, rq, rk)
    q0 = q.copy()
    q0[..., h:] = 0.0  # zero queries: uniform attention
    V = orc.reconstruct(v[..., :h].astype(np.float64), v[..., h:].astype(np.float64))
    o, lse = orc.tpa_reference(q0, k, v, None, None, h, causal=True)
    running_mean = np.cumsum(V, axis=1) / np.arange(1, l + 1)[None, :, None, None]
    np.testing.assert_allclose(o, running_mean, rtol=1e-12, atol=1e-14)
    np.testing.assert_allclose(lse, np.broadcast_to(np.log(np.arange(1, l + 1))[None, :, None], lse.shape), rtol=1e-12, atol=1e-14)
    o, lse = orc.tpa_reference(q0, k, v, None, None, h, causal=False)
    np.testing.assert_allclose(o, np.broadcast_to(V.mean(1, keepdims=True), o.shape), rtol=1e-12)
    np.testing.assert_allclose(lse, np.log(l), rtol=1e-12)
    # a single key: o = V[0], lse = the logit
    o, lse = orc.tpa_reference(q, k[:, :1], v[:, :1], None, None, h, sm_scale=0.5)
    np.testing.assert_allclose(o, np.broadcast_to(V[:, :1], o.shape), rtol=1e-12)
    Q = orc.reconstruct(q[..., :h].astype(np.float64), q[..., h:].astype(np.float64))
    K = orc.reconstruct(k[..., :h].astype(np.float64), k[..., h:].astype(np.float64))
    np.testing.assert_allclose(lse, 0.5 * np.einsum("bqhd,bhd->bqh", Q, K[:, 0]), rtol=1e-12)


def test_rank_invariances():
    b, lq, lk, h, dk, dv, rq, rk = 2, 9, 11, 2, 4, 3, 3, 2
    q, k, v = make_factors(13, b, lq, lk, h, dk, dv, rq, rk)
    base, base_l = orc.tpa_reference(q, k, v, None, None, h, sm_scale=0.9)
    # duplicating every rank leaves (1/R) sum unchanged
    o, l = orc.tpa_reference(np.concatenate([q, q], 2), np.concatenate([k, k], 2), np.concatenate([v, v], 2), None, None, h, sm_scale=0.9)
    np.testing.assert_allclose(o, base, rtol=1e-12)
    np.testing.assert_allclose(l, base_l, rtol=1e-12)
    # permuting ranks
    o, _ = orc.tpa_reference(q[:, :, ::-1], k[:, :, ::-1], v[:, :, ::-1], None, None, h, sm_scale=0.9)
    np.testing.assert_allclose(o, base, rtol=1e-12)
    # a * c with b / c
    k2 = k.astype(np.float64).copy()
    k2[..., :h] *= 4.0
    k2[..., h:] /= 4.0
    o, _ = orc.tpa_reference(q, k2, v, None, None, h, sm_scale=0.9)
    np.testing.assert_allclose(o, base, rtol=1e-12)
    # rank 1 with a == 1: every head shares b (multi-query attention)
    k1 = k[:, :, :1].copy()
    k1[..., :h] = 1.0
    K = orc.reconstruct(k1[..., :h].astype(np.float64), k1[..., h:].astype(np.float64))
    np.testing.assert_allclose(K[:, :, 0], K[:, :, 1], rtol=0)


def test_causal_prefix_and_decode_row():
    b, l, h, dk, dv, rq, rk = 1, 24, 2, 8, 8, 6, 2
    q, k, v = make_factors(17, b, l, l, h, dk, dv, rq, rk)
    full, full_l = orc.tpa_reference(q, k, v, None, None, h, sm_scale=0.4, causal=True)
    part, part_l = orc.tpa_reference(q[:, :10], k[:, :10], v[:, :10], None, None, h, sm_scale=0.4, causal=True)
    np.testing.assert_allclose(full[:, :10], part, rtol=1e-12)
    np.testing.assert_allclose(full_l[:, :10], part_l, rtol=1e-12)
    # the last causal row equals an unmasked single-query call over the whole cache
    dec, dec_l = orc.tpa_reference(q[:, -1:], k, v, None, None, h, sm_scale=0.4, causal=False)
    np.testing.assert_allclose(full[:, -1:], dec, rtol=1e-12)
    np.testing.assert_allclose(full_l[:, -1:], dec_l, rtol=1e-12)


def test_rows_variant_matches_full():
    b, lq, lk, h, dk, dv, rq, rk = 2, 37, 29, 3, 4, 6, 2, 2
    q, k, v = make_factors(19, b, lq, lk, h, dk, dv, rq, rk)
    qseg, kvseg = segment_ids(lq, 9, b), segment_ids(lk, 9, b)
    rows = np.array([0, 5, 28, 36])
    for causal in (False, True):
        full, full_l = orc.tpa_reference(q, k, v, qseg, kvseg, h, sm_scale=0.3, causal=causal)
        sub, sub_l = orc.tpa_reference_rows(q, k, v, qseg, kvseg, h, rows, sm_scale=0.3, causal=causal)
        np.testing.assert_array_equal(np.isnan(sub), np.isnan(full[:, rows]))
        np.testing.assert_allclose(sub, full[:, rows], rtol=1e-12)
        np.testing.assert_allclose(sub_l, full_l[:, rows], rtol=1e-12)


def test_lse_helpers():
    rng = np.random.default_rng(0)
    x = rng.standard_normal((4, 9))
    np.testing.assert_allclose(orc.lse(x), scipy.special.logsumexp(x, axis=-1), rtol=1e-13)
    # split-and-merge gives the logsumexp of the whole (tpa/tpa.py:228-242)
    np.testing.assert_allclose(orc.lse_accum(orc.lse(x[:, :4]), orc.lse(x[:, 4:])), orc.lse(x), rtol=1e-13)
    ninf = np.full((4,), -np.inf)
    assert np.isneginf(orc.lse(np.full((4, 3), -np.inf))).all()
    assert np.isneginf(orc.lse_accum(ninf, ninf)).all()
    np.testing.assert_allclose(orc.lse_accum(ninf, x[:, 0]), x[:, 0])


# ---------------------------------------------------------------- backward
def torch_tpa_loss(q, k, v, qseg, kvseg, h, sm_scale, causal, do):
    """An independently written dense attention in torch (float64), differentiated by autograd:
    sum(nan_to_zero(o) * do), the scalar whose gradient `_tpa_bwd` returns (tpa/tpa_test.py:170-197
    uses nansum(o), i.e. do = 1)."""
    tq, tk, tv = (torch.tensor(x, dtype=torch.float64, requires_grad=True) for x in (q, k, v))
    rec = lambda t: torch.einsum("blrh,blrd->blhd", t[..., :h], t[..., h:]) / t.shape[2]
    Q, K, V = rec(tq), rec(tk), rec(tv)
    x = sm_scale * torch.einsum("bqhd,bkhd->bhqk", Q, K)
    lq, lk = q.shape[1], k.shape[1]
    keep = torch.ones((q.shape[0], lq, lk), dtype=torch.bool)
    if qseg is not None:
        keep &= torch.tensor(qseg)[:, :, None] == torch.tensor(kvseg)[:, None, :]
    if causal:
        keep &= torch.arange(lq)[:, None] >= torch.arange(lk)[None, :]
    live = keep.any(-1)  # rows with at least one visible key
    x = x.masked_fill(~keep[:, None], -1e300)  # finite, so autograd never meets inf - inf
    p = torch.softmax(x, dim=-1) * keep[:, None]
    o = torch.einsum("bhqk,bkhd->bqhd", p, V) * live[:, :, None, None]
    loss = (o * torch.tensor(do, dtype=torch.float64)).sum()
    loss.backward()
    return tq.grad.numpy(), tk.grad.numpy(), tv.grad.numpy()


@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("seg", [None, 5])
@pytest.mark.parametrize("lq,lk", [(24, 24), (30, 12)])  # (30, 12) with seg = 5: rows whose segment has no key
def test_backward_against_torch_autograd(causal, seg, lq, lk):
    b, h, dk, dv, rq, rk = 2, 3, 7, 5, 4, 2
    q, k, v = make_factors(11, b, lq, lk, h, dk, dv, rq, rk)
    rng = np.random.default_rng(5)
    do = rng.standard_normal((b, lq, h, dv))
    qseg = segment_ids(lq, seg, b) if seg else None
    kvseg = segment_ids(lk, seg, b) if seg else None
    got = orc.tpa_backward(q, k, v, qseg, kvseg, h, do, sm_scale=0.4, causal=causal)
    want = torch_tpa_loss(q, k, v, qseg, kvseg, h, 0.4, causal, do)
    for g, w in zip(got, want):
        np.testing.assert_allclose(g, w, rtol=1e-9, atol=1e-11)


def test_backward_against_finite_differences():
    """Central differences of sum(o * do) on the forward oracle, every input element of a tiny case."""
    b, lq, lk, h, dk, dv, rq, rk = 1, 4, 5, 2, 3, 2, 2, 3
    q, k, v = (x.astype(np.float64) for x in make_factors(12, b, lq, lk, h, dk, dv, rq, rk))
    do = np.random.default_rng(6).standard_normal((b, lq, h, dv))
    f = lambda q_, k_, v_: float(np.sum(orc.tpa_reference(q_, k_, v_, None, None, h, sm_scale=0.7, causal=True)[0] * do))
    grads = orc.tpa_backward(q, k, v, None, None, h, do, sm_scale=0.7, causal=True)
    eps = 1e-6
    for which, (x, g) in enumerate(zip((q, k, v), grads)):
        num = np.zeros_like(x)
        for idx in np.ndindex(*x.shape):
            args = [q.copy(), k.copy(), v.copy()]
            args[which][idx] += eps
            up = f(*args)
            args[which][idx] -= 2 * eps
            num[idx] = (up - f(*args)) / (2 * eps)
        np.testing.assert_allclose(g, num, rtol=1e-6, atol=1e-8)


def test_backward_known_answer_from_reference_mha_test():
    """tpa/mha_test.py:87-118 (commented out upstream): gradients of nansum(o) on the literal case."""
    q = np.array([[2, 1], [1, 1], [1, 1]], dtype=float)[None, :, None, :]
    k = np.ones((3, 2))[None, :, None, :]
    v = np.ones((3, 2))[None, :, None, :]
    ninf = -np.inf
    bias = np.array([[0, ninf, 0], [0, ninf, 0], [ninf, ninf, ninf]])[None]
    dq, dk, dv = orc.mha_backward(q, k, v, bias, 1.0, np.ones((1, 3, 1, 2)))
    np.testing.assert_allclose(dq, np.zeros_like(q), atol=1e-15)
    np.testing.assert_allclose(dk, np.zeros_like(k), atol=1e-15)
    np.testing.assert_allclose(dv[0, :, 0], [[1, 1], [0, 0], [1, 1]], atol=1e-15)


def test_mha_backward_with_finite_bias_against_autograd():
    """tpa/mha_test.py:9-41: dense attention with a random additive bias."""
    b, lq, lk, h, dk, dv = 2, 4, 6, 3, 8, 8
    rng = np.random.default_rng(7)
    q, k, v = rng.standard_normal((b, lq, h, dk)), rng.standard_normal((b, lk, h, dk)), rng.standard_normal((b, lk, h, dv))
    bias, do = rng.standard_normal((b, lq, lk)), rng.standard_normal((b, lq, h, dv))
    for scale in (0.5, 1.0, 2.0):
        tq, tk, tv = (torch.tensor(x, requires_grad=True) for x in (q, k, v))
        x = scale * torch.einsum("bqhd,bkhd->bhqk", tq, tk) + torch.tensor(bias)[:, None]
        o = torch.einsum("bhqk,bkhd->bqhd", torch.softmax(x, -1), tv)
        (o * torch.tensor(do)).sum().backward()
        got = orc.mha_backward(q, k, v, bias, scale, do)
        for g, w in zip(got, (tq.grad, tk.grad, tv.grad)):
            np.testing.assert_allclose(g, w.numpy(), rtol=1e-10, atol=1e-12)


# ---------------------------------------------------------------- the producer step (projections + rotary embedding)
def _rope_tables(rope_len, d, base=10000.0):
    inv = base ** (-np.arange(0, d, 2, dtype=np.float64) / d)
    ang = np.arange(rope_len, dtype=np.float64)[:, None] * inv[None, :]
    return np.cos(ang), np.sin(ang)


def test_append_reference_against_loops():
    rng = np.random.default_rng(5)
    b, n, dm, h, d, rq, rk = 2, 3, 7, 2, 4, 2, 3
    x = rng.standard_normal((b, n, dm))
    w = rng.standard_normal((rq * (h + d) + 2 * rk * (h + d), dm))
    cos, sin = _rope_tables(16, d)
    pos = rng.integers(0, 16, (b, n))
    got = orc.tpa_append_reference(x, w, cos, sin, pos, h, d, rq, rk)
    row = 0
    for name, r_, inner in (("qa", rq, h), ("qb", rq, d), ("ka", rk, h), ("kb", rk, d), ("va", rk, h), ("vb", rk, d)):
        want = np.zeros((b, n, r_, inner))
        for bi in range(b):
            for i in range(n):
                for r in range(r_):
                    for e in range(inner):
                        want[bi, i, r, e] = sum(x[bi, i, k] * w[row + r * inner + e, k] for k in range(dm))
                    if name in ("qb", "kb"):
                        y = want[bi, i, r].copy()
                        for j in range(inner // 2):
                            c, s_ = cos[pos[bi, i], j], sin[pos[bi, i], j]
                            want[bi, i, r, 2 * j] = y[2 * j] * c - y[2 * j + 1] * s_
                            want[bi, i, r, 2 * j + 1] = y[2 * j + 1] * c + y[2 * j] * s_
        row += r_ * inner
        np.testing.assert_allclose(got[name], want, rtol=1e-12, atol=1e-12, err_msg=name)


def test_rope_closed_forms():
    rng = np.random.default_rng(6)
    d = 8
    cos, sin = _rope_tables(64, d)
    y = rng.standard_normal((5, d))
    # position 0 is the identity
    np.testing.assert_allclose(orc.rope_rotate(y, cos[0], sin[0]), y, atol=1e-15)
    # a rotation: the norm of every pair is preserved
    r = orc.rope_rotate(y, cos[17], sin[17])
    np.testing.assert_allclose(r[:, 0::2] ** 2 + r[:, 1::2] ** 2, y[:, 0::2] ** 2 + y[:, 1::2] ** 2, rtol=1e-12)
    # angles add: rotating by position 5 and then by position 9 is rotating by position 14
    np.testing.assert_allclose(orc.rope_rotate(orc.rope_rotate(y, cos[5], sin[5]), cos[9], sin[9]), orc.rope_rotate(y, cos[14], sin[14]), atol=1e-12)
    # the dot product of a rotated query and key depends on the distance of their positions only
    q, k = rng.standard_normal(d), rng.standard_normal(d)
    dots = [orc.rope_rotate(q, cos[m], sin[m]) @ orc.rope_rotate(k, cos[m - 7], sin[m - 7]) for m in (7, 20, 63)]
    np.testing.assert_allclose(dots, dots[0], rtol=1e-12)
    # ... and it is not the unrotated one (a sign slip in the rotation would pass the norm test)
    assert abs(dots[0] - q @ k) > 1e-3
    # direction: the first pair of (1, 0) at position p is (cos p, sin p) for frequency 1
    e = np.zeros(d); e[0] = 1.0
    np.testing.assert_allclose(orc.rope_rotate(e, cos[3], sin[3])[:2], [np.cos(3.0), np.sin(3.0)], atol=1e-12)
