"""Seeded random problems through tpa_factors / tpa_factors_bwd with `kernel = AUTO`, against the oracle.

The parametrised tests elsewhere walk the shapes the kernels were written for; these walk shapes nobody
picked: lengths that are not multiples of anything, head counts and head sizes on and off the matrix-core
kernels' grid, every mask the interface takes (segment ids in runs of random length, causal with an offset,
per-sequence key lengths, bottom-right alignment) in random combination, with and without the optional
workspace, both storage types.  Whatever kernel the dispatcher picks must meet the same bounds as in
tests/test_gpu_parity.py: fp32 1e-4 / 1e-3, bf16 the per-row bound of its rounding points.
"""

import numpy as np
import pytest
import torch

from conftest import make_factors
from error_model import tpa_bounds
from oracle import tpa_oracle as orc
from test_gpu_parity import BF16_TOL, F32_TOL, as_f64, check, split, to_gpu, visible_bias

pytestmark = pytest.mark.gpu


def _runs(rng, b, length, mean_run):
    """ids [b, length] in runs of random length (non-decreasing: packed documents)"""
    out = np.zeros((b, length), np.int32)
    for i in range(b):
        pos, sid = 0, int(rng.integers(0, 3))
        while pos < length:
            n = int(rng.integers(1, 2 * mean_run))
            out[i, pos : pos + n] = sid
            pos += n
            sid += int(rng.integers(1, 3))
    return out


def _problem(rng):
    mfma_grid = rng.random() < 0.75
    d = int(rng.choice([64, 128])) if mfma_grid else int(rng.choice([8, 24, 40, 72, 96]))
    dv = d if mfma_grid or rng.random() < 0.5 else int(rng.choice([16, 48, 80]))
    h = int(rng.choice([8, 16, 24, 32, 40])) if mfma_grid else int(rng.choice([1, 3, 5, 12]))
    b = int(rng.integers(1, 4))
    lq = int(rng.choice([1, 2, 5, 17, 64, 100, 129, 256, 300, 511, 640]))
    lk = int(rng.choice([1, 7, 63, 64, 65, 200, 257, 512, 700, 1100, 2050]))
    rq, rk = int(rng.choice([1, 2, 3, 6])), int(rng.choice([1, 2, 3, 4, 8]))
    dtype = torch.bfloat16 if rng.random() < 0.6 else torch.float32
    mask = rng.choice(["none", "causal", "causal_offset", "bottom_right", "segments", "segments_causal", "lengths"])
    return dict(b=b, lq=lq, lk=lk, h=h, d=d, dv=dv, rq=rq, rk=rk, dtype=dtype, mask=str(mask), ws=bool(rng.random() < 0.5),
                sharp=bool(rng.random() < 0.2))


def _masks(rng, c):
    b, lq, lk = c["b"], c["lq"], c["lk"]
    qseg = kvseg = lengths = None
    causal, offset = False, 0
    m = c["mask"]
    if m in ("causal", "segments_causal"):
        causal = True
    if m == "causal_offset":
        causal, offset = True, int(rng.integers(-3, max(lk - lq, 0) + 4))
    if m == "bottom_right":
        causal = 2
        lengths = [int(x) for x in rng.integers(min(lq, lk), lk + 1, size=b)]
    if m == "lengths":
        lengths = [int(x) for x in rng.integers(0, lk + 1, size=b)]
        lengths[0] = lk
    if m.startswith("segments"):
        # one run pattern cut to both lengths, so that queries and keys of a document line up as in a packed batch
        ids = _runs(rng, b, max(lq, lk), int(rng.choice([20, 90, 300])))
        qseg, kvseg = ids[:, :lq].copy(), ids[:, :lk].copy()
    bias = visible_bias(b, lq, lk, qseg, kvseg, causal=bool(causal), offset=offset, lengths=lengths, bottom_right=causal == 2)
    return qseg, kvseg, lengths, causal, offset, bias


@pytest.mark.parametrize("seed", range(160))
def test_random_forward_problem(gpu, seed):
    from tpa import tpa

    rng = np.random.default_rng(1000 + seed)
    c = _problem(rng)
    b, lq, lk, h, d, dv, rq, rk, dtype = (c[k] for k in ("b", "lq", "lk", "h", "d", "dv", "rq", "rk", "dtype"))
    q, k, v = make_factors(seed, b, lq, lk, h, d, dv, rq, rk, scale_by_rank=not c["sharp"])
    qseg, kvseg, lengths, causal, offset, bias = _masks(rng, c)
    tq, tk, tv = (to_gpu(x, dtype, gpu) for x in (q, k, v))
    sm_scale = d**-0.5
    o, lse = tpa.tpa_factors(
        *split(tq, tk, tv, h),
        None if qseg is None else torch.from_numpy(qseg).to(gpu), None if kvseg is None else torch.from_numpy(kvseg).to(gpu),
        sm_scale, causal, use_workspace=c["ws"], kv_lengths=lengths, causal_offset=offset,
    )
    fq, fk, fv = as_f64(tq), as_f64(tk), as_f64(tv)
    dense = [orc.reconstruct(*orc.split_factors(x, h)) for x in (fq, fk, fv)]
    o_ref, l_ref = orc.mha_forward(*dense, bias=bias, sm_scale=sm_scale)
    bf16 = dtype == torch.bfloat16
    # which kernel ran is the dispatcher's business: the factored bound covers the split-key kernels too
    bounds = tpa_bounds(fq, fk, fv, h, sm_scale, form="factored") if bf16 else None
    check(o, lse, o_ref, l_ref, BF16_TOL if bf16 else F32_TOL, bounds)


@pytest.mark.parametrize("seed", range(64))
def test_random_backward_problem(gpu, seed):
    from tpa import tpa

    rng = np.random.default_rng(5000 + seed)
    c = _problem(rng)
    c["lq"], c["lk"] = min(c["lq"], 300), min(c["lk"], 700)  # the oracle's backward holds [b, h, lq, lk] several times over
    if c["mask"] == "bottom_right":
        c["mask"] = "causal_offset"  # the backward takes lengths with top-left alignment only
    b, lq, lk, h, d, dv, rq, rk, dtype = (c[k] for k in ("b", "lq", "lk", "h", "d", "dv", "rq", "rk", "dtype"))
    q, k, v = make_factors(seed, b, lq, lk, h, d, dv, rq, rk, scale_by_rank=True)
    qseg, kvseg, lengths, causal, offset, bias = _masks(rng, c)
    tq, tk, tv = (to_gpu(x, dtype, gpu) for x in (q, k, v))
    sm_scale = d**-0.5
    tqs = None if qseg is None else torch.from_numpy(qseg).to(gpu)
    tks = None if kvseg is None else torch.from_numpy(kvseg).to(gpu)
    fs = split(tq, tk, tv, h)
    o, lse = tpa.tpa_factors(*fs, tqs, tks, sm_scale, causal, kv_lengths=lengths, causal_offset=offset)
    do = torch.from_numpy(np.random.default_rng(seed).standard_normal((b, lq, h, dv)).astype(np.float32)).to(dtype).to(gpu)
    grads = tpa.tpa_factors_bwd(*fs, tqs, tks, o, lse, do, sm_scale, causal, kv_lengths=lengths, causal_offset=offset)
    # oracle: gradients of sum(o * do) through the dense attention with the same additive bias, projected onto the factors
    fq, fk, fv = as_f64(tq), as_f64(tk), as_f64(tv)
    (qa, qb), (ka, kb), (va, vb) = (orc.split_factors(x, h) for x in (fq, fk, fv))
    dq, dk, dv_ = orc.mha_backward(orc.reconstruct(qa, qb), orc.reconstruct(ka, kb), orc.reconstruct(va, vb), bias, sm_scale, as_f64(do))
    want = []
    for dx, (a, bb) in ((dq, (qa, qb)), (dk, (ka, kb)), (dv_, (va, vb))):
        want += list(orc.project_to_factors(np.nan_to_num(dx), a, bb))
    # bf16 matrix-core kernels: dense Q, K, V, P and dS are rounded to bf16, so the probabilities carry the relative
    # error E that the forward's error law gives the exponent (tests/error_model.py; 3e-3 for benchmark-like
    # inputs, 0.1 where low ranks make the softmax sharp), and the gradients inherit it: 2e-2 + 2 E of the largest
    # entry.  fp32: 3e-4.  A gradient array that is exactly zero (a row that sees a single key has p = 1 and
    # dS = 0, so nothing reaches q and k) is held against a fiftieth of the largest entry of all six instead of
    # against itself.
    if dtype == torch.bfloat16:
        tol = 2e-2 + 2.0 * float(tpa_bounds(fq, fk, fv, h, sm_scale)[0].max())
    else:
        tol = 3e-4
    floor = 0.02 * max(np.abs(w).max() for w in want)
    for name, g, w in zip(("dqa", "dqb", "dka", "dkb", "dva", "dvb"), grads, want):
        g = as_f64(g)
        assert np.isfinite(g).all(), name
        scale = max(np.abs(w).max(), floor, 1e-30)
        assert np.abs(g - w).max() <= tol * scale, (name, float(np.abs(g - w).max() / scale), tol, c)


@pytest.mark.parametrize("seed", range(64))
def test_random_decode_problem(gpu, seed):
    """tpa_decode with whatever the interface takes: several query rows, key ranges, ragged and paged caches,
    a causal limit per row (offset or aligned with the end of each cache)."""
    from tpa import tpa

    rng = np.random.default_rng(9000 + seed)
    b, lq = int(rng.integers(1, 6)), int(rng.choice([1, 1, 2, 3, 4, 7]))
    h, d = int(rng.choice([8, 16, 32, 40, 64])), int(rng.choice([64, 128]))
    rq, rk = int(rng.choice([1, 2, 6])), int(rng.choice([1, 2, 4, 8]))
    dtype = torch.bfloat16 if rng.random() < 0.7 else torch.float32
    paged = rng.random() < 0.4
    page_size = int(rng.choice([32, 64, 256])) if paged else 0
    lk = int(rng.choice([2, 5, 8, 17, 33])) * page_size if paged else int(rng.choice([37, 300, 1024, 1500, 4100]))
    q, k, v = make_factors(seed, b, lq, lk, h, d, d, rq, rk, scale_by_rank=rng.random() < 0.8)
    tq, tk, tv = (to_gpu(x, dtype, gpu) for x in (q, k, v))
    lengths = None
    if rng.random() < 0.6:
        lengths = [int(x) for x in rng.integers(lq, lk + 1, size=b)]
    mode = str(rng.choice(["none", "offset", "bottom_right"]))
    causal, offset = False, 0
    if mode == "offset":
        causal, offset = True, lk - lq - int(rng.integers(0, 4))
    if mode == "bottom_right":
        causal = 2
    qa, qb, ka, kb, va, vb = split(tq, tk, tv, h)
    table = None
    if paged:
        pps = lk // page_size
        npages = b * pps + 3
        table = torch.from_numpy(rng.permutation(npages)[: b * pps].astype(np.int32)).reshape(b, pps).to(gpu)
        pool = lambda x: torch.full((npages, page_size) + tuple(x.shape[2:]), float("nan"), dtype=x.dtype, device=gpu).index_copy_(
            0, table.reshape(-1).long(), x.reshape(b * pps, page_size, *x.shape[2:]))
        ka, kb, va, vb = (pool(x) for x in (ka, kb, va, vb))
    sm_scale = d**-0.5
    o, lse = tpa.tpa_decode(qa, qb, ka, kb, va, vb, sm_scale=sm_scale, num_splits=int(rng.choice([0, 0, 1, 3, 9])),
                            kv_lengths=lengths, page_table=table, causal=causal, causal_offset=offset)
    bias = visible_bias(b, lq, lk, causal=bool(causal), offset=offset, lengths=lengths, bottom_right=causal == 2)
    fq, fk, fv = as_f64(tq), as_f64(tk), as_f64(tv)
    dense = [orc.reconstruct(*orc.split_factors(x, h)) for x in (fq, fk, fv)]
    o_ref, l_ref = orc.mha_forward(*dense, bias=bias, sm_scale=sm_scale)
    bf16 = dtype == torch.bfloat16
    check(o, lse, o_ref, l_ref, BF16_TOL if bf16 else F32_TOL, tpa_bounds(fq, fk, fv, h, sm_scale, form="factored") if bf16 else None)


@pytest.mark.parametrize("seed", range(48))
def test_random_append_problem(gpu, seed):
    """tpa_cache_append on layers and batches nobody picked: every output factor against the oracle, the rest of
    the cache untouched, tokens past the capacity dropped; contiguous and paged caches, given positions."""
    from test_gpu_append import f64, make_layer, rope_tables
    from tpa import tpa

    rng = np.random.default_rng(13000 + seed)
    b, n = int(rng.integers(1, 9)), int(rng.choice([1, 1, 2, 3, 7, 16, 33, 70, 129, 300, 1100]))
    dm = int(rng.choice([64, 128, 192, 256, 512, 1024, 1536]))
    h, d = int(rng.choice([8, 16, 24, 32])), int(rng.choice([64, 96, 128]))
    rq, rk = int(rng.choice([1, 2, 3, 6])), int(rng.choice([1, 2, 4]))
    dtype = torch.bfloat16 if rng.random() < 0.75 else torch.float32
    x, w = make_layer(seed, b, n, dm, h, d, rq, rk, dtype, gpu)
    page_size = int(rng.choice([8, 16, 64]))
    cache_len = (n + int(rng.integers(0, 40)) + page_size - 1) // page_size * page_size
    cos, sin = rope_tables(cache_len + 9, d)
    lengths = rng.integers(0, max(cache_len - n, 0) + 1, size=b).astype(np.int32)
    if rng.random() < 0.3:
        lengths[-1] = min(max(cache_len - n + 2, 0), cache_len)  # the last tokens of the last sequence do not fit
    pos = None
    if rng.random() < 0.4:
        pos = (lengths[:, None] + np.arange(n)[None, :] + rng.integers(0, 5, size=(b, 1))).astype(np.int32)
    paged = rng.random() < 0.5
    if paged:
        pps = cache_len // page_size
        table = torch.from_numpy(rng.permutation(b * pps + 2)[: b * pps].astype(np.int32)).reshape(b, pps).to(gpu)
        caches = [torch.full((b * pps + 2, page_size, rk, inner), float("nan"), dtype=dtype, device=gpu) for inner in (h, d, h, d)]
    else:
        table = None
        caches = [torch.full((b, cache_len, rk, inner), float("nan"), dtype=dtype, device=gpu) for inner in (h, d, h, d)]
    qa, qb, new_len = tpa.tpa_cache_append(x, w, cos, sin, *caches, lengths, rank_q=rq, positions=pos, page_table=table,
                                           use_workspace=bool(rng.random() < 0.5))
    used = pos if pos is not None else lengths[:, None] + np.arange(n)[None, :]
    want = orc.tpa_append_reference(f64(x), f64(w), cos, sin, np.minimum(used, cos.shape[0] - 1), h, d, rq, rk)
    rel = 2.0**-8 if dtype == torch.bfloat16 else 1e-5
    for name, got in (("qa", qa), ("qb", qb)):
        assert np.abs(f64(got) - want[name]).max() <= rel * np.abs(want[name]).max(), name
    for name, cache in zip(("ka", "kb", "va", "vb"), caches):
        c = f64(cache[table.long()].reshape(b, cache_len, rk, -1) if paged else cache)
        for bi in range(b):
            fits = max(min(n, cache_len - int(lengths[bi])), 0)
            rows = c[bi, lengths[bi] : lengths[bi] + fits]
            assert np.abs(rows - want[name][bi, :fits]).max(initial=0.0) <= rel * np.abs(want[name]).max(), (name, bi)
            assert np.isnan(c[bi, : lengths[bi]]).all() and np.isnan(c[bi, lengths[bi] + fits :]).all(), (name, bi)
    assert new_len.cpu().tolist() == [min(int(l) + n, cache_len) for l in lengths]


@pytest.mark.parametrize("seed", range(48))
def test_random_dense_attention_problem(gpu, seed):
    """mha (tpa/mha.py) forward and backward: head sizes on and off the matrix-core grid, dk != dv, a dense bias
    with -inf entries (rows without any visible key among them) or the causal flag, few rows over many keys."""
    from error_model import dense_bounds
    from tpa import mha

    rng = np.random.default_rng(17000 + seed)
    b, h = int(rng.integers(1, 4)), int(rng.choice([1, 2, 4, 8, 16]))
    lq = int(rng.choice([1, 3, 16, 65, 128, 200, 384]))
    lk = int(rng.choice([1, 9, 64, 100, 257, 640, 1500]))
    mfma_grid = rng.random() < 0.7
    dk = int(rng.choice([64, 128])) if mfma_grid else int(rng.choice([8, 24, 40, 96]))
    dv = dk if mfma_grid or rng.random() < 0.5 else int(rng.choice([16, 48, 72]))
    dtype = torch.bfloat16 if rng.random() < 0.6 else torch.float32
    mode = str(rng.choice(["none", "causal", "bias"]))
    g = np.random.Generator(np.random.Philox(seed))
    q, k, v, do = (g.standard_normal(s, dtype=np.float32) for s in ((b, lq, h, dk), (b, lk, h, dk), (b, lk, h, dv), (b, lq, h, dv)))
    bias = None
    if mode == "bias":
        bias = g.standard_normal((b, lq, lk), dtype=np.float32)
        bias[g.random((b, lq, lk)) < 0.3] = -np.inf
        bias[:, lq // 2] = -np.inf  # a row that sees nothing
    sm_scale = dk**-0.5
    tq, tk, tv, tdo = (to_gpu(x, dtype, gpu) for x in (q, k, v, do))
    o, res = mha._mha_fwd(tq, tk, tv, None if bias is None else torch.from_numpy(bias).to(gpu), sm_scale, causal=mode == "causal")
    lse = res[0]
    fq, fk, fv = as_f64(tq), as_f64(tk), as_f64(tv)
    full_bias = np.zeros((b, lq, lk)) if bias is None else bias.astype(np.float64)
    if mode == "causal":
        full_bias = full_bias + visible_bias(b, lq, lk, causal=True)
    o_ref, l_ref = orc.mha_forward(fq, fk, fv, bias=full_bias, sm_scale=sm_scale)
    bf16 = dtype == torch.bfloat16
    check(o, lse, o_ref, l_ref, BF16_TOL if bf16 else F32_TOL, dense_bounds(fq, fk, fv, sm_scale) if bf16 else None)
    dq, dk_, dv_, _, _ = mha._mha_bwd(res, tdo)
    want = orc.mha_backward(fq, fk, fv, full_bias, sm_scale, as_f64(tdo))
    tol = 2e-2 + 2.0 * float(dense_bounds(fq, fk, fv, sm_scale)[0].max()) if bf16 else 3e-4
    # a gradient that is exactly zero (one visible key: p = 1, dS = p (dp - delta) = 0) comes out as the rounding of
    # o inside delta, 2^-8 of |dp| - with these unscaled N(0, 1) inputs a few percent of the largest gradient
    floor = 0.1 * max(np.abs(w).max() for w in want)
    for name, got, w in zip(("dq", "dk", "dv"), (dq, dk_, dv_), want):
        got = as_f64(got)
        assert np.isfinite(got).all(), name
        scale = max(np.abs(w).max(), floor, 1e-30)
        # (gradients come back in the input dtype: a bf16 rounding of their own on top)
        assert np.abs(got - w).max() <= (tol + (2.0**-8 if bf16 else 0.0)) * scale, (name, float(np.abs(got - w).max() / scale), tol)
