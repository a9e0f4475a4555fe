"""Parity of the fp32 MFMA prefill kernel (fp32 inputs, the reference's default dtype) against the
CPU oracle, through the Python API -> C ABI.  kernel=2 makes a fall-back to the vector-ALU kernel
an error, so every case here really runs the matrix-core kernel.  Tolerance: 1e-4 on outputs,
1e-3 on the logsumexp, as for every fp32 path.
"""

import numpy as np
import pytest
import torch

from conftest import make_factors, segment_ids
from oracle import tpa_oracle as orc
from test_gpu_parity import F32_TOL, _varlen_reference, as_f64, check, split, to_gpu

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("d", [128, 64])
@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize(
    "b,lq,lk,h,rq,rk",
    [
        (2, 512, 512, 4, 6, 2),   # the benchmark ranks
        (1, 300, 300, 2, 6, 2),   # ragged tails in both directions
        (1, 257, 130, 2, 1, 1),   # lq > lk, rank 1
        (1, 100, 700, 3, 3, 4),   # lk > lq
        (1, 256, 256, 2, 16, 8),  # the high-rank configuration's ranks
    ],
)
def test_prefill_f32_mfma(gpu, d, causal, b, lq, lk, h, rq, rk):
    from tpa import tpa

    q, k, v = make_factors(12, b, lq, lk, h, d, d, rq, rk)
    scale = d**-0.5
    tq, tk, tv = (to_gpu(x, torch.float32, gpu) for x in (q, k, v))
    o, lse = tpa.tpa_factors(*split(tq, tk, tv, h), sm_scale=scale, causal=causal, kernel=2)
    o_ref, l_ref = orc.tpa_reference(q, k, v, None, None, h, sm_scale=scale, causal=causal)
    check(o, lse, o_ref, l_ref, F32_TOL)


def test_prefill_f32_mfma_concatenated_layout_in_place(gpu):
    """The reference's q[b, l, r, h + d] arrays read in place (A = base, B = base + h), default
    kernel choice: identical to the explicit MFMA request on split copies."""
    from tpa import tpa

    b, t, h, d = 2, 384, 8, 64
    q, k, v = make_factors(13, b, t, t, h, d, d, 6, 2)
    tq, tk, tv = (to_gpu(x, torch.float32, gpu) for x in (q, k, v))
    o, res = tpa._tpa_fwd(tq, tk, tv, h, None, None, d**-0.5, True, None, False, False, False)
    o2, lse2 = tpa.tpa_factors(*split(tq, tk, tv, h), sm_scale=d**-0.5, causal=True, kernel=2)
    assert torch.equal(o, o2) and torch.equal(res[-1].permute(0, 2, 1), lse2)
    o_ref, l_ref = orc.tpa_reference(q, k, v, None, None, h, sm_scale=d**-0.5, causal=True)
    check(o, res[-1].permute(0, 2, 1), o_ref, l_ref, F32_TOL)


@pytest.mark.parametrize(
    "b,lq,lk,h,d,rk,seg,causal",
    [
        (2, 512, 512, 4, 128, 2, 100, True),
        (2, 640, 384, 2, 64, 2, 77, False),    # query rows whose segment has no key at all: NaN / -inf
        (1, 1024, 1024, 2, 128, 2, 321, True),  # the segment size of tpa/tpa_test.py:72
        (1, 256, 1024, 2, 64, 4, 42, False),    # tpa/tpa_test.py:69-70 style: lq != lk
    ],
)
def test_prefill_f32_mfma_segment_ids(gpu, b, lq, lk, h, d, rk, seg, causal):
    from tpa import tpa

    q, k, v = make_factors(14, b, lq, lk, h, d, d, 6, rk)
    qseg, kvseg = segment_ids(lq, seg, b), segment_ids(lk, seg, b)
    tq, tk, tv = (to_gpu(x, torch.float32, gpu) for x in (q, k, v))
    tqs, tks = torch.from_numpy(qseg).to(gpu), torch.from_numpy(kvseg).to(gpu)
    o, lse = tpa.tpa_factors(*split(tq, tk, tv, h), tqs, tks, d**-0.5, causal, 2)
    o_ref, l_ref = orc.tpa_reference(q, k, v, qseg, kvseg, h, sm_scale=d**-0.5, causal=causal)
    check(o, lse, o_ref, l_ref, F32_TOL)
    if lq > lk:
        assert np.isnan(o_ref).any()  # the case really has empty rows


@pytest.mark.parametrize("causal", [False, True])
def test_prefill_f32_mfma_per_sequence_key_lengths(gpu, causal):
    """A padded batch: keys past kv_lengths[b] are never read as values (they are NaN here)."""
    from tpa import tpa

    b, lq, lk, h, d = 4, 400, 700, 8, 64
    lengths = [700, 333, 64, 0]
    q, k, v = make_factors(15, b, lq, lk, h, d, d, 3, 2)
    tq, tk, tv = (to_gpu(x, torch.float32, gpu) for x in (q, k, v))
    for bi, n in enumerate(lengths):
        tk[bi, n:] = float("nan")
        tv[bi, n:] = float("nan")
    o, lse = tpa.tpa_factors(*split(tq, tk, tv, h), None, None, d**-0.5, causal, 2, kv_lengths=lengths)
    o_ref, l_ref = _varlen_reference(as_f64(tq), np.nan_to_num(as_f64(tk)), np.nan_to_num(as_f64(tv)), lengths, h, d**-0.5, causal)
    check(o, lse, o_ref, l_ref, F32_TOL)


def test_prefill_f32_mfma_sharp_softmax_large_logits(gpu):
    """sm_scale = 1 on N(0,1) factors: logits of order ten and more, row maxima that keep moving
    from tile to tile (the rescale path), still within the fp32 tolerance."""
    from tpa import tpa

    b, t, h, d = 1, 640, 2, 64
    q, k, v = make_factors(16, b, t, t, h, d, d, 2, 2)
    tq, tk, tv = (to_gpu(x, torch.float32, gpu) for x in (q, k, v))
    o, lse = tpa.tpa_factors(*split(tq, tk, tv, h), sm_scale=1.0, causal=False, kernel=2)
    o_ref, l_ref = orc.tpa_reference(q, k, v, None, None, h, sm_scale=1.0, causal=False)
    check(o, lse, o_ref, l_ref, F32_TOL)
    assert np.abs(l_ref).max() > 10  # the logits really are large


@pytest.mark.parametrize("d", [128, 64])
@pytest.mark.parametrize("causal", [False, True])
def test_mha_f32_mfma_vs_oracle(gpu, d, causal):
    """The dense baseline (tpa/mha.py:23-37) through the same kernel."""
    from tpa.mha import _mha_fwd

    b, lq, lk, h = 2, 320, 450, 3
    rng = np.random.Generator(np.random.Philox(17))
    q = rng.standard_normal((b, lq, h, d))
    k = rng.standard_normal((b, lk, h, d))
    v = rng.standard_normal((b, lk, h, d))
    tq, tk, tv = (to_gpu(x, torch.float32, gpu) for x in (q, k, v))
    o, (lse, *_) = _mha_fwd(tq, tk, tv, None, d**-0.5, causal=causal, kernel=2)
    bias = np.where(np.tril(np.ones((lq, lk), bool)), 0.0, -np.inf)[None].repeat(b, 0) if causal else None
    o_ref, l_ref = orc.mha_forward(as_f64(tq), as_f64(tk), as_f64(tv), bias, d**-0.5)
    check(o, lse, o_ref, l_ref, F32_TOL)


def test_f32_mfma_few_query_rows_and_refusals(gpu):
    from tpa import _dispatch as dsp
    from tpa import tpa

    # a handful of query rows over a short cache (no decode route below 1024 keys): still the
    # matrix-core kernel, whose waves without rows only help rebuild the tiles
    q, k, v = make_factors(18, 2, 3, 500, 2, 64, 64, 2, 2)
    tq, tk, tv = (to_gpu(x, torch.float32, gpu) for x in (q, k, v))
    o, lse = tpa.tpa_factors(*split(tq, tk, tv, 2), sm_scale=0.125, kernel=2, use_workspace=False)
    o_ref, l_ref = orc.tpa_reference(q, k, v, None, None, 2, sm_scale=0.125)
    check(o, lse, o_ref, l_ref, F32_TOL)
    # a head size the matrix-core kernels do not take: explicit request refused, default falls back
    q, k, v = make_factors(19, 1, 70, 90, 2, 32, 32, 2, 2)
    tq, tk, tv = (to_gpu(x, torch.float32, gpu) for x in (q, k, v))
    with pytest.raises(dsp.TpaError) as e:
        tpa.tpa_factors(*split(tq, tk, tv, 2), sm_scale=0.125, kernel=2)
    assert e.value.code == -6
    o, lse = tpa.tpa_factors(*split(tq, tk, tv, 2), sm_scale=0.125)
    o_ref, l_ref = orc.tpa_reference(q, k, v, None, None, 2, sm_scale=0.125)
    check(o, lse, o_ref, l_ref, F32_TOL)


# ---------------------------------------------------------------- fp32 decode over the factored cache
def _decode_f32(gpu, q, k, v, h, sm_scale, num_splits=0, kernel=2, **kw):
    from tpa import tpa

    tq, tk, tv = (to_gpu(x, torch.float32, gpu) for x in (q, k, v))
    o, lse = tpa.tpa_decode(*split(tq, tk, tv, h), sm_scale=sm_scale, num_splits=num_splits, kernel=kernel, **kw)
    return (tq, tk, tv), o, lse


@pytest.mark.parametrize("d", [128, 64])
@pytest.mark.parametrize(
    "b,lq,lk,h,rq,rk",
    [
        (3, 1, 1024, 32, 6, 2),
        (2, 1, 1000, 32, 6, 2),  # cache length not a multiple of the block
        (2, 1, 37, 32, 6, 2),    # shorter than one block per wave
        (1, 2, 777, 16, 3, 1),   # two query tokens, 16 heads, rank 1
        (1, 1, 515, 64, 2, 4),   # two head blocks, rank 4
        (2, 1, 640, 5, 6, 2),    # a head count that is no multiple of anything
    ],
)
def test_decode_f32_mfma(gpu, d, b, lq, lk, h, rq, rk):
    q, k, v = make_factors(26, b, lq, lk, h, d, d, rq, rk)
    scale = d**-0.5
    _, o, lse = _decode_f32(gpu, q, k, v, h, scale)
    assert o.dtype == torch.float32
    o_ref, l_ref = orc.tpa_reference(q, k, v, None, None, h, sm_scale=scale)
    check(o, lse, o_ref, l_ref, F32_TOL)


def test_decode_f32_split_invariance_and_vector_kernel(gpu):
    b, lk, h, d = 2, 2048, 32, 128
    q, k, v = make_factors(28, b, 1, lk, h, d, d, 6, 2)
    scale = d**-0.5
    o_ref, l_ref = orc.tpa_reference(q, k, v, None, None, h, sm_scale=scale)
    results = []
    for s in (1, 2, 3, 8):
        _, o, lse = _decode_f32(gpu, q, k, v, h, scale, num_splits=s)
        check(o, lse, o_ref, l_ref, F32_TOL)
        results.append((as_f64(o), as_f64(lse)))
    for o, lse in results[1:]:  # any number of key ranges: the same answer up to fp32 re-association
        assert np.abs(o - results[0][0]).max() <= 1e-5 and np.abs(lse - results[0][1]).max() <= 1e-5
    _, og, lg = _decode_f32(gpu, q, k, v, h, scale, kernel=1)  # the vector-ALU kernel on the same inputs
    assert np.abs(as_f64(og) - results[0][0]).max() <= F32_TOL and np.abs(as_f64(lg) - results[0][1]).max() <= F32_TOL


def test_decode_f32_per_sequence_cache_lengths(gpu):
    """A padded fp32 cache: entry b reads only its first kv_lengths[b] tokens (the padding is NaN)."""
    from tpa import tpa

    b, lk, h, d, rk = 5, 3000, 32, 128, 2
    lengths = [3000, 1777, 9, 640, 0]
    q, k, v = make_factors(29, b, 1, lk, h, d, d, 6, rk)
    tq, tk, tv = (to_gpu(x, torch.float32, gpu) for x in (q, k, v))
    for bi, n in enumerate(lengths):
        tk[bi, n:] = float("nan")
        tv[bi, n:] = float("nan")
    o, lse = tpa.tpa_decode(*split(tq, tk, tv, h), sm_scale=d**-0.5, kv_lengths=torch.tensor(lengths, dtype=torch.int32), kernel=2)
    o_ref, l_ref = _varlen_reference(as_f64(tq), np.nan_to_num(as_f64(tk)), np.nan_to_num(as_f64(tv)), lengths, h, d**-0.5, False)
    check(o, lse, o_ref, l_ref, F32_TOL)


def test_tpa_entry_point_serves_fp32_decode_with_the_split_key_kernel(gpu):
    """tpa() with one query token over a long fp32 cache: the library's decode route (it gets a
    workspace from the wrapper); the result equals the explicit tpa_decode call bit for bit."""
    from tpa import tpa

    b, lk, h, d = 2, 4096, 32, 128
    q, k, v = make_factors(30, b, 1, lk, h, d, d, 6, 2)
    tq, tk, tv = (to_gpu(x, torch.float32, gpu) for x in (q, k, v))
    o = tpa.tpa(tq, tk, tv, num_heads=h, sm_scale=d**-0.5)
    o2, _ = tpa.tpa_decode(*split(tq, tk, tv, h), sm_scale=d**-0.5, kernel=2)
    assert torch.equal(o, o2)
    o_ref, _ = orc.tpa_reference(q, k, v, None, None, h, sm_scale=d**-0.5)
    assert np.abs(as_f64(o) - o_ref).max() <= F32_TOL


# ---------------------------------------------------------------- random problems
@pytest.mark.parametrize("seed", range(12))
def test_random_shapes_f32_mfma_forward_and_backward(gpu, seed):
    """Random problems the fp32 matrix-core kernels take, forward and backward (kernel=2 makes a
    silent fallback an error): any lengths, head counts, ranks, masks."""
    from tpa import tpa

    rng = np.random.default_rng(7000 + seed)
    b, lq, lk = int(rng.integers(1, 4)), int(rng.integers(64, 700)), int(rng.integers(64, 700))
    h, d = int(rng.integers(1, 6)), int(rng.choice([64, 128]))
    rq, rk = int(rng.integers(1, 7)), int(rng.integers(1, 6))
    causal = bool(rng.integers(0, 2))
    seg = int(rng.integers(20, 400)) if rng.integers(0, 3) == 0 else None
    q, k, v = make_factors(8000 + seed, b, lq, lk, h, d, d, rq, rk)
    do = rng.standard_normal((b, lq, h, d)).astype(np.float32)
    qseg = segment_ids(lq, seg, b) if seg else None
    kvseg = segment_ids(lk, seg, b) if seg else None
    tq, tk, tv, tdo = (to_gpu(x, torch.float32, gpu) for x in (q, k, v, do))
    tqs = torch.from_numpy(qseg).to(gpu) if seg else None
    tks = torch.from_numpy(kvseg).to(gpu) if seg else None
    # the head factors sit at 4 h bytes into a row: split copies keep the B factors 16-byte aligned
    parts = split(tq, tk, tv, h)
    o, lse = tpa.tpa_factors(*parts, tqs, tks, d**-0.5, causal, 2)
    o_ref, l_ref = orc.tpa_reference(q, k, v, qseg, kvseg, h, sm_scale=d**-0.5, causal=causal)
    check(o, lse, o_ref, l_ref, F32_TOL)
    grads = tpa.tpa_factors_bwd(*parts, tqs, tks, o, lse, tdo, d**-0.5, causal, kernel=2)
    want = orc.tpa_backward(q, k, v, qseg, kvseg, h, do, sm_scale=d**-0.5, causal=causal)
    for n, w in enumerate(want):
        g = np.concatenate([x.cpu().numpy() for x in grads[2 * n : 2 * n + 2]], axis=-1).astype(np.float64)
        assert np.isfinite(g).all()
        assert np.max(np.abs(g - w)) <= 2e-4 * max(1e-30, np.max(np.abs(w))), "qkv"[n]
