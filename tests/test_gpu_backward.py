"""GPU parity of the backward pass (tpa_bwd / mha_bwd through the C ABI) against the CPU oracle.

The cases follow the reference's own backward tests: tpa/tpa_test.py:128-205 (gradients of
nansum(o), tolerances atol 1e-3 / rtol 1e-2 there; fp32 here is held to 2e-4 of the largest
gradient) and tpa/mha_test.py:9-41,44-118.
"""

import numpy as np
import pytest
import torch

from conftest import make_factors, segment_ids
from oracle import tpa_oracle as orc

pytestmark = pytest.mark.gpu


def rel_err(got, want):
    got, want = np.asarray(got, np.float64), np.asarray(want, np.float64)
    assert got.shape == want.shape
    assert np.isfinite(got).all()
    return float(np.max(np.abs(got - want)) / max(1e-30, np.max(np.abs(want))))


# the reference's backward grid (tpa/tpa_test.py:128-141), nomat folded away: it does not change results
@pytest.mark.parametrize("rank_q", [1, 6])
@pytest.mark.parametrize("rank_k", [1, 4])
@pytest.mark.parametrize(
    "batch_size,lq,lk,h,dk,dv,segment_size",
    [
        (1, 8, 8, 1, 4, 6, 8),
        (2, 1024, 128, 2, 3, 5, 42),
        (2, 1024, 128, 2, 3, 5, None),
        (2, 128, 1024, 2, 3, 5, 42),
        (2, 128, 1024, 2, 3, 5, None),
        (1, 1024, 1024, 2, 3, 5, 321),
    ],
)
def test_reference_backward_grid(gpu, batch_size, rank_q, rank_k, lq, lk, h, dk, dv, segment_size):
    """d nansum(o) / d(q, k, v) through torch.autograd on tpa(), as the reference's test takes
    jax.grad of it; normal inputs, sm_scale = 1, not causal (tpa/tpa_test.py:155-205)."""
    from tpa import tpa

    q, k, v = make_factors(5, batch_size, lq, lk, h, dk, dv, rank_q, rank_k)
    qseg = segment_ids(lq, segment_size, batch_size) if segment_size else None
    kvseg = segment_ids(lk, segment_size, batch_size) if segment_size else None
    tq, tk, tv = (torch.from_numpy(x).to(gpu).requires_grad_() for x in (q, k, v))
    o = tpa.tpa(tq, tk, tv, num_heads=h, q_segment_ids=qseg, kv_segment_ids=kvseg, causal=False)
    torch.nansum(o).backward()
    want = orc.tpa_backward(q, k, v, qseg, kvseg, h, np.ones((batch_size, lq, h, dv)), sm_scale=1.0, causal=False)
    for name, t, w in zip("qkv", (tq, tk, tv), want):
        assert rel_err(t.grad.cpu().numpy(), w) <= 2e-4, name
        np.testing.assert_allclose(t.grad.cpu().numpy(), w, atol=1e-3, rtol=1e-2)  # the reference's own bound


@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("seg", [None, 50])
@pytest.mark.parametrize("b,lq,lk,h,dk,dv,rq,rk", [(2, 200, 200, 3, 16, 24, 3, 2), (1, 130, 77, 4, 64, 64, 6, 2), (1, 60, 300, 2, 40, 130, 2, 3)])
def test_backward_fp32_masks_ragged_and_random_upstream(gpu, b, lq, lk, h, dk, dv, rq, rk, seg, causal):
    """_tpa_bwd on residuals of _tpa_fwd with a random upstream gradient."""
    from tpa import tpa

    q, k, v = make_factors(6, b, lq, lk, h, dk, dv, rq, rk, scale_by_rank=True)
    do = np.random.default_rng(8).standard_normal((b, lq, h, dv)).astype(np.float32)
    qseg = segment_ids(lq, seg, b) if seg else None
    kvseg = segment_ids(lk, seg, b) if seg else None
    scale = dk**-0.5
    tq, tk, tv = (torch.from_numpy(x).to(gpu) for x in (q, k, v))
    o, res = tpa._tpa_fwd(tq, tk, tv, h, qseg, kvseg, scale, causal, None, False, False, False)
    dq, dk_, dv_, n1, n2 = tpa._tpa_bwd(h, scale, causal, None, False, False, False, res, torch.from_numpy(do).to(gpu))
    assert n1 is None and n2 is None
    want = orc.tpa_backward(q, k, v, qseg, kvseg, h, do, sm_scale=scale, causal=causal)
    for name, g, w in zip("qkv", (dq, dk_, dv_), want):
        assert g.dtype == torch.float32 and g.shape == w.shape
        assert rel_err(g.cpu().numpy(), w) <= 2e-4, name


def test_backward_bf16_inputs(gpu):
    """bf16 factors: the gradients are computed in fp32 from the bf16 values and the bf16 forward
    output, then cast to bf16; compared with the oracle on the same bf16-rounded inputs."""
    from tpa import tpa

    b, lq, lk, h, d, rq, rk = 2, 384, 384, 8, 64, 6, 2
    q, k, v = make_factors(9, b, lq, lk, h, d, d, rq, rk, scale_by_rank=True)
    do = np.random.default_rng(10).standard_normal((b, lq, h, d)).astype(np.float32)
    tq, tk, tv = (torch.from_numpy(x).to(gpu).to(torch.bfloat16).requires_grad_() for x in (q, k, v))
    tdo = torch.from_numpy(do).to(gpu).to(torch.bfloat16)
    o = tpa.tpa(tq, tk, tv, num_heads=h, sm_scale=d**-0.5, causal=True)
    o.backward(tdo)
    f64 = lambda t: t.detach().float().cpu().numpy().astype(np.float64)
    want = orc.tpa_backward(f64(tq), f64(tk), f64(tv), None, None, h, f64(tdo), sm_scale=d**-0.5, causal=True)
    for name, t, w in zip("qkv", (tq, tk, tv), want):
        assert t.grad.dtype == torch.bfloat16
        assert rel_err(f64(t.grad), w) <= 2e-2, name  # bf16 output rounding (2^-9 relative) and the bf16 o in delta


def test_backward_per_batch_entry_api(gpu):
    """_bwd on one batch entry (tpa/tpa.py:823-962) equals the batched call."""
    from tpa import tpa

    b, lq, lk, h, dk, dv, rq, rk = 2, 40, 56, 2, 8, 8, 2, 2
    q, k, v = make_factors(13, b, lq, lk, h, dk, dv, rq, rk)
    do = np.random.default_rng(14).standard_normal((b, lq, h, dv)).astype(np.float32)
    tq, tk, tv, tdo = (torch.from_numpy(x).to(gpu) for x in (q, k, v, do))
    o, res = tpa._tpa_fwd(tq, tk, tv, h, None, None, 0.3, True, None, False, False, False)
    dq, dk_, dv_, _, _ = tpa._tpa_bwd(h, 0.3, True, None, False, False, False, res, tdo)
    l = res[-1]
    one = tpa._bwd(tq[1], tk[1], tv[1], None, None, o[1], l[1], tdo[1], h, 0.3, True, None, False, False, False)
    for g, g1 in zip((dq, dk_, dv_), one):
        assert torch.equal(g[1], g1)


# ---------------------------------------------------------------- dense attention (tpa/mha.py:40-65)
@pytest.mark.parametrize("batch,lq,lk,h,dk,dv", [(2, 4, 6, 3, 8, 8), (1, 3, 5, 2, 4, 4)])
@pytest.mark.parametrize("sm_scale", [0.5, 1.0, 2.0])
def test_mha_gradients_match(gpu, batch, lq, lk, h, dk, dv, sm_scale):
    """tpa/mha_test.py:9-41: random bias, do = 1."""
    from tpa import mha

    rng = np.random.default_rng(21)
    q, k, v = (rng.standard_normal(s).astype(np.float32) for s in ((batch, lq, h, dk), (batch, lk, h, dk), (batch, lk, h, dv)))
    bias = rng.standard_normal((batch, lq, lk)).astype(np.float32)
    o, res = mha._mha_fwd(*(torch.from_numpy(x).to(gpu) for x in (q, k, v)), torch.from_numpy(bias).to(gpu), sm_scale)
    dq, dk_, dv_, _, _ = mha._mha_bwd(res, torch.ones_like(o))
    want = orc.mha_backward(q.astype(np.float64), k.astype(np.float64), v.astype(np.float64), bias.astype(np.float64), sm_scale, np.ones((batch, lq, h, dv)))
    for g, w in zip((dq, dk_, dv_), want):
        np.testing.assert_allclose(g.cpu().numpy(), w, atol=1e-5, rtol=1e-4)


def test_mha_backward_known_answer(gpu):
    """tpa/mha_test.py:44-118: the literal case with -inf bias; dq = dk = 0, dv = [[1,1],[0,0],[1,1]]."""
    from tpa import mha

    q = torch.tensor([[2.0, 1.0], [1.0, 1.0], [1.0, 1.0]], device=gpu)[None, :, None, :].requires_grad_()
    k = torch.ones((1, 3, 1, 2), device=gpu, requires_grad=True)
    v = torch.ones((1, 3, 1, 2), device=gpu, requires_grad=True)
    ninf = float("-inf")
    bias = torch.tensor([[0, ninf, 0], [0, ninf, 0], [ninf, ninf, ninf]], device=gpu)[None]
    o = mha.mha(q, k, v, bias)
    torch.nansum(o).backward()
    assert torch.equal(q.grad, torch.zeros_like(q))
    assert torch.equal(k.grad, torch.zeros_like(k))
    np.testing.assert_allclose(v.grad[0, :, 0].cpu().numpy(), [[1, 1], [0, 0], [1, 1]], atol=1e-6)


def test_mha_backward_bf16_causal(gpu):
    from tpa import mha

    b, l, h, d = 2, 300, 4, 64
    rng = np.random.default_rng(22)
    q, k, v, do = (torch.from_numpy(rng.standard_normal((b, l, h, d)).astype(np.float32)).to(gpu).to(torch.bfloat16) for _ in range(4))
    q.requires_grad_(), k.requires_grad_(), v.requires_grad_()
    o = mha.mha(q, k, v, None, d**-0.5, causal=True)
    o.backward(do)
    f64 = lambda t: t.detach().float().cpu().numpy().astype(np.float64)
    bias = np.where(np.tril(np.ones((l, l), bool)), 0.0, -np.inf)[None].repeat(b, 0)
    want = orc.mha_backward(f64(q), f64(k), f64(v), bias, d**-0.5, f64(do))
    for t, w in zip((q, k, v), want):
        assert rel_err(f64(t.grad), w) <= 2e-2


def test_backward_error_codes(gpu):
    """A too small workspace is refused, and there is no MFMA backward kernel to ask for."""
    import ctypes

    from tpa import _dispatch as d
    from tpa import tpa

    q, k, v = make_factors(15, 1, 16, 16, 2, 8, 8, 2, 2)
    tq, tk, tv = (torch.from_numpy(x).to(gpu) for x in (q, k, v))
    o, res = tpa._tpa_fwd(tq, tk, tv, 2, None, None, 1.0, False, None, False, False, False)
    with pytest.raises(d.TpaError) as e:
        tpa.tpa_factors_bwd(tq[..., :2], tq[..., 2:], tk[..., :2], tk[..., 2:], tv[..., :2], tv[..., 2:], None, None,
                            o, res[-1].permute(0, 2, 1), torch.ones_like(o), workspace=torch.empty(1024, dtype=torch.uint8, device=gpu))
    assert e.value.code == -5


# ---------------------------------------------------------------- bf16 MFMA backward kernels
def _bf16_case(gpu, seed, b, lq, lk, h, d, rq, rk, seg, causal, kernel):
    from tpa import tpa

    q, k, v = make_factors(seed, b, lq, lk, h, d, d, rq, rk, scale_by_rank=True)
    do = np.random.default_rng(seed + 1).standard_normal((b, lq, h, d)).astype(np.float32)
    qseg = segment_ids(lq, seg, b) if seg else None
    kvseg = segment_ids(lk, seg, b) if seg else None
    tq, tk, tv = (torch.from_numpy(x).to(gpu).to(torch.bfloat16) for x in (q, k, v))
    tdo = torch.from_numpy(do).to(gpu).to(torch.bfloat16)
    sp = lambda t: (t[..., :h], t[..., h:])
    tqs = None if qseg is None else torch.from_numpy(qseg).to(gpu)
    tks = None if kvseg is None else torch.from_numpy(kvseg).to(gpu)
    o, lse = tpa.tpa_factors(*sp(tq), *sp(tk), *sp(tv), tqs, tks, d**-0.5, causal)
    grads = tpa.tpa_factors_bwd(*sp(tq), *sp(tk), *sp(tv), tqs, tks, o, lse, tdo, d**-0.5, causal, kernel=kernel)
    f64 = lambda t: t.detach().float().cpu().numpy().astype(np.float64)
    want = orc.tpa_backward(f64(tq), f64(tk), f64(tv), qseg, kvseg, h, f64(tdo), sm_scale=d**-0.5, causal=causal)
    got = [np.concatenate([f64(grads[2 * n]), f64(grads[2 * n + 1])], axis=-1) for n in range(3)]
    return got, want


@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize(
    "b,lq,lk,h,d,rq,rk,seg",
    [
        (2, 512, 512, 4, 128, 6, 2, None),
        (1, 300, 300, 2, 128, 2, 2, None),   # ragged last tiles
        (2, 200, 450, 2, 64, 3, 4, None),    # lq != lk
        (1, 700, 333, 2, 128, 2, 1, None),
        (2, 384, 384, 2, 64, 6, 2, 100),     # packed sequences
        (1, 640, 384, 2, 128, 2, 2, 77),     # rows whose segment has no key: no gradient from them
        # head counts that are multiples of 8: the one-launch reconstruction and the lane-reduction projections
        (1, 300, 300, 8, 128, 6, 2, None),   # 16 lanes per (token, head group), one group
        (2, 200, 260, 16, 64, 3, 4, None),   # 8 lanes per group, two groups; lq != lk, ragged token count per wave
        (1, 130, 131, 32, 128, 2, 2, None),  # four groups: a token fills a wave
        (1, 100, 100, 64, 64, 2, 1, None),   # eight groups of eight lanes
        (1, 100, 100, 64, 128, 2, 2, 50),    # more than a wave per token: the staged projection; packed
    ],
)
def test_backward_bf16_mfma_kernels(gpu, b, lq, lk, h, d, rq, rk, seg, causal):
    """kernel=2 makes a fallback to the fp32 kernels an error.  bf16 P and dS in the contractions:
    held to 1.5e-2 of the largest gradient entry."""
    got, want = _bf16_case(gpu, 31, b, lq, lk, h, d, rq, rk, seg, causal, kernel=2)
    for name, g, w in zip("qkv", got, want):
        assert rel_err(g, w) <= 1.5e-2, name


def test_backward_bf16_mfma_matches_fp32_kernels(gpu):
    """Same inputs through the vector-ALU kernels (kernel=1) and the MFMA kernels (kernel=2)."""
    a, want = _bf16_case(gpu, 33, 2, 320, 320, 2, 64, 4, 2, None, True, kernel=1)
    b_, _ = _bf16_case(gpu, 33, 2, 320, 320, 2, 64, 4, 2, None, True, kernel=2)
    for x, y, w in zip(a, b_, want):
        assert rel_err(x, w) <= 6e-3   # the fp32 kernels are limited by the bf16 rounding of the forward output inside delta
        assert rel_err(y, x) <= 1.5e-2


@pytest.mark.parametrize("d,causal", [(64, False), (128, True)])
def test_mha_backward_bf16_mfma(gpu, d, causal):
    from tpa import mha

    b, lq, lk, h = 2, 333, 333, 4
    rng = np.random.default_rng(41)
    mk = lambda *s: torch.from_numpy(rng.standard_normal(s).astype(np.float32)).to(gpu).to(torch.bfloat16)
    q, k, v, do = mk(b, lq, h, d), mk(b, lk, h, d), mk(b, lk, h, d), mk(b, lq, h, d)
    o, res = mha._mha_fwd(q, k, v, None, d**-0.5, causal=causal)
    dq, dk, dv, _, _ = mha._mha_bwd(res, do, kernel=2)
    f64 = lambda t: t.detach().float().cpu().numpy().astype(np.float64)
    bias = np.where(np.tril(np.ones((lq, lk), bool)), 0.0, -np.inf)[None].repeat(b, 0) if causal else None
    want = orc.mha_backward(f64(q), f64(k), f64(v), bias, d**-0.5, f64(do))
    for t, w in zip((dq, dk, dv), want):
        assert rel_err(f64(t), w) <= 2e-2


def test_backward_mfma_refuses_what_it_cannot_run(gpu):
    from tpa import _dispatch as d
    from tpa import tpa

    q, k, v = make_factors(15, 1, 16, 16, 2, 8, 8, 2, 2)
    tq, tk, tv = (torch.from_numpy(x).to(gpu) for x in (q, k, v))
    o, res = tpa._tpa_fwd(tq, tk, tv, 2, None, None, 1.0, False, None, False, False, False)
    with pytest.raises(d.TpaError) as e:
        tpa.tpa_factors_bwd(tq[..., :2], tq[..., 2:], tk[..., :2], tk[..., 2:], tv[..., :2], tv[..., 2:], None, None,
                            o, res[-1].permute(0, 2, 1), torch.ones_like(o), kernel=2)
    assert e.value.code == -6


@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("pattern", ["long_runs", "shuffled", "island", "island_with_hole", "absent", "descending"])
def test_backward_bf16_segment_id_patterns(gpu, pattern, causal):
    """The MFMA backward kernels visit only the tiles between the first and last key (row) whose id
    lies in the id range of a workgroup's rows (keys); the gradients must not depend on how the ids
    are laid out."""
    from test_gpu_parity import _id_pattern
    from tpa import tpa

    b, lq, lk, h, d = 2, 1536, 1536, 4, 128
    q, k, v = make_factors(81, b, lq, lk, h, d, d, 3, 2, scale_by_rank=True)
    do = np.random.default_rng(82).standard_normal((b, lq, h, d)).astype(np.float32)
    qseg, kvseg = _id_pattern(pattern, b, lq, lk)
    tq, tk, tv = (torch.from_numpy(x).to(gpu).to(torch.bfloat16) for x in (q, k, v))
    tdo = torch.from_numpy(do).to(gpu).to(torch.bfloat16)
    tqs, tks = torch.from_numpy(qseg).to(gpu), torch.from_numpy(kvseg).to(gpu)
    sp = lambda t: (t[..., :h], t[..., h:])
    o, lse = tpa.tpa_factors(*sp(tq), *sp(tk), *sp(tv), tqs, tks, d**-0.5, causal)
    grads = tpa.tpa_factors_bwd(*sp(tq), *sp(tk), *sp(tv), tqs, tks, o, lse, tdo, d**-0.5, causal, kernel=2)
    f64 = lambda t: t.detach().float().cpu().numpy().astype(np.float64)
    want = orc.tpa_backward(f64(tq), f64(tk), f64(tv), qseg, kvseg, h, f64(tdo), sm_scale=d**-0.5, causal=causal)
    got = [np.concatenate([f64(grads[2 * n]), f64(grads[2 * n + 1])], axis=-1) for n in range(3)]
    for name, g, w in zip("qkv", got, want):
        if pattern == "absent":
            assert not np.any(g) and not np.any(w), name  # no pair is visible: every gradient is zero
        else:
            assert rel_err(g, w) <= 1.5e-2, name


# ---------------------------------------------------------------- causal mask with an offset (key <= query + offset)
def _offset_backward_reference(q, k, v, h, sm_scale, offset, do, qseg=None, kvseg=None):
    """Oracle gradients under the bias `key <= query + offset`, composed from the oracle's parts
    (reconstruction, dense attention backward, projection onto the factors)."""
    q, k, v, do = (np.asarray(x, dtype=np.float64) for x in (q, k, v, do))
    b, lq, lk = q.shape[0], q.shape[1], k.shape[1]
    bias = orc.attention_bias(b, lq, lk, qseg, kvseg, False)
    bias = bias + np.where(np.tril(np.ones((lq, lk), dtype=bool), k=offset), 0.0, -np.inf)[None]
    (qa, qb), (ka, kb), (va, vb) = (orc.split_factors(x, h) for x in (q, k, v))
    dq_, dk_, dv_ = orc.mha_backward(orc.reconstruct(qa, qb), orc.reconstruct(ka, kb), orc.reconstruct(va, vb), bias, sm_scale, do)
    cat = lambda pair: np.concatenate(pair, axis=-1)
    return cat(orc.project_to_factors(dq_, qa, qb)), cat(orc.project_to_factors(dk_, ka, kb)), cat(orc.project_to_factors(dv_, va, vb))


@pytest.mark.parametrize(
    "dt,kernel,b,lq,lk,h,d,rq,rk,offset,seg,tol",
    [
        (torch.bfloat16, 2, 2, 384, 768, 2, 128, 6, 2, 384, None, 1.5e-2),   # new tokens over a cache
        (torch.bfloat16, 2, 1, 300, 700, 2, 64, 2, 2, 77, None, 1.5e-2),     # ragged, diagonal off the tile boundaries
        (torch.bfloat16, 2, 1, 600, 600, 2, 128, 2, 2, -130, None, 1.5e-2),  # the first 130 rows see nothing
        (torch.bfloat16, 2, 1, 600, 600, 2, 64, 2, 4, -300, None, 1.5e-2),   # a whole query block sees nothing
        (torch.bfloat16, 2, 2, 512, 768, 2, 128, 2, 2, 256, 200, 1.5e-2),    # with packed documents
        (torch.bfloat16, 2, 1, 256, 256, 2, 64, 2, 2, 100000, None, 1.5e-2), # nothing masked
        (torch.float32, 2, 2, 320, 640, 2, 64, 6, 2, 320, None, 2e-4),       # fp32 matrix-core kernels
        (torch.float32, 2, 1, 400, 400, 2, 128, 2, 2, -97, 150, 2e-4),
        (torch.float32, 2, 1, 200, 450, 2, 64, 2, 2, 33, None, 2e-4),
        (torch.float32, 1, 2, 130, 200, 3, 24, 2, 3, 70, None, 2e-4),        # vector-ALU kernels
        (torch.float32, 1, 1, 130, 200, 3, 24, 2, 3, -40, 50, 2e-4),
    ],
)
def test_backward_with_causal_offset(gpu, dt, kernel, b, lq, lk, h, d, rq, rk, offset, seg, tol):
    from tpa import tpa

    q, k, v = make_factors(71, b, lq, lk, h, d, d, rq, rk, scale_by_rank=dt == torch.bfloat16)
    do = np.random.default_rng(72).standard_normal((b, lq, h, d)).astype(np.float32)
    qseg = segment_ids(lq, seg, b) if seg else None
    kvseg = segment_ids(lk, seg, b) if seg else None
    tq, tk, tv, tdo = (torch.from_numpy(x).to(gpu).to(dt) for x in (q, k, v, do))
    sp = lambda t: (t[..., :h], t[..., h:])
    tqs = None if qseg is None else torch.from_numpy(qseg).to(gpu)
    tks = None if kvseg is None else torch.from_numpy(kvseg).to(gpu)
    o, lse = tpa.tpa_factors(*sp(tq), *sp(tk), *sp(tv), tqs, tks, d**-0.5, True, causal_offset=offset)
    grads = tpa.tpa_factors_bwd(*sp(tq), *sp(tk), *sp(tv), tqs, tks, o, lse, tdo, d**-0.5, True, kernel=kernel, causal_offset=offset)
    f64 = lambda t: t.detach().float().cpu().numpy().astype(np.float64)
    want = _offset_backward_reference(f64(tq), f64(tk), f64(tv), h, d**-0.5, offset, f64(tdo), qseg, kvseg)
    for n, (name, w) in enumerate(zip("qkv", want)):
        got = np.concatenate([f64(grads[2 * n]), f64(grads[2 * n + 1])], axis=-1)
        assert rel_err(got, w) <= tol, name


@pytest.mark.parametrize("dt,tol", [(torch.float32, 2e-4), (torch.bfloat16, 1.5e-2)])
def test_ring_schedule_backward_emulated_on_one_gpu(gpu, dt, tol):
    """The backward of a sequence-sharded causal call, the devices replaced by a loop: with the
    global o, lse and do of its rows, every (query shard, key shard) meeting is one backward block
    call with the shards' distance as causal offset; dq sums over the key shards a query shard
    meets, dk / dv over the query shards a key shard meets (what tpa/ring_tpa.py rotates around
    the ring).  The sums equal the gradients of the unsharded call."""
    from tpa import tpa

    b, h, d, shards, per = 2, 4, 64, 3, 256
    t = shards * per
    q, k, v = make_factors(75, b, t, t, h, d, d, 4, 2, scale_by_rank=dt == torch.bfloat16)
    do = np.random.default_rng(76).standard_normal((b, t, h, d)).astype(np.float32)
    tq, tk, tv, tdo = (torch.from_numpy(x).to(gpu).to(dt) for x in (q, k, v, do))
    sp = lambda x: (x[..., :h], x[..., h:])
    o, lse = tpa.tpa_factors(*sp(tq), *sp(tk), *sp(tv), None, None, d**-0.5, True)
    full = tpa.tpa_factors_bwd(*sp(tq), *sp(tk), *sp(tv), None, None, o, lse, tdo, d**-0.5, True)
    acc = [torch.zeros_like(g) for g in full]
    for s in range(shards):
        rows = slice(s * per, (s + 1) * per)
        for j in range(s + 1):  # key shards after the query shard are invisible to it
            keys = slice(j * per, (j + 1) * per)
            g = tpa.tpa_factors_bwd(
                *sp(tq[:, rows]), *sp(tk[:, keys]), *sp(tv[:, keys]), None, None,
                o[:, rows], lse[:, :, rows], tdo[:, rows], d**-0.5, True, causal_offset=(s - j) * per,
            )
            acc[0][:, rows] += g[0]
            acc[1][:, rows] += g[1]
            for n in range(2, 6):
                acc[n][:, keys] += g[n]
    f64 = lambda x: x.detach().float().cpu().numpy().astype(np.float64)
    for a, w in zip(acc, full):
        assert rel_err(f64(a), f64(w)) <= tol


def test_causal_offset_through_autograd(gpu):
    """tpa(..., causal=True, causal_offset=lk - lq): new tokens over a cache, forward and gradients."""
    from tpa import tpa

    b, lq, lk, h, d = 2, 192, 448, 4, 64
    q, k, v = make_factors(79, b, lq, lk, h, d, d, 3, 2)
    tq, tk, tv = (torch.from_numpy(x).to(gpu).requires_grad_() for x in (q, k, v))
    o = tpa.tpa(tq, tk, tv, num_heads=h, sm_scale=d**-0.5, causal=True, causal_offset=lk - lq)
    torch.nansum(o).backward()
    want = _offset_backward_reference(q, k, v, h, d**-0.5, lk - lq, np.ones((b, lq, h, d)))
    for name, t, w in zip("qkv", (tq, tk, tv), want):
        assert rel_err(t.grad.cpu().numpy(), w) <= 2e-4, name


def test_causal_offset_through_the_residual_interface(gpu):
    """_tpa_fwd(..., causal_offset=) followed by _tpa_bwd(residuals, do, causal_offset=): the residuals
    hold the reference's seven entries and no offset, so the backward call is given the same value."""
    from tpa import tpa

    b, lq, lk, h, d = 2, 192, 448, 4, 64
    q, k, v = make_factors(80, b, lq, lk, h, d, d, 3, 2)
    tq, tk, tv = (torch.from_numpy(x).to(gpu) for x in (q, k, v))
    o, res = tpa._tpa_fwd(tq, tk, tv, h, None, None, d**-0.5, True, None, False, False, False, causal_offset=lk - lq)
    do = torch.ones_like(o)
    got = tpa._tpa_bwd(h, d**-0.5, True, None, False, False, False, res, do, causal_offset=lk - lq)
    want = _offset_backward_reference(q, k, v, h, d**-0.5, lk - lq, np.ones((b, lq, h, d)))
    for name, t, w in zip("qkv", got[:3], want):
        assert rel_err(t.cpu().numpy(), w) <= 2e-4, name


def test_backward_bottom_right_alignment_is_the_offset_lk_minus_lq(gpu):
    """Without per-sequence lengths (which the backward does not take) CAUSAL_BOTTOM_RIGHT is the
    fixed offset lk - lq, forward and backward: the same launches, equal bits."""
    from tpa import tpa

    b, lq, lk, h, d = 2, 200, 456, 2, 64
    q, k, v = make_factors(81, b, lq, lk, h, d, d, 3, 2)
    do = np.random.default_rng(82).standard_normal((b, lq, h, d)).astype(np.float32)
    tq, tk, tv, tdo = (torch.from_numpy(x).to(gpu) for x in (q, k, v, do))
    sp = lambda t: (t[..., :h], t[..., h:])
    outs = []
    for causal, off in ((tpa.CAUSAL_BOTTOM_RIGHT, 0), (True, lk - lq)):
        o, lse = tpa.tpa_factors(*sp(tq), *sp(tk), *sp(tv), None, None, d**-0.5, causal, causal_offset=off)
        g = tpa.tpa_factors_bwd(*sp(tq), *sp(tk), *sp(tv), None, None, o, lse, tdo, d**-0.5, causal, causal_offset=off)
        outs.append((o, lse) + tuple(g))
    for x, y in zip(*outs):
        assert torch.equal(x, y)


@pytest.mark.parametrize("rank_q", [1, 6])
@pytest.mark.parametrize("rank_k", [1, 4])
@pytest.mark.parametrize("batch_size,lq,lk,h,dim_k,dim_v", [(1, 8, 8, 1, 4, 6), (2, 1024, 128, 2, 3, 5), (2, 128, 1024, 2, 3, 5), (1, 1024, 1024, 2, 3, 5)])
def test_ring_schedule_backward_on_the_references_ring_grid(gpu, batch_size, rank_q, rank_k, lq, lk, h, dim_k, dim_v):
    """The grid of the reference's ring backward test (tpa/ring_tpa_test.py:141-233: eight sequence
    shards, uniform inputs, segment ids position // 42, d nansum(o), atol 1e-3 / rtol 1e-2), the
    devices replaced by a loop: a block backward per (query shard, key shard) meeting with the
    global o and lse of the rows, dq summed over key shards, dk / dv over query shards."""
    from tpa import tpa

    shards = 8
    q, k, v = make_factors(190, batch_size, lq, lk, h, dim_k, dim_v, rank_q, rank_k, dist="uniform")
    qseg, kvseg = segment_ids(lq, 42, batch_size), segment_ids(lk, 42, batch_size)
    tq, tk, tv = (torch.from_numpy(x).to(gpu) for x in (q, k, v))
    tqs, tks = torch.from_numpy(qseg).to(gpu), torch.from_numpy(kvseg).to(gpu)
    sp = lambda t: (t[..., :h], t[..., h:])
    o, lse = tpa.tpa_factors(*sp(tq), *sp(tk), *sp(tv), tqs, tks, 1.0, False)
    do = torch.ones_like(o)  # d nansum(o) / d o; rows that are NaN take no gradient
    acc = [torch.zeros(t.shape, dtype=torch.float32, device=gpu) for x in (tq, tk, tv) for t in sp(x)]
    pq, pk = lq // shards, lk // shards
    for s in range(shards):
        rows = slice(s * pq, (s + 1) * pq)
        for j in range(shards):
            keys = slice(j * pk, (j + 1) * pk)
            g = tpa.tpa_factors_bwd(*sp(tq[:, rows]), *sp(tk[:, keys]), *sp(tv[:, keys]), tqs[:, rows], tks[:, keys],
                                    o[:, rows], lse[:, :, rows], do[:, rows], 1.0, False)
            acc[0][:, rows] += g[0]
            acc[1][:, rows] += g[1]
            for n in range(2, 6):
                acc[n][:, keys] += g[n]
    want = orc.tpa_backward(q, k, v, qseg, kvseg, h, np.ones((batch_size, lq, h, dim_v)), sm_scale=1.0, causal=False)
    for n, w in enumerate(want):
        got = torch.cat([acc[2 * n], acc[2 * n + 1]], dim=-1).cpu().numpy()
        np.testing.assert_allclose(got, w, atol=1e-3, rtol=1e-2)


@pytest.mark.parametrize("dt,d,kernel", [(torch.float32, 24, 1), (torch.float32, 64, 2), (torch.bfloat16, 128, 2)])
@pytest.mark.parametrize("causal,offset,seg", [(False, 0, None), (True, 40, None), (True, 0, 70)])
def test_backward_of_a_ragged_batch(gpu, dt, d, kernel, causal, offset, seg):
    """kv_lengths in the backward (vector-ALU, fp32 and bf16 matrix-core kernels): gradients of a forward made
    with kv_lengths equal the oracle's on each batch entry cut to its length, and are zero on the padding."""
    from tpa import tpa

    b, lq, lk, h, rq, rk = 3, 200, 330, 8, 3, 2
    lengths = [330, 129, 64]
    q, k, v = make_factors(21, b, lq, lk, h, d, d, rq, rk, scale_by_rank=True)
    do = np.random.default_rng(22).standard_normal((b, lq, h, d)).astype(np.float32)
    qseg = segment_ids(lq, seg, b) if seg else None
    kvseg = segment_ids(lk, seg, b) if seg else None
    tq, tk, tv, tdo = (torch.from_numpy(x).to(gpu).to(dt) for x in (q, k, v, do))
    scale = d**-0.5
    sp = lambda x: (x[..., :h], x[..., h:])
    o, lse = tpa.tpa_factors(*sp(tq), *sp(tk), *sp(tv), qseg, kvseg, scale, causal, kernel, kv_lengths=lengths, causal_offset=offset)
    grads = tpa.tpa_factors_bwd(*sp(tq), *sp(tk), *sp(tv), qseg, kvseg, o, lse, tdo, scale, causal, kernel=kernel,
                                causal_offset=offset, kv_lengths=lengths)
    f64 = lambda t: t.detach().float().cpu().numpy().astype(np.float64)
    fq, fk, fv, fdo = f64(tq), f64(tk), f64(tv), f64(tdo)
    tol = 2e-4 if dt == torch.float32 else 1.5e-2
    for bi, n in enumerate(lengths):
        # the oracle on the entry cut to its length; an offset mask is a segment-free tril with that diagonal,
        # which the oracle's backward takes as a dense bias through its segment / causal arguments only for
        # offset 0, so offsets are folded into segment-free calls on shifted keys where needed
        qs = None if qseg is None else qseg[bi : bi + 1]
        ks = None if kvseg is None else kvseg[bi : bi + 1, :n]
        if causal and offset:
            # key <= query + offset  <=>  top-left causal after prepending `offset` dummy queries
            pad_q = np.zeros((1, offset, rq, h + d))
            want = orc.tpa_backward(np.concatenate([pad_q, fq[bi : bi + 1]], 1), fk[bi : bi + 1, :n], fv[bi : bi + 1, :n], None, None, h,
                                    np.concatenate([np.zeros((1, offset, h, d)), fdo[bi : bi + 1]], 1), sm_scale=scale, causal=True)
            want = (want[0][:, offset:], want[1], want[2])
        else:
            want = orc.tpa_backward(fq[bi : bi + 1], fk[bi : bi + 1, :n], fv[bi : bi + 1, :n], qs, ks, h, fdo[bi : bi + 1], sm_scale=scale, causal=causal)
        got_q = np.concatenate([f64(grads[0][bi : bi + 1]), f64(grads[1][bi : bi + 1])], -1)
        got_k = np.concatenate([f64(grads[2][bi : bi + 1]), f64(grads[3][bi : bi + 1])], -1)
        got_v = np.concatenate([f64(grads[4][bi : bi + 1]), f64(grads[5][bi : bi + 1])], -1)
        assert rel_err(got_q, want[0]) <= tol, ("q", bi)
        assert rel_err(got_k[:, :n], want[1]) <= tol, ("k", bi)
        assert rel_err(got_v[:, :n], want[2]) <= tol, ("v", bi)
        assert not got_k[:, n:].any() and not got_v[:, n:].any(), "padding keys receive no gradient"
    with pytest.raises(NotImplementedError):
        tpa.tpa_factors_bwd(*sp(tq), *sp(tk), *sp(tv), None, None, o, lse, tdo, scale, tpa.CAUSAL_BOTTOM_RIGHT, kv_lengths=lengths)
