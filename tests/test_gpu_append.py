"""tpa_cache_append (projections to the rank factors, rotary embedding, append to the factored cache)
through the Python API -> C ABI, against the CPU oracle, and end to end with tpa_decode.

Tolerances: the factors are sums of d_model products of bf16 values accumulated in fp32 and rounded
once to bf16: max-abs <= 2^-8 of the largest factor entry (fp32 inputs: 1e-5 of it).  Decode over
an appended cache against decode over a cache built on the host: bf16 outputs <= 2e-2, logsumexp <= 1e-3.
"""

import numpy as np
import pytest
import torch

from oracle import tpa_oracle as orc
from tpa import tpa

pytestmark = pytest.mark.gpu


def rope_tables(rope_len, d, base=10000.0):
    inv = base ** (-np.arange(0, d, 2, dtype=np.float64) / d)
    ang = np.arange(rope_len, dtype=np.float64)[:, None] * inv[None, :]
    return np.cos(ang).astype(np.float32), np.sin(ang).astype(np.float32)


def f64(t):
    return t.detach().float().cpu().numpy().astype(np.float64)


def make_layer(seed, b, n, dm, h, d, rq, rk, dtype, gpu):
    rng = np.random.Generator(np.random.Philox(seed))
    x = torch.from_numpy(rng.standard_normal((b, n, dm), dtype=np.float32)).to(dtype).to(gpu)
    w = torch.from_numpy(rng.standard_normal((rq * (h + d) + 2 * rk * (h + d), dm), dtype=np.float32) / np.sqrt(dm)).to(dtype).to(gpu)
    return x, w


@pytest.mark.parametrize("dtype,kernel", [(torch.bfloat16, 2), (torch.bfloat16, 1), (torch.float32, 0)])
@pytest.mark.parametrize(
    "b,n,dm,h,d,rq,rk",
    [
        (3, 5, 256, 16, 64, 6, 2),     # 15 tokens: the decode-step kernel (k split over the waves), one k step per wave
        (2, 70, 128, 8, 128, 3, 4),    # 140 tokens: 64 x 64 tiles
        (1, 1, 64, 32, 128, 6, 2),     # d_model too short for the k split: tiles
        (64, 1, 1024, 32, 128, 6, 2),  # a decode step of 64 sequences: all four blocks of 16 tokens
        (7, 3, 512, 8, 64, 2, 1),      # 21 tokens: the second block of 16 is ragged
        (5, 2, 256, 8, 64, 1, 1),      # 216 output columns: the last workgroup owns half a block of columns
        (8, 2, 2048, 16, 128, 2, 2),   # with a workspace: 8 slabs of k, one k step per wave
        (4, 9, 4096, 8, 64, 3, 1),     # 8 slabs, two k steps per wave; 200 columns: the last workgroup owns 8 of its 64
        (2, 3, 1536, 8, 64, 2, 2),     # 2 slabs, three k steps per wave
    ],
)
@pytest.mark.parametrize("use_workspace", [False, True])
def test_append_matches_the_oracle(gpu, dtype, kernel, b, n, dm, h, d, rq, rk, use_workspace):
    """With `use_workspace` a decode step whose d_model is a multiple of 512 runs as two kernels (partial sums of
    2, 4 or 8 slabs of k in the workspace, then a finishing kernel); every other case ignores it."""
    x, w = make_layer(1, b, n, dm, h, d, rq, rk, dtype, gpu)
    if use_workspace and kernel == 2 and b * n <= 64 and dm % 512 == 0:
        slabs = next(sl for sl in (8, 4, 2) if dm % (256 * sl) == 0)
        assert tpa.cache_append_workspace_bytes(b, n, dm, h, d, rq, rk) == slabs * 64 * (rq + 2 * rk) * (h + d) * 4
    cache_len = 96
    cos, sin = rope_tables(256, d)
    lengths = np.array([(7 * i + 3) % (cache_len - n - 1) for i in range(b)], dtype=np.int32)
    caches = [torch.full((b, cache_len, rk, inner), float("nan"), dtype=dtype, device=gpu) for inner in (h, d, h, d)]
    qa, qb, new_len = tpa.tpa_cache_append(x, w, cos, sin, *caches, lengths, rank_q=rq, kernel=kernel, use_workspace=use_workspace)
    pos = lengths[:, None] + np.arange(n)[None, :]
    want = orc.tpa_append_reference(f64(x), f64(w), cos, sin, pos, h, d, rq, rk)
    rel = 2.0**-8 if dtype == torch.bfloat16 else 1e-5
    for name, got in (("qa", qa), ("qb", qb)):
        assert np.abs(f64(got) - want[name]).max() <= rel * np.abs(want[name]).max(), name
    for name, cache in zip(("ka", "kb", "va", "vb"), caches):
        c = f64(cache)
        for bi in range(b):
            rows = c[bi, lengths[bi] : lengths[bi] + n]
            assert np.abs(rows - want[name][bi]).max() <= rel * np.abs(want[name]).max(), name
            # nothing else of the cache was touched
            assert np.isnan(c[bi, : lengths[bi]]).all() and np.isnan(c[bi, lengths[bi] + n :]).all(), name
    assert new_len.cpu().tolist() == (lengths + n).tolist()


def test_append_positions_override_and_capacity(gpu):
    """`positions` replaces kv_lengths[b] + i for the rotation only; tokens past the capacity are dropped."""
    b, n, dm, h, d, rq, rk = 2, 4, 64, 8, 64, 2, 2
    x, w = make_layer(2, b, n, dm, h, d, rq, rk, torch.bfloat16, gpu)
    cos, sin = rope_tables(64, d)
    cache_len = 10
    lengths = np.array([8, 0], dtype=np.int32)  # entry 0 has room for two of its four tokens
    pos = np.array([[40, 41, 42, 43], [0, 9, 9, 63]], dtype=np.int32)
    caches = [torch.full((b, cache_len, rk, inner), float("nan"), dtype=torch.bfloat16, device=gpu) for inner in (h, d, h, d)]
    qa, qb, new_len = tpa.tpa_cache_append(x, w, cos, sin, *caches, lengths, rank_q=rq, positions=pos)
    want = orc.tpa_append_reference(f64(x), f64(w), cos, sin, pos, h, d, rq, rk)
    assert np.abs(f64(qb) - want["qb"]).max() <= 2.0**-8 * np.abs(want["qb"]).max()
    kb = f64(caches[1])
    assert np.abs(kb[0, 8:10] - want["kb"][0, :2]).max() <= 2.0**-8 * np.abs(want["kb"]).max()
    assert np.abs(kb[1, 0:4] - want["kb"][1]).max() <= 2.0**-8 * np.abs(want["kb"]).max()
    assert np.isnan(kb[0, :8]).all() and np.isnan(kb[1, 4:]).all()
    assert new_len.cpu().tolist() == [10, 4]


@pytest.mark.parametrize("paged", [False, True])
def test_append_then_decode_equals_decode_over_a_host_built_cache(gpu, paged):
    """Prefill a cache token by token group (three appends of different sizes), then decode the last
    token: the same through a cache whose factors the oracle computed on the host."""
    b, dm, h, d, rq, rk = 4, 256, 32, 128, 6, 2
    steps = [37, 64, 1]
    total = sum(steps)
    cache_len, page_size = 128, 16
    cos, sin = rope_tables(cache_len, d)
    rng = np.random.Generator(np.random.Philox(3))
    xs = torch.from_numpy(rng.standard_normal((b, total, dm), dtype=np.float32)).to(torch.bfloat16).to(gpu)
    w = torch.from_numpy(rng.standard_normal((rq * (h + d) + 2 * rk * (h + d), dm), dtype=np.float32) / np.sqrt(dm)).to(torch.bfloat16).to(gpu)
    if paged:
        pages_per_seq = cache_len // page_size
        npages = 2 * b * pages_per_seq
        table = torch.from_numpy(np.random.default_rng(4).permutation(npages)[: b * pages_per_seq].astype(np.int32)).reshape(b, pages_per_seq).to(gpu)
        caches = [torch.zeros((npages, page_size, rk, inner), dtype=torch.bfloat16, device=gpu) for inner in (h, d, h, d)]
    else:
        table = None
        caches = [torch.zeros((b, cache_len, rk, inner), dtype=torch.bfloat16, device=gpu) for inner in (h, d, h, d)]
    lengths = torch.zeros(b, dtype=torch.int32, device=gpu)
    t0 = 0
    for n in steps:
        qa, qb, lengths = tpa.tpa_cache_append(xs[:, t0 : t0 + n], w, cos, sin, *caches, lengths, rank_q=rq, page_table=table)
        t0 += n
    assert lengths.cpu().tolist() == [total] * b
    sm_scale = d**-0.5
    o, lse = tpa.tpa_decode(qa, qb, *caches, sm_scale=sm_scale, kv_lengths=lengths, page_table=table, kernel=2)
    # the same layer on the host: factors of all tokens, rounded to bf16 like the cache rows
    pos = np.tile(np.arange(total)[None], (b, 1))
    fac = orc.tpa_append_reference(f64(xs), f64(w), cos, sin, pos, h, d, rq, rk)
    r16 = lambda a: torch.from_numpy(a.astype(np.float32)).to(torch.bfloat16).to(gpu)
    hq = (r16(fac["qa"][:, -1:]), r16(fac["qb"][:, -1:]))
    hc = [r16(fac[name]) for name in ("ka", "kb", "va", "vb")]
    o_h, lse_h = tpa.tpa_decode(*hq, *hc, sm_scale=sm_scale, kernel=2)
    assert np.abs(f64(o) - f64(o_h)).max() <= 2e-2
    assert np.abs(f64(lse) - f64(lse_h)).max() <= 1e-3
    # and against the oracle's attention on the host factors
    cat = lambda a, bb: np.concatenate([a, bb], axis=-1)
    o_ref, l_ref = orc.tpa_reference(cat(f64(hq[0]), f64(hq[1])), cat(f64(hc[0]), f64(hc[1])), cat(f64(hc[2]), f64(hc[3])), None, None, h, sm_scale=sm_scale)
    assert np.abs(f64(o) - o_ref).max() <= 2e-2
    assert np.abs(f64(lse).transpose(0, 2, 1) - l_ref).max() <= 1e-3


def test_append_contiguous_and_paged_caches_hold_the_same_rows(gpu):
    b, n, dm, h, d, rq, rk = 3, 33, 128, 16, 64, 4, 2
    x, w = make_layer(5, b, n, dm, h, d, rq, rk, torch.bfloat16, gpu)
    cos, sin = rope_tables(128, d)
    cache_len, page_size = 64, 8
    lengths = torch.tensor([0, 5, 31], dtype=torch.int32, device=gpu)
    cont = [torch.zeros((b, cache_len, rk, inner), dtype=torch.bfloat16, device=gpu) for inner in (h, d, h, d)]
    pages_per_seq = cache_len // page_size
    table = torch.from_numpy(np.random.default_rng(8).permutation(b * pages_per_seq).astype(np.int32)).reshape(b, pages_per_seq).to(gpu)
    pool = [torch.zeros((b * pages_per_seq, page_size, rk, inner), dtype=torch.bfloat16, device=gpu) for inner in (h, d, h, d)]
    out_c = tpa.tpa_cache_append(x, w, cos, sin, *cont, lengths, rank_q=rq)
    out_p = tpa.tpa_cache_append(x, w, cos, sin, *pool, lengths, rank_q=rq, page_table=table)
    for a, bb in zip(out_c, out_p):
        assert torch.equal(a, bb)
    for c, p_ in zip(cont, pool):
        gathered = p_[table.long()].reshape(b, cache_len, rk, -1)  # [b, pages, page_size, rk, x] -> [b, cache_len, rk, x]
        assert torch.equal(gathered, c)


@pytest.mark.parametrize(
    "b,n,dm,h,d,rq,rk",
    [
        (3, 2731, 128, 32, 128, 6, 2),  # 8193 tokens: the last token tile holds one; 1600 columns: the last column tile a quarter
        (2, 4900, 64, 32, 96, 6, 2),    # 1280 columns = five whole column tiles; one k step
        (5, 2000, 192, 16, 128, 7, 1),  # 1296 columns: rank rows and factors change inside a wave's 64-column pieces
        (2, 1025, 128, 32, 128, 6, 2),  # 2050 tokens: too few for the 256 x 256 tiles, enough for the 128 x 128 ones
        (3, 700, 64, 16, 128, 6, 2),    # 128 x 128 tiles: 1440 columns (the last tile a quarter), one k step
    ],
)
@pytest.mark.parametrize("paged", [False, True])
def test_prefill_chunks_take_the_large_tiles(gpu, b, n, dm, h, d, rq, rk, paged):
    """Enough new tokens to fill the chip with 256 x 256 or 128 x 128 tiles (the kernels a prefill chunk gets): every output
    against the oracle, ragged last tiles in both directions, tokens past the capacity dropped, contiguous
    and paged caches, explicit positions."""
    x, w = make_layer(11, b, n, dm, h, d, rq, rk, torch.bfloat16, gpu)
    page_size = 64
    cache_len = (n + 5 + page_size - 1) // page_size * page_size
    cos, sin = rope_tables(cache_len + 7, d)
    lengths = np.array([(3 * i) % 7 for i in range(b)], dtype=np.int32)
    lengths[-1] = cache_len - n + 2  # the last two tokens of the last sequence do not fit
    rng = np.random.default_rng(12)
    pos = (lengths[:, None] + np.arange(n)[None, :] + rng.integers(0, 3, size=(b, 1))).astype(np.int32)
    if paged:
        pages_per_seq = cache_len // page_size
        table = torch.from_numpy(rng.permutation(b * pages_per_seq).astype(np.int32)).reshape(b, pages_per_seq).to(gpu)
        caches = [torch.full((b * pages_per_seq, page_size, rk, inner), float("nan"), dtype=torch.bfloat16, device=gpu) for inner in (h, d, h, d)]
    else:
        table = None
        caches = [torch.full((b, cache_len, rk, inner), float("nan"), dtype=torch.bfloat16, device=gpu) for inner in (h, d, h, d)]
    qa, qb, new_len = tpa.tpa_cache_append(x, w, cos, sin, *caches, lengths, rank_q=rq, positions=pos, page_table=table, kernel=2)
    want = orc.tpa_append_reference(f64(x), f64(w), cos, sin, np.minimum(pos, cos.shape[0] - 1), h, d, rq, rk)
    rel = 2.0**-8
    for name, got in (("qa", qa), ("qb", qb)):
        assert np.abs(f64(got) - want[name]).max() <= rel * np.abs(want[name]).max(), name
    for name, cache in zip(("ka", "kb", "va", "vb"), caches):
        c = f64(cache[table.long()].reshape(b, cache_len, rk, -1) if paged else cache)
        for bi in range(b):
            fits = min(n, cache_len - lengths[bi])
            rows = c[bi, lengths[bi] : lengths[bi] + fits]
            assert np.abs(rows - want[name][bi, :fits]).max() <= rel * np.abs(want[name]).max(), (name, bi)
            assert np.isnan(c[bi, : lengths[bi]]).all() and np.isnan(c[bi, lengths[bi] + fits :]).all(), (name, bi)
    assert new_len.cpu().tolist() == [min(int(l) + n, cache_len) for l in lengths]
