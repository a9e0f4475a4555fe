"""The entry points only enqueue kernels on the caller's stream (no allocation, no synchronisation, no memset), so a
caller may record them into a HIP graph: prefill, decode and the producer step captured once and replayed, with
eager work and synchronisations between the replays, give the eager results bit for bit every time."""

import pytest
import torch

from conftest import make_factors
from test_gpu_parity import split, to_gpu

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("rk", [2, 4])  # rank 4: the prefill goes through dense Q, K, V (two launches)
def test_prefill_decode_and_append_replay_from_a_graph(gpu, rk):
    from tpa import tpa

    b, t, h, d, rq = 2, 640, 8, 128, 6
    q, k, v = make_factors(3, b, t, t, h, d, d, rq, rk, scale_by_rank=True)
    tq, tk, tv = (to_gpu(x, torch.bfloat16, gpu) for x in (q, k, v))
    qa, qb, ka, kb, va, vb = split(tq, tk, tv, h)
    scale = d**-0.5
    # decode: the last token of q against all keys; producer step: four new tokens per sequence into a cache
    dq = (qa[:, -1:].contiguous(), qb[:, -1:].contiguous())
    lk_dec = 2048
    _, kd, vd = make_factors(4, b, 1, lk_dec, h, d, d, rq, rk, scale_by_rank=True)
    dk_, dv_ = (to_gpu(x, torch.bfloat16, gpu) for x in (kd, vd))
    dka, dkb, dva, dvb = dk_[..., :h].contiguous(), dk_[..., h:].contiguous(), dv_[..., :h].contiguous(), dv_[..., h:].contiguous()
    ws = torch.empty(max(tpa.decode_workspace_bytes(b, 1, lk_dec, h, d), 16), dtype=torch.uint8, device=gpu)
    dm, n_new, cache_len = 256, 4, 64
    g = torch.Generator(device=gpu)
    g.manual_seed(5)
    x = torch.randn((b, n_new, dm), generator=g, device=gpu).to(torch.bfloat16)
    w = (torch.randn(((rq + 2 * rk) * (h + d), dm), generator=g, device=gpu) / dm**0.5).to(torch.bfloat16)
    ang = torch.arange(cache_len, device=gpu, dtype=torch.float32)[:, None] * (10000.0 ** (-torch.arange(0, d, 2, device=gpu, dtype=torch.float32) / d))[None]
    cos, sin = torch.cos(ang).contiguous(), torch.sin(ang).contiguous()
    lengths = torch.tensor([3, 17], dtype=torch.int32, device=gpu)

    def work(caches):
        o, lse = tpa.tpa_factors(qa, qb, ka, kb, va, vb, sm_scale=scale, causal=True, kernel=2)
        od, lsed = tpa.tpa_decode(*dq, dka, dkb, dva, dvb, sm_scale=scale, workspace=ws, kernel=2)
        aq, bq, new_len = tpa.tpa_cache_append(x, w, cos, sin, *caches, lengths, rank_q=rq, kernel=2)
        return o, lse, od, lsed, aq, bq, new_len

    new_caches = lambda: [torch.zeros((b, cache_len, rk, inner), dtype=torch.bfloat16, device=gpu) for inner in (h, d, h, d)]
    eager_caches = new_caches()
    eager = work(eager_caches)
    torch.cuda.synchronize()

    graph_caches = new_caches()
    stream = torch.cuda.Stream()
    with torch.cuda.stream(stream):
        work(graph_caches)  # warm up on the capture stream (library set-up, allocator)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=stream):
            captured = work(graph_caches)
    torch.cuda.synchronize()
    for replay in range(3):
        for c in graph_caches:
            c.fill_(float("nan"))  # eager work between the replays; every replay has to write the rows again
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for name, got, want in zip(("o", "lse", "o_decode", "lse_decode", "qa", "qb", "new_lengths"), captured, eager):
            assert torch.equal(got, want), (replay, name)
        for got, want in zip(graph_caches, eager_caches):
            for bi in range(b):
                lo = int(lengths[bi])
                assert torch.equal(got[bi, lo : lo + n_new], want[bi, lo : lo + n_new]), replay
