"""The library's launches inside a captured HIP graph (what a serving loop does with the decode
step): the C ABI only enqueues kernels on the stream it is given - no allocation, no memset, no
synchronisation - so a capture records them, and every replay must equal the eager call on the
inputs of that moment.  Replays alternate with eager work and synchronisations.
"""

import numpy as np
import pytest
import torch

from conftest import make_factors

pytestmark = pytest.mark.gpu


def _capture(gpu, fn):
    """Warm up on a side stream (first-use set-up of the kernels happens outside the capture), then capture fn."""
    side = torch.cuda.Stream(device=gpu)
    side.wait_stream(torch.cuda.current_stream(gpu))
    with torch.cuda.stream(side):
        fn()
    torch.cuda.current_stream(gpu).wait_stream(side)
    torch.cuda.synchronize(gpu)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        out = fn()
    return graph, out


def _same(x, y):
    return torch.equal(torch.nan_to_num(x.float(), nan=7.0), torch.nan_to_num(y.float(), nan=7.0))


@pytest.mark.parametrize("lq,causal", [(1, False), (4, 2)])
def test_decode_replays_in_a_graph(gpu, lq, causal):
    from tpa import tpa

    b, lk, h, d, rq, rk = 4, 2048, 16, 128, 6, 2
    q, k, v = make_factors(170, b, lq, lk, h, d, d, rq, rk, scale_by_rank=True)
    bf = lambda x: torch.from_numpy(x).to(gpu).to(torch.bfloat16)
    tq, tk, tv = bf(q), bf(k), bf(v)
    ops = [t.contiguous() for x in (tq, tk, tv) for t in (x[..., :h], x[..., h:])]
    lengths = torch.tensor([lk, 1500, 700, 64], dtype=torch.int32, device=gpu)
    ws = torch.empty(tpa.decode_workspace_bytes(b, lq, lk, h, d) + 256, dtype=torch.uint8, device=gpu)
    call = lambda: tpa.tpa_decode(*ops, sm_scale=d**-0.5, workspace=ws, kernel=2, kv_lengths=lengths, causal=causal)
    graph, (o_g, lse_g) = _capture(gpu, call)
    gen = torch.Generator(device=gpu)
    gen.manual_seed(171)
    for rep in range(4):
        # the serving loop's own work between replays: new queries, one more token in every cache
        ops[0].copy_(torch.randn(ops[0].shape, generator=gen, device=gpu))
        ops[1].copy_(torch.randn(ops[1].shape, generator=gen, device=gpu))
        lengths.add_(torch.tensor([0, 1, 1, 1], dtype=torch.int32, device=gpu))
        graph.replay()
        torch.cuda.synchronize(gpu)
        o_e, lse_e = call()
        torch.cuda.synchronize(gpu)
        assert _same(o_g, o_e) and torch.equal(lse_g, lse_e), rep


def test_prefill_and_backward_replay_in_a_graph(gpu):
    from tpa import tpa

    b, t, h, d = 2, 512, 4, 128
    q, k, v = make_factors(172, b, t, t, h, d, d, 6, 2, scale_by_rank=True)
    bf = lambda x: torch.from_numpy(x).to(gpu).to(torch.bfloat16)
    ops = [p.contiguous() for x in (bf(q), bf(k), bf(v)) for p in (x[..., :h], x[..., h:])]
    do = torch.randn((b, t, h, d), device=gpu).to(torch.bfloat16)
    bws = torch.empty(tpa.bwd_workspace_bytes(b, t, t, h, d, d) + 256, dtype=torch.uint8, device=gpu)

    def call():
        o, lse = tpa.tpa_factors(*ops, sm_scale=d**-0.5, causal=True, kernel=2)
        grads = tpa.tpa_factors_bwd(*ops, None, None, o, lse, do, d**-0.5, True, workspace=bws, kernel=2)
        return (o, lse) + tuple(grads)

    graph, outs_g = _capture(gpu, call)
    gen = torch.Generator(device=gpu)
    gen.manual_seed(173)
    for rep in range(3):
        for x in ops:
            x.copy_(torch.randn(x.shape, generator=gen, device=gpu) * 0.5)
        graph.replay()
        torch.cuda.synchronize(gpu)
        outs_e = call()
        torch.cuda.synchronize(gpu)
        for g_, e_ in zip(outs_g, outs_e):
            assert _same(g_, e_), rep
