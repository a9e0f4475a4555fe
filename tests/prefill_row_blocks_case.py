"""Run in a child process by test_gpu_parity.py with TPA_PREFILL_ROW_BLOCKS=2 (the library reads the
variable once per process): the four-wave prefill kernel with 64 query rows per wave and its
generated tile loop, against the oracle, on shapes that reach every part of it (plain tiles,
interleaved tiles, the causal diagonal, a ragged last tile, reference moves, the dense loader)."""

import os
import sys

import numpy as np
import torch

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
from conftest import make_factors  # noqa: E402  (also puts the package and the oracle on the path)
from error_model import dense_bounds, tpa_bounds  # noqa: E402
from oracle import tpa_oracle as orc  # noqa: E402
from tpa import tpa  # noqa: E402
from tpa.mha import _mha_fwd  # noqa: E402

assert os.environ.get("TPA_PREFILL_ROW_BLOCKS") == "2"
dev = torch.device("cuda:0")
f64 = lambda t: t.detach().float().cpu().numpy().astype(np.float64)


def within(o, lse_bhl, o_ref, l_ref, bounds):
    lse_b, o_b = bounds
    o, lse = f64(o), f64(lse_bhl).transpose(0, 2, 1)
    assert (np.isnan(o) == np.isnan(o_ref)).all()
    ok = ~np.isnan(o_ref)
    assert (np.where(ok, np.abs(o - o_ref) - o_b[..., None], 0.0) <= 0).all()
    assert (np.abs(lse - l_ref) <= lse_b).all()


for seed, (b, lq, lk, h, causal, scaled) in enumerate(
    [(2, 700, 700, 8, True, True), (1, 512, 1100, 16, False, True), (1, 300, 3000, 8, False, False), (1, 1536, 1536, 8, True, False)]
):
    d = 128
    q, k, v = make_factors(500 + seed, b, lq, lk, h, d, d, 6 if scaled else 1, 2, scale_by_rank=scaled)
    if seed == 3:  # logits that climb along the keys: the reference moves inside the interleaved tiles
        k[..., h] += np.linspace(0.0, 30.0, lk, dtype=np.float32)[None, :, None]
        q[..., h] = 1.0
    tq, tk, tv = (torch.from_numpy(x).to(torch.bfloat16).to(dev) for x in (q, k, v))
    sp = lambda t: (t[..., :h], t[..., h:])
    o, lse = tpa.tpa_factors(*sp(tq), *sp(tk), *sp(tv), sm_scale=d**-0.5, causal=causal, kernel=2, use_workspace=False)
    o_ref, l_ref = orc.tpa_reference(f64(tq), f64(tk), f64(tv), None, None, h, sm_scale=d**-0.5, causal=causal)
    within(o, lse, o_ref, l_ref, tpa_bounds(f64(tq), f64(tk), f64(tv), h, d**-0.5))

rng = np.random.Generator(np.random.Philox(7))
for causal in (False, True):
    qd, kd, vd = (torch.from_numpy(rng.standard_normal((2, 900, 4, 128), dtype=np.float32)).to(torch.bfloat16).to(dev) for _ in range(3))
    bias = np.where(np.tril(np.ones((900, 900), bool)), 0.0, -np.inf)[None].repeat(2, 0) if causal else None
    o_ref, l_ref = orc.mha_forward(f64(qd), f64(kd), f64(vd), bias, 128**-0.5)
    o, (lse, *_) = _mha_fwd(qd, kd, vd, None, 128**-0.5, causal=causal, kernel=2)
    within(o, lse, o_ref, l_ref, dense_bounds(f64(qd), f64(kd), f64(vd), 128**-0.5))
print("ok")
