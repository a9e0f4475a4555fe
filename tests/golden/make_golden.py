#!/usr/bin/env python3
"""Writes the fixtures of this directory:  python tests/golden/make_golden.py

The upstream implementation needs jax, which is not installed where this build runs, so the
vectors are written from the float64 CPU restatement in oracle/ (itself pinned by
tests/test_oracle.py against brute force, closed forms, library routines and the one literal
answer upstream holds, tpa/mha_test.py:44-118).  They freeze that behaviour: a later change to
the oracle or to the seeded input recipe shows up as a fixture mismatch.

small_cases.npz  inputs and full outputs of small problems, among them the upstream test shape
                 (1, 8, 8, 1, 4, 6) of tpa/tpa_test.py:66 and the literal case of tpa/mha_test.py
sampled_rows.npz for larger seeded problems: the seed recipe, a checksum of the inputs and the
                 outputs of a few query rows
backward_cases.npz  for the small problems: a seeded upstream gradient and the gradients of the three
                 factor arrays (what _tpa_bwd returns, tpa/tpa.py:168-214), and the literal gradients
                 upstream keeps in tpa/mha_test.py:87-118
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

from conftest import make_factors, segment_ids  # noqa: E402
from oracle import tpa_oracle as orc  # noqa: E402

# name: (seed, b, lq, lk, h, dk, dv, rq, rk, segment_size or 0, causal, sm_scale, dist)
SMALL = {
    "upstream_tiny_causal": (11, 1, 8, 8, 1, 4, 6, 2, 3, 0, True, 1.0, "uniform"),
    "upstream_tiny_segments": (12, 1, 8, 8, 1, 4, 6, 1, 1, 3, False, 1.0, "uniform"),
    "ragged_cross": (13, 2, 19, 37, 3, 8, 5, 6, 2, 0, False, 0.5, "normal"),
    "segments_causal_empty_rows": (14, 2, 24, 16, 2, 8, 8, 2, 2, 5, True, 0.7, "normal"),
    "decode_one_row": (15, 3, 1, 77, 4, 16, 16, 6, 2, 0, False, 0.25, "normal"),
}

# name: (seed, b, lq, lk, h, dk, dv, rq, rk, causal, sm_scale, dist, scale_by_rank, rows)
SAMPLED = {
    "c1_fp32": (0, 1, 512, 512, 8, 64, 64, 6, 2, True, 0.125, "normal", False, [0, 1, 63, 64, 255, 300, 511]),
    "upstream_long_segments": (42, 2, 1024, 128, 2, 3, 5, 4, 2, False, 1.0, "uniform", False, [0, 41, 42, 167, 168, 1023]),
    "sharp_bf16_prefill": (7, 2, 512, 512, 4, 128, 128, 6, 2, True, 0.0883883, "normal", False, [0, 31, 32, 257, 511]),
}


def checksum(*arrays):
    """Sum of the float64 values and of their squares: cheap, order-free, sensitive to the stream."""
    s = sum(float(np.sum(a.astype(np.float64))) for a in arrays)
    s2 = sum(float(np.sum(a.astype(np.float64) ** 2)) for a in arrays)
    return np.array([s, s2])


def main():
    small = {}
    for name, (seed, b, lq, lk, h, dk, dv, rq, rk, seg, causal, scale, dist) in SMALL.items():
        q, k, v = make_factors(seed, b, lq, lk, h, dk, dv, rq, rk, dist=dist)
        qs = segment_ids(lq, seg, b) if seg else None
        ks = segment_ids(lk, seg, b) if seg else None
        o, lse = orc.tpa_reference(q, k, v, qs, ks, h, sm_scale=scale, causal=causal)
        small.update({f"{name}.q": q, f"{name}.k": k, f"{name}.v": v, f"{name}.o": o, f"{name}.lse": lse,
                      f"{name}.meta": np.array([h, seg, int(causal)]), f"{name}.sm_scale": np.array(scale)})
    # the literal case upstream keeps in tpa/mha_test.py:44-118 (dense attention with a -inf bias)
    ninf = -np.inf
    small["upstream_mha_literal.q"] = np.array([[2, 1], [1, 1], [1, 1]], dtype=np.float64)[None, :, None, :]
    small["upstream_mha_literal.k"] = np.ones((1, 3, 1, 2))
    small["upstream_mha_literal.v"] = np.ones((1, 3, 1, 2))
    small["upstream_mha_literal.bias"] = np.array([[0, ninf, 0], [0, ninf, 0], [ninf, ninf, ninf]])[None]
    small["upstream_mha_literal.o"] = np.array([[1.0, 1.0], [1.0, 1.0], [np.nan, np.nan]])[None, :, None, :]
    np.savez_compressed(os.path.join(HERE, "small_cases.npz"), **small)

    back = {}
    for name, (seed, b, lq, lk, h, dk, dv, rq, rk, seg, causal, scale, dist) in SMALL.items():
        q, k, v = make_factors(seed, b, lq, lk, h, dk, dv, rq, rk, dist=dist)
        qs = segment_ids(lq, seg, b) if seg else None
        ks = segment_ids(lk, seg, b) if seg else None
        do = np.random.Generator(np.random.Philox(seed + 1000)).standard_normal((b, lq, h, dv)).astype(np.float32)
        dq, dk_, dv_ = orc.tpa_backward(q, k, v, qs, ks, h, do, sm_scale=scale, causal=causal)
        back.update({f"{name}.do": do, f"{name}.dq": dq, f"{name}.dk": dk_, f"{name}.dv": dv_})
    # tpa/mha_test.py:87-118: gradients of nansum(o) on the literal case
    back["upstream_mha_literal.dq"] = np.zeros((1, 3, 1, 2))
    back["upstream_mha_literal.dk"] = np.zeros((1, 3, 1, 2))
    back["upstream_mha_literal.dv"] = np.array([[1.0, 1.0], [0.0, 0.0], [1.0, 1.0]])[None, :, None, :]
    np.savez_compressed(os.path.join(HERE, "backward_cases.npz"), **back)

    sampled = {}
    for name, (seed, b, lq, lk, h, dk, dv, rq, rk, causal, scale, dist, sbr, rows) in SAMPLED.items():
        q, k, v = make_factors(seed, b, lq, lk, h, dk, dv, rq, rk, dist=dist, scale_by_rank=sbr)
        seg = 42 if name == "upstream_long_segments" else 0  # tpa/tpa_test.py:71
        qs = segment_ids(lq, seg, b) if seg else None
        ks = segment_ids(lk, seg, b) if seg else None
        o, lse = orc.tpa_reference_rows(q, k, v, qs, ks, h, rows, sm_scale=scale, causal=causal)
        sampled.update({f"{name}.recipe": np.array([seed, b, lq, lk, h, dk, dv, rq, rk, seg, int(causal), int(sbr)]),
                        f"{name}.dist": np.array(dist), f"{name}.sm_scale": np.array(scale),
                        f"{name}.rows": np.array(rows), f"{name}.input_checksum": checksum(q, k, v),
                        f"{name}.o": o, f"{name}.lse": lse})
    np.savez_compressed(os.path.join(HERE, "sampled_rows.npz"), **sampled)
    print("wrote", sorted(os.listdir(HERE)))


if __name__ == "__main__":
    main()
