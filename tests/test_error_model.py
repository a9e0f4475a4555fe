"""The bf16 error model (tests/error_model.py) against a numpy emulation of the bf16 prefill
kernel's rounding points: the bound holds, is not vacuous, and on benchmark-like inputs the
emulated errors stay inside the absolute gates stated for the benchmark configurations."""

import numpy as np
import torch

from conftest import bf16_round, make_factors
from error_model import emulate_bf16_prefill, round_bf16, tight_violations, tpa_bounds
from oracle import tpa_oracle as orc


def test_round_bf16_matches_torch():
    rng = np.random.default_rng(0)
    x = np.concatenate([rng.standard_normal(4096) * 10.0 ** rng.integers(-6, 6, 4096), [0.0, 1.0, 1.00390625, 1.01171875, -3.0]])
    want = torch.from_numpy(x.astype(np.float32)).to(torch.bfloat16).to(torch.float64).numpy()
    np.testing.assert_array_equal(round_bf16(x), want)


def _errors(seed, b, lq, lk, h, d, rq, rk, scaled, causal):
    q, k, v = (bf16_round(x) for x in make_factors(seed, b, lq, lk, h, d, d, rq, rk, scale_by_rank=scaled))
    scale = d**-0.5
    o_ref, l_ref = orc.tpa_reference(q, k, v, None, None, h, sm_scale=scale, causal=causal)
    o, l, _ = emulate_bf16_prefill(q, k, v, h, scale, causal)
    lse_b, o_b = tpa_bounds(q, k, v, h, scale)
    return np.abs(o - o_ref).max(-1), np.abs(l - l_ref), o_b, lse_b


def test_bound_holds_and_is_not_vacuous_on_sharp_inputs():
    # unscaled N(0,1) factors, query rank one: logits of order ten
    eo, el, o_b, lse_b = _errors(1, 2, 96, 160, 4, 128, 1, 2, False, True)
    assert (eo <= o_b).all() and (el <= lse_b).all()
    assert el.max() > 2e-3, "this distribution is the one where the absolute 1e-3 does not hold"
    # the worst row comes within a factor of 80 of its bound (the bound is a sum of absolute
    # values, the error a sum of signed terms: sqrt(D) apart at best)
    assert (el / lse_b).max() > 1 / 80 and (eo / o_b).max() > 1 / 80


def test_bound_stays_inside_the_absolute_gates_on_benchmark_like_inputs():
    # N(0,1)/sqrt(R) factors, ranks 6/2, D = 128: the distribution of the benchmark configurations
    eo, el, o_b, lse_b = _errors(2, 1, 128, 256, 4, 128, 6, 2, True, True)
    assert (eo <= o_b).all() and (el <= lse_b).all()
    # the worst-case bound (sums of absolute values) is up to 1e-2 here; the errors themselves
    # (signed sums) stay inside the absolute gates stated for the benchmark configurations
    assert lse_b.max() <= 1e-2 and o_b.max() <= 1e-1
    assert el.max() <= 1e-3 and eo.max() <= 2e-2
    # the factored form (decode kernels) bounds the materialised one
    q, k, v = (bf16_round(x) for x in make_factors(2, 1, 128, 256, 4, 128, 128, 6, 2, scale_by_rank=True))
    lse_f, o_f = tpa_bounds(q, k, v, 4, 128**-0.5, form="factored")
    assert (lse_f >= lse_b).all() and (o_f >= o_b).all()


CASES = {  # seed, b, lq, lk, h, d, rq, rk, factors scaled by 1/sqrt(R), causal
    "sharp": (1, 2, 96, 160, 4, 128, 1, 2, False, True),
    "benchmark-like": (2, 1, 128, 256, 4, 128, 6, 2, True, True),
}


def test_tight_gate_rejects_one_extra_rounding():
    """The gate that holds the GPU kernels to the emulation (tests/test_gpu_parity.py: check_tight) fails an
    emulation with one mistake in its rounding points: P rounded twice, P truncated, Q rounded before its
    scale factor is applied.  The unmodified emulation passes against itself trivially; what the GPU kernels
    measure against it is written beside the TIGHT_* constants."""
    for name, (seed, b, lq, lk, h, d, rq, rk, scaled, causal) in CASES.items():
        q, k, v = (bf16_round(x) for x in make_factors(seed, b, lq, lk, h, d, d, rq, rk, scale_by_rank=scaled))
        o, l, slack = emulate_bf16_prefill(q, k, v, h, d**-0.5, causal)
        assert not tight_violations(o, l, o, l, slack)
        for fault in ("p_twice", "p_trunc", "q_unscaled_round"):
            o2, l2, _ = emulate_bf16_prefill(q, k, v, h, d**-0.5, causal, faults=(fault,))
            assert tight_violations(o2, l2, o, l, slack), (name, fault)


def test_whole_number_reference_changes_no_bit():
    """P = bf16(2^(x - m)) has the same mantissa for every whole number m, so neither the output nor any
    rounding depends on which whole number the kernels use as the softmax reference: the emulation with the
    reference three above the row maximum returns the same bits."""
    seed, b, lq, lk, h, d, rq, rk, scaled, causal = CASES["sharp"]
    q, k, v = (bf16_round(x) for x in make_factors(seed, b, lq, lk, h, d, d, rq, rk, scale_by_rank=scaled))
    o, l, _ = emulate_bf16_prefill(q, k, v, h, d**-0.5, causal)
    o3, l3, _ = emulate_bf16_prefill(q, k, v, h, d**-0.5, causal, reference_shift=3)
    np.testing.assert_array_equal(o, o3)
    np.testing.assert_allclose(l, l3, rtol=0, atol=1e-12)
    # a reference that is not a whole number does change roundings of P
    import error_model as em

    assert em.round_bf16(2.0**-0.37 * 1.2345) != em.round_bf16(1.2345) * 2.0**-0.37


DECODE_CASES = {  # seed, b, lq, lk, h, d, rq, rk, factors scaled by 1/sqrt(R)
    "sharp": (3, 2, 2, 300, 8, 128, 1, 2, False),
    "benchmark-like": (4, 2, 1, 700, 8, 128, 6, 2, True),
    "rank 4, head size 64": (5, 1, 3, 257, 16, 64, 6, 4, True),
}


def test_decode_emulation_follows_the_oracle_and_its_gate_rejects_one_extra_rounding():
    """The decode twin of the tight gate: the split-key kernels round the folded query once and every
    (probability x head factor of V) product once; the emulation of exactly that stays inside the worst-case
    law against the float64 oracle, and the gate that compares the GPU kernels with it fails an emulation that
    rounds p before the product, truncates the product, or rounds the query sum before its scale factor."""
    from error_model import emulate_bf16_decode

    for name, (seed, b, lq, lk, h, d, rq, rk, scaled) in DECODE_CASES.items():
        q, k, v = (bf16_round(x) for x in make_factors(seed, b, lq, lk, h, d, d, rq, rk, scale_by_rank=scaled))
        scale = d**-0.5
        o, l, slack = emulate_bf16_decode(q, k, v, h, scale)
        o_ref, l_ref = orc.tpa_reference(q, k, v, None, None, h, sm_scale=scale)
        lse_b, o_b = tpa_bounds(q, k, v, h, scale, form="factored")
        assert (np.abs(o - o_ref).max(-1) <= o_b).all() and (np.abs(l - l_ref) <= lse_b).all(), name
        assert not tight_violations(o, l, o, l, slack)
        for fault in ("p_before_av", "p_trunc", "q_unscaled_round"):
            o2, l2, _ = emulate_bf16_decode(q, k, v, h, scale, faults=(fault,))
            assert tight_violations(o2, l2, o, l, slack), (name, fault)
