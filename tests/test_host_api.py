"""Host-side behaviour of the Python operator API that needs no GPU."""

import numpy as np
import pytest
import torch

from oracle import tpa_oracle as orc


def test_module_layout_mirrors_the_reference():
    from tpa import mha, tpa

    # names other code reaches for (tpa/ring_tpa.py:82,241,244; tpa/mha_test.py:6)
    for name in ("tpa", "BlockSizes", "_fwd", "_tpa_fwd", "_bwd", "_tpa_bwd", "_precompute_delta", "_lse", "_lse_accum"):
        assert hasattr(tpa, name), name
    for name in ("mha", "_mha_fwd", "_mha_bwd"):
        assert hasattr(mha, name), name
    bs = tpa.BlockSizes()
    assert (bs.block_q, bs.block_kv, bs.block_h) == (128, 128, 4)  # tpa/tpa.py:39-70


def test_signature_matches_the_reference():
    import inspect

    from tpa import mha, tpa

    sig = inspect.signature(tpa.tpa)
    params = list(sig.parameters)
    assert params[:12] == [
        "q", "k", "v", "num_heads", "q_segment_ids", "kv_segment_ids", "sm_scale", "causal",
        "block_sizes", "nomat", "debug", "interpret",
    ]  # tpa/tpa.py:74-87
    # additions can only be named, so a positional call of the reference means the same here
    assert all(sig.parameters[n].kind is inspect.Parameter.KEYWORD_ONLY for n in params[12:])
    assert sig.parameters["sm_scale"].default == 1.0 and sig.parameters["causal"].default is False
    assert list(inspect.signature(mha.mha).parameters)[:5] == ["q", "k", "v", "bias", "sm_scale"]  # tpa/mha.py:11-17


def test_lse_helpers_match_the_oracle():
    from tpa import tpa

    rng = np.random.default_rng(1)
    x = rng.standard_normal((5, 7)).astype(np.float32)
    x[2] = -np.inf
    got = tpa._lse(torch.from_numpy(x)).numpy()
    np.testing.assert_allclose(got, orc.lse(x.astype(np.float64)), rtol=1e-6)
    a = torch.tensor([0.3, -np.inf, -np.inf, 2.0])
    b = torch.tensor([1.1, -np.inf, 0.5, -np.inf])
    np.testing.assert_allclose(tpa._lse_accum(a, b).numpy(), orc.lse_accum(a.numpy().astype(np.float64), b.numpy().astype(np.float64)), rtol=1e-6)


def test_backward_signatures_and_delta():
    import inspect

    from tpa import tpa

    # tpa/tpa.py:168-178 and tpa/tpa.py:823-839
    # (the reference's positional parameters, then the keyword-only addition for the causal offset)
    params = inspect.signature(tpa._tpa_bwd).parameters
    assert list(params) == [
        "num_heads", "sm_scale", "causal", "block_sizes", "nomat", "debug", "interpret", "residuals", "do", "causal_offset"]
    assert params["causal_offset"].kind is inspect.Parameter.KEYWORD_ONLY and params["causal_offset"].default == 0
    assert list(inspect.signature(tpa._bwd).parameters) == [
        "q", "k", "v", "q_segment_ids", "kv_segment_ids", "o", "l", "do", "num_heads", "sm_scale", "causal",
        "block_sizes", "nomat", "debug", "interpret"]
    # tpa/tpa.py:965-995: nansum(out * do) per row, NaN rows of an empty query contribute 0
    rng = np.random.default_rng(2)
    out, do = rng.standard_normal((6, 5)).astype(np.float32), rng.standard_normal((6, 5)).astype(np.float32)
    out[3] = np.nan
    got = tpa._precompute_delta(torch.from_numpy(out), torch.from_numpy(do), torch.zeros(6)).numpy()
    np.testing.assert_allclose(got, np.nansum(out * do, axis=1), rtol=1e-6)
    assert got[3] == 0.0


def test_no_gpu_means_an_error_not_a_fallback():
    from tpa import tpa

    if torch.cuda.is_available():
        pytest.skip("a GPU is visible")
    x = np.zeros((1, 4, 1, 6), dtype=np.float32)
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        tpa.tpa(x, x, x, num_heads=2)


def test_product_package_never_imports_the_oracle():
    import os
    import re

    from conftest import PKG_PARENT

    pat = re.compile(r"^\s*(from|import)\s+\.*oracle\b|tpa_oracle|oracle/", re.M)
    for dirpath, _, files in os.walk(PKG_PARENT):
        for f in files:
            if f.endswith((".py", ".hip", ".h", ".cc", "Makefile")):
                text = open(os.path.join(dirpath, f)).read()
                assert not pat.search(text), os.path.join(dirpath, f)


def test_causal_argument_values():
    """False / True as in the reference (tpa/tpa.py:82), CAUSAL_BOTTOM_RIGHT as the one addition; anything else raises."""
    from tpa import tpa

    assert tpa._causal_code(False) == 0 and tpa._causal_code(True) == 1
    assert tpa._causal_code(np.bool_(True)) == 1 and tpa._causal_code(0) == 0
    assert tpa._causal_code(tpa.CAUSAL_BOTTOM_RIGHT) == 2
    for bad in (3, -1):
        with pytest.raises(ValueError):
            tpa._causal_code(bad)
