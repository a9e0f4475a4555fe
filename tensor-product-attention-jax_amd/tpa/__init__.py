"""Tensor Product Attention forward for MI355X (gfx950).

The package mirrors the module layout of the reference so that its call sites read the same:

    from tpa import tpa            # the module of tpa/tpa.py
    o = tpa.tpa(q, k, v, num_heads=h, sm_scale=s, causal=True)
    from tpa.mha import mha        # tpa/mha.py
"""

from . import mha, tpa  # noqa: F401  (submodules, as in the reference's `from ... import tpa`)

__all__ = ["tpa", "mha"]
