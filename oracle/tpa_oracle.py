"""CPU oracle for the Tensor Product Attention forward path.  TEST INFRASTRUCTURE ONLY.

This file restates, in plain numpy, the arithmetic of the reference's jnp oracle so that
the HIP kernels can be checked against it.  Only tests, the smoke check and the benchmark's
`cpu_baseline` leg may import it; the product package never does.

What follows what (reference file:line):
  * `split_factors`      - tpa/tpa_test.py:35-37  (A factor = first `num_heads` columns)
  * `reconstruct`        - tpa/tpa_test.py:42-44  (X = (1/R) * sum_r a_r (x) b_r)
  * `attention_bias`     - tpa/tpa_test.py:46-55  (segment equality, then top-left tril; additive -inf)
  * `mha_forward`        - tpa/mha.py:23-37       (dot, scale AFTER the dot, + bias broadcast over heads,
                                                   softmax over keys, p @ v, output [b, lq, h, dv])
  * `lse` / `lse_accum`  - tpa/tpa.py:220-242     (-inf safe logsumexp and its pairwise merge)
  * empty rows           - tpa/tpa.py:437-439     (O = NaN, LSE = -inf), same as softmax of an all -inf row
  * shape rules          - tpa/tpa.py:474-479

The reference returns LSE as l[b, lq, h] (tpa/tpa.py:255,443); this oracle returns it in that
layout too (`lse_blh`); callers transpose when they compare with the kernels' [b, h, lq].

Backward (the gradients of the same functions):
  * `mha_backward`       - tpa/mha.py:40-65       (p with NaN -> 0, dv = p^T do, dp = do v^T,
                                                   dx = scale * p * (dp - sum(dp * p)), dq = dx k, dk = dx^T q)
  * `project_to_factors` - tpa/tpa.py:781-783,793-799 (da = dX . b / R, db = dX . a / R, the chain rule
                                                   through X = (1/R) sum_r a_r (x) b_r)
  * `tpa_backward`       - tpa/tpa.py:168-214,546-962 (what `_tpa_bwd` returns: dq, dk, dv in the
                                                   concatenated factor layout; rows without a visible key
                                                   contribute nothing, tpa/tpa.py:675-676,979)
  pinned by tests/test_oracle.py against torch autograd (float64, CPU) of an independently written
  dense attention, central finite differences on a tiny case, and the literal gradients the
  reference holds (tpa/mha_test.py:87-118: dq = dk = 0, dv = [[1,1],[0,0],[1,1]]).

Producer step (no counterpart in the reference, which takes the factors as given; arXiv 2501.06425,
section 3, is what is restated):
  * `rope_rotate`          - rotary position embedding on adjacent pairs (y[2j], y[2j+1])
  * `tpa_append_reference` - the six factors of new tokens as linear maps of the hidden state, with
                             the B factors of Q and K rotated
  pinned by tests/test_oracle.py: float64 loops over every output element on a tiny case, and the
  closed forms of a rotation (position 0 is the identity, pair norms are preserved, angles add,
  the dot product of a rotated query and key depends on the distance of their positions only).

How this oracle is pinned (tests/test_oracle.py): brute-force float64 loops on tiny shapes,
torch's scaled_dot_product_attention and scipy's softmax/logsumexp as independent library
routines, closed forms (zero queries -> running mean of V and LSE = ln(count); lk = 1), rank
invariances (duplicated / permuted ranks, a*c with b/c), the causal prefix property, and the
only literal known-answer the reference holds (tpa/mha_test.py:44-118, forward part).
Parity against the bit-stream of jax itself is unpinned (jax is not installable here); the
mathematical contract is pinned by the checks above.
"""

from __future__ import annotations

import numpy as np

__all__ = [
    "split_factors",
    "reconstruct",
    "attention_bias",
    "mha_forward",
    "tpa_reference",
    "tpa_reference_rows",
    "lse",
    "lse_accum",
    "mha_backward",
    "project_to_factors",
    "tpa_backward",
    "rope_rotate",
    "tpa_append_reference",
]


def split_factors(x: np.ndarray, num_heads: int):
    """x[b, l, r, h + d] -> (a[b, l, r, h], b[b, l, r, d]).  tpa/tpa_test.py:35-37."""
    return x[..., :num_heads], x[..., num_heads:]


def reconstruct(a: np.ndarray, b: np.ndarray) -> np.ndarray:
    """(1/R) * sum_r a[b,l,r,h] * b[b,l,r,d] -> [b, l, h, d].  tpa/tpa_test.py:42-44."""
    rank = a.shape[2]
    # per token an [h, r] x [r, d] product
    return np.matmul(np.swapaxes(a, 2, 3), b) / rank


def attention_bias(batch, lq, lk, q_segment_ids, kv_segment_ids, causal, dtype=np.float64):
    """Additive bias [b, lq, lk] of 0 / -inf.  tpa/tpa_test.py:46-55."""
    bias = np.zeros((batch, lq, lk), dtype=dtype)
    if q_segment_ids is not None:
        assert kv_segment_ids is not None
        same = np.asarray(q_segment_ids)[:, :, None] == np.asarray(kv_segment_ids)[:, None, :]
        bias = bias + np.where(same, 0.0, -np.inf)
    if causal:
        tril = np.tril(np.ones((lq, lk), dtype=bool))
        bias = bias + np.where(tril, 0.0, -np.inf)[None]
    return bias


def lse(x: np.ndarray) -> np.ndarray:
    """-inf safe logsumexp over the last axis.  tpa/tpa.py:220-226."""
    m = np.max(x, axis=-1)
    with np.errstate(invalid="ignore", divide="ignore"):
        val = m + np.log(np.sum(np.exp(x - m[..., None]), axis=-1))
    return np.where(np.isneginf(m), -np.inf, val)


def lse_accum(a: np.ndarray, b: np.ndarray) -> np.ndarray:
    """log(exp(a) + exp(b)), -inf safe.  tpa/tpa.py:228-242."""
    assert a.shape == b.shape
    hi = np.maximum(a, b)
    lo = np.minimum(a, b)
    with np.errstate(invalid="ignore"):
        val = hi + np.log(1 + np.exp(lo - hi))
    return np.where(np.isneginf(hi), -np.inf, val)


def mha_forward(q, k, v, bias=None, sm_scale=1.0):
    """Dense attention, tpa/mha.py:23-37, plus the logsumexp the kernels also emit.

    q[b,lq,h,dk] k[b,lk,h,dk] v[b,lk,h,dv] bias[b,lq,lk] -> (o[b,lq,h,dv], lse[b,lq,h]).
    A row whose logits are all -inf gives o = NaN and lse = -inf.
    """
    # the two contractions go through matmul (BLAS) rather than einsum's scalar loops
    x = np.matmul(np.transpose(q, (0, 2, 1, 3)), np.transpose(k, (0, 2, 3, 1)))  # b h lq lk
    x = sm_scale * x
    if bias is not None:
        x = x + bias[:, None, :, :]
    m = np.max(x, axis=-1, keepdims=True)
    with np.errstate(invalid="ignore", divide="ignore"):
        e = np.exp(x - m)  # all -inf row: -inf - -inf = NaN, as jax.nn.softmax gives
        s = np.sum(e, axis=-1, keepdims=True)
        p = e / s
        l_ = np.where(np.isneginf(m[..., 0]), -np.inf, m[..., 0] + np.log(s[..., 0]))
    o = np.transpose(np.matmul(p, np.transpose(v, (0, 2, 1, 3))), (0, 2, 1, 3))  # b lq h dv
    return o, np.transpose(l_, (0, 2, 1))


def tpa_reference(
    q, k, v, q_segment_ids, kv_segment_ids, num_heads, sm_scale=1.0, causal=False, dtype=np.float64
):
    """The reference's `reference()` (tpa/tpa_test.py:22-57) on concatenated factors.

    q[b,lq,rq,h+dk] k[b,lk,rk,h+dk] v[b,lk,rk,h+dv] -> (o[b,lq,h,dv], lse[b,lq,h]), computed in `dtype`.
    """
    q = np.asarray(q, dtype=dtype)
    k = np.asarray(k, dtype=dtype)
    v = np.asarray(v, dtype=dtype)
    qa, qb = split_factors(q, num_heads)
    ka, kb = split_factors(k, num_heads)
    va, vb = split_factors(v, num_heads)
    b, lq = qa.shape[:2]
    lk = ka.shape[1]
    assert k.shape[:3] == v.shape[:3], (k.shape, v.shape)  # tpa/tpa.py:474-475
    q_ = reconstruct(qa, qb)
    k_ = reconstruct(ka, kb)
    v_ = reconstruct(va, vb)
    bias = attention_bias(b, lq, lk, q_segment_ids, kv_segment_ids, causal, dtype=dtype)
    return mha_forward(q_, k_, v_, bias=bias, sm_scale=sm_scale)


def tpa_reference_rows(
    q, k, v, q_segment_ids, kv_segment_ids, num_heads, rows, sm_scale=1.0, causal=False, dtype=np.float64
):
    """Same result as `tpa_reference(...)[:, rows]`, computed for the listed query rows only.

    Each output row depends only on its own row of logits, so this is exact; it lets long
    sequences be checked without materialising [b, h, lq, lk].  The causal mask uses the
    absolute row index (top-left aligned tril, tpa/tpa_test.py:53).
    """
    rows = np.asarray(rows)
    q = np.asarray(q)[:, rows].astype(dtype)
    k = np.asarray(k, dtype=dtype)
    v = np.asarray(v, dtype=dtype)
    qa, qb = split_factors(q, num_heads)
    ka, kb = split_factors(k, num_heads)
    va, vb = split_factors(v, num_heads)
    b = q.shape[0]
    lk = k.shape[1]
    q_ = reconstruct(qa, qb)
    k_ = reconstruct(ka, kb)
    v_ = reconstruct(va, vb)
    bias = np.zeros((b, len(rows), lk), dtype=dtype)
    if q_segment_ids is not None:
        same = np.asarray(q_segment_ids)[:, rows][:, :, None] == np.asarray(kv_segment_ids)[:, None, :]
        bias = bias + np.where(same, 0.0, -np.inf)
    if causal:
        keep = rows[:, None] >= np.arange(lk)[None, :]
        bias = bias + np.where(keep, 0.0, -np.inf)[None]
    return mha_forward(q_, k_, v_, bias=bias, sm_scale=sm_scale)


def mha_backward(q, k, v, bias, sm_scale, do):
    """Gradients of dense attention, tpa/mha.py:40-65.

    q[b,lq,h,dk] k[b,lk,h,dk] v[b,lk,h,dv] bias[b,lq,lk]|None do[b,lq,h,dv] -> (dq, dk, dv), same
    shapes as q, k, v.  The softmax is recomputed; rows whose logits are all -inf have p = 0
    (tpa/mha.py:55) and so contribute nothing.
    """
    qt = np.transpose(q, (0, 2, 1, 3))   # b h lq dk
    kt = np.transpose(k, (0, 2, 1, 3))   # b h lk dk
    vt = np.transpose(v, (0, 2, 1, 3))   # b h lk dv
    dot = np.transpose(do, (0, 2, 1, 3))  # b h lq dv
    x = sm_scale * np.matmul(qt, np.swapaxes(kt, 2, 3))
    if bias is not None:
        x = x + bias[:, None, :, :]
    m = np.max(x, axis=-1, keepdims=True)
    with np.errstate(invalid="ignore", divide="ignore"):
        e = np.exp(x - m)
        p = e / np.sum(e, axis=-1, keepdims=True)
    p = np.where(np.isnan(p), 0.0, p)
    dot = np.where(np.isnan(dot), 0.0, dot)
    dv = np.matmul(np.swapaxes(p, 2, 3), dot)                # b h lk dv
    dp = np.matmul(dot, np.swapaxes(vt, 2, 3))               # b h lq lk
    dx = sm_scale * p * (dp - np.sum(dp * p, axis=-1, keepdims=True))
    dq = np.matmul(dx, kt)                                   # b h lq dk
    dk = np.matmul(np.swapaxes(dx, 2, 3), qt)                # b h lk dk
    back = lambda t: np.transpose(t, (0, 2, 1, 3))
    return back(dq), back(dk), back(dv)


def project_to_factors(dx, a, b):
    """Chain rule through X = (1/R) sum_r a[b,l,r,h] b[b,l,r,d]: dX[b,l,h,d] -> (da, db).

    da[b,l,r,h] = (1/R) sum_d dX[b,l,h,d] b[b,l,r,d];  db[b,l,r,d] = (1/R) sum_h dX[b,l,h,d] a[b,l,r,h]
    (tpa/tpa.py:781-783 for q, 793-799 for k).
    """
    rank = a.shape[2]
    da = np.matmul(b, np.swapaxes(dx, 2, 3)) / rank   # [r, d] x [d, h] per token
    db = np.matmul(a, dx) / rank                       # [r, h] x [h, d] per token
    return da, db


def tpa_backward(q, k, v, q_segment_ids, kv_segment_ids, num_heads, do, sm_scale=1.0, causal=False, dtype=np.float64):
    """What the reference's `_tpa_bwd` returns (tpa/tpa.py:168-214): (dq, dk, dv) in the layout of q, k, v.

    q[b,lq,rq,h+dk] k[b,lk,rk,h+dk] v[b,lk,rk,h+dv] do[b,lq,h,dv].
    """
    q = np.asarray(q, dtype=dtype)
    k = np.asarray(k, dtype=dtype)
    v = np.asarray(v, dtype=dtype)
    do = np.asarray(do, dtype=dtype)
    qa, qb = split_factors(q, num_heads)
    ka, kb = split_factors(k, num_heads)
    va, vb = split_factors(v, num_heads)
    b, lq = qa.shape[:2]
    lk = ka.shape[1]
    bias = attention_bias(b, lq, lk, q_segment_ids, kv_segment_ids, causal, dtype=dtype)
    dq_, dk_, dv_ = mha_backward(reconstruct(qa, qb), reconstruct(ka, kb), reconstruct(va, vb), bias, sm_scale, do)
    cat = lambda pair: np.concatenate(pair, axis=-1)
    return cat(project_to_factors(dq_, qa, qb)), cat(project_to_factors(dk_, ka, kb)), cat(project_to_factors(dv_, va, vb))


def rope_rotate(y, cos, sin):
    """Rotate adjacent pairs: y[..., 2j] c - y[..., 2j+1] s, y[..., 2j+1] c + y[..., 2j] s with
    c = cos[..., j], s = sin[..., j] (cos / sin broadcast against y's leading dimensions)."""
    y = np.asarray(y, dtype=np.float64)
    even, odd = y[..., 0::2], y[..., 1::2]
    out = np.empty_like(y)
    out[..., 0::2] = even * cos - odd * sin
    out[..., 1::2] = odd * cos + even * sin
    return out


def tpa_append_reference(x, w, rope_cos, rope_sin, positions, num_heads, head_dim, rank_q, rank_k):
    """Factors of new tokens: y = x w^T with w[n_out, d_model], y's columns in the order
    qa[rq*h] qb[rq*d] ka[rk*h] kb[rk*d] va[rk*h] vb[rk*d]; qb and kb rotated at `positions[b, i]`.

    x[b, n, d_model], rope_cos / rope_sin[rope_len, d/2], positions[b, n] ->
    dict of float64 arrays qa[b,n,rq,h], qb[b,n,rq,d], ka[b,n,rk,h], kb[b,n,rk,d], va, vb."""
    x = np.asarray(x, dtype=np.float64)
    w = np.asarray(w, dtype=np.float64)
    b, n, _ = x.shape
    h, d = num_heads, head_dim
    y = x @ w.T
    widths = [rank_q * h, rank_q * d, rank_k * h, rank_k * d, rank_k * h, rank_k * d]
    assert w.shape[0] == sum(widths), (w.shape, widths)
    out, c0 = {}, 0
    for name, width, r, inner in zip(("qa", "qb", "ka", "kb", "va", "vb"), widths, (rank_q,) * 2 + (rank_k,) * 4, (h, d) * 3):
        out[name] = y[..., c0 : c0 + width].reshape(b, n, r, inner)
        c0 += width
    pos = np.asarray(positions)
    c = np.asarray(rope_cos, dtype=np.float64)[pos][:, :, None, :]  # [b, n, 1, d/2]
    s_ = np.asarray(rope_sin, dtype=np.float64)[pos][:, :, None, :]
    out["qb"] = rope_rotate(out["qb"], c, s_)
    out["kb"] = rope_rotate(out["kb"], c, s_)
    return out
