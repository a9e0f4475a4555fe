"""Error bounds of the bf16 matrix-core kernels against a float64 oracle that reads the same
bf16 inputs.  Test infrastructure.

What the kernels round, and nothing else: the reconstructed (and pre-scaled) Q once to bf16, the
reconstructed K and V once to bf16 (prefill; the decode kernels leave the cache factors as they
are and round only Q), the probabilities P once to bf16 before O += P V, and the output once to
bf16.  Everything else is fp32.  A bf16 rounding moves a value by at most 2^-9 of its size, so with
c = sm_scale:

  logit      x = c sum_d Q_d K_d        |dx|   <= 2 * 2^-9 * c * sum_d |Q_d| |K_d|          =: E
  logsumexp  is 1-Lipschitz in the sup norm of the logits of its row
                                        |dlse| <= max over the row's keys of E   (+ 2.5e-4 for the fp32 sums)
  softmax    p = exp(x - lse)           |dp|/p <= 2 E (first order)
  output     o = sum_k p_k V_k, P, V and o rounded once each
                                        |do|   <= (2 E + 3 * 2^-9) * max_k |V_k|  <= (2 E + 2^-7) max_k |V_k|

E is a worst case (a sum of absolute values; the error itself is a sum of signed terms, about
sqrt(d) smaller).  For the benchmark configurations' N(0,1)/sqrt(R) factors E is 1e-3 .. 4e-3
and the kernels' logsumexp error about 1e-4 (their tests keep the absolute bounds 2e-2 / 1e-3);
for unscaled N(0,1) factors with a query rank of one E reaches 0.1 and the kernels' logsumexp
error 1e-2 .. 5e-2 (measured: 1.3e-2 at |lse| ~ 10, 4.9e-2 at |lse| ~ 33).

`form="factored"` bounds the decode kernels, which never form K or V: there |K_d| is replaced by
(1/R) sum_r |a_r| |b_r,d| (and V likewise), which also bounds the materialised form.
"""

from __future__ import annotations

import numpy as np

EPS = 2.0**-9  # largest relative move of a round-to-nearest bf16 rounding


def _recon(x, num_heads, absolute_factors):
    a, b = x[..., :num_heads], x[..., num_heads:]
    if absolute_factors:
        a, b = np.abs(a), np.abs(b)
    out = np.matmul(np.swapaxes(a, 2, 3), b) / a.shape[2]  # [b, l, h, d]
    return np.abs(out)


def dense_bounds(q, k, v, sm_scale):
    """|q|, |k|, |v| dense [b, l, h, d] (absolute values taken here) -> (lse_bound[b, lq, h], o_bound[b, lq, h])."""
    q, k, v = (np.abs(np.nan_to_num(np.asarray(x, dtype=np.float64))) for x in (q, k, v))
    b, lq, h, _ = q.shape
    a_max = np.empty((b, lq, h))
    for bi in range(b):  # [h, lq, lk] at a time
        x = np.matmul(np.transpose(q[bi], (1, 0, 2)), np.transpose(k[bi], (1, 2, 0)))
        a_max[bi] = x.max(axis=-1).T
    e = 2.0 * EPS * sm_scale * a_max
    vmax = v.max(axis=(1, 3))[:, None, :]  # [b, 1, h]
    return 2.5e-4 + e, (2.0 * e + 2.0**-7) * vmax + 1e-6


def tpa_bounds(q, k, v, num_heads, sm_scale, form="materialised"):
    """Concatenated factors q[b,lq,rq,h+dk], k[b,lk,rk,h+dk], v[b,lk,rk,h+dv] (the bf16-rounded
    values the kernel reads) -> (lse_bound[b, lq, h], o_bound[b, lq, h])."""
    assert form in ("materialised", "factored")
    q, k, v = (np.nan_to_num(np.asarray(x, dtype=np.float64)) for x in (q, k, v))
    fact = form == "factored"
    return dense_bounds(_recon(q, num_heads, False), _recon(k, num_heads, fact), _recon(v, num_heads, fact), sm_scale)


def round_bf16(x):
    """float64/float32 array -> nearest bfloat16 (ties to even), returned as float64."""
    u = np.asarray(x, dtype=np.float32).view(np.uint32).astype(np.uint64)
    u = ((u + 0x7FFF + ((u >> 16) & 1)) & 0xFFFF0000).astype(np.uint32)
    return u.view(np.float32).astype(np.float64)


def emulate_bf16_prefill(q, k, v, num_heads, sm_scale, causal=False):
    """The rounding points of the bf16 prefill kernel in numpy (float64 between them): bf16 of the
    pre-scaled Q, of K, V, P and of the output.  -> (o[b,lq,h,dv], lse[b,lq,h])"""
    q, k, v = (np.asarray(x, dtype=np.float64) for x in (q, k, v))
    rec = lambda x: np.matmul(np.swapaxes(x[..., :num_heads], 2, 3), x[..., num_heads:]) / x.shape[2]
    log2e = 1.4426950408889634
    qs = round_bf16(rec(q) * (sm_scale * log2e))
    kk, vv = round_bf16(rec(k)), round_bf16(rec(v))
    x = np.einsum("bqhd,bkhd->bhqk", qs, kk)  # log2 domain
    if causal:
        lq, lk = x.shape[-2:]
        x = np.where(np.tril(np.ones((lq, lk), bool)), x, -np.inf)
    m = x.max(-1, keepdims=True)
    p = np.exp2(x - m)
    l = p.sum(-1, keepdims=True)
    o = np.einsum("bhqk,bkhd->bqhd", round_bf16(p), vv) / np.transpose(l, (0, 2, 1, 3))
    lse = (m[..., 0] + np.log2(l[..., 0])) / log2e
    return round_bf16(o), np.transpose(lse, (0, 2, 1))
