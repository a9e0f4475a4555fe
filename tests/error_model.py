"""Error bounds of the bf16 matrix-core kernels against a float64 oracle that reads the same
bf16 inputs.  Test infrastructure.

What the kernels round, and nothing else: the reconstructed (and pre-scaled) Q once to bf16, the
reconstructed K and V once to bf16 (prefill; the decode kernels leave the cache factors as they
are and round only Q), the probabilities P once to bf16 before O += P V, and the output once to
bf16.  Everything else is fp32.  A bf16 rounding (8 significant bits, round to nearest) moves a value by at
most 2^-8 of its size - half a spacing, relative to a value just above a power of two - so with c = sm_scale:

  logit      x = c sum_d Q_d K_d        |dx|   <= 2 * 2^-8 * c * sum_d |Q_d| |K_d|          =: E
  logsumexp  is 1-Lipschitz in the sup norm of the logits of its row
                                        |dlse| <= max over the row's keys of E   (+ 2.5e-4 for the fp32 sums)
  softmax    p = exp(x - lse)           |dp|/p <= 2 E (first order)
  output     o = sum_k p_k V_k, P, V and o rounded once each
                                        |do|   <= (2 E + 3 * 2^-8) * max_k |V_k|

The three roundings of the output term do line up where a row sees a single key (o = V_k: the softmax
reference is a whole number, so even the one probability, 2^(x - ceil x), is rounded); E is a worst case of
another kind (a sum of absolute values; the error itself is a sum of signed terms, about sqrt(d) smaller).
For the benchmark configurations' N(0,1)/sqrt(R) factors E is 2e-3 .. 8e-3 and the kernels' logsumexp error
about 1e-4 (their tests keep the absolute bounds 2e-2 / 1e-3); for unscaled N(0,1) factors with a query rank
of one E reaches 0.2 and the kernels' logsumexp error 1e-2 .. 5e-2 (measured: 1.3e-2 at |lse| ~ 10, 4.9e-2
at |lse| ~ 33).

`form="factored"` bounds the decode kernels, which never form K or V: there |K_d| is replaced by
(1/R) sum_r |a_r| |b_r,d| (and V likewise), which also bounds the materialised form.
"""

from __future__ import annotations

import numpy as np

EPS = 2.0**-8  # largest relative move of a round-to-nearest bf16 rounding (unit roundoff of 8 significant bits)


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
    return 2.5e-4 + e, (2.0 * e + 3.0 * EPS) * vmax + 1e-6


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


def truncate_bf16(x):
    """float64/float32 array -> bfloat16 by dropping the low 16 bits of the float32 (round toward zero)."""
    u = np.asarray(x, dtype=np.float32).view(np.uint32) & np.uint32(0xFFFF0000)
    return u.view(np.float32).astype(np.float64)


def bf16_ulp(x):
    """spacing of bfloat16 (8 significand bits) at |x|; the spacing at the smallest normal number below it"""
    ax = np.maximum(np.abs(np.asarray(x, dtype=np.float64)), 2.0**-126)
    return 2.0 ** (np.floor(np.log2(ax)) - 7)


LOG2E_F32 = float(np.float32(1.4426950408889634))


def emulate_bf16_attention(qd, kd, vd, sm_scale, bias=None, q_prescaled=False, faults=(), reference_shift=0):
    """The rounding points of the bf16 matrix-core prefill kernels in numpy, float64 between them, on dense
    qd[b,lq,h,d], kd[b,lk,h,d], vd[b,lk,h,dv] (float64, not yet rounded):

        Q' = bf16(Q * sm_scale * log2 e)   K' = bf16(K)   V' = bf16(V)
        x  = Q' . K' (+ bias, 0 / -inf)                       the exponent, base 2
        p  = 2^(x - m),  m a WHOLE number (here: ceil of the row maximum)
        l  = sum_k p_k (unrounded)          P = bf16(p)
        o  = bf16( (sum_k P_k V'_k) / l )   lse = (m + log2 l) / log2 e

    Because m is a whole number, P has the mantissa of bf16(2^x) whatever m is: the kernels' choice of
    reference (the first tile's maximum rounded up, moved by whole numbers) changes no bit of P, so this
    emulation and a kernel differ only by fp32 summation order, the fp32 accuracy of exp2 and rare double
    roundings - a few output elements in a thousand, by one bf16 spacing.

    `faults` injects mistakes for the tests of the gate itself: "p_twice" rounds P a second time at another
    scale, "p_trunc" truncates P instead of rounding it, "q_unscaled_round" rounds Q before the scale factor
    is applied and again after.

    -> (o[b,lq,h,dv] (bf16 values), lse[b,lq,h], slack[b,lq,h,dv]): slack is what an output element may move
    by before its last rounding without any rounding point being wrong: TIGHT_REL of sum_k p_k |V'_k| / l (fp32
    summation order), plus one bf16 spacing (2^-7 of the value at most) of the row's largest p_k / l times the largest |V'| of the column
    (the rounding of one P or V' element flipped, because an exponent or a reconstructed value that lies on a
    rounding boundary in float64 lies beside it in fp32; with many keys of similar weight this is nothing,
    with one dominant key it is the spacing of V')"""
    qd, kd, vd = (np.asarray(x, dtype=np.float64) for x in (qd, kd, vd))
    c = 1.0 if q_prescaled else float(np.float32(np.float32(sm_scale) * np.float32(LOG2E_F32)))
    if "q_unscaled_round" in faults:
        qd = round_bf16(qd)
    qs, kk, vv = round_bf16(qd * c), round_bf16(kd), round_bf16(vd)
    x = np.matmul(np.transpose(qs, (0, 2, 1, 3)), np.transpose(kk, (0, 2, 3, 1)))  # b h lq lk
    if bias is not None:
        x = x + np.asarray(bias, dtype=np.float64)[:, None, :, :]
    with np.errstate(invalid="ignore", divide="ignore", over="ignore"):
        m = np.ceil(x.max(-1, keepdims=True)) + int(reference_shift)  # any whole number gives the same bits
        p = np.exp2(x - m)  # a row without a visible key: -inf - -inf = NaN, as the kernels give
        l = p.sum(-1, keepdims=True)
        if "p_trunc" in faults:
            pr = truncate_bf16(p)
        elif "p_twice" in faults:
            pr = round_bf16(round_bf16(p * 0.75) / 0.75)
        else:
            pr = round_bf16(p)
        vt = np.transpose(vv, (0, 2, 1, 3))  # b h lk dv
        o = np.matmul(pr, vt) / l
        slack = TIGHT_REL * np.matmul(p, np.abs(vt)) / l + 2.0**-7 * (p.max(-1, keepdims=True) / l) * np.abs(vt).max(-2, keepdims=True)
        lse = np.where(np.isneginf(m[..., 0]), -np.inf, (m[..., 0] + np.log2(l[..., 0])) / LOG2E_F32)
    o = np.transpose(o, (0, 2, 1, 3))
    return round_bf16(o), np.transpose(lse, (0, 2, 1)), np.transpose(slack, (0, 2, 1, 3))


def reconstruct_dense(x, num_heads):
    """concatenated factors x[b,l,r,h+d] -> (1/R) sum_r a_r (x) b_r as [b,l,h,d], exact in float64"""
    x = np.asarray(x, dtype=np.float64)
    return np.matmul(np.swapaxes(x[..., :num_heads], 2, 3), x[..., num_heads:]) / x.shape[2]


def emulate_bf16_prefill(q, k, v, num_heads, sm_scale, causal=False, bias=None, faults=(), reference_shift=0):
    """emulate_bf16_attention on concatenated factors q[b,lq,rq,h+dk], k[b,lk,rk,h+dk], v[b,lk,rk,h+dv] (the
    bf16 values the kernel reads): Q, K and V are reconstructed exactly and rounded once, as both prefill
    routes do.  `bias` [b,lq,lk] of 0 / -inf is added to a top-left causal mask where `causal` is set.
    -> (o, lse[b,lq,h], slack)"""
    qd, kd, vd = (reconstruct_dense(x, num_heads) for x in (q, k, v))
    if causal:
        lq, lk = qd.shape[1], kd.shape[1]
        tri = np.where(np.tril(np.ones((lq, lk), bool)), 0.0, -np.inf)[None]
        bias = tri if bias is None else np.asarray(bias, dtype=np.float64) + tri
    return emulate_bf16_attention(qd, kd, vd, sm_scale, bias=bias, faults=faults, reference_shift=reference_shift)


def emulate_bf16_decode(q, k, v, num_heads, sm_scale, bias=None, faults=()):
    """The rounding points of the bf16 split-key decode kernels in numpy, float64 between them, on concatenated
    factors q[b,lq,rq,h+d], k[b,lk,rk,h+d], v[b,lk,rk,h+dv] (the bf16 values the kernel reads).  The cache
    factors are used as they are; K and V are never formed:

        Qm[h]  = bf16( (sm_scale log2 e / (rq rk)) * sum_r qa_r[h] qb_r )          the only rounding of the query
        x[h,t] = sum_j ka_j[t,h] (Qm[h] . kb_j[t])  (+ bias, 0 / -inf)             the exponent, base 2
        p      = 2^(x - m),  m a WHOLE number (ceil of the row maximum);  l = sum_t p (unrounded)
        P'_j   = bf16( p * va_j[t,h] )                                              one rounding per (key, rank)
        o      = bf16( (sum_t sum_j P'_j vb_j[t]) / (rk l) )       lse = (m + log2 l) / log2 e

    With m a whole number P' has the same significand whatever m is, so the split of the keys over waves and
    ranges changes no bit of it.  `faults`: "p_before_av" rounds p and then the product again, "p_trunc"
    truncates P', "q_unscaled_round" rounds the query sum before the scale factor and again after.
    -> (o[b,lq,h,dv], lse[b,lq,h], slack[b,lq,h,dv]) as emulate_bf16_attention."""
    q, k, v = (np.asarray(x, dtype=np.float64) for x in (q, k, v))
    h = num_heads
    rq, rk = q.shape[2], k.shape[2]
    c = float(np.float32(np.float32(np.float32(sm_scale) * np.float32(LOG2E_F32)) / (np.float32(rq) * np.float32(rk))))
    qsum = np.einsum("blrh,blrd->blhd", q[..., :h], q[..., h:])
    if "q_unscaled_round" in faults:
        qsum = round_bf16(qsum)
    qm = round_bf16(qsum * c)  # b lq h d
    t = np.einsum("bqhd,bkjd->bhqkj", qm, k[..., h:])  # Qm . kb_j
    x = np.einsum("bhqkj,bkjh->bhqk", t, k[..., :h])
    if bias is not None:
        x = x + np.asarray(bias, dtype=np.float64)[:, None, :, :]
    with np.errstate(invalid="ignore", divide="ignore", over="ignore"):
        m = np.ceil(x.max(-1, keepdims=True))
        p = np.exp2(x - m)
        l = p.sum(-1, keepdims=True)
        va = np.transpose(v[..., :h], (0, 3, 1, 2))[:, :, None]  # b h 1 lk rk
        pa = p[..., None] * va  # b h lq lk rk
        if "p_trunc" in faults:
            pr = truncate_bf16(pa)
        elif "p_before_av" in faults:
            pr = round_bf16(round_bf16(p)[..., None] * va)
        else:
            pr = round_bf16(pa)
        vb = v[..., h:]  # b lk rk dv
        o = np.einsum("bhqkj,bkjd->bhqd", pr, vb) / (rk * l)
        mass = np.einsum("bhqkj,bkjd->bhqd", np.abs(pa), np.abs(vb)) / (rk * l)
        one = 2.0**-7 * (np.abs(pa).max(axis=(-1, -2))[..., None] / l) * np.abs(vb).max(axis=(1, 2))[:, None, None, :] / rk
        slack = TIGHT_REL * mass + one
        lse = np.where(np.isneginf(m[..., 0]), -np.inf, (m[..., 0] + np.log2(l[..., 0])) / LOG2E_F32)
    return round_bf16(np.transpose(o, (0, 2, 1, 3))), np.transpose(lse, (0, 2, 1)), np.transpose(slack, (0, 2, 1, 3))


# The gate that holds a bf16 kernel to its emulation: per output element two bf16 spacings (a flipped last
# rounding, and the neighbouring value where the element sits at a power of two) plus the emulation's slack
# (fp32 summation order, one flipped P or V' rounding), at most TIGHT_FRAC of the elements different at all,
# and the logsumexp within TIGHT_LSE (+ its own fp32 rounding).  Measured on the GPU over benchmark-like,
# sharp, packed and high-rank problems on both prefill routes: 0.002 - 0.17 % of the elements differ,
# logsumexp by at most 7e-5; a second rounding of P, a truncated P or Q rounded before its scale factor make
# 9 - 65 % of the elements differ (tests/test_error_model.py).
TIGHT_SPACINGS = 2.0
TIGHT_REL = 1e-4
TIGHT_FRAC = 0.01
TIGHT_LSE = 2e-4


def tight_violations(o, lse_blh, o_emu, lse_emu, slack):
    """-> list of strings, empty if (o, lse) agree with the emulation (see TIGHT_*).  All arrays float64;
    o / o_emu hold bf16 values."""
    bad = []
    o, o_emu = np.asarray(o, dtype=np.float64), np.asarray(o_emu, dtype=np.float64)
    if not np.array_equal(np.isnan(o), np.isnan(o_emu)):
        return ["NaN rows differ"]
    if not np.array_equal(np.isneginf(lse_blh), np.isneginf(lse_emu)):
        return ["-inf logsumexp rows differ"]
    ok = ~np.isnan(o_emu)
    if ok.any():
        d = np.abs(np.where(ok, o - o_emu, 0.0))
        tol = np.where(ok, TIGHT_SPACINGS * np.maximum(bf16_ulp(o_emu), bf16_ulp(o)) + np.nan_to_num(slack), np.inf)
        worst = (d / tol).max()
        if worst > 1.0:
            bad.append(f"an output element is {worst:.2f} x ({TIGHT_SPACINGS:.0f} bf16 spacings + slack) away from the emulation")
        frac = (d > 0).sum() / ok.sum()
        if frac > TIGHT_FRAC:
            bad.append(f"{100 * frac:.1f} % of the output elements differ from the emulation (gate {100 * TIGHT_FRAC:.0f} %)")
    okl = ~np.isneginf(lse_emu)
    if okl.any():
        with np.errstate(invalid="ignore"):
            dl = np.abs(np.where(okl, lse_blh - lse_emu, 0.0))
        told = TIGHT_LSE + 1e-6 * np.abs(np.where(okl, lse_emu, 0.0))
        if (dl > told).any():
            bad.append(f"logsumexp off by {dl.max():.2e} (gate {TIGHT_LSE:.0e})")
    return bad
