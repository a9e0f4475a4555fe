"""Tensor Product Attention forward: the operator API of the reference's tpa/tpa.py.

Same names, argument meaning and error behaviour as tpa/tpa.py:35-165,220-242,446-543; the
work is done by the gfx950 HIP kernels behind the C ABI (include/tpa_abi.h).  Arrays are torch
tensors that live on the GPU (numpy arrays are copied there and back).  Differences from the
reference, all on purpose:

  * accumulation is always fp32 (the reference accumulates in the input dtype, tpa/tpa.py:433-434);
  * the logsumexp residual is fp32 (the reference keeps it in the input dtype, tpa/tpa.py:530);
  * sequence lengths need not be multiples of the block sizes (tpa/tpa.py:489-490 asserts that);
    `block_sizes` is accepted and ignored because the kernels fix their own tiles;
  * `nomat` picks an evaluation order, as in the reference (tpa/tpa.py:250), and changes no
    result: `nomat=True` runs the kernels that never form K or V (the split-key decode kernels,
    over windows of 64 query rows, two launches per window) wherever they take the problem, and
    the plain kernel elsewhere.  Those kernels form Q per head and share one pass over the kb / vb
    rows between the heads.  `tpa_factors(nomat="pairs")` runs the reference's own arithmetic: a
    table bb = qb_r . kb_s per rank pair shared by the heads of a workgroup, combined per head with
    qa_r ka_s (tpa/tpa.py:333-359; csrc/tpa_nomat.hip); it is the slowest of the three.  The default rebuilds
    K/V tiles in LDS, which is the faster order on matrix cores except for a few query rows over
    a long cache (`tpa_decode`);
  * `interpret=True` (the Pallas CPU interpreter upstream) selects the plain fp32-arithmetic
    kernel instead of the MFMA kernels; `debug` is ignored;
  * the backward pass (tpa/tpa.py:168-214,546-995) goes through dense Q, K, V and dense gradients
    in a workspace (bf16 MFMA kernels for bf16 inputs and fp32 MFMA kernels for fp32 inputs of
    head sizes 64 and 128, fp32 vector-ALU kernels otherwise); gradients are accumulated in fp32
    and cast to the input dtype; torch.autograd reaches it through `tpa()`.
"""

from __future__ import annotations

import dataclasses

import numpy as np
import torch

from . import _dispatch as _d

__all__ = [
    "BlockSizes", "tpa", "tpa_factors", "tpa_decode", "tpa_cache_append", "tpa_factors_bwd", "_tpa_fwd", "_tpa_bwd", "_fwd", "_bwd",
    "_precompute_delta", "_lse", "_lse_accum",
]


# Whether forward calls bring the optional workspace with which the library reconstructs dense Q, K, V
# once and runs its fastest prefill loop (`tpa_factors(use_workspace=...)` overrides it per call).
USE_WORKSPACE = True


@dataclasses.dataclass
class BlockSizes:
    """Tile configuration of the reference kernels (tpa/tpa.py:35-70).  Kept for signature
    compatibility; the HIP kernels use fixed tiles and ignore it."""

    block_q: int = 128
    block_kv: int = 128
    block_h: int = 4


def _lse(x: torch.Tensor) -> torch.Tensor:
    """Logsumexp over the last dimension, -inf for all -inf input (tpa/tpa.py:220-226)."""
    m = torch.amax(x, dim=-1)
    safe = torch.where(torch.isneginf(m), torch.zeros_like(m), m)
    l_ = safe + torch.log(torch.sum(torch.exp(x - safe[..., None]), dim=-1))
    return torch.where(torch.isneginf(m), m, l_)


def _lse_accum(a: torch.Tensor, b: torch.Tensor) -> torch.Tensor:
    """log(exp(a) + exp(b)), -inf safe (tpa/tpa.py:228-242)."""
    assert a.shape == b.shape, f"mismatching shapes: {a.shape}, {b.shape}"
    hi = torch.maximum(a, b)
    lo = torch.minimum(a, b)
    safe = torch.where(torch.isneginf(hi), torch.zeros_like(hi), hi)
    lse = safe + torch.log(1 + torch.exp(lo - safe))
    return torch.where(torch.isneginf(hi), hi, lse)


CAUSAL_BOTTOM_RIGHT = 2  # value of `causal`: the last query aligned with the last key of each batch entry
# `nomat` of tpa_factors: True / 1 = the split-key kernels over windows of query rows, "pairs" / 2 = the
# reference's own arithmetic, a table per rank pair shared by the heads of a workgroup (tpa/tpa.py:333-359)
NOMAT_SPLIT_KEYS = 1
NOMAT_RANK_PAIRS = 2


def _causal_code(causal) -> int:
    """False / True as in the reference (tpa/tpa.py:82; True = top-left aligned mask), or
    CAUSAL_BOTTOM_RIGHT (an addition): the mask counted from the end of each batch entry's keys
    (`kv_lengths[b]` where given), so that the last query sees every key, the one before it all
    but the last, ... - freshly appended tokens over caches of different lengths."""
    if causal is True or causal is False:
        return int(causal)
    code = int(causal)
    if code not in (0, 1, CAUSAL_BOTTOM_RIGHT):
        raise ValueError(f"causal must be False, True or CAUSAL_BOTTOM_RIGHT, got {causal!r}")
    return code


def _as_device_tensor(x, device):
    """torch GPU tensors pass through; numpy arrays / CPU tensors are copied to `device`."""
    if isinstance(x, torch.Tensor):
        return x if x.is_cuda else x.to(device)
    return torch.as_tensor(np.asarray(x)).to(device)


def _pick_device(*xs) -> torch.device:
    for x in xs:
        if isinstance(x, torch.Tensor) and x.is_cuda:
            return x.device
    if not torch.cuda.is_available():
        raise RuntimeError("tpa needs an AMD GPU: no HIP device is visible and there is no CPU fallback")
    return torch.device("cuda", torch.cuda.current_device())


def _segment_ids(ids, batch: int, length: int, device) -> torch.Tensor | None:
    if ids is None:
        return None
    t = _as_device_tensor(ids, device).to(torch.int32)
    if t.dim() == 1:  # the reference vmaps with in_axes=None for unbatched ids (tpa/tpa.py:144-163)
        t = t[None].expand(batch, length)
    if tuple(t.shape) != (batch, length):
        raise ValueError(f"segment ids must have shape {(batch, length)}, got {tuple(t.shape)}")
    return t.contiguous()


def _lengths(kv_lengths, batch: int, device) -> torch.Tensor | None:
    if kv_lengths is None:
        return None
    t = _as_device_tensor(kv_lengths, device).to(torch.int32).contiguous()
    if tuple(t.shape) != (batch,):
        raise ValueError(f"kv_lengths must have shape {(batch,)}, got {tuple(t.shape)}")
    return t


def tpa_factors(
    qa, qb, ka, kb, va, vb,
    q_segment_ids=None,
    kv_segment_ids=None,
    sm_scale: float = 1.0,
    causal: bool = False,
    kernel: int = _d.KERNEL_AUTO,
    return_lse: bool = True,
    use_workspace: bool | None = None,
    kv_lengths=None,
    causal_offset: int = 0,
    nomat: bool = False,
):
    """Forward pass on the six split factor arrays, the operands of the reference's kernel
    launch (tpa/tpa.py:246-251,543) with a leading batch dimension:

        qa[b,lq,rq,h] qb[b,lq,rq,dk] ka[b,lk,rk,h] kb[b,lk,rk,dk] va[b,lk,rk,h] vb[b,lk,rk,dv]

    Returns (o[b,lq,h,dv] in the input dtype, lse[b,h,lq] fp32 or None).  The arrays may be
    views (e.g. slices of the concatenated tensors); only the last dimension must be contiguous.
    `use_workspace=False` withholds the optional scratch memory, which keeps the call on the
    fused prefill kernel whatever the problem (None: the module's `USE_WORKSPACE`, True unless changed).  `kv_lengths` (int32 [b], an addition): batch
    entry i attends to its first kv_lengths[i] keys only; the rest of its k / v rows is padding
    that is never read.  `causal_offset` (an addition, also taken by `tpa_factors_bwd`): with `causal`, query i
    sees keys up to i + causal_offset; 0 is the reference's top-left alignment
    (tpa/tpa.py:377-379), lk - lq aligns the last query with the last key (new tokens over a
    cache), and a sequence shard of a ring (tpa/ring_tpa.py:73-79) passes the distance from the
    first key of the shard it meets to its own first query.  `nomat` (tpa/tpa.py:250): never
    form K or V - same results, the rank-space order of operations (see the module docstring).
    """
    if use_workspace is None:
        use_workspace = USE_WORKSPACE
    device = _pick_device(qa, qb, ka, kb, va, vb)
    qa, qb, ka, kb, va, vb = (_as_device_tensor(x, device) for x in (qa, qb, ka, kb, va, vb))
    dtype = qa.dtype
    for name, t in (("qb", qb), ("ka", ka), ("kb", kb), ("va", va), ("vb", vb)):
        if t.dtype != dtype:
            raise TypeError(f"{name} has dtype {t.dtype}, expected {dtype}")
    b, lq, rq, h = qa.shape
    _, lk, rk, dv = vb.shape
    dk = qb.shape[-1]
    # shape rules of tpa/tpa.py:474-475: k and v share length and rank, q and k share h + dk
    assert tuple(qb.shape) == (b, lq, rq, dk), qb.shape
    assert tuple(ka.shape) == (b, lk, rk, h), ka.shape
    assert tuple(kb.shape) == (b, lk, rk, dk), kb.shape
    assert tuple(va.shape) == (b, lk, rk, h), va.shape
    qseg = _segment_ids(q_segment_ids, b, lq, device)
    kvseg = _segment_ids(kv_segment_ids, b, lk, device)
    if (qseg is None) != (kvseg is None):
        raise ValueError("q_segment_ids and kv_segment_ids must be given together")

    kvlen = _lengths(kv_lengths, b, device)
    o = torch.empty((b, lq, h, dv), dtype=dtype, device=device)
    lse = torch.empty((b, h, lq), dtype=torch.float32, device=device) if return_lse else None
    lib = _d.load_library()
    # hand the library the workspace with which it can pick its fastest kernel (split partials for
    # a decode through this entry point, dense Q, K and V for prefills that are long enough); it decides whether
    # the problem qualifies
    ws, ws_ptr, ws_bytes = None, None, 0
    # (fp32 inputs: only the split-key decode kernel takes a workspace)
    nomat = NOMAT_RANK_PAIRS if nomat in ("pairs", NOMAT_RANK_PAIRS) and nomat is not True else int(bool(nomat))
    if nomat == NOMAT_RANK_PAIRS:
        pass  # one launch, no workspace
    elif nomat:
        # the split partials of the non-materialising kernels: required, not optional
        need = lib.tpa_fwd_nomat_workspace_bytes(b, lq, lk, h, dk, dv, rq, rk) if kernel != _d.KERNEL_GENERIC else 0
        if need:
            ws = torch.empty(need + 256, dtype=torch.uint8, device=device)
            pad = (-ws.data_ptr()) % 256
            ws_ptr, ws_bytes = ws.data_ptr() + pad, need
    elif use_workspace and kernel != _d.KERNEL_GENERIC and (dtype == torch.bfloat16 or lq <= 16):
        need = lib.tpa_fwd_workspace_bytes(b, lq, lk, h, dk, dv, rq, rk)
        if need:
            ws = torch.empty(need + 256, dtype=torch.uint8, device=device)
            pad = (-ws.data_ptr()) % 256
            ws_ptr, ws_bytes = ws.data_ptr() + pad, need
    args = _d.TpaFwdArgs(
        qa=_d.factor(qa), qb=_d.factor(qb), ka=_d.factor(ka), kb=_d.factor(kb), va=_d.factor(va), vb=_d.factor(vb),
        q_segment_ids=qseg.data_ptr() if qseg is not None else None,
        kv_segment_ids=kvseg.data_ptr() if kvseg is not None else None,
        o=o.data_ptr(), lse=lse.data_ptr() if lse is not None else None,
        B=b, lq=lq, lk=lk, H=h, dk=dk, dv=dv, rq=rq, rk=rk,
        dtype=_d.dtype_code(dtype), sm_scale=float(sm_scale), causal=_causal_code(causal), kernel=int(kernel),
        workspace=ws_ptr, workspace_bytes=ws_bytes, num_splits=0,
        kv_lengths=kvlen.data_ptr() if kvlen is not None else None,
        causal_offset=int(causal_offset), nomat=nomat,
    )
    with torch.cuda.device(device):
        _d.check("tpa_fwd", lib.tpa_fwd(args, _d.current_stream_ptr(device)))
    return o, lse


def tpa_decode(
    qa, qb, ka, kb, va, vb,
    sm_scale: float = 1.0,
    num_splits: int = 0,
    workspace: torch.Tensor | None = None,
    kernel: int = _d.KERNEL_AUTO,
    kv_lengths=None,
    page_table=None,
    causal: bool = False,
    causal_offset: int = 0,
):
    """Few query tokens against a long factored KV cache, split over key ranges.

    The reference has no separate entry point for this: it is tpa() with lq = 1
    (block_q = min(128, lq), tpa/tpa.py:485).  Same operands as `tpa_factors`; the cache is
    ka/kb/va/vb.  `workspace` (uint8, at least `decode_workspace_bytes(...)`) may be passed to
    avoid the allocation.  `kv_lengths` (int32 [b]): how many tokens of each batch entry's cache
    are filled (sequences of different lengths in one padded cache); the rest is not read.
    `page_table` (int32 [b, pages_per_seq]): the cache arrays are then page pools
    [pages, page_size, rk, x] shared by all sequences, and token t of entry i lives in page
    page_table[i, t // page_size]; the logical cache length is pages_per_seq * page_size.
    `causal` with `causal_offset` (see `tpa_factors`): query i sees keys up to i + causal_offset,
    e.g. lq freshly appended tokens that must not see each other's successors
    (causal_offset = lk - lq); segment ids are not taken here.
    Returns (o[b,lq,h,dv], lse[b,h,lq]).
    """
    device = _pick_device(qa, qb, ka, kb, va, vb)
    qa, qb, ka, kb, va, vb = (_as_device_tensor(x, device) for x in (qa, qb, ka, kb, va, vb))
    dtype = qa.dtype
    b, lq, rq, h = qa.shape
    dk = qb.shape[-1]
    pt, page_size, pages_per_seq = None, 0, 0
    if page_table is None:
        _, lk, rk, dv = vb.shape
        assert tuple(kb.shape) == (b, lk, rk, dk), kb.shape
        assert tuple(ka.shape) == (b, lk, rk, h) and tuple(va.shape) == (b, lk, rk, h)
    else:
        pt = _as_device_tensor(page_table, device).to(torch.int32).contiguous()
        assert pt.dim() == 2 and pt.shape[0] == b, pt.shape
        npages, page_size, rk, dv = vb.shape
        pages_per_seq = pt.shape[1]
        lk = pages_per_seq * page_size
        assert tuple(kb.shape) == (npages, page_size, rk, dk), kb.shape
        assert tuple(ka.shape) == (npages, page_size, rk, h) and tuple(va.shape) == (npages, page_size, rk, h)
    kvlen = _lengths(kv_lengths, b, device)
    lib = _d.load_library()
    need = lib.tpa_decode_workspace_bytes(b, lq, lk, h, dv, num_splits)
    if workspace is None:
        workspace = torch.empty(max(need, 16), dtype=torch.uint8, device=device)
    o = torch.empty((b, lq, h, dv), dtype=dtype, device=device)
    lse = torch.empty((b, h, lq), dtype=torch.float32, device=device)
    args = _d.TpaFwdArgs(
        qa=_d.factor(qa), qb=_d.factor(qb), ka=_d.factor(ka), kb=_d.factor(kb), va=_d.factor(va), vb=_d.factor(vb),
        q_segment_ids=None, kv_segment_ids=None, o=o.data_ptr(), lse=lse.data_ptr(),
        B=b, lq=lq, lk=lk, H=h, dk=dk, dv=dv, rq=rq, rk=rk,
        dtype=_d.dtype_code(dtype), sm_scale=float(sm_scale), causal=_causal_code(causal), kernel=int(kernel),
        workspace=workspace.data_ptr(), workspace_bytes=workspace.numel() * workspace.element_size(),
        num_splits=int(num_splits),
        kv_lengths=kvlen.data_ptr() if kvlen is not None else None,
        page_table=pt.data_ptr() if pt is not None else None, page_size=int(page_size), pages_per_seq=int(pages_per_seq),
        causal_offset=int(causal_offset),
    )
    with torch.cuda.device(device):
        _d.check("tpa_decode", lib.tpa_decode(args, _d.current_stream_ptr(device)))
    return o, lse


def tpa_cache_append(
    x, w, rope_cos, rope_sin, ka, kb, va, vb,
    kv_lengths=None,
    *,
    rank_q: int,
    positions=None,
    page_table=None,
    kernel: int = _d.KERNEL_AUTO,
    workspace: torch.Tensor | None = None,
    use_workspace: bool | None = None,
):
    """The producer step for `n` new tokens per sequence (an addition: the reference takes the
    factors as given): y = x w^T gives the six rank factors of every token, the B factors of Q and
    K are rotated by the rotary tables at the token's position, and the K / V factors are written
    into the cache `ka, kb, va, vb` at token `kv_lengths[b] + i` - the arrays `tpa_decode` reads.

    x[b, n, d_model]; w[rq*(h+d) + 2*rk*(h+d), d_model] (rows in the order qa, qb, ka, kb, va, vb,
    as torch.nn.Linear keeps its weight); rope_cos, rope_sin[rope_len, d/2] fp32; the cache arrays
    [b, cache_len, rk, h|d], or page pools [pages, page_size, rk, h|d] with `page_table`
    [b, pages_per_seq]; `positions` [b, n] defaults to kv_lengths[b] + i.  A decode step (at most 64 new
    tokens in all) is faster with scratch memory for partial sums: `workspace` (uint8, at least
    `cache_append_workspace_bytes(...)`; a serving loop passes the same one every step) or, with
    `use_workspace` (default: the module's `USE_WORKSPACE`), one allocated here.
    Returns (qa[b, n, rq, h], qb[b, n, rq, d], new_kv_lengths[b])."""
    device = _pick_device(x, w, ka, kb, va, vb)
    x, w, ka, kb, va, vb = (_as_device_tensor(t, device) for t in (x, w, ka, kb, va, vb))
    dtype = x.dtype
    for name, t in (("w", w), ("ka", ka), ("kb", kb), ("va", va), ("vb", vb)):
        if t.dtype != dtype:
            raise TypeError(f"{name} has dtype {t.dtype}, expected {dtype}")
    b, n, d_model = x.shape
    rk, h = ka.shape[2], ka.shape[3]
    d = kb.shape[3]
    rq = int(rank_q)
    assert tuple(w.shape) == (rq * (h + d) + 2 * rk * (h + d), d_model), w.shape
    assert kb.shape[:3] == ka.shape[:3] and va.shape == ka.shape and vb.shape == kb.shape, (ka.shape, kb.shape, va.shape, vb.shape)
    cos = _as_device_tensor(rope_cos, device).to(torch.float32).contiguous()
    sin = _as_device_tensor(rope_sin, device).to(torch.float32).contiguous()
    assert cos.shape == sin.shape and cos.dim() == 2 and cos.shape[1] == d // 2, (cos.shape, d)
    pt, page_size, pages_per_seq = None, 0, 0
    if page_table is None:
        assert ka.shape[0] == b, ka.shape
        cache_len = ka.shape[1]
    else:
        pt = _as_device_tensor(page_table, device).to(torch.int32).contiguous()
        assert pt.dim() == 2 and pt.shape[0] == b, pt.shape
        page_size, pages_per_seq = ka.shape[1], pt.shape[1]
        cache_len = pages_per_seq * page_size
    kvlen = _lengths(kv_lengths, b, device)
    pos = None
    if positions is not None:
        pos = _as_device_tensor(positions, device).to(torch.int32).contiguous()
        assert tuple(pos.shape) == (b, n), pos.shape
    x, w = x.contiguous(), w.contiguous()
    qa = torch.empty((b, n, rq, h), dtype=dtype, device=device)
    qb = torch.empty((b, n, rq, d), dtype=dtype, device=device)
    new_len = torch.empty((b,), dtype=torch.int32, device=device)
    lib = _d.load_library()
    ws_ptr, ws_bytes = None, 0
    if use_workspace is None:
        use_workspace = USE_WORKSPACE
    if workspace is None and use_workspace and kernel != _d.KERNEL_GENERIC:
        need = lib.tpa_cache_append_workspace_bytes(b, n, d_model, h, d, rq, rk, _d.dtype_code(dtype))
        if need:
            workspace = torch.empty(need + 16, dtype=torch.uint8, device=device)
    if workspace is not None:
        pad = (-workspace.data_ptr()) % 16
        ws_ptr, ws_bytes = workspace.data_ptr() + pad, workspace.numel() * workspace.element_size() - pad
    args = _d.TpaAppendArgs(
        x=x.data_ptr(), w=w.data_ptr(), rope_cos=cos.data_ptr(), rope_sin=sin.data_ptr(),
        positions=None if pos is None else pos.data_ptr(), kv_lengths=None if kvlen is None else kvlen.data_ptr(),
        new_kv_lengths=new_len.data_ptr(),
        qa=_d.factor(qa), qb=_d.factor(qb), ka=_d.factor(ka), kb=_d.factor(kb), va=_d.factor(va), vb=_d.factor(vb),
        page_table=None if pt is None else pt.data_ptr(), page_size=int(page_size), pages_per_seq=int(pages_per_seq),
        B=b, n=n, d_model=d_model, H=h, D=d, rq=rq, rk=rk, cache_len=int(cache_len), rope_len=int(cos.shape[0]),
        dtype=_d.dtype_code(dtype), kernel=int(kernel), workspace=ws_ptr, workspace_bytes=ws_bytes,
    )
    with torch.cuda.device(device):
        _d.check("tpa_cache_append", lib.tpa_cache_append(args, _d.current_stream_ptr(device)))
    return qa, qb, new_len


def cache_append_workspace_bytes(b: int, n: int, d_model: int, h: int, d: int, rq: int, rk: int, dtype=torch.bfloat16) -> int:
    return int(_d.load_library().tpa_cache_append_workspace_bytes(b, n, d_model, h, d, rq, rk, _d.dtype_code(dtype)))


def decode_workspace_bytes(b: int, lq: int, lk: int, h: int, dv: int, num_splits: int = 0) -> int:
    return int(_d.load_library().tpa_decode_workspace_bytes(b, lq, lk, h, dv, num_splits))


def tpa_factors_bwd(
    qa, qb, ka, kb, va, vb,
    q_segment_ids, kv_segment_ids,
    o, lse, do,
    sm_scale: float = 1.0,
    causal: bool = False,
    grads=None,
    workspace: torch.Tensor | None = None,
    kernel: int = _d.KERNEL_AUTO,
    causal_offset: int = 0,
    kv_lengths=None,
):
    """Backward pass on the split factor arrays: the operands of the reference's backward kernel
    launch (tpa/tpa.py:872-958) with a leading batch dimension, `lse` as [b, h, lq] fp32.

    Returns the six fp32 gradients (dqa, dqb, dka, dkb, dva, dvb), each shaped like its factor.
    `grads` may hold six fp32 tensors (or views, e.g. the two parts of a concatenated
    dq[b, lq, rq, h+dk]) to be written in place.  `causal_offset`: the value the forward call
    was made with (see `tpa_factors`).  `kv_lengths` (int32 [b]): the value the forward call was made
    with.  The backward kernels take a ragged batch as a mask: the padding keys get a segment id that no
    query carries (ids are made up here where the call has none), so they receive zero gradients and the
    tiles that hold only padding are skipped.  Unlike the forward, the backward does read the padding rows of
    k and v: they must hold finite values.  `causal=CAUSAL_BOTTOM_RIGHT` together with `kv_lengths` (an
    offset per batch entry) is not available here and raises NotImplementedError.
    """
    device = _pick_device(qa, qb, ka, kb, va, vb)
    qa, qb, ka, kb, va, vb, o, lse, do = (_as_device_tensor(x, device) for x in (qa, qb, ka, kb, va, vb, o, lse, do))
    dtype = qa.dtype
    b, lq, rq, h = qa.shape
    _, lk, rk, dv = vb.shape
    dk = qb.shape[-1]
    assert tuple(kb.shape) == (b, lk, rk, dk), kb.shape
    assert tuple(o.shape) == (b, lq, h, dv) and tuple(do.shape) == (b, lq, h, dv), (o.shape, do.shape)
    assert tuple(lse.shape) == (b, h, lq), lse.shape
    qseg = _segment_ids(q_segment_ids, b, lq, device)
    kvseg = _segment_ids(kv_segment_ids, b, lk, device)
    kvlen = _lengths(kv_lengths, b, device)
    if kvlen is not None:
        if _causal_code(causal) == CAUSAL_BOTTOM_RIGHT:
            raise NotImplementedError("tpa_factors_bwd: kv_lengths with causal=CAUSAL_BOTTOM_RIGHT needs an offset per batch entry")
        padding = torch.arange(lk, device=device, dtype=torch.int32)[None, :] >= kvlen[:, None]
        if qseg is None:
            qseg = torch.zeros((b, lq), dtype=torch.int32, device=device)
            kvseg = padding.to(torch.int32).contiguous()
        else:
            below = torch.minimum(qseg.min(), kvseg.min()) - 1  # an id that no query carries
            kvseg = torch.where(padding, below.to(torch.int32), kvseg).contiguous()
    o = o.to(dtype).contiguous()
    do = do.to(dtype).contiguous()
    lse = lse.to(torch.float32).contiguous()
    if grads is None:
        grads = tuple(torch.empty(t.shape, dtype=torch.float32, device=device) for t in (qa, qb, ka, kb, va, vb))
    lib = _d.load_library()
    need = lib.tpa_bwd_workspace_bytes(b, lq, lk, h, dk, dv)
    if workspace is None:
        workspace = torch.empty(need + 256, dtype=torch.uint8, device=device)
    pad = (-workspace.data_ptr()) % 256
    args = _d.TpaBwdArgs(
        qa=_d.factor(qa), qb=_d.factor(qb), ka=_d.factor(ka), kb=_d.factor(kb), va=_d.factor(va), vb=_d.factor(vb),
        q_segment_ids=None if qseg is None else qseg.data_ptr(),
        kv_segment_ids=None if kvseg is None else kvseg.data_ptr(),
        o=o.data_ptr(), lse=lse.data_ptr(), d_o=do.data_ptr(),
        dqa=_d.grad(grads[0]), dqb=_d.grad(grads[1]), dka=_d.grad(grads[2]), dkb=_d.grad(grads[3]),
        dva=_d.grad(grads[4]), dvb=_d.grad(grads[5]),
        B=b, lq=lq, lk=lk, H=h, dk=dk, dv=dv, rq=rq, rk=rk,
        dtype=_d.dtype_code(dtype), sm_scale=float(sm_scale), causal=_causal_code(causal), kernel=int(kernel),
        workspace=workspace.data_ptr() + pad, workspace_bytes=workspace.numel() - pad,
        causal_offset=int(causal_offset),
    )
    with torch.cuda.device(device):
        _d.check("tpa_bwd", lib.tpa_bwd(args, _d.current_stream_ptr(device)))
    return tuple(grads)


def bwd_workspace_bytes(b: int, lq: int, lk: int, h: int, dk: int, dv: int) -> int:
    return int(_d.load_library().tpa_bwd_workspace_bytes(b, lq, lk, h, dk, dv))


def _bwd_concat(q, k, v, qseg, kvseg, o, lse_bhl, do, num_heads, sm_scale, causal, causal_offset=0):
    """Gradients in the concatenated layout of q, k, v (fp32), written in place by the kernels."""
    h = num_heads
    dq, dk, dv = (torch.empty(t.shape, dtype=torch.float32, device=t.device) for t in (q, k, v))
    views = (dq[..., :h], dq[..., h:], dk[..., :h], dk[..., h:], dv[..., :h], dv[..., h:])
    tpa_factors_bwd(
        q[..., :h], q[..., h:], k[..., :h], k[..., h:], v[..., :h], v[..., h:],
        qseg, kvseg, o, lse_bhl, do, sm_scale, causal, grads=views, causal_offset=causal_offset,
    )
    return dq, dk, dv


class _TpaFunction(torch.autograd.Function):
    """The operator with its vjp, as tpa.defvjp(_tpa_fwd, _tpa_bwd) registers it (tpa/tpa.py:217)."""

    @staticmethod
    def forward(ctx, q, k, v, num_heads, qseg, kvseg, sm_scale, causal, kernel, causal_offset=0, nomat=False):
        qa, qb = q[..., :num_heads], q[..., num_heads:]
        ka, kb = k[..., :num_heads], k[..., num_heads:]
        va, vb = v[..., :num_heads], v[..., num_heads:]
        o, lse = tpa_factors(qa, qb, ka, kb, va, vb, qseg, kvseg, sm_scale, causal, kernel, causal_offset=causal_offset, nomat=nomat)
        ctx.mark_non_differentiable(lse)
        ctx.save_for_backward(q, k, v, o, lse)
        ctx.statics = (num_heads, qseg, kvseg, sm_scale, causal, causal_offset)
        return o, lse

    @staticmethod
    def backward(ctx, do, _dlse):
        q, k, v, o, lse = ctx.saved_tensors
        num_heads, qseg, kvseg, sm_scale, causal, causal_offset = ctx.statics
        dq, dk, dv = _bwd_concat(q, k, v, qseg, kvseg, o, lse, do, num_heads, sm_scale, causal, causal_offset)
        return dq.to(q.dtype), dk.to(k.dtype), dv.to(v.dtype), None, None, None, None, None, None, None, None


def _tpa_fwd(
    q, k, v, num_heads, q_segment_ids, kv_segment_ids, sm_scale, causal, block_sizes, nomat, debug, interpret,
    causal_offset: int = 0,
):
    """tpa/tpa.py:124-165: returns (o, residuals) with residuals (q, k, v, qseg, kvseg, o, l),
    l[b, lq, h] being the logsumexp in the reference's layout (a transposed view, fp32)."""
    del block_sizes, debug
    device = _pick_device(q, k, v)
    q, k, v = (_as_device_tensor(x, device) for x in (q, k, v))
    if q.dim() != 4 or k.dim() != 4 or v.dim() != 4:
        raise ValueError("q, k, v must be [b, l, r, h + d]")
    b, lq, rq, h_dk = q.shape
    _, lk, rk, _ = v.shape  # rank and length of the keys are read from v (tpa/tpa.py:474)
    assert tuple(k.shape) == (b, lk, rk, h_dk), k.shape  # tpa/tpa.py:475
    assert 0 < num_heads < h_dk and num_heads < v.shape[-1], (num_heads, q.shape, v.shape)
    kernel = _d.KERNEL_GENERIC if interpret else _d.KERNEL_AUTO
    o, lse = _TpaFunction.apply(q, k, v, int(num_heads), q_segment_ids, kv_segment_ids, float(sm_scale), _causal_code(causal), kernel, int(causal_offset), bool(nomat))
    l = lse.permute(0, 2, 1)
    return o, (q, k, v, q_segment_ids, kv_segment_ids, o, l)


def tpa(
    q, k, v,
    num_heads: int,
    q_segment_ids=None,
    kv_segment_ids=None,
    sm_scale: float = 1.0,
    causal: bool = False,
    block_sizes: BlockSizes | None = None,
    nomat: bool = False,
    debug: bool = False,
    interpret: bool = False,
    *,
    causal_offset: int = 0,
):
    """Tensor Product Attention (tpa/tpa.py:73-121).

    q[b,lq,rq,h+dk], k[b,lk,rk,h+dk], v[b,lk,rk,h+dv]: rank factors concatenated along the
    last dimension, head factor first.  Returns o[b,lq,h,dv] in q's dtype.  numpy inputs give a
    numpy result.  `causal_offset` (an addition, differentiable like the rest): with `causal`,
    query i sees keys up to i + causal_offset instead of i (see `tpa_factors`).
    """
    was_numpy = not isinstance(q, torch.Tensor)
    o, _ = _tpa_fwd(
        q, k, v, num_heads, q_segment_ids, kv_segment_ids, sm_scale, causal, block_sizes, nomat, debug, interpret,
        causal_offset=causal_offset,
    )
    return o.cpu().numpy() if was_numpy and o.dtype != torch.bfloat16 else o


def _fwd(
    q, k, v, q_segment_ids, kv_segment_ids, num_heads, sm_scale, causal, block_sizes, nomat, debug, interpret
):
    """Per-batch-element forward (tpa/tpa.py:446-543): q[lq,rq,h+dk] ... -> (o[lq,h,dv], l[lq,h])."""
    qs = None if q_segment_ids is None else torch.as_tensor(q_segment_ids)[None]
    ks = None if kv_segment_ids is None else torch.as_tensor(kv_segment_ids)[None]
    device = _pick_device(q, k, v)
    q, k, v = (_as_device_tensor(x, device)[None] for x in (q, k, v))
    o, res = _tpa_fwd(q, k, v, num_heads, qs, ks, sm_scale, causal, block_sizes, nomat, debug, interpret)
    return o[0], res[-1][0]


def _tpa_bwd(num_heads, sm_scale, causal, block_sizes, nomat, debug, interpret, residuals, do, *, causal_offset: int = 0):
    """tpa/tpa.py:168-214: (dq, dk, dv, None, None) from the residuals `_tpa_fwd` returned, in the
    dtype and the concatenated layout of q, k, v.  The residuals carry no causal offset (they have
    the reference's seven entries), so a forward made with `causal_offset != 0` must hand the same
    value to this call."""
    del block_sizes, nomat, debug, interpret
    q, k, v, q_segment_ids, kv_segment_ids, o, l = residuals
    device = _pick_device(q, k, v)
    q, k, v, o, l, do = (_as_device_tensor(x, device) for x in (q, k, v, o, l, do))
    dq, dk, dv = _bwd_concat(q, k, v, q_segment_ids, kv_segment_ids, o, l.permute(0, 2, 1), do, int(num_heads), float(sm_scale), _causal_code(causal),
                             int(causal_offset))
    return dq.to(q.dtype), dk.to(k.dtype), dv.to(v.dtype), None, None


def _bwd(
    q, k, v, q_segment_ids, kv_segment_ids, o, l, do, num_heads, sm_scale, causal, block_sizes, nomat, debug, interpret
):
    """Per-batch-element backward (tpa/tpa.py:823-962): q[lq,rq,h+dk] ... o[lq,h,dv] l[lq,h]
    do[lq,h,dv] -> (dq, dk, dv) shaped like q, k, v."""
    qs = None if q_segment_ids is None else torch.as_tensor(q_segment_ids)[None]
    ks = None if kv_segment_ids is None else torch.as_tensor(kv_segment_ids)[None]
    device = _pick_device(q, k, v)
    q, k, v, o, l, do = (_as_device_tensor(x, device)[None] for x in (q, k, v, o, l, do))
    dq, dk, dv, _, _ = _tpa_bwd(num_heads, sm_scale, causal, block_sizes, nomat, debug, interpret, (q, k, v, qs, ks, o, l), do)
    return dq[0], dk[0], dv[0]


def _precompute_delta(out, do, lse, block_q=None, debug=False, interpret=False):
    """tpa/tpa.py:965-995: delta[lq] = nansum(out * do, axis=1) for one head, out/do [lq, dv].
    (The backward kernels compute it themselves; kept because callers of the reference name it.)"""
    del block_q, debug, interpret
    out, do = torch.as_tensor(out), torch.as_tensor(do)
    return torch.nansum(out.float() * do.float(), dim=1).to(torch.as_tensor(lse).dtype)
