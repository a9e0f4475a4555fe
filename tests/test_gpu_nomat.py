"""`nomat`: the evaluation orders that never form K or V (tpa/tpa.py:250,333-359,398-413).

The reference runs one test grid over nomat in {False, True} against the same dense reference
(tpa/tpa_test.py:60-125): the switch changes the order of operations, never the function.  Here
it selects the split-key kernels over windows of 64 query rows; `kernel=2` (matrix-core kernels
only, no fallback) makes a test fail with an error if anything else would have served the call.
Tolerances as in tests/test_gpu_parity.py: fp32 1e-4 / 1e-3, bf16 the per-row bounds of
tests/error_model.py in their `factored` form (these kernels round Q only).  `nomat="pairs"`
selects the reference's own arithmetic instead (a table per rank pair shared by the heads of a
workgroup, csrc/tpa_nomat.hip), which rounds nothing before the probabilities; same tests, same bounds.
"""

import numpy as np
import pytest
import torch

from conftest import make_factors, segment_ids
from oracle import tpa_oracle as orc
from test_gpu_parity import BF16_TOL, F32_TOL, LSE_TOL, _bottom_right_reference, _offset_reference, as_f64, bf16_bounds, check, split, to_gpu

pytestmark = pytest.mark.gpu

MFMA_ONLY = 2


# the lengths, batch sizes and ranks of the reference's grid (tpa/tpa_test.py:60-76) at head sizes the
# split-key kernels take; the segment-id half of that grid runs in test_gpu_parity.py (plain kernel)
@pytest.mark.parametrize("rank_q", [1, 6])
@pytest.mark.parametrize("rank_k", [1, 4])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize(
    "batch_size,lq,lk,h,d",
    [
        (1, 8, 8, 8, 64),
        (2, 1024, 128, 8, 64),
        (2, 128, 1024, 8, 128),
        (1, 1024, 1024, 16, 64),
    ],
)
def test_reference_grid_shapes_without_materialising(gpu, batch_size, rank_q, rank_k, dtype, lq, lk, h, d):
    from tpa import tpa

    q, k, v = make_factors(0, batch_size, lq, lk, h, d, d, rank_q, rank_k, dist="uniform")
    tq, tk, tv = (to_gpu(x, dtype, gpu) for x in (q, k, v))
    o_ref, l_ref = orc.tpa_reference(as_f64(tq), as_f64(tk), as_f64(tv), None, None, h)
    o, lse = tpa.tpa_factors(*split(tq, tk, tv, h), sm_scale=1.0, kernel=MFMA_ONLY, nomat=True)
    if dtype == torch.float32:
        check(o, lse, o_ref, l_ref, F32_TOL)
    else:
        check(o, lse, o_ref, l_ref, BF16_TOL, bf16_bounds(tq, tk, tv, h, 1.0, form="factored"))
    # the two evaluation orders agree (the property the reference's grid states by running both)
    o_m, lse_m = tpa.tpa_factors(*split(tq, tk, tv, h), sm_scale=1.0)
    if dtype == torch.float32:
        assert (o - o_m).abs().max().item() <= 2 * F32_TOL
        assert (lse - lse_m).abs().max().item() <= 2 * LSE_TOL
    else:
        lb, ob = bf16_bounds(tq, tk, tv, h, 1.0, form="factored")
        assert (o.float() - o_m.float()).abs().max().item() <= 2 * ob.max()
        assert (lse - lse_m).abs().max().item() <= 2 * lb.max()


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("lq,lk,causal_offset", [(130, 130, 0), (257, 400, 143), (100, 300, -20), (65, 64, 3)])
def test_causal_windows(gpu, dtype, lq, lk, causal_offset):
    """Window boundaries (row 64, 128, ...) under a causal mask with an offset, ragged lengths; rows that see no
    key (negative offset) end as NaN / -inf in every window."""
    from tpa import tpa

    b, h, d, rq, rk = 2, 8, 64, 3, 2
    q, k, v = make_factors(5, b, lq, lk, h, d, d, rq, rk, scale_by_rank=True)
    tq, tk, tv = (to_gpu(x, dtype, gpu) for x in (q, k, v))
    o_ref, l_ref = _offset_reference(as_f64(tq), as_f64(tk), as_f64(tv), h, d**-0.5, causal_offset)
    o, lse = tpa.tpa_factors(*split(tq, tk, tv, h), sm_scale=d**-0.5, causal=True, kernel=MFMA_ONLY, causal_offset=causal_offset, nomat=True)
    if dtype == torch.float32:
        check(o, lse, o_ref, l_ref, F32_TOL)
    else:
        check(o, lse, o_ref, l_ref, BF16_TOL, bf16_bounds(tq, tk, tv, h, d**-0.5, form="factored"))


def test_ragged_batch_bottom_right(gpu):
    """Sequences of different lengths, the last query aligned with each sequence's last key: the alignment counts
    from the whole call's query rows, not from a window's."""
    from tpa import tpa

    b, lq, lk, h, d, rq, rk = 3, 150, 500, 8, 128, 2, 2
    lengths = [500, 151, 320]
    q, k, v = make_factors(9, b, lq, lk, h, d, d, rq, rk, scale_by_rank=True)
    tq, tk, tv = (to_gpu(x, torch.bfloat16, gpu) for x in (q, k, v))
    kvl = torch.tensor(lengths, dtype=torch.int32, device=gpu)
    o, lse = tpa.tpa_factors(*split(tq, tk, tv, h), sm_scale=d**-0.5, causal=tpa.CAUSAL_BOTTOM_RIGHT, kernel=MFMA_ONLY, kv_lengths=kvl, nomat=True)
    o_ref, l_ref = _bottom_right_reference(as_f64(tq), as_f64(tk), as_f64(tv), lengths, h, d**-0.5, 0)
    check(o, lse, o_ref, l_ref, BF16_TOL, bf16_bounds(tq, tk, tv, h, d**-0.5, form="factored"))


def test_shapes_outside_the_split_key_kernels_run_the_plain_kernel(gpu):
    """Segment ids or other head sizes: nomat is honoured as `same results` by the plain kernel; asking for the
    matrix-core kernels only is refused."""
    from tpa import _dispatch as dd
    from tpa import tpa

    b, lq, lk, h, dk, dv = 2, 128, 1024, 2, 3, 5
    q, k, v = make_factors(0, b, lq, lk, h, dk, dv, 6, 4, dist="uniform")
    qseg, kvseg = segment_ids(lq, 42, b), segment_ids(lk, 42, b)
    tq, tk, tv = (to_gpu(x, torch.float32, gpu) for x in (q, k, v))
    o, lse = tpa.tpa_factors(*split(tq, tk, tv, h), qseg, kvseg, 1.0, nomat=True)
    o_ref, l_ref = orc.tpa_reference(q, k, v, qseg, kvseg, h)
    check(o, lse, o_ref, l_ref, F32_TOL)
    with pytest.raises(dd.TpaError):
        tpa.tpa_factors(*split(tq, tk, tv, h), qseg, kvseg, 1.0, kernel=MFMA_ONLY, nomat=True)
    assert dd.load_library().tpa_fwd_nomat_workspace_bytes(b, lq, lk, h, dk, dv, 6, 4) == 0


def test_workspace_is_required_and_sized_for_every_window(gpu):
    from tpa import _dispatch as dd

    lib = dd.load_library()
    one = lib.tpa_fwd_nomat_workspace_bytes(2, 64, 4096, 8, 64, 64, 6, 2)
    assert one == lib.tpa_decode_workspace_bytes(2, 64, 4096, 8, 64, 0)
    both = lib.tpa_fwd_nomat_workspace_bytes(2, 64 * 3 + 5, 4096, 8, 64, 64, 6, 2)
    assert both == max(one, lib.tpa_decode_workspace_bytes(2, 5, 4096, 8, 64, 0))
    # the C ABI refuses a call that brings none
    t = torch.zeros((2, 70, 2, 8 + 64), dtype=torch.bfloat16, device=gpu)
    o = torch.empty((2, 70, 8, 64), dtype=torch.bfloat16, device=gpu)
    f = [dd.factor(x) for x in (t[..., :8], t[..., 8:])]
    args = dd.TpaFwdArgs(qa=f[0], qb=f[1], ka=f[0], kb=f[1], va=f[0], vb=f[1], o=o.data_ptr(), lse=None, B=2, lq=70, lk=70, H=8,
                         dk=64, dv=64, rq=2, rk=2, dtype=dd.dtype_code(torch.bfloat16), sm_scale=1.0, causal=0, kernel=0,
                         workspace=None, workspace_bytes=0, num_splits=0, nomat=1)
    assert lib.tpa_fwd(args, None) == -5  # TPA_ERR_WORKSPACE


def test_config5_full_size_against_the_materialising_route(gpu):
    """B=8, T=2048, H=64, D=64, Rq=16, Rk=Rv=8, non-causal, at full size: sampled rows against the oracle and the
    whole output against the default route (which forms K and V)."""
    from tpa import tpa

    b, t, h, d, rq, rk = 8, 2048, 64, 64, 16, 8
    q, k, v = make_factors(0, b, t, t, h, d, d, rq, rk, scale_by_rank=True)
    tq, tk, tv = (to_gpu(x, torch.bfloat16, gpu) for x in (q, k, v))
    o, lse = tpa.tpa_factors(*split(tq, tk, tv, h), sm_scale=d**-0.5, kernel=MFMA_ONLY, nomat=True)
    rows = np.array([0, 63, 64, 1023, 2047])
    for bi in (0, 7):
        sl = slice(bi, bi + 1)
        o_ref, l_ref = orc.tpa_reference_rows(as_f64(tq[sl]), as_f64(tk[sl]), as_f64(tv[sl]), None, None, h, rows, sm_scale=d**-0.5, causal=False, dtype=np.float32)
        assert np.abs(as_f64(o[sl][:, rows]) - o_ref).max() <= BF16_TOL
        assert np.abs(as_f64(lse[sl][:, :, rows]).transpose(0, 2, 1) - l_ref).max() <= LSE_TOL
    o_m, lse_m = tpa.tpa_factors(*split(tq, tk, tv, h), sm_scale=d**-0.5)
    assert (o.float() - o_m.float()).abs().max().item() <= BF16_TOL
    assert (lse - lse_m).abs().max().item() <= LSE_TOL


# ---------------------------------------------------------------- nomat="pairs": the reference's rank-pair tables
@pytest.mark.parametrize("rank_q", [1, 6])
@pytest.mark.parametrize("rank_k", [1, 2, 4])
@pytest.mark.parametrize(
    "batch_size,lq,lk,h,d",
    [
        (1, 8, 8, 8, 64),
        (2, 1024, 128, 8, 64),
        (2, 128, 1024, 8, 128),
        (1, 1024, 1024, 16, 64),
        (1, 300, 333, 3, 128),   # ragged lengths, a head block that is not full
    ],
)
def test_reference_grid_shapes_with_rank_pair_tables(gpu, batch_size, rank_q, rank_k, lq, lk, h, d):
    """The lengths, batch sizes and ranks of the reference's grid (tpa/tpa_test.py:60-76) through the kernel that
    computes what the reference's nomat branch computes (tpa/tpa.py:333-359, 398-413)."""
    from tpa import tpa

    q, k, v = make_factors(0, batch_size, lq, lk, h, d, d, rank_q, rank_k, dist="uniform")
    tq, tk, tv = (to_gpu(x, torch.bfloat16, gpu) for x in (q, k, v))
    o_ref, l_ref = orc.tpa_reference(as_f64(tq), as_f64(tk), as_f64(tv), None, None, h)
    o, lse = tpa.tpa_factors(*split(tq, tk, tv, h), sm_scale=1.0, kernel=MFMA_ONLY, nomat="pairs")
    check(o, lse, o_ref, l_ref, BF16_TOL, bf16_bounds(tq, tk, tv, h, 1.0, form="factored"))
    # the three evaluation orders agree
    lb, ob = bf16_bounds(tq, tk, tv, h, 1.0, form="factored")
    for other in (False, True):
        o_m, lse_m = tpa.tpa_factors(*split(tq, tk, tv, h), sm_scale=1.0, nomat=other)
        assert (o.float() - o_m.float()).abs().max().item() <= 2 * ob.max()
        assert (lse - lse_m).abs().max().item() <= 2 * lb.max()


@pytest.mark.parametrize("lq,lk,causal_offset", [(130, 130, 0), (257, 400, 143), (100, 300, -20), (65, 64, 3), (600, 600, -259)])
def test_rank_pair_tables_under_a_causal_mask(gpu, lq, lk, causal_offset):
    """Diagonal blocks, an offset between query and key positions, rows that see no key (NaN / -inf)."""
    from tpa import tpa

    b, h, d, rq, rk = 2, 8, 64, 6, 2
    q, k, v = make_factors(5, b, lq, lk, h, d, d, rq, rk, scale_by_rank=True)
    tq, tk, tv = (to_gpu(x, torch.bfloat16, gpu) for x in (q, k, v))
    o_ref, l_ref = _offset_reference(as_f64(tq), as_f64(tk), as_f64(tv), h, d**-0.5, causal_offset)
    o, lse = tpa.tpa_factors(*split(tq, tk, tv, h), sm_scale=d**-0.5, causal=True, kernel=MFMA_ONLY, causal_offset=causal_offset, nomat="pairs")
    check(o, lse, o_ref, l_ref, BF16_TOL, bf16_bounds(tq, tk, tv, h, d**-0.5, form="factored"))


def test_rank_pair_tables_on_a_ragged_batch(gpu):
    from tpa import tpa

    b, lq, lk, h, d, rq, rk = 4, 150, 500, 8, 128, 6, 2
    lengths = [500, 151, 320, 0]
    q, k, v = make_factors(9, b, lq, lk, h, d, d, rq, rk, scale_by_rank=True)
    tq, tk, tv = (to_gpu(x, torch.bfloat16, gpu) for x in (q, k, v))
    kvl = torch.tensor(lengths, dtype=torch.int32, device=gpu)
    o, lse = tpa.tpa_factors(*split(tq, tk, tv, h), sm_scale=d**-0.5, causal=tpa.CAUSAL_BOTTOM_RIGHT, kernel=MFMA_ONLY, kv_lengths=kvl, nomat="pairs")
    o_ref, l_ref = _bottom_right_reference(as_f64(tq), as_f64(tk), as_f64(tv), lengths, h, d**-0.5, 0)
    check(o, lse, o_ref, l_ref, BF16_TOL, bf16_bounds(tq, tk, tv, h, d**-0.5, form="factored"))


def test_rank_pair_tables_where_no_instance_exists(gpu):
    """Other ranks, fp32 or segment ids: the plain kernel serves the call (same results); matrix cores only is refused."""
    from tpa import _dispatch as dd
    from tpa import tpa

    b, lq, lk, h, d = 1, 96, 200, 8, 64
    q, k, v = make_factors(3, b, lq, lk, h, d, d, 3, 2, scale_by_rank=True)
    tq, tk, tv = (to_gpu(x, torch.bfloat16, gpu) for x in (q, k, v))
    o_ref, l_ref = orc.tpa_reference(as_f64(tq), as_f64(tk), as_f64(tv), None, None, h, sm_scale=d**-0.5)
    o, lse = tpa.tpa_factors(*split(tq, tk, tv, h), sm_scale=d**-0.5, nomat="pairs")
    check(o, lse, o_ref, l_ref, BF16_TOL, bf16_bounds(tq, tk, tv, h, d**-0.5, form="factored"))
    with pytest.raises(dd.TpaError):
        tpa.tpa_factors(*split(tq, tk, tv, h), sm_scale=d**-0.5, kernel=MFMA_ONLY, nomat="pairs")


def test_rank_pair_tables_at_the_config5_shape(gpu):
    """B=8, T=2048, H=64, D=64 with the ranks 6 / 2 the kernel is instantiated for: sampled rows against the oracle,
    the whole output against the default route (which forms K and V)."""
    from tpa import tpa

    b, t, h, d, rq, rk = 8, 2048, 64, 64, 6, 2
    q, k, v = make_factors(0, b, t, t, h, d, d, rq, rk, scale_by_rank=True)
    tq, tk, tv = (to_gpu(x, torch.bfloat16, gpu) for x in (q, k, v))
    o, lse = tpa.tpa_factors(*split(tq, tk, tv, h), sm_scale=d**-0.5, kernel=MFMA_ONLY, nomat="pairs")
    rows = np.array([0, 31, 32, 255, 256, 1023, 2047])
    for bi in (0, 7):
        sl = slice(bi, bi + 1)
        o_ref, l_ref = orc.tpa_reference_rows(as_f64(tq[sl]), as_f64(tk[sl]), as_f64(tv[sl]), None, None, h, rows, sm_scale=d**-0.5, causal=False, dtype=np.float32)
        assert np.abs(as_f64(o[sl][:, rows]) - o_ref).max() <= BF16_TOL
        assert np.abs(as_f64(lse[sl][:, :, rows]).transpose(0, 2, 1) - l_ref).max() <= LSE_TOL
    o_m, lse_m = tpa.tpa_factors(*split(tq, tk, tv, h), sm_scale=d**-0.5)
    assert (o.float() - o_m.float()).abs().max().item() <= BF16_TOL
    assert (lse - lse_m).abs().max().item() <= LSE_TOL
