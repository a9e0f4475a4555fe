"""CPU-side checks of the C ABI: the library loads, exports every function include/tpa_abi.h
declares, and the ctypes structures have the layout the C compiler gives the header's."""

import ctypes
import os
import re
import subprocess

import pytest

from conftest import ROOT

HEADER = os.path.join(ROOT, "include", "tpa_abi.h")


def declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    body = text[text.index('extern "C" {'):]
    names = re.findall(r"^\s*(?:const\s+)?[A-Za-z_][\w\s\*]*?\b(\w+)\s*\([^;{]*\)\s*;", body, flags=re.M)
    return sorted(set(names))


def test_header_declares_the_expected_entry_points():
    names = declared_functions()
    for f in ("tpa_fwd", "tpa_decode", "mha_fwd", "tpa_decode_workspace_bytes", "tpa_strerror", "tpa_abi_version",
              "tpa_bwd", "mha_bwd", "tpa_bwd_workspace_bytes", "mha_bwd_workspace_bytes", "tpa_cache_append",
              "tpa_cache_append_workspace_bytes", "tpa_fwd_nomat_workspace_bytes", "tpa_decode_noalloc"):
        assert f in names, names


def test_library_exports_every_declared_symbol():
    from tpa import _dispatch

    lib = _dispatch.load_library()
    for name in declared_functions():
        assert hasattr(lib, name), f"{name} is declared in tpa_abi.h but not exported"
    assert lib.tpa_abi_version() == _dispatch.ABI_VERSION
    assert lib.tpa_strerror(0) == b"ok"
    assert b"workspace" in lib.tpa_strerror(-5)


def test_struct_layout_matches_the_c_compiler(tmp_path):
    from tpa import _dispatch as d

    fields = {"TpaFactor": d.TpaFactor, "TpaFwdArgs": d.TpaFwdArgs, "MhaFwdArgs": d.MhaFwdArgs,
              "TpaGrad": d.TpaGrad, "TpaBwdArgs": d.TpaBwdArgs, "MhaBwdArgs": d.MhaBwdArgs,
              "TpaAppendArgs": d.TpaAppendArgs}
    lines = ['#include <stdio.h>', '#include <stddef.h>', '#include "tpa_abi.h"', "int main(void) {"]
    for sname, cls in fields.items():
        lines.append(f'printf("{sname} %zu\\n", sizeof({sname}));')
        for fname, _ in cls._fields_:
            lines.append(f'printf("{sname}.{fname} %zu\\n", offsetof({sname}, {fname}));')
    lines.append("return 0; }")
    src = tmp_path / "layout.c"
    src.write_text("\n".join(lines))
    exe = tmp_path / "layout"
    subprocess.run(["gcc", "-I", os.path.join(ROOT, "include"), str(src), "-o", str(exe)], check=True)
    out = subprocess.run([str(exe)], check=True, capture_output=True, text=True).stdout
    got = dict(line.split() for line in out.strip().splitlines())
    for sname, cls in fields.items():
        assert int(got[sname]) == ctypes.sizeof(cls), sname
        for fname, _ in cls._fields_:
            assert int(got[f"{sname}.{fname}"]) == getattr(cls, fname).offset, f"{sname}.{fname}"


def test_size_queries_need_no_gpu():
    import torch

    from tpa import _dispatch

    lib = _dispatch.load_library()
    # config 4: 64 sequences, one query token, 32 heads -> 4 key ranges fill the 256 CUs
    assert lib.tpa_decode_default_splits(64, 1, 8192, 32) == 4
    assert lib.tpa_decode_workspace_bytes(64, 1, 8192, 32, 128, 0) == 64 * 4 * 32 * (128 + 2) * 4
    assert lib.tpa_decode_workspace_bytes(64, 1, 8192, 32, 128, 7) == 64 * 7 * 32 * (128 + 2) * 4
    assert lib.tpa_decode_default_splits(0, 1, 8192, 32) == 0
    # optional forward workspace: decode partials, or dense bf16 K and V when the rank is not 2
    assert lib.tpa_fwd_workspace_bytes(64, 1, 8192, 32, 128, 128, 6, 2) == lib.tpa_decode_workspace_bytes(64, 1, 8192, 32, 128, 0)
    assert lib.tpa_fwd_workspace_bytes(8, 2048, 2048, 64, 64, 64, 16, 8) == 3 * 8 * 2048 * 64 * 64 * 2  # dense Q, K, V
    assert lib.tpa_fwd_workspace_bytes(4, 4096, 4096, 16, 128, 128, 6, 2) == 3 * 4 * 4096 * 16 * 128 * 2
    assert lib.tpa_fwd_workspace_bytes(1, 32768, 32768, 32, 128, 128, 6, 2) == 3 * 32768 * 32 * 128 * 2
    assert lib.tpa_fwd_workspace_bytes(2, 1024, 4096, 16, 128, 128, 6, 2) == 0   # rank 2 below 2048 rows: the fused kernel
    assert lib.tpa_fwd_workspace_bytes(2, 257, 4096, 16, 128, 128, 6, 4) > 0    # other ranks: from the second query block on
    assert lib.tpa_fwd_workspace_bytes(2, 512, 512, 4, 48, 48, 6, 4) == 0        # not an MFMA head size
    # backward: dense Q, K, V and their gradients (fp32, each rounded up to 256 bytes) plus delta
    r = lambda n: (n + 255) // 256 * 256
    nq, nk, nv, nd = 2 * 10 * 3 * 5 * 4, 2 * 7 * 3 * 5 * 4, 2 * 7 * 3 * 6 * 4, 2 * 3 * 10 * 4
    assert lib.tpa_bwd_workspace_bytes(2, 10, 7, 3, 5, 6) == 2 * (r(nq) + r(nk) + r(nv)) + r(nd)
    assert lib.mha_bwd_workspace_bytes(2, 10, 7, 3, 5, 6, 0) == r(nd)
    assert lib.mha_bwd_workspace_bytes(2, 10, 7, 3, 5, 6, 1) == r(nd) + r(nq) + r(nk) + r(nv)
    assert lib.tpa_bwd_workspace_bytes(2, 0, 7, 3, 5, 6) == 0
    # producer step: partial sums of a decode step whose contraction is split over 2, 4 or 8 slabs of d_model
    bf16, f32 = _dispatch.dtype_code(torch.bfloat16), _dispatch.dtype_code(torch.float32)
    n_out = (6 + 2 * 2) * (32 + 128)
    assert lib.tpa_cache_append_workspace_bytes(64, 1, 4096, 32, 128, 6, 2, bf16) == 8 * 64 * n_out * 4
    assert lib.tpa_cache_append_workspace_bytes(8, 2, 1024, 32, 128, 6, 2, bf16) == 4 * 64 * n_out * 4
    assert lib.tpa_cache_append_workspace_bytes(8, 2, 1536, 32, 128, 6, 2, bf16) == 2 * 64 * n_out * 4
    assert lib.tpa_cache_append_workspace_bytes(8, 2, 256, 32, 128, 6, 2, bf16) == 0    # d_model too short to split
    assert lib.tpa_cache_append_workspace_bytes(65, 1, 4096, 32, 128, 6, 2, bf16) == 0  # more than 64 new tokens
    assert lib.tpa_cache_append_workspace_bytes(64, 1, 4096, 32, 128, 6, 2, f32) == 0
    # nomat: the split-key kernels' partials for one window of 64 query rows
    assert lib.tpa_fwd_nomat_workspace_bytes(2, 200, 4096, 8, 64, 64, 6, 2) == lib.tpa_decode_workspace_bytes(2, 64, 4096, 8, 64, 0)
    assert lib.tpa_fwd_nomat_workspace_bytes(2, 200, 4096, 2, 3, 5, 6, 2) == 0


def test_null_and_shape_errors_are_reported_before_any_launch():
    """Validation happens on the host: these calls return error codes without touching a GPU."""
    from tpa import _dispatch as d

    lib = d.load_library()
    assert lib.tpa_fwd(None, None) == -1
    args = d.TpaFwdArgs()
    args.dtype = 5
    assert lib.tpa_fwd(ctypes.byref(args), None) == -3
    args.dtype = d.TPA_DTYPE_BF16
    assert lib.tpa_fwd(ctypes.byref(args), None) == -2  # all dimensions are zero
    args.B = args.lq = args.lk = args.H = args.dk = args.dv = args.rq = args.rk = 1
    assert lib.tpa_fwd(ctypes.byref(args), None) == -1  # factor pointers are NULL
    args.dk = 1000
    assert lib.tpa_decode(ctypes.byref(args), None) == -2
    margs = d.MhaFwdArgs()
    assert lib.mha_fwd(ctypes.byref(margs), None) == -2
    assert lib.mha_fwd(None, None) == -1
    bargs = d.TpaBwdArgs()
    assert lib.tpa_bwd(None, None) == -1
    assert lib.tpa_bwd(ctypes.byref(bargs), None) == -2
    bargs.B = bargs.lq = bargs.lk = bargs.H = bargs.dk = bargs.dv = bargs.rq = bargs.rk = 1
    assert lib.tpa_bwd(ctypes.byref(bargs), None) == -1  # pointers are NULL
    mb = d.MhaBwdArgs()
    assert lib.mha_bwd(ctypes.byref(mb), None) == -2
    assert lib.mha_bwd(None, None) == -1
    assert lib.tpa_cache_append(None, None) == -1
    ap = d.TpaAppendArgs()
    ap.dtype = 7
    assert lib.tpa_cache_append(ctypes.byref(ap), None) == -3
    ap.dtype = d.TPA_DTYPE_BF16
    assert lib.tpa_cache_append(ctypes.byref(ap), None) == -2  # all dimensions are zero
    ap.B = ap.n = ap.d_model = ap.rq = ap.rk = ap.cache_len = ap.rope_len = 1
    ap.H, ap.D = 8, 12
    assert lib.tpa_cache_append(ctypes.byref(ap), None) == -2  # head size not a multiple of 8
    ap.D = 16
    assert lib.tpa_cache_append(ctypes.byref(ap), None) == -1  # pointers are NULL
    assert lib.tpa_decode_noalloc(None, None) == -1
    assert lib.tpa_decode_noalloc(ctypes.byref(d.TpaFwdArgs()), None) == -2


def test_unknown_causal_values_are_refused_by_every_entry_point():
    """`causal` outside the declared values is an error in the forward and in the backward calls
    (checked before the workspace and before any launch; the pointers below are never read)."""
    from tpa import _dispatch as d

    lib = d.load_library()
    fake = d.TpaFactor(256, 0, 0, 0)
    fwd = d.TpaFwdArgs(qa=fake, qb=fake, ka=fake, kb=fake, va=fake, vb=fake, o=256, B=1, lq=1, lk=1, H=1, dk=1, dv=1, rq=1, rk=1,
                       dtype=d.TPA_DTYPE_F32, causal=3)
    assert lib.tpa_fwd(ctypes.byref(fwd), None) == -6
    assert lib.tpa_decode(ctypes.byref(fwd), None) == -6
    assert lib.tpa_decode_noalloc(ctypes.byref(fwd), None) == -6
    g = d.TpaGrad(256, 0, 0, 0)
    for bad in (3, -1):
        bwd = d.TpaBwdArgs(qa=fake, qb=fake, ka=fake, kb=fake, va=fake, vb=fake, o=256, lse=256, d_o=256,
                           dqa=g, dqb=g, dka=g, dkb=g, dva=g, dvb=g, B=1, lq=1, lk=1, H=1, dk=1, dv=1, rq=1, rk=1,
                           dtype=d.TPA_DTYPE_F32, causal=bad)
        assert lib.tpa_bwd(ctypes.byref(bwd), None) == -6
    bwd.causal = 2  # a known value passes this check and stops at the missing workspace
    assert lib.tpa_bwd(ctypes.byref(bwd), None) == -5
    mf = d.MhaFwdArgs(q=256, k=256, v=256, o=256, B=1, lq=1, lk=1, H=1, dk=1, dv=1, dtype=d.TPA_DTYPE_F32, causal=2)
    assert lib.mha_fwd(ctypes.byref(mf), None) == -6
    mb = d.MhaBwdArgs(q=256, k=256, v=256, o=256, lse=256, d_o=256, dq=256, dk_out=256, dv_out=256,
                      B=1, lq=1, lk=1, H=1, dk=1, dv=1, dtype=d.TPA_DTYPE_F32, causal=2)
    assert lib.mha_bwd(ctypes.byref(mb), None) == -6


def test_missing_library_fails_loudly(tmp_path):
    from tpa import _dispatch

    with pytest.raises(RuntimeError, match="not built"):
        _dispatch.load_library(str(tmp_path / "nope.so"))
