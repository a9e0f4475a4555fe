"""The generated tile loops of the prefill kernel (csrc/gen_prefill_loop.py) against the C++ side that hands
them their registers (csrc/tpa_prefill.hip), without a GPU: every register an instruction of a loop writes
is an in/out operand of its asm statement or a listed clobber, every register it reads is an operand or was
written earlier in the loop, input-only operands are never written, each copy of the iteration passes
exactly one workgroup barrier, and nothing beyond the 256 registers of a wave is named."""

import os
import re
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "tensor-product-attention-jax_amd", "csrc")
REG = re.compile(r"\b([vs])(?:(\d+)|\[(\d+):(\d+)\])")


def regs(text):
    out = set()
    for m in REG.finditer(text):
        lo, hi = (int(m.group(2)),) * 2 if m.group(2) is not None else (int(m.group(3)), int(m.group(4)))
        out.update(f"{m.group(1)}{i}" for i in range(lo, hi + 1))
    return out


def generate(tmp_path, d, loader):
    out = tmp_path / f"loop_{d}_{loader}.inc"
    subprocess.run([sys.executable, os.path.join(CSRC, "gen_prefill_loop.py"), str(d), loader, str(out)], check=True, capture_output=True)
    lines = [ln.strip()[1:].split("\\n")[0] for ln in out.read_text().splitlines() if ln.startswith('"')]
    clob = re.findall(r'"([^"]+)"', (tmp_path / f"loop_{d}_{loader}_clobbers.inc").read_text())
    return lines, set(clob)


def asm_operands(d, loader):
    """(in/out registers, input-only registers) of the asm statement in tpa_prefill.hip that includes the loop"""
    src = open(os.path.join(CSRC, "tpa_prefill.hip")).read()
    start = src.index(f'#include "gen/prefill_loop_{d}_{loader}.inc"')
    stmt = src[start : src.index(");", start)]
    outs, ins, _ = stmt.split("\n            :")[1:4] if stmt.count("\n            :") >= 3 else (None, None, None)
    assert outs is not None, "operand list of the asm statement not found"
    inout = set().union(*(regs(c) for c in re.findall(r'"\+\{([^}]+)\}"', outs)))
    assert not re.findall(r'"=\{', outs), "write-only operands are not expected"
    inputs = set().union(*(regs(c) for c in re.findall(r'"\{([^}]+)\}"', ins)))
    return inout, inputs


def dst_and_src(line):
    """(registers written, registers read) of one instruction line, None for labels and control flow"""
    if line.endswith(":") or line.startswith(("s_nop", "s_waitcnt", "s_barrier", "s_branch", "s_cbranch")):
        return None
    op, _, rest = line.partition(" ")
    opnds = [o.strip() for o in rest.split(",")]
    opnds = [o.split(" offset:")[0].replace(" offen", "") for o in opnds]
    if op.startswith(("ds_write", "s_cmp")):
        return set(), set().union(*(regs(o) for o in opnds))
    if op.startswith("v_cmp"):
        return {"vcc"}, set().union(*(regs(o) for o in opnds[1:]))
    if op.startswith("v_permlane32_swap"):
        both = regs(opnds[0]) | regs(opnds[1])
        return both, both
    return regs(opnds[0]), set().union(*(regs(o) for o in opnds[1:])) if len(opnds) > 1 else set()


@pytest.mark.parametrize("loader", ["dense", "r2"])
@pytest.mark.parametrize("d", [128, 64])
def test_generated_loop_matches_its_asm_statement(tmp_path, d, loader):
    lines, clob = generate(tmp_path, d, loader)
    inout, inputs = asm_operands(d, loader)
    assert {"vcc", "scc", "memory"} <= clob
    clob_regs = {c for c in clob if REG.fullmatch(c)}
    assert not (inout & inputs) and not (clob_regs & (inout | inputs)), "an operand is listed twice"
    defined = set(inout) | set(inputs)
    n_mfma = 0
    for ln in lines:
        ds = dst_and_src(ln)
        if ds is None:
            continue
        dst, src = ds
        n_mfma += ln.startswith("v_mfma")
        for r in dst | src:
            if r != "vcc":
                assert int(r[1:]) < (256 if r[0] == "v" else 102), f"{r} in `{ln}`"
        assert not (dst & inputs), f"`{ln}` writes an input-only operand"
        stray = {r for r in dst if r != "vcc"} - inout - clob_regs
        assert not stray, f"`{ln}` writes {sorted(stray)}: neither an in/out operand nor a clobber"
        undefined = {r for r in src if r != "vcc"} - defined
        assert not undefined, f"`{ln}` reads {sorted(undefined)} before anything wrote them"
        defined |= dst
    # two copies of the iteration (tile parity), one workgroup barrier each, and the matrix instructions of two tiles
    assert sum(ln == "s_barrier" for ln in lines) == 2
    assert n_mfma == 2 * (2 * (d // 16) + 4 * (d // 32))
    # every clobbered register is really used (a stale clobber would hide a register the compiler could have)
    used = set()
    for ln in lines:
        ds = dst_and_src(ln)
        if ds:
            used |= ds[0] | ds[1]
    assert clob_regs <= used, sorted(clob_regs - used)


def test_generator_takes_no_environment_input():
    """The product generator is a function of its arguments only (experiment switches live elsewhere)."""
    text = open(os.path.join(CSRC, "gen_prefill_loop.py")).read()
    assert "environ" not in text and "getenv" not in text
