#!/usr/bin/env python3
"""Writes the assembly of the interleaved tile loop of the prefill kernel with two row blocks per
wave (prefill_kernel<D, LOADER, false, 2> in tpa_prefill.hip) as a C string-literal include file.

Why assembly: the wave owns all 512 registers of its SIMD and the loop needs most of them in a
fixed split - O^T accumulators and Q fragments in the accumulation registers, logits, factor
loads and vector temporaries in the architectural ones - which the compiler's allocator does not
find (it spills the Q fragments and copies the accumulators back and forth).  Every register in
the loop is therefore named here, and the C++ side hands the state over in exactly these
registers (inline-assembly operands pinned to physical registers).

One iteration = one tile of 64 keys for the wave's 64 query rows (row blocks r = 0, 1):
    S^T block 0 (16 MFMAs) | rebuild of K tile j+1, refill of the K factor registers
    S^T block 1 (16)       | softmax of block 0 for both row blocks
    O^T keys 0-31 (16)     | softmax of block 1
    O^T keys 32-63 (16)    | rebuild of V tile j+1, refill of the V factor registers
    publish head factors of tile j+2, fetch those of tile j+3, barrier
Every fragment read from LDS feeds two MFMAs (one per row block).  It is the instruction stream of
hot_iteration() + tail() in tpa_prefill.hip, whose comments give the meaning of each step.

The script keeps track of outstanding LDS / memory operations and of the software-visible hazards
of gfx950 (results of matrix instructions, dot instructions, transcendental instructions, lane
swaps) and inserts the s_waitcnt / s_nop instructions they need.

usage: gen_prefill_loop.py <D: 128|64> <loader: r2|dense> <output.inc>
"""
import re
import sys

import os
KO = set(filter(None, os.environ.get("PF_KO", "").split(",")))  # experiment switches: leave parts of the loop out (timing only)
D = int(sys.argv[1])
DENSE = sys.argv[2] == "dense"
OUT = sys.argv[3]
assert D in (128, 64)

KTK = 64
KS, VS = D + 8, D + 32                  # LDS row strides (elements)
NKS, NDB = D // 16, D // 32
CPR = D // 8
TPP = 256 // CPR                         # tokens per loader pass (256 threads)
NPASS = KTK // TPP
NLOAD = 1 if DENSE else 2                # factor loads per pass and matrix (ranks)
K_OFF, V_OFF = 0, KTK * KS * 2           # byte offsets inside one LDS set
A_OFF = V_OFF + KTK * VS * 2             # head-factor slot [K|V][token][rank] bf16
SET_STRIDE = 0x10000                     # second LDS set = first + 64 KiB (toggled with one xor)

# ---- register map (must match the operand list of the asm statement in tpa_prefill.hip)
def S(r, mb): return 16 * (2 * mb + r)           # logits of (row block, key block): v[S : S+15]
NMREF = [64, 80]                                  # v: -reference tuples
KREG, VREG = 96, 128                              # v: factor registers [pass][rank][4]
RING = 160                                        # v: fragment buffers of 4: v[160:171] and v[232:255]
RING_BUFS = [160, 164, 168] + [232 + 4 * k for k in range(6)]
LA = int(os.environ.get("PF_LA", "2"))            # fragments read ahead of the MFMAs that consume them
assert 1 <= LA < len(RING_BUFS)
CH = 172                                          # v: 8 rebuild temporaries
AAK, AAV = 180, 184                               # v: packed halved head factors per pass
MREF = [188, 189]; LSUM = [190, 191]; APEND = 192  # v[188:195] state tuple
KFRAG, VFRAG, KW, VW, AA, ASTORE, KVOFF, VVOFF, AVOFF = range(196, 205)  # v[196:211] address tuple
TMP = 212                                         # v[212:231] temporaries
O = lambda r, db: 16 * (r * NDB + db)            # a: O^T accumulators
Q = lambda r, ks: 16 * 2 * NDB + 4 * (r * NKS + ks)  # a: Q fragments
# s[32:47] scalar tuple
S_J, S_HOT_END, S_LAST, S_KTILE, S_VTILE, S_ATILE, S_KPASS, S_KRANK, S_VPASS, S_VRANK, S_SEL_LO, S_SEL_HI = range(32, 44)
S_KB, S_VB, S_AR = 48, 52, 56                     # buffer resources s[48:51], s[52:55], s[56:59]
S_T0, S_T1, S_T2, S_T3, S_SLACK = 60, 61, 62, 63, 64

def vt(n, c=4): return f"v[{n}:{n + c - 1}]"
def at(n, c=4): return f"a[{n}:{n + c - 1}]"
def st(n, c=4): return f"s[{n}:{n + c - 1}]"

REG_RE = re.compile(r"\b([vas])(?:(\d+)|\[(\d+):(\d+)\])")

def regs_of(opnd):
    out = set()
    for m in REG_RE.finditer(opnd):
        f = m.group(1)
        if m.group(2) is not None:
            out.add(f + m.group(2))
        else:
            out.update(f"{f}{i}" for i in range(int(m.group(3)), int(m.group(4)) + 1))
    if "vcc" in opnd:
        out.add("vcc")
    return out


class Stream:
    """Instruction list with automatic s_waitcnt / s_nop insertion."""

    def __init__(self):
        self.lines = []
        self.ws = 0                      # wait states issued so far
        self.writer = {}                 # reg -> (wait state index of its last writer, kind)
        self.mfma_c_read = {}            # reg -> wait state index of the last MFMA that read it as C
        self.lds = []                    # outstanding LDS operations (ids, oldest first)
        self.vm = []                     # outstanding memory loads
        self.pending = {}                # reg -> ('lds' | 'vm', id)
        self.next_id = 0

    def raw(self, text):
        self.lines.append(text)

    def nop(self, n):
        while n > 0:
            k = min(n, 8)
            self.lines.append(f"s_nop {k - 1}")
            self.ws += k
            n -= k

    def _wait_for(self, regs):
        need_l = need_v = None
        for r in regs:
            if r in self.pending:
                q, i = self.pending[r]
                lst = self.lds if q == "lds" else self.vm
                if i in lst:
                    after = len(lst) - 1 - lst.index(i)
                    if q == "lds":
                        need_l = after if need_l is None else min(need_l, after)
                    else:
                        need_v = after if need_v is None else min(need_v, after)
        parts = []
        if need_v is not None:
            parts.append(f"vmcnt({need_v})")
            self.vm = self.vm[len(self.vm) - need_v:] if need_v else []
        if need_l is not None:
            need_l = min(need_l, 15)     # the counter has four bits: waiting for fewer is always allowed
            parts.append(f"lgkmcnt({need_l})")
            self.lds = self.lds[len(self.lds) - need_l:] if need_l else []
        if parts:
            self.lines.append("s_waitcnt " + " ".join(parts))
            self.ws += 1
        for r in list(self.pending):
            q, i = self.pending[r]
            if i not in (self.lds if q == "lds" else self.vm):
                del self.pending[r]

    def ins(self, op, *opnds, ndst=1):
        """Emit `op opnds...`; the first ndst operands are destinations."""
        text = op + " " + ", ".join(opnds) if opnds else op
        base = op.split("_e32")[0].split("_e64")[0]
        if base.startswith("v_mfma"):
            kind = "mfma"
        elif base.startswith("v_dot2"):
            kind = "dot"
        elif base in ("v_exp_f32", "v_log_f32", "v_rcp_f32"):
            kind = "trans"
        elif base.startswith("v_permlane32_swap"):
            kind = "swap"
        elif base.startswith("v_"):
            kind = "valu"
        elif base.startswith("ds_read"):
            kind = "ds_read"
        elif base.startswith("ds_write"):
            kind = "ds_write"
        elif base.startswith("buffer_load"):
            kind = "vmem"
        elif base.startswith("s_"):
            kind = "salu"
        else:
            raise ValueError(op)
        dst, src = set(), set()
        for k, o in enumerate(opnds):
            o = o.split(" offset:")[0].replace(" offen", "")
            (dst if k < ndst and kind != "ds_write" else src).update(regs_of(o))
        if kind == "swap":           # both operands are read and written
            src |= dst
        if kind == "mfma":           # v_mfma d, a, b, c
            c_regs = regs_of(opnds[3])
            ab_regs = regs_of(opnds[1]) | regs_of(opnds[2])
            src = c_regs | ab_regs
        # ---- memory results
        self._wait_for(src | dst)
        # ---- hazards: wait states needed between a producer and this instruction
        need = 0
        for r in src | dst:
            if r not in self.writer:
                continue
            w_ws, w_kind = self.writer[r]
            gap = self.ws - w_ws - 1         # wait states already between them
            req = 0
            if w_kind == "dot":
                req = 3
            elif w_kind == "trans" and kind not in ("trans",):
                req = 1
            elif w_kind == "mfma":
                if kind == "mfma" and r in (c_regs if kind == "mfma" else ()) and r in dst:
                    req = 0                  # accumulation into the same tuple: back to back
                else:
                    req = 12
            elif w_kind in ("valu", "swap") and kind == "mfma":
                req = 2
            elif w_kind in ("valu", "swap", "trans") and kind == "swap":
                req = 2
            need = max(need, req - gap)
        if kind in ("valu", "trans", "dot", "swap", "ds_read", "vmem"):
            for r in dst:                    # a matrix instruction may still be reading it as C
                if r in self.mfma_c_read:
                    need = max(need, 14 - (self.ws - self.mfma_c_read[r] - 1))
        if need > 0:
            self.nop(need)
        self.lines.append(text)
        me = self.ws
        self.ws += 1
        for r in dst:
            self.writer[r] = (me, kind)
            self.mfma_c_read.pop(r, None)
        if kind == "mfma":
            for r in c_regs - dst:
                self.mfma_c_read[r] = me
        if kind in ("ds_read", "ds_write"):
            i = self.next_id; self.next_id += 1
            self.lds.append(i)
            for r in dst:
                self.pending[r] = ("lds", i)
        if kind == "vmem":
            i = self.next_id; self.next_id += 1
            self.vm.append(i)
            for r in dst:
                self.pending[r] = ("vm", i)

    def prime_vm(self, reg_groups):
        """Loads issued by the previous iteration (or, on entry, by nobody: the waits then fall through)."""
        for regs in reg_groups:
            i = self.next_id; self.next_id += 1
            self.vm.append(i)
            for r in regs:
                self.pending[r] = ("vm", i)

    def barrier(self):
        self.lines.append("s_waitcnt lgkmcnt(0)")
        if "barrier" not in KO:
            self.lines.append("s_barrier")
        self.lds = []
        self.pending = {r: p for r, p in self.pending.items() if p[0] != "lds"}
        self.ws += 2


def load_groups():
    """Registers of the factor loads in flight at the top of an iteration, oldest first."""
    g = []
    for base in (KREG, VREG):
        for ps in range(NPASS):
            for rr in range(NLOAD):
                n = base + (ps * 2 + rr) * 4
                g.append([f"v{n + k}" for k in range(4)])
    if not DENSE:
        g.append([f"v{APEND}"])
    return g


def frag_buf(f): return RING_BUFS[f % (LA + 1)]

def emit_frag_load(e, f):
    if "frag" in KO:
        return
    b = frag_buf(f)
    if f < 2 * NKS:
        mb, kk = divmod(f, NKS)
        e.ins("ds_read_b128", vt(b), f"v{KFRAG} offset:{mb * 32 * KS * 2 + kk * 32}")
    else:
        kk, db = divmod(f - 2 * NKS, NDB)
        off = kk * 16 * VS * 2 + db * 64
        e.ins("ds_read_b64_tr_b16", vt(b, 2), f"v{VFRAG} offset:{off}")
        e.ins("ds_read_b64_tr_b16", vt(b + 2, 2), f"v{VFRAG} offset:{off + 8 * VS * 2}")

def emit_mfma(e, f, r):
    if "mfma" in KO:
        return
    b = frag_buf(f)
    if f < 2 * NKS:
        mb, kk = divmod(f, NKS)
        s = S(r, mb)
        e.ins("v_mfma_f32_32x32x16_bf16", vt(s, 16), vt(b), at(Q(r, kk)), vt(NMREF[r], 16) if kk == 0 else vt(s, 16))
    else:
        kk, db = divmod(f - 2 * NKS, NDB)
        p = S(r, kk // 2) + 4 * (kk % 2)     # P fragment kk lives in the registers of the logits it was made from
        e.ins("v_mfma_f32_32x32x16_bf16", at(O(r, db), 16), vt(b), vt(p), at(O(r, db), 16))

# ---- rebuild of one loader pass of one matrix: three pieces
def piece(e, is_v, ps, part):
    base, aa, waddr, rstride = (VREG, AAV, VW, VS) if is_v else (KREG, AAK, KW, KS)
    b0, b1 = base + (ps * 2) * 4, base + (ps * 2 + 1) * 4
    woff = ps * TPP * rstride * 2
    wt = TMP + 8 + 4 * (ps % 2)              # packed result, two tuples in turn
    if "rebuild" in KO and not DENSE:
        if part == 2:
            e.ins("ds_write_b128", f"v{waddr}", vt(b0) + f" offset:{woff}")
        return
    if DENSE:
        if part == 2:
            e.ins("ds_write_b128", f"v{waddr}", vt(b0) + f" offset:{woff}")
        return
    if part == 0:
        for k in range(4):
            e.ins("v_perm_b32", f"v{CH + 2 * k}", f"v{b1 + k}", f"v{b0 + k}", f"s{S_SEL_LO}")
            e.ins("v_perm_b32", f"v{CH + 2 * k + 1}", f"v{b1 + k}", f"v{b0 + k}", f"s{S_SEL_HI}")
    elif part == 1:
        for k in range(8):
            if "dot" in KO:
                e.ins("v_mul_f32", f"v{CH + k}", f"v{CH + k}", f"v{aa + ps}")
            else:
                e.ins("v_dot2_f32_bf16", f"v{CH + k}", f"v{CH + k}", f"v{aa + ps}", "0")
    else:
        for k in range(4):
            e.ins("v_cvt_pk_bf16_f32", f"v{wt + k}", f"v{CH + 2 * k}", f"v{CH + 2 * k + 1}")
        e.ins("ds_write_b128", f"v{waddr}", vt(wt) + f" offset:{woff}")

def issue_loads(e, is_v):
    base, rs, voff, tile, pss, rks = (VREG, S_VB, VVOFF, S_VTILE, S_VPASS, S_VRANK) if is_v else (KREG, S_KB, KVOFF, S_KTILE, S_KPASS, S_KRANK)
    # tile = min(j + 2, last); byte offset of its first token
    e.ins("s_add_u32", f"s{S_T0}", f"s{S_J}", "2")
    e.ins("s_min_u32", f"s{S_T0}", f"s{S_T0}", f"s{S_LAST}")
    e.ins("s_mul_i32", f"s{S_T1}", f"s{S_T0}", f"s{tile}")
    for ps in range(NPASS):
        if "vmem" in KO:
            continue
        e.ins("buffer_load_dwordx4", vt(base + ps * 8), f"v{voff}", st(rs), f"s{S_T1} offen")
        if not DENSE:
            e.ins("s_add_u32", f"s{S_T2}", f"s{S_T1}", f"s{rks}")
            e.ins("buffer_load_dwordx4", vt(base + ps * 8 + 4), f"v{voff}", st(rs), f"s{S_T2} offen")
        if ps + 1 < NPASS:
            e.ins("s_add_u32", f"s{S_T1}", f"s{S_T1}", f"s{pss}")

# ---- softmax pieces of block (r, mb)
def sm_max(e, r, mb, label):
    if "softmax" in KO or "max" in KO:
        return
    s = S(r, mb)
    ta, tb = TMP + 2 * r, TMP + 2 * r + 1
    e.ins("v_max3_f32", f"v{ta}", f"v{s}", f"v{s + 1}", f"v{s + 2}")
    e.ins("v_max3_f32", f"v{tb}", f"v{s + 3}", f"v{s + 4}", f"v{s + 5}")
    for k in range(6, 16, 4):
        e.ins("v_max3_f32", f"v{ta}", f"v{ta}", f"v{s + k}", f"v{s + k + 1}")
        if k + 3 < 16:
            e.ins("v_max3_f32", f"v{tb}", f"v{tb}", f"v{s + k + 2}", f"v{s + k + 3}")
    # (6,7 | 8,9) (10,11 | 12,13) (14,15)
    e.ins("v_max_f32", f"v{ta}", f"v{ta}", f"v{tb}")
    e.ins("v_mov_b32", f"v{tb}", f"v{ta}")
    e.ins("v_permlane32_swap_b32", f"v{ta}", f"v{tb}", ndst=2)
    e.ins("v_max_f32", f"v{ta}", f"v{ta}", f"v{tb}")
    e.ins("v_cmp_lt_f32", "vcc", f"s{S_SLACK}", f"v{ta}")
    e.raw(f"s_cbranch_vccnz .Lpf_rare_{r}{mb}_%=")
    e.raw(f".Lpf_cont_{r}{mb}_%=:")

def sm_exp(e, r, mb, q):
    if "softmax" in KO:
        return
    s = S(r, mb)
    t0, t1 = TMP + 4 + 2 * r, TMP + 5 + 2 * r
    for k in range(4):
        e.ins("v_mov_b32" if "exp" in KO else "v_exp_f32", f"v{s + 4 * q + k}", f"v{s + 4 * q + k}")
    e.ins("v_add_f32", f"v{t0}", f"v{s + 4 * q}", f"v{s + 4 * q + 1}")
    e.ins("v_add_f32", f"v{t1}", f"v{s + 4 * q + 2}", f"v{s + 4 * q + 3}")
    e.ins("v_cvt_pk_bf16_f32", f"v{s + 2 * q}", f"v{s + 4 * q}", f"v{s + 4 * q + 1}")
    e.ins("v_add_f32", f"v{t0}", f"v{t0}", f"v{t1}")
    e.ins("v_cvt_pk_bf16_f32", f"v{s + 2 * q + 1}", f"v{s + 4 * q + 2}", f"v{s + 4 * q + 3}")
    e.ins("v_add_f32", f"v{LSUM[r]}", f"v{LSUM[r]}", f"v{t0}")

def rare_path(r, mb):
    """Row maximum left the slack (rare): move the reference of row block r up by a whole number
    and rescale what was accumulated against the old one (move_reference() in tpa_prefill.hip)."""
    e = Stream()
    t = TMP + 2 * r                  # the row maximum
    d, al, x0, x1 = TMP + 16, TMP + 17, TMP + 18, TMP + 19
    e.raw(f".Lpf_rare_{r}{mb}_%=:")
    e.nop(16)                        # matrix instructions in flight: their results and their C reads
    e.ins("v_ceil_f32", f"v{d}", f"v{t}")
    e.ins("v_max_f32", f"v{d}", "0", f"v{d}")                 # delta = tmax > 0 ? ceil(tmax) : 0
    e.ins("v_exp_f32_e64", f"v{al}", f"-v{d}")                # alpha = 2^-delta
    e.ins("v_add_f32", f"v{MREF[r]}", f"v{MREF[r]}", f"v{d}")
    for k in range(16):
        e.ins("v_sub_f32", f"v{NMREF[r] + k}", "0", f"v{MREF[r]}")
    e.ins("v_mul_f32", f"v{LSUM[r]}", f"v{LSUM[r]}", f"v{al}")
    for db in range(NDB):
        for k in range(16):
            a, x = O(r, db) + k, (x0, x1)[k % 2]
            e.ins("v_accvgpr_read_b32", f"v{x}", f"a{a}")
            e.ins("v_mul_f32", f"v{x}", f"v{x}", f"v{al}")
            e.ins("v_accvgpr_write_b32", f"a{a}", f"v{x}")
    s0, s1 = S(r, 0), S(r, 1)
    if mb == 0:                      # nothing of this tile is packed yet: both blocks move
        for k in range(16):
            e.ins("v_sub_f32", f"v{s0 + k}", f"v{s0 + k}", f"v{d}")
    else:                            # block 0 has become packed P (s0[0..7]): scale it
        for k in range(8):
            e.ins("v_lshlrev_b32", f"v{x0}", "16", f"v{s0 + k}")
            e.ins("v_and_b32", f"v{x1}", "0xffff0000", f"v{s0 + k}")
            e.ins("v_mul_f32", f"v{x0}", f"v{x0}", f"v{al}")
            e.ins("v_mul_f32", f"v{x1}", f"v{x1}", f"v{al}")
            e.ins("v_cvt_pk_bf16_f32", f"v{s0 + k}", f"v{x0}", f"v{x1}")
    for k in range(16):
        e.ins("v_sub_f32", f"v{s1 + k}", f"v{s1 + k}", f"v{d}")
    e.nop(4)
    e.raw(f"s_branch .Lpf_cont_{r}{mb}_%=")
    return e.lines


def softmax_items(mb):
    items = [("max", 0), ("max", 1)]
    for q in range(4):
        items += [("exp", 0, q), ("exp", 1, q)]
    return items

def place(items, slots):
    """item k of len(items) goes behind MFMA slot k * slots / len(items)"""
    out = [[] for _ in range(slots)]
    for k, it in enumerate(items):
        out[k * slots // len(items)].append(it)
    return out


def iteration():
    e = Stream()
    e.prime_vm(load_groups())
    NF = 2 * NKS + 4 * NDB
    G1, G2, G3, G4 = 2 * NKS, 2 * NKS, 4 * NDB, 4 * NDB          # slots (MFMAs) per group
    # first fragments, then the head factors of the tile that is rebuilt in this iteration
    for f in range(LA):
        emit_frag_load(e, f)
    if not DENSE:
        for ps in range(NPASS):
            e.ins("ds_read_b32", f"v{AAK + ps}", f"v{AA} offset:{ps * TPP * 4}")
        for ps in range(NPASS):
            e.ins("ds_read_b32", f"v{AAV + ps}", f"v{AA} offset:{2 * KTK * 2 + ps * TPP * 4}")
    NP = 3 * NPASS
    g1 = place([("piece", False, k // 3, k % 3) for k in range(NP)] + [("issue", False)], G1)
    g2 = place(softmax_items(0), G2)
    g3 = place(softmax_items(1), G3)
    g4 = place([("piece", True, k // 3, k % 3) for k in range(NP)] + [("issue", True)], G4)
    slices = g1 + g2 + g3 + g4
    for f in range(NF):
        if f + LA < NF:
            emit_frag_load(e, f + LA)
        for r in range(2):
            emit_mfma(e, f, r)
            for it in slices[2 * f + r]:
                if it[0] == "piece":
                    piece(e, it[1], it[2], it[3])
                elif it[0] == "issue":
                    issue_loads(e, it[1])
                elif it[0] == "max":
                    mb = 0 if 2 * f + r < G1 + G2 else 1
                    sm_max(e, it[1], mb, None)
                else:
                    mb = 0 if 2 * f + r < G1 + G2 else 1
                    sm_exp(e, it[1], mb, it[2])
    # ---- tail: head factors of tile j+2 into the other slot (halved: the 1/R of rank 2), fetch
    # those of tile j+3, flip the LDS sets, barrier
    if not DENSE:
        e.ins("v_lshlrev_b32", f"v{TMP}", "16", f"v{APEND}")
        e.ins("v_mul_f32", f"v{TMP}", "0.5", f"v{TMP}")
        e.ins("ds_write_b16_d16_hi", f"v{ASTORE}", f"v{TMP}")
        e.ins("s_add_u32", f"s{S_T0}", f"s{S_J}", "3")
        e.ins("s_min_u32", f"s{S_T0}", f"s{S_T0}", f"s{S_LAST}")
        e.ins("s_mul_i32", f"s{S_T1}", f"s{S_T0}", f"s{S_ATILE}")
        e.ins("buffer_load_ushort", f"v{APEND}", f"v{AVOFF}", st(S_AR), f"s{S_T1} offen")
    for a in (KFRAG, VFRAG, AA, KW, VW, ASTORE):
        e.ins("v_xor_b32", f"v{a}", f"0x{SET_STRIDE:x}", f"v{a}")
    e.barrier()
    # the loads in flight now are those the next iteration expects
    assert "vmem" in KO or len(e.vm) == len(load_groups()), (len(e.vm), len(load_groups()))
    return e.lines


def main():
    lines = []
    # ---- entry: the address registers arrive for LDS set 0; point them at the sets of tile j
    lines += [
        f"s_mov_b32 s{S_SLACK}, 0x41000000",             # 8.0: the slack of the reference
        f"s_and_b32 s{S_T0}, s{S_J}, 1",
        f"s_lshl_b32 s{S_T0}, s{S_T0}, 16",              # (j & 1) << 16: set of tile j
        f"s_xor_b32 s{S_T1}, s{S_T0}, 0x{SET_STRIDE:x}",  # set of tile j + 1
    ]
    for a in (KFRAG, VFRAG, AA):
        lines.append(f"v_xor_b32 v{a}, s{S_T0}, v{a}")
    for a in (KW, VW, ASTORE):
        lines.append(f"v_xor_b32 v{a}, s{S_T1}, v{a}")
    lines.append(".Lpf_loop_%=:")
    lines += iteration()
    lines += [
        f"s_add_u32 s{S_J}, s{S_J}, 1",
        f"s_cmp_lt_u32 s{S_J}, s{S_HOT_END}",
        "s_cbranch_scc1 .Lpf_loop_%=",
        "s_branch .Lpf_done_%=",
    ]
    for r in range(2):
        for mb in range(2):
            if not ({"softmax", "max"} & KO):
                lines += rare_path(r, mb)
    lines += [
        ".Lpf_done_%=:",
        "s_waitcnt vmcnt(0)",                             # the factor registers go back to the compiler
        "s_nop 7", "s_nop 7",                             # ... and so do the accumulators
    ]
    with open(OUT, "w") as f:
        f.write(f"// generated by gen_prefill_loop.py {D} {'dense' if DENSE else 'r2'}: do not edit\n")
        for ln in lines:
            f.write(f'"{ln}\\n\\t"\n')
    # registers the loop uses beyond its operands
    ring = [b + k for b in RING_BUFS[:LA + 1] for k in range(4)]
    clob = [f"v{n}" for n in sorted(set(list(range(0, 64)) + list(range(RING, MREF[0])) + list(range(TMP, TMP + 20)) + ring))]
    clob += [f"s{n}" for n in range(S_T0, S_SLACK + 1)] + ["vcc", "scc", "memory"]
    with open(OUT.replace(".inc", "_clobbers.inc"), "w") as f:
        f.write("// generated by gen_prefill_loop.py: do not edit\n")
        f.write(", ".join(f'"{c}"' for c in clob) + "\n")
    n_mfma = sum("v_mfma" in ln for ln in lines)
    print(f"{OUT}: {len(lines)} lines, {n_mfma} MFMAs", file=sys.stderr)


main()
