#!/usr/bin/env python3
"""Writes the assembly of the pipelined tile loop of the prefill kernel (dense K/V loader,
prefill_kernel<D, LOAD_DENSE, false> in tpa_prefill.hip) as a C string-literal include file.

One iteration j belongs to one wave (32 query rows) and overlaps two tiles of 64 keys:

    S^T of tile j+1  (2 D/16 MFMAs, into the logit registers the previous iteration freed)
    softmax of tile j (row maximum, exponentials, packing to bf16), spread behind those MFMAs
    O^T += V^T P^T of tile j  (4 D/32 MFMAs)
    loader: K tile j+2 and V tile j+1 from registers to LDS, K tile j+3 and V tile j+2 requested
    one barrier

so no matrix instruction of an iteration waits for vector work of the same iteration: the logits
a softmax reads were finished an iteration earlier.  There are two sets of logit registers (tile
parity), hence two copies of the iteration in the loop body; K tiles rotate through three LDS
buffers whose byte offsets travel in scalar registers, V tiles through two that the copies
address with immediates.  It is the instruction stream of cold_compute() + advance_tiles() +
tail() in tpa_prefill.hip, whose comments give the meaning of each step.

Why assembly: the two sets of logits, the accumulators, the Q fragments and the loads in flight
fill the 256 registers a wave has with two waves per SIMD, in a fixed assignment that the
compiler's allocator does not find.  Every register in the loop is named here, and the C++ side
hands the state over in exactly these registers (inline-assembly operands pinned to physical
registers).

The script keeps track of outstanding LDS / memory operations and of the software-visible hazards
of gfx950 (results of matrix instructions, transcendental instructions, lane swaps, vector
writes read by matrix instructions) and inserts the s_waitcnt / s_nop instructions they need.

usage: gen_prefill_loop.py <D: 128|64> dense <output.inc>
"""
import os
import re
import sys

KO = set(filter(None, os.environ.get("PF_KO", "").split(",")))  # experiment switches: leave parts of the loop out (timing only)
D = int(sys.argv[1])
assert sys.argv[2] == "dense" and D in (128, 64)
OUT = sys.argv[3]

KTK = 64
KS, VS = D + 8, D + 32                  # LDS row strides (elements)
NKS, NDB = D // 16, D // 32
CPR = D // 8
TPP = 512 // CPR                        # tokens per loader pass (512 threads)
NPASS = KTK // TPP
KBUF, VBUF = KTK * KS * 2, KTK * VS * 2  # bytes of one K / V buffer
NF = 2 * NKS + 4 * NDB                  # matrix instructions per iteration
LA = int(os.environ.get("PF_LA", "2"))  # fragments read ahead of the MFMAs that consume them

# ---- register map (must match the operand list of the asm statement in tpa_prefill.hip)
def S(p, mb): return 32 * p + 16 * mb             # v: logits of (tile parity, 32-key block)
NMREF = 64                                        # v[64:79]: -reference in all 16 registers
def O(db): return 80 + 16 * db                    # v[80:143]: O^T accumulators
def Q(ks): return 144 + 4 * ks                    # v[144:175]: Q fragments
def KREG(ps): return 176 + 4 * ps                 # v[176:183]: K rows on their way (one tuple per loader pass)
def VREG(ps): return 184 + 4 * ps                 # v[184:191]: V rows
RING_BUFS = [192, 196, 200, 212]                  # v[192:203], v[212:215]: fragment buffers
BATCH = int(os.environ.get("PF_BATCH", "1"))      # fragments fetched, and waited for, together
assert 1 <= LA < len(RING_BUFS) and BATCH in (1, 2)
MREF, LSUM, KFRAG0, VFRAG, KW0, VW, KVOFF, VVOFF = range(204, 212)   # v[204:219]: state / address tuple
TA, TB, T0A, T1A, KFRAG, KW, RD, RAL, T0B, T1B = range(220, 230)        # v[220:229]: temporaries
# s[32:47] scalar tuple
S_J, S_END, S_LAST, S_KTILE, S_VTILE, S_KPASS, S_VPASS, S_KR, S_KWB = range(32, 41)
S_KB, S_VB = 48, 52                               # buffer resources s[48:51], s[52:55]
S_T0, S_T1, S_SLACK = 60, 61, 64

def vt(n, c=4): return f"v[{n}:{n + c - 1}]"
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
        c_regs = set()
        if kind == "mfma":           # v_mfma d, a, b, c
            c_regs = regs_of(opnds[3])
            src = c_regs | regs_of(opnds[1]) | regs_of(opnds[2])
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
            if w_kind == "trans" and kind != "trans":
                req = 1
            elif w_kind == "mfma":
                if kind == "mfma" and r in c_regs and r in dst:
                    req = 0                  # accumulation into the same tuple: back to back
                else:
                    req = 12
            elif w_kind in ("valu", "swap", "trans") and kind == "mfma":
                req = 2
            elif w_kind in ("valu", "swap", "trans") and kind == "swap":
                req = 2
            need = max(need, req - gap)
        if kind in ("valu", "trans", "swap", "ds_read", "vmem"):
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


class Rec:
    """Records instructions instead of emitting them, so that a group of them can be dealt out
    one by one behind the matrix instructions.  A label or branch stays glued to the instruction
    in front of it."""

    def __init__(self):
        self.items = []

    def ins(self, *a, **k):
        self.items.append([("ins", a, k)])

    def raw(self, text):
        self.items[-1].append(("raw", text))


def replay(e, item):
    for kind, *rest in item:
        if kind == "ins":
            e.ins(*rest[0], **rest[1])
        else:
            e.raw(rest[0])


def load_groups():
    """Registers of the loads in flight at the top of an iteration, oldest first."""
    g = []
    for base in (KREG, VREG):
        for ps in range(NPASS):
            g.append([f"v{base(ps) + k}" for k in range(4)])
    return g


def frag_buf(f): return RING_BUFS[f % (LA + 1)] if BATCH == 1 else RING_BUFS[f % 4]

def qk_of(f):
    """(32-key block, k step) of S^T instruction f: the two blocks alternate, so that consecutive
    matrix instructions accumulate into different tuples (back-to-back accumulation into one tuple
    costs 37 cycles an instruction instead of 32)"""
    return (f % 2, f // 2) if "qkchain" not in KO else divmod(f, NKS)

def emit_frag_load(e, f, p):
    if "frag" in KO:
        return
    b = frag_buf(f)
    if f < 2 * NKS:                       # rows of K tile j+1
        mb, kk = qk_of(f)
        e.ins("ds_read_b128", vt(b), f"v{KFRAG} offset:{mb * 32 * KS * 2 + kk * 32}")
    else:                                 # columns of V tile j (buffer p)
        kk, db = divmod(f - 2 * NKS, NDB)
        off = p * VBUF + kk * 16 * VS * 2 + db * 64
        if "vtr" in KO:                    # timing only: one plain 16-byte read in place of the two transposed ones
            e.ins("ds_read_b128", vt(b), f"v{KFRAG} offset:{(db % 2) * 32 * KS * 2 + ((kk * NDB + db) % NKS) * 32}")
            return
        e.ins("ds_read_b64_tr_b16", vt(b, 2), f"v{VFRAG} offset:{off}")
        e.ins("ds_read_b64_tr_b16", vt(b + 2, 2), f"v{VFRAG} offset:{off + 8 * VS * 2}")

def emit_mfma(e, f, p):
    if "mfma" in KO:
        return
    b = frag_buf(f)
    if f < 2 * NKS:                       # logits of tile j+1 into the other set
        mb, kk = qk_of(f)
        s = S(1 - p, mb)
        e.ins("v_mfma_f32_32x32x16_bf16", vt(s, 16), vt(b), vt(Q(kk)), vt(NMREF, 16) if kk == 0 else vt(s, 16))
    else:                                 # O^T += V^T P^T of tile j
        kk, db = divmod(f - 2 * NKS, NDB)
        pr = S(p, kk // 2) + 4 * (kk % 2)  # P fragment kk lives in the registers of the logits it was made from
        e.ins("v_mfma_f32_32x32x16_bf16", vt(O(db), 16), vt(b), vt(pr), vt(O(db), 16))

# ---- loader
def write_tile(e, is_v, p):
    for ps in range(NPASS):
        if is_v:                          # V tile j+1 -> buffer 1-p
            e.ins("ds_write_b128", f"v{VW}", vt(VREG(ps)) + f" offset:{(1 - p) * VBUF + ps * TPP * VS * 2}")
        else:                             # K tile j+2 -> the buffer s_KWB names
            e.ins("ds_write_b128", f"v{KW}", vt(KREG(ps)) + f" offset:{ps * TPP * KS * 2}")

def issue_loads(e, is_v):
    base, rs, voff, tile, pss = (VREG, S_VB, VVOFF, S_VTILE, S_VPASS) if is_v else (KREG, S_KB, KVOFF, S_KTILE, S_KPASS)
    # tile = min(j + 2 (V) or j + 3 (K), last); byte offset of its first token
    e.ins("s_add_u32", f"s{S_T0}", f"s{S_J}", "2" if is_v else "3")
    e.ins("s_min_u32", f"s{S_T0}", f"s{S_T0}", f"s{S_LAST}")
    e.ins("s_mul_i32", f"s{S_T1}", f"s{S_T0}", f"s{tile}")
    for ps in range(NPASS):
        if "vmem" not in KO:
            e.ins("buffer_load_dwordx4", vt(base(ps)), f"v{voff}", st(rs), f"s{S_T1} offen")
        if ps + 1 < NPASS:
            e.ins("s_add_u32", f"s{S_T1}", f"s{S_T1}", f"s{pss}")

# ---- softmax of tile j (set p): one maximum over the tile's 32 logits of this lane's row
def sm_max(e, p):
    s = S(p, 0)
    e.ins("v_max3_f32", f"v{TA}", f"v{s}", f"v{s + 1}", f"v{s + 2}")
    e.ins("v_max3_f32", f"v{TB}", f"v{s + 3}", f"v{s + 4}", f"v{s + 5}")
    for k in range(6, 32, 4):
        e.ins("v_max3_f32", f"v{TA}", f"v{TA}", f"v{s + k}", f"v{s + k + 1}")
        if k + 3 < 32:
            e.ins("v_max3_f32", f"v{TB}", f"v{TB}", f"v{s + k + 2}", f"v{s + k + 3}")
    e.ins("v_max_f32", f"v{TA}", f"v{TA}", f"v{TB}")
    e.ins("v_mov_b32", f"v{TB}", f"v{TA}")
    e.ins("v_permlane32_swap_b32", f"v{TA}", f"v{TB}", ndst=2)
    e.ins("v_max_f32", f"v{TA}", f"v{TA}", f"v{TB}")
    e.ins("v_cmp_lt_f32", "vcc", f"s{S_SLACK}", f"v{TA}")
    e.raw(f"s_cbranch_vccnz .Lpf_rare_{p}_%=")
    e.raw(f".Lpf_cont_{p}_%=:")

def sm_exp(e, p, mb, q):
    s = S(p, mb)
    T0, T1 = ((T0A, T1A), (T0B, T1B))[mb]   # the two blocks' instructions interleave: a pair of temporaries each
    for k in range(4):
        e.ins("v_mov_b32" if "exp" in KO else "v_exp_f32", f"v{s + 4 * q + k}", f"v{s + 4 * q + k}")
    if "lsum" in KO:
        e.ins("v_cvt_pk_bf16_f32", f"v{s + 2 * q}", f"v{s + 4 * q}", f"v{s + 4 * q + 1}")
        e.ins("v_cvt_pk_bf16_f32", f"v{s + 2 * q + 1}", f"v{s + 4 * q + 2}", f"v{s + 4 * q + 3}")
        return
    e.ins("v_add_f32", f"v{T0}", f"v{s + 4 * q}", f"v{s + 4 * q + 1}")
    e.ins("v_add_f32", f"v{T1}", f"v{s + 4 * q + 2}", f"v{s + 4 * q + 3}")
    e.ins("v_cvt_pk_bf16_f32", f"v{s + 2 * q}", f"v{s + 4 * q}", f"v{s + 4 * q + 1}")
    e.ins("v_add_f32", f"v{T0}", f"v{T0}", f"v{T1}")
    e.ins("v_cvt_pk_bf16_f32", f"v{s + 2 * q + 1}", f"v{s + 4 * q + 2}", f"v{s + 4 * q + 3}")
    e.ins("v_add_f32", f"v{LSUM}", f"v{LSUM}", f"v{T0}")

def rare_path(p, started):
    """Row maximum of tile j left the slack (rare): move the reference up by a whole number and
    rescale what was accumulated against the old one (do_softmax() in tpa_prefill.hip).  `started`
    = the blocks of tile j+1 whose first matrix instruction was issued before the branch: their
    accumulation began at the old reference."""
    e = Stream()
    e.raw(f".Lpf_rare_{p}_%=:")
    e.nop(64)                        # matrix instructions in flight: their results and their operand reads
    e.ins("v_ceil_f32", f"v{RD}", f"v{TA}")
    e.ins("v_max_f32", f"v{RD}", "0", f"v{RD}")               # delta = tmax > 0 ? ceil(tmax) : 0
    e.ins("v_exp_f32_e64", f"v{RAL}", f"-v{RD}")              # alpha = 2^-delta
    e.ins("v_add_f32", f"v{MREF}", f"v{MREF}", f"v{RD}")
    for k in range(16):
        e.ins("v_sub_f32", f"v{NMREF + k}", "0", f"v{MREF}")
    e.ins("v_mul_f32", f"v{LSUM}", f"v{LSUM}", f"v{RAL}")
    for db in range(NDB):
        for k in range(16):
            e.ins("v_mul_f32", f"v{O(db) + k}", f"v{O(db) + k}", f"v{RAL}")
    for mb in range(2):              # nothing of tile j is packed yet
        for k in range(16):
            e.ins("v_sub_f32", f"v{S(p, mb) + k}", f"v{S(p, mb) + k}", f"v{RD}")
    for mb in started:
        for k in range(16):
            e.ins("v_sub_f32", f"v{S(1 - p, mb) + k}", f"v{S(1 - p, mb) + k}", f"v{RD}")
    e.nop(4)
    e.raw(f"s_branch .Lpf_cont_{p}_%=")
    return e.lines


def spread(items, lo, hi, out):
    """item k of len(items) goes behind MFMA slot lo + k (hi - lo) / len(items)"""
    n = len(items)
    for k, it in enumerate(items):
        out[lo + k * (hi - lo) // n].append(it)


def half(e, p, rare):
    """iteration j with j & 1 == p"""
    e.ins("v_add_u32", f"v{KFRAG}", f"s{S_KR}", f"v{KFRAG0}")
    e.ins("v_add_u32", f"v{KW}", f"s{S_KWB}", f"v{KW0}")
    for f in range(LA if BATCH == 1 else 2):
        emit_frag_load(e, f, p)
    slots = [[] for _ in range(NF)]
    N_QK = 2 * NKS
    ga, gb, gc, gd = Rec(), Rec(), Rec(), Rec()
    if not ({"softmax", "max"} & KO):
        sm_max(ga, p)
    n_max = len(ga.items)
    if "softmax" not in KO:
        for q in range(4):
            sm_exp(ga, p, 0, q)
        for q in range(4):
            sm_exp(gb, p, 1, q)
    write_tile(gc, False, p); issue_loads(gc, False)
    write_tile(gd, True, p); issue_loads(gd, True)
    # P of keys 0-31 must be packed before the first O^T instruction, P of keys 32-63 before the
    # O^T instructions of the second half of the tile
    spread(ga.items, 0, N_QK - 1, slots)
    spread(gb.items, N_QK // 2, N_QK + 2 * NDB - 1, slots)
    spread(gc.items, N_QK, N_QK + 2 * NDB, slots)
    spread(gd.items, N_QK + 2 * NDB, NF, slots)
    # the slot behind which the maximum's branch sits decides which blocks of tile j+1 have started
    if n_max:
        branch_slot = (n_max - 1) * (N_QK - 1) // len(ga.items)
        assert branch_slot < N_QK // 2     # before the first exponential of block 1
        rare[p] = sorted({qk_of(f)[0] for f in range(branch_slot + 1)})
    for f in range(NF):
        if BATCH == 1:
            if f + LA < NF:
                emit_frag_load(e, f + LA, p)
        elif f % 2 == 0:                 # the next pair on its way, then one wait for this pair
            for g in (f + 2, f + 3):
                if g < NF:
                    emit_frag_load(e, g, p)
            e._wait_for({f"v{frag_buf(g) + k}" for g in (f, f + 1) for k in range(4)})
        emit_mfma(e, f, p)
        for it in slots[f]:
            replay(e, it)
    # the K buffers rotate: next iteration reads what this one wrote beside, and writes the one after
    e.ins("s_mov_b32", f"s{S_KR}", f"s{S_KWB}")
    e.ins("s_add_u32", f"s{S_KWB}", f"s{S_KWB}", f"0x{KBUF:x}")
    e.ins("s_cmp_eq_u32", f"s{S_KWB}", f"0x{3 * KBUF:x}")
    e.ins("s_cselect_b32", f"s{S_KWB}", "0", f"s{S_KWB}")
    e.ins("s_add_u32", f"s{S_J}", f"s{S_J}", "1")
    e.barrier()


def main():
    rare = {}
    e = Stream()
    e.raw(f"s_mov_b32 s{S_SLACK}, 0x41000000")       # 8.0: the slack of the reference
    e.raw("s_nop 7")                                  # the logits of tile 1 come from matrix instructions issued just before
    e.raw("s_nop 7")
    e.raw(".Lpf_loop_%=:")
    e.prime_vm(load_groups())
    n_vm = len(e.vm)
    half(e, 1, rare)                                  # entry with an odd tile
    e.raw(f"s_cmp_lt_u32 s{S_J}, s{S_END}")
    e.raw("s_cbranch_scc0 .Lpf_done_%=")
    half(e, 0, rare)
    assert "vmem" in KO or len(e.vm) == n_vm, (len(e.vm), n_vm)   # the loads in flight are those the next iteration expects
    e.raw(f"s_cmp_lt_u32 s{S_J}, s{S_END}")
    e.raw("s_cbranch_scc1 .Lpf_loop_%=")
    e.raw("s_branch .Lpf_done_%=")
    lines = e.lines
    for p in sorted(rare):
        lines += rare_path(p, rare[p])
    lines += [
        ".Lpf_done_%=:",
        "s_waitcnt vmcnt(0)",                             # the load registers go back to the compiler
        "s_nop 7", "s_nop 7",                             # ... and so do the accumulators
    ]
    with open(OUT, "w") as f:
        f.write(f"// generated by gen_prefill_loop.py {D} dense: do not edit\n")
        for ln in lines:
            f.write(f'"{ln}\\n\\t"\n')
    # registers the loop uses beyond its operands
    ring = [b + k for b in (RING_BUFS[:LA + 1] if BATCH == 1 else RING_BUFS) for k in range(4)]
    # (a buffer inside the state tuple v[204:219] is part of an in/out operand already)
    clob = [f"v{n}" for n in sorted((set(ring) | set(range(TA, T1B + 1))) - set(range(204, 220)))]
    clob += [f"s{n}" for n in (S_T0, S_T1, S_SLACK)] + ["vcc", "scc", "memory"]
    with open(OUT.replace(".inc", "_clobbers.inc"), "w") as f:
        f.write("// generated by gen_prefill_loop.py: do not edit\n")
        f.write(", ".join(f'"{c}"' for c in clob) + "\n")
    n_mfma = sum("v_mfma" in ln for ln in lines)
    print(f"{OUT}: {len(lines)} lines, {n_mfma} MFMAs", file=sys.stderr)


main()
