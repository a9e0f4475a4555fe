#!/usr/bin/env python3
"""Writes the assembly of the pipelined tile loops of the prefill kernel (tpa_prefill.hip) as C
string-literal include files: one loop for the dense K/V loader, one for the rank-2 factor loader.

Both loops belong to one wave (32 query rows) and overlap neighbouring pieces of the key axis so
that no matrix instruction of an iteration waits for vector work of the same iteration: the logits a
softmax reads were finished one step earlier.

dense loader (prefill_kernel<D, LOAD_DENSE, false>), one iteration j = one tile of 64 keys:

    S^T of tile j+1  (2 D/16 MFMAs, into the logit registers the previous iteration freed)
    softmax of tile j (row maximum, exponentials, packing to bf16), spread behind those MFMAs
    O^T += V^T P^T of tile j  (4 D/32 MFMAs)
    loader: K tile j+2 and V tile j+1 from registers to LDS, K tile j+3 and V tile j+2 requested
    one barrier

There are two sets of logit registers (tile parity), hence two copies of the iteration in the loop
body; K tiles rotate through three LDS buffers whose byte offsets travel in scalar registers, V
tiles through two that the copies address with immediates.

rank-2 factor loader (prefill_kernel<D, LOAD_TPA_R2, false>): the rows in flight are two ranks of B
factors per tile (twice the registers) and the loader's share of an iteration is the rebuild
K = a_0/2 b_0 + a_1/2 b_1, so the logits are pipelined in blocks of 32 keys, with two sets of 16
logit registers.  Iteration j (tile j = blocks 2j, 2j+1) enters with the logits of block 2j finished:

    S^T of block 2j+1 (D/16 MFMAs)  | softmax of block 2j
    O^T += V^T P^T of block 2j (2 D/32 MFMAs)  | rebuild of K tile j+2 into LDS, K tile j+3 requested
    S^T of block 2j+2 (first half of K tile j+1)  | softmax of block 2j+1
    O^T of block 2j+1  | rebuild of V tile j+1, V tile j+2 requested; head factors of K tile j+3 / V tile j+2
                         into their LDS slot, those of K tile j+4 / V tile j+3 requested
    one barrier

Again two copies of the iteration (the V buffers and the head-factor slots alternate and are
addressed with immediates); the three K buffers rotate through three scalar registers.

It is the instruction stream of cold_compute() + advance_tiles() + tail() in tpa_prefill.hip, whose
comments give the meaning of each step.

Why assembly: the logits, the accumulators, the Q fragments and the loads in flight fill the 256
registers a wave has with two waves per SIMD, in a fixed assignment that the compiler's allocator
does not find.  Every register in the loop is named here, and the C++ side hands the state over in
exactly these registers (inline-assembly operands pinned to physical registers).

The script keeps track of outstanding LDS / memory operations and of the software-visible hazards
of gfx950 (results of matrix, dot and transcendental instructions, lane swaps, vector writes read by
matrix instructions) and inserts the s_waitcnt / s_nop instructions they need.

usage: gen_prefill_loop.py <D: 128|64> <dense|r2> <output.inc>
"""
import re
import sys

D = int(sys.argv[1])
LOADER = sys.argv[2]
assert LOADER in ("dense", "r2") and D in (128, 64)
OUT = sys.argv[3]
R2 = LOADER == "r2"

KTK = 64
KS, VS = D + 8, D + 32                  # LDS row strides (elements)
NKS, NDB = D // 16, D // 32
CPR = D // 8
TPP = 512 // CPR                        # tokens per loader pass (512 threads)
NPASS = KTK // TPP
KBUF, VBUF = KTK * KS * 2, KTK * VS * 2  # bytes of one K / V buffer
NF = 2 * NKS + 4 * NDB                  # matrix instructions per iteration
LA = 2                                  # fragments read ahead of the MFMAs that consume them
ASLOT = 2 * KTK * 2 * 2                 # bytes of one slot of head factors: [K|V][token][rank] bf16

# ---- register maps (must match the operand lists of the asm statements in tpa_prefill.hip)
if not R2:
    def S(p, mb): return 32 * p + 16 * mb             # v: logits of (tile parity, 32-key block)
    NMREF = 64                                        # v[64:79]: -reference in all 16 registers
    def O(db): return 80 + 16 * db                    # v[80:143]: O^T accumulators
    def Q(ks): return 144 + 4 * ks                    # v[144:175]: Q fragments
    def KREG(ps): return 176 + 4 * ps                 # v[176:183]: K rows on their way (one tuple per loader pass)
    def VREG(ps): return 184 + 4 * ps                 # v[184:191]: V rows
    RING_BUFS = [192, 196, 200]                       # v[192:203]: fragment buffers
    MREF, LSUM, KFRAG0, VFRAG, KW0, VW, KVOFF, VVOFF = range(204, 212)   # v[204:219]: state / address tuple
    STATE = range(204, 220)
    TA, TB, T0A, T1A, KFRAG, KW, RD, RAL, T0B, T1B = range(220, 230)        # v[220:229]: temporaries
    TEMPS = range(220, 230)
    # s[32:47] scalar tuple
    S_J, S_END, S_LAST, S_KTILE, S_VTILE, S_KPASS, S_VPASS, S_KR, S_KWB = range(32, 41)
    S_KB, S_VB = 48, 52                               # buffer resources s[48:51], s[52:55]
    S_T0, S_T1, S_SLACK = 60, 61, 64
    S_CLOB = (S_T0, S_T1, S_SLACK)
else:
    def SET(b): return 16 * b                         # v[0:31]: logits of the block with parity b
    NMREF = 32                                        # v[32:47]
    def O(db): return 48 + 16 * db                    # v[48:111]
    def Q(ks): return 112 + 4 * ks                    # v[112:143]
    def KREG(ps, r): return 144 + 8 * ps + 4 * r      # v[144:159]: B-factor rows of K on their way (pass, rank)
    def VREG(ps, r): return 160 + 8 * ps + 4 * r      # v[160:175]
    RING_BUFS = [176, 180, 184]                       # v[176:187]
    # v[188:203]: state / address tuple
    MREF, LSUM, KFRAG0, VFRAG, KW0, VW, KVOFF, VVOFF, A_RD, A_WR, A_VOFF, A_PEND = range(188, 200)
    STATE = range(188, 204)
    # v[204:221]: temporaries
    TA, TB, T0A, T1A, T0B, T1B, KFA, KFB, KW, RD, RAL, AAK0, AAK1, AAV0, AAV1, PT, PT2, AT = range(204, 222)
    TEMPS = range(204, 222)
    # s[32:47] scalar tuple
    S_J, S_END, S_LAST, S_KTILE, S_VTILE, S_KPASS, S_VPASS, S_K0, S_K1, S_K2, S_KRANK, S_VRANK, S_ATILE, S_AAHEAD = range(32, 46)
    S_KB, S_VB, S_AB = 48, 52, 56                     # buffer resources s[48:51], s[52:55], s[56:59]
    S_T0, S_T1, S_SLACK, S_SELLO, S_SELHI, S_T2 = 60, 61, 64, 65, 66, 67
    S_CLOB = (S_T0, S_T1, S_SLACK, S_SELLO, S_SELHI, S_T2)

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
            elif w_kind == "dot":
                req = 3                      # a dot result may be read (or overwritten) three wait states later
            elif w_kind == "mfma":
                if kind == "mfma" and r in c_regs and r in dst:
                    req = 0                  # accumulation into the same tuple: back to back
                else:
                    req = 12
            elif w_kind in ("valu", "swap", "trans") and kind in ("mfma", "dot"):
                req = 2
            elif w_kind in ("valu", "swap", "trans") and kind == "swap":
                req = 2
            need = max(need, req - gap)
        if kind in ("valu", "trans", "swap", "dot", "ds_read", "vmem"):
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


def spread(items, lo, hi, out):
    """item k of len(items) goes behind MFMA slot lo + k (hi - lo) / len(items)"""
    n = len(items)
    for k, it in enumerate(items):
        out[lo + k * (hi - lo) // n].append(it)


def frag_buf(f): return RING_BUFS[f % (LA + 1)]


# =====================================================================================================
# dense loader
# =====================================================================================================
def load_groups():
    """Registers of the loads in flight at the top of an iteration, oldest first."""
    g = []
    if R2:
        for base in (KREG, VREG):
            for ps in range(NPASS):
                for r in range(2):
                    g.append([f"v{base(ps, r) + k}" for k in range(4)])
        g.append([f"v{A_PEND}"])
    else:
        for base in (KREG, VREG):
            for ps in range(NPASS):
                g.append([f"v{base(ps) + k}" for k in range(4)])
    return g


def qk_of(f):
    """(32-key block, k step) of S^T instruction f: the two blocks alternate, so that consecutive
    matrix instructions accumulate into different tuples (back-to-back accumulation into one tuple
    costs 37 cycles an instruction instead of 32)"""
    return (f % 2, f // 2)

def emit_frag_load(e, f, p):
    b = frag_buf(f)
    if f < 2 * NKS:                       # rows of K tile j+1
        mb, kk = qk_of(f)
        e.ins("ds_read_b128", vt(b), f"v{KFRAG} offset:{mb * 32 * KS * 2 + kk * 32}")
    else:                                 # columns of V tile j (buffer p)
        kk, db = divmod(f - 2 * NKS, NDB)
        off = p * VBUF + kk * 16 * VS * 2 + db * 64
        e.ins("ds_read_b64_tr_b16", vt(b, 2), f"v{VFRAG} offset:{off}")
        e.ins("ds_read_b64_tr_b16", vt(b + 2, 2), f"v{VFRAG} offset:{off + 8 * VS * 2}")

def emit_mfma(e, f, p):
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

def sm_exp_regs(e, s, q, T0, T1):
    """exponentials, row sum and bf16 packing of logits 4q .. 4q+3 of the 16 in v[s:s+15]"""
    for k in range(4):
        e.ins("v_exp_f32", f"v{s + 4 * q + k}", f"v{s + 4 * q + k}")
    e.ins("v_add_f32", f"v{T0}", f"v{s + 4 * q}", f"v{s + 4 * q + 1}")
    e.ins("v_add_f32", f"v{T1}", f"v{s + 4 * q + 2}", f"v{s + 4 * q + 3}")
    e.ins("v_cvt_pk_bf16_f32", f"v{s + 2 * q}", f"v{s + 4 * q}", f"v{s + 4 * q + 1}")
    e.ins("v_add_f32", f"v{T0}", f"v{T0}", f"v{T1}")
    e.ins("v_cvt_pk_bf16_f32", f"v{s + 2 * q + 1}", f"v{s + 4 * q + 2}", f"v{s + 4 * q + 3}")
    e.ins("v_add_f32", f"v{LSUM}", f"v{LSUM}", f"v{T0}")

def sm_exp(e, p, mb, q):
    T0, T1 = ((T0A, T1A), (T0B, T1B))[mb]   # the two blocks' instructions interleave: a pair of temporaries each
    sm_exp_regs(e, S(p, mb), q, T0, T1)

def rescale(e, sets):
    """the reference moves up by ceil(row maximum) (a whole number, so every factor is an exact power of
    two): O and the row sum shrink, the logit registers listed in `sets` move down"""
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
    for s in sets:
        for k in range(16):
            e.ins("v_sub_f32", f"v{s + k}", f"v{s + k}", f"v{RD}")

def rare_path(p, started):
    """Row maximum of tile j left the slack (rare): move the reference up by a whole number and
    rescale what was accumulated against the old one (do_softmax() in tpa_prefill.hip).  `started`
    = the blocks of tile j+1 whose first matrix instruction was issued before the branch: their
    accumulation began at the old reference."""
    e = Stream()
    e.raw(f".Lpf_rare_{p}_%=:")
    e.nop(64)                        # matrix instructions in flight: their results and their operand reads
    # nothing of tile j is packed yet: both its blocks move
    rescale(e, [S(p, 0), S(p, 1)] + [S(1 - p, mb) for mb in started])
    e.nop(4)
    e.raw(f"s_branch .Lpf_cont_{p}_%=")
    return e.lines


def half(e, p, rare):
    """iteration j with j & 1 == p"""
    e.ins("v_add_u32", f"v{KFRAG}", f"s{S_KR}", f"v{KFRAG0}")
    e.ins("v_add_u32", f"v{KW}", f"s{S_KWB}", f"v{KW0}")
    for f in range(LA):
        emit_frag_load(e, f, p)
    slots = [[] for _ in range(NF)]
    N_QK = 2 * NKS
    ga, gb, gc, gd = Rec(), Rec(), Rec(), Rec()
    sm_max(ga, p)
    n_max = len(ga.items)
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
    branch_slot = (n_max - 1) * (N_QK - 1) // len(ga.items)
    assert branch_slot < N_QK // 2     # before the first exponential of block 1
    rare[p] = sorted({qk_of(f)[0] for f in range(branch_slot + 1)})
    for f in range(NF):
        if f + LA < NF:
            emit_frag_load(e, f + LA, p)
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


# =====================================================================================================
# rank-2 factor loader
# =====================================================================================================
def r2_step(f):
    """matrix instruction f of an iteration -> (phase, index within the phase): phases 0 / 2 are the
    S^T of blocks 2j+1 / 2j+2, phases 1 / 3 the O^T of blocks 2j / 2j+1"""
    bounds = [NKS, NKS + 2 * NDB, 2 * NKS + 2 * NDB, NF]
    lo = 0
    for ph, hi in enumerate(bounds):
        if f < hi:
            return ph, f - lo
        lo = hi
    raise ValueError(f)

def r2_frag_load(e, f, p):
    b = frag_buf(f)
    ph, k = r2_step(f)
    if ph == 0:                           # rows 32 .. 63 of K tile j
        e.ins("ds_read_b128", vt(b), f"v{KFA} offset:{32 * KS * 2 + k * 32}")
    elif ph == 2:                         # rows 0 .. 31 of K tile j+1
        e.ins("ds_read_b128", vt(b), f"v{KFB} offset:{k * 32}")
    else:                                 # columns of V tile j (buffer p), keys 16 kk .. 16 kk + 15
        kk, db = divmod(k, NDB)
        kk += 2 * (ph // 2)
        off = p * VBUF + kk * 16 * VS * 2 + db * 64
        e.ins("ds_read_b64_tr_b16", vt(b, 2), f"v{VFRAG} offset:{off}")
        e.ins("ds_read_b64_tr_b16", vt(b + 2, 2), f"v{VFRAG} offset:{off + 8 * VS * 2}")

def r2_mfma(e, f, p):
    b = frag_buf(f)
    ph, k = r2_step(f)
    if ph in (0, 2):                      # logits of block 2j+1 into set 1, of block 2j+2 into set 0
        s = SET(1 if ph == 0 else 0)
        e.ins("v_mfma_f32_32x32x16_bf16", vt(s, 16), vt(b), vt(Q(k)), vt(NMREF, 16) if k == 0 else vt(s, 16))
    else:                                 # O^T += V^T P^T of block 2j (set 0) / 2j+1 (set 1)
        kk, db = divmod(k, NDB)
        pr = SET(ph // 2) + 4 * kk         # P fragment kk of the block lives in the registers of the logits it was made from
        e.ins("v_mfma_f32_32x32x16_bf16", vt(O(db), 16), vt(b), vt(pr), vt(O(db), 16))

def r2_sm_max(e, p, blk):
    """row maximum over the 16 logits of this lane's row in set blk, and the test against the slack"""
    s = SET(blk)
    e.ins("v_max3_f32", f"v{TA}", f"v{s}", f"v{s + 1}", f"v{s + 2}")
    e.ins("v_max3_f32", f"v{TB}", f"v{s + 3}", f"v{s + 4}", f"v{s + 5}")
    e.ins("v_max3_f32", f"v{TA}", f"v{TA}", f"v{s + 6}", f"v{s + 7}")
    e.ins("v_max3_f32", f"v{TB}", f"v{TB}", f"v{s + 8}", f"v{s + 9}")
    e.ins("v_max3_f32", f"v{TA}", f"v{TA}", f"v{s + 10}", f"v{s + 11}")
    e.ins("v_max3_f32", f"v{TB}", f"v{TB}", f"v{s + 12}", f"v{s + 13}")
    e.ins("v_max3_f32", f"v{TA}", f"v{TA}", f"v{s + 14}", f"v{s + 15}")
    e.ins("v_max_f32", f"v{TA}", f"v{TA}", f"v{TB}")
    e.ins("v_mov_b32", f"v{TB}", f"v{TA}")
    e.ins("v_permlane32_swap_b32", f"v{TA}", f"v{TB}", ndst=2)
    e.ins("v_max_f32", f"v{TA}", f"v{TA}", f"v{TB}")
    e.ins("v_cmp_lt_f32", "vcc", f"s{S_SLACK}", f"v{TA}")
    e.raw(f"s_cbranch_vccnz .Lpf_rare_{p}{blk}_%=")
    e.raw(f".Lpf_cont_{p}{blk}_%=:")

def r2_rare_path(p, blk):
    """Row maximum of a block left the slack (rare).  The block's own logits are not packed yet; the
    other set holds the partial sums of the next block, whose accumulation began at the old
    reference (its first matrix instruction is always issued before the branch)."""
    e = Stream()
    e.raw(f".Lpf_rare_{p}{blk}_%=:")
    e.nop(64)                        # matrix instructions in flight: their results and their operand reads
    rescale(e, [SET(blk), SET(1 - blk)])
    e.nop(4)
    e.raw(f"s_branch .Lpf_cont_{p}{blk}_%=")
    return e.lines

def r2_rebuild(e, is_v, p):
    """K tile j+2 (into the buffer s_K2 names) or V tile j+1 (into buffer 1-p) from the B-factor rows
    in registers and the halved head factors aa = (a_0/2, a_1/2) of this thread's tokens: per 16-byte
    chunk 8 v_perm_b32 pair b_0[d] with b_1[d] (in place, two temporaries), 8 v_dot2_f32_bf16 form
    a_0/2 b_0[d] + a_1/2 b_1[d], 4 v_cvt_pk_bf16_f32 pack; then the next tile's rows are requested."""
    base, aa = (VREG, (AAV0, AAV1)) if is_v else (KREG, (AAK0, AAK1))
    rs, voff, tile, pss, rank = (S_VB, VVOFF, S_VTILE, S_VPASS, S_VRANK) if is_v else (S_KB, KVOFF, S_KTILE, S_KPASS, S_KRANK)
    # tile = min(j + 2 (V) or j + 3 (K), last); byte offset of its first token
    e.ins("s_add_u32", f"s{S_T0}", f"s{S_J}", "2" if is_v else "3")
    e.ins("s_min_u32", f"s{S_T0}", f"s{S_T0}", f"s{S_LAST}")
    e.ins("s_mul_i32", f"s{S_T1}", f"s{S_T0}", f"s{tile}")
    for ps in range(NPASS):
        b0, b1 = base(ps, 0), base(ps, 1)
        # (b0[i], b1[i]) -> pairs (b_0[d], b_1[d]) of elements 2i and 2i+1, each multiplied with (a_0/2, a_1/2):
        # element 2i ends in b0[i], element 2i+1 in b1[i]
        def dots(i):
            e.ins("v_dot2_f32_bf16", f"v{b1 + i}", f"v{(PT, PT2)[i % 2]}", f"v{aa[ps]}", "0")
            e.ins("v_dot2_f32_bf16", f"v{b0 + i}", f"v{b0 + i}", f"v{aa[ps]}", "0")
        for i in range(4):
            e.ins("v_perm_b32", f"v{(PT, PT2)[i % 2]}", f"v{b1 + i}", f"v{b0 + i}", f"s{S_SELHI}")
            e.ins("v_perm_b32", f"v{b0 + i}", f"v{b1 + i}", f"v{b0 + i}", f"s{S_SELLO}")
            if i >= 1:
                dots(i - 1)
        dots(3)
        for i in range(4):
            e.ins("v_cvt_pk_bf16_f32", f"v{b0 + i}", f"v{b0 + i}", f"v{b1 + i}")
        if is_v:
            e.ins("ds_write_b128", f"v{VW}", vt(b0) + f" offset:{(1 - p) * VBUF + ps * TPP * VS * 2}")
        else:
            e.ins("ds_write_b128", f"v{KW}", vt(b0) + f" offset:{ps * TPP * KS * 2}")
        # the pass's registers are free: request its rows of the next tile right away, so that the eight waves'
        # loads reach the memory pipeline a few at a time (a burst of them stalls the waves at issue)
        e.ins("s_add_u32", f"s{S_T2}", f"s{S_T1}", f"s{rank}")
        e.ins("buffer_load_dwordx4", vt(base(ps, 0)), f"v{voff}", st(rs), f"s{S_T1} offen")
        e.ins("buffer_load_dwordx4", vt(base(ps, 1)), f"v{voff}", st(rs), f"s{S_T2} offen")
        if ps + 1 < NPASS:
            e.ins("s_add_u32", f"s{S_T1}", f"s{S_T1}", f"s{pss}")

def r2_head_factors(e, p):
    """this thread's head factor of K tile j+3 / V tile j+2 (requested an iteration ago) halved (the 1/R
    of the reconstruction, exact in bf16) into slot 1-p; the one of K tile j+4 / V tile j+3 requested
    (s_AAHEAD = 4 for the waves that serve K, 3 for those that serve V)"""
    e.ins("v_lshlrev_b32", f"v{AT}", "16", f"v{A_PEND}")
    e.ins("v_mul_f32", f"v{AT}", "0.5", f"v{AT}")
    e.ins("v_cvt_pk_bf16_f32", f"v{AT}", f"v{AT}", "0")
    e.ins("ds_write_b16", f"v{A_WR}", f"v{AT}" + f" offset:{(1 - p) * ASLOT}")
    e.ins("s_add_u32", f"s{S_T0}", f"s{S_J}", f"s{S_AAHEAD}")
    e.ins("s_min_u32", f"s{S_T0}", f"s{S_T0}", f"s{S_LAST}")
    e.ins("s_mul_i32", f"s{S_T1}", f"s{S_T0}", f"s{S_ATILE}")
    e.ins("buffer_load_ushort", f"v{A_PEND}", f"v{A_VOFF}", st(S_AB), f"s{S_T1} offen")

def half_r2(e, p):
    """iteration j with j & 1 == p"""
    e.ins("v_add_u32", f"v{KFA}", f"s{S_K0}", f"v{KFRAG0}")
    e.ins("v_add_u32", f"v{KFB}", f"s{S_K1}", f"v{KFRAG0}")
    e.ins("v_add_u32", f"v{KW}", f"s{S_K2}", f"v{KW0}")
    # halved head factors (a_0, a_1) of this thread's tokens in K tile j+2 and V tile j+1: slot p
    for ps in range(NPASS):
        e.ins("ds_read_b32", f"v{(AAK0, AAK1)[ps]}", f"v{A_RD} offset:{p * ASLOT + ps * TPP * 4}")
    for ps in range(NPASS):
        e.ins("ds_read_b32", f"v{(AAV0, AAV1)[ps]}", f"v{A_RD} offset:{p * ASLOT + KTK * 4 + ps * TPP * 4}")
    for f in range(LA):
        r2_frag_load(e, f, p)
    slots = [[] for _ in range(NF)]
    P1, P2, P3 = NKS, NKS + 2 * NDB, 2 * NKS + 2 * NDB     # first instruction of phases 1, 2, 3
    g0, g0b, g1, g1b, gk, gv = Rec(), Rec(), Rec(), Rec(), Rec(), Rec()
    # softmax of block 2j (set 0): maximum and the first 8 keys before the O^T instructions of keys
    # 0-15 of the block, the other 8 keys before those of keys 16-31
    r2_sm_max(g0, p, 0)
    for q in range(2):
        sm_exp_regs(g0, SET(0), q, T0A, T1A)
    for q in range(2, 4):
        sm_exp_regs(g0b, SET(0), q, T0B, T1B)
    r2_sm_max(g1, p, 1)
    for q in range(2):
        sm_exp_regs(g1, SET(1), q, T0A, T1A)
    for q in range(2, 4):
        sm_exp_regs(g1b, SET(1), q, T0B, T1B)
    r2_rebuild(gk, False, p)
    r2_rebuild(gv, True, p)
    r2_head_factors(gv, p)
    spread(g0.items, 0, P1, slots)
    spread(g0b.items, P1 - NKS // 4, P1 + NDB, slots)
    spread(gk.items, P1, P2, slots)
    spread(g1.items, P2, P3, slots)
    spread(g1b.items, P3 - NKS // 4, P3 + NDB, slots)
    spread(gv.items, P3, NF, slots)
    for f in range(NF):
        if f + LA < NF:
            r2_frag_load(e, f + LA, p)
        r2_mfma(e, f, p)
        for it in slots[f]:
            replay(e, it)
    # the K buffers rotate: (tile j, tile j+1, free) -> (tile j+1, tile j+2, free)
    e.ins("s_mov_b32", f"s{S_T0}", f"s{S_K0}")
    e.ins("s_mov_b32", f"s{S_K0}", f"s{S_K1}")
    e.ins("s_mov_b32", f"s{S_K1}", f"s{S_K2}")
    e.ins("s_mov_b32", f"s{S_K2}", f"s{S_T0}")
    e.ins("s_add_u32", f"s{S_J}", f"s{S_J}", "1")
    e.barrier()


def main():
    e = Stream()
    e.raw(f"s_mov_b32 s{S_SLACK}, 0x41000000")       # 8.0: the slack of the reference
    if R2:
        e.raw(f"s_mov_b32 s{S_SELLO}, 0x05040100")   # v_perm_b32 selectors: low halves / high halves of two registers
        e.raw(f"s_mov_b32 s{S_SELHI}, 0x07060302")
    e.raw("s_nop 7")                                  # the logits handed in come from matrix instructions issued just before
    e.raw("s_nop 7")
    e.raw(".Lpf_loop_%=:")
    e.prime_vm(load_groups())
    n_vm = len(e.vm)
    rare_lines = []
    if R2:
        half_r2(e, 1)                                 # entry with an odd tile
        e.raw(f"s_cmp_lt_u32 s{S_J}, s{S_END}")
        e.raw("s_cbranch_scc0 .Lpf_done_%=")
        half_r2(e, 0)
        for p in (0, 1):
            for blk in (0, 1):
                rare_lines += r2_rare_path(p, blk)
    else:
        rare = {}
        half(e, 1, rare)                              # entry with an odd tile
        e.raw(f"s_cmp_lt_u32 s{S_J}, s{S_END}")
        e.raw("s_cbranch_scc0 .Lpf_done_%=")
        half(e, 0, rare)
        for p in sorted(rare):
            rare_lines += rare_path(p, rare[p])
    assert len(e.vm) == n_vm, (len(e.vm), n_vm)       # the loads in flight are those the next iteration expects
    e.raw(f"s_cmp_lt_u32 s{S_J}, s{S_END}")
    e.raw("s_cbranch_scc1 .Lpf_loop_%=")
    e.raw("s_branch .Lpf_done_%=")
    lines = e.lines + rare_lines
    lines += [
        ".Lpf_done_%=:",
        "s_waitcnt vmcnt(0)",                             # the load registers go back to the compiler
        "s_nop 7", "s_nop 7",                             # ... and so do the accumulators
    ]
    with open(OUT, "w") as f:
        f.write(f"// generated by gen_prefill_loop.py {D} {LOADER}: do not edit\n")
        for ln in lines:
            f.write(f'"{ln}\\n\\t"\n')
    # registers the loop uses beyond its operands (the state tuple is an in/out operand)
    ring = [b + k for b in RING_BUFS for k in range(4)]
    named = set().union(*(regs_of(ln) for ln in lines))     # a head size with one loader pass leaves some unused
    clob = [f"v{n}" for n in sorted((set(ring) | set(TEMPS)) - set(STATE)) if f"v{n}" in named]
    clob += [f"s{n}" for n in S_CLOB] + ["vcc", "scc", "memory"]
    with open(OUT.replace(".inc", "_clobbers.inc"), "w") as f:
        f.write("// generated by gen_prefill_loop.py: do not edit\n")
        f.write(", ".join(f'"{c}"' for c in clob) + "\n")
    n_mfma = sum("v_mfma" in ln for ln in lines)
    print(f"{OUT}: {len(lines)} lines, {n_mfma} MFMAs", file=sys.stderr)


main()
