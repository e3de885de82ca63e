#!/usr/bin/env python3
"""Writes the main loop of the four-wave prefill kernel (w4a16_prefill_wide.hip)
as one inline-assembly statement with fixed registers.

Why assembly: a wave of that kernel owns a 128 x 128 fp32 accumulator, i.e. all
256 AGPRs, next to about 170 live VGPRs.  With no register to spare the
compiler's allocator moves accumulators around and spills inside the loop; with
the registers named here nothing moves.  The schedule is also exactly the one
written down here: which unpack operation, LDS access or load is issued behind
which MFMA, and every s_waitcnt is computed from the order of issue.

The statement covers prologue, loop and the first part of the epilogue:
  prologue  requests of stages 0 and 1, slab 0 to LDS, unpack of the first k step
  loop      two 64-deep stages per turn (stage parity u is static), see stage()
  epilogue  row blocks 4..7 of the accumulator go to LDS for the other k half,
            row blocks 0..3 to v[0:127], which are the statement's outputs

Register map (v = VGPR, a = AGPR, s = SGPR):
  a[32i+4o : +3]   accumulator of row block i, operand o = 2j+h (16-column group j, half h)
  v[32b+4o : +3]   unpacked weights, buffer b (k step parity), operand o
  v[64+4x : +3]    activation operand ring, x = row block % 4
  v[80+4i : +3]    activation slab staging register i (8 per thread)
  v[112+16u+4r:+3] packed weights of stage parity u, 16-deep row r of the stage
  v[144+4u : +3]   group scales of stage parity u
  v[152+i]         byte offset of this thread's row i in A (or the out-of-range flag)
  v160 v161        per-lane byte offsets into B and into the scale rows
  v162 v163        LDS addresses: operand reads, slab writes
  v164 v165        shifted words of the unpack;  v166 0x64006400;  v167 -72 (fp16 x2)
  v168             LDS address for the accumulators that go to the other k half
  s[40:43] s[44:47] s[48:51]   buffer resources of A (tile rows), B, scales
  s52 s53 s54      first stage, end stage of this k half; stages the loop runs
  s55 s56          bytes per packed row of B; bytes per scale row
  s57..s67         loop state and constants (see below)
"""
import sys

# Schedule knobs (key=value on the command line overrides; the defaults are
# the measured best):
#   ahead    row blocks between an operand's LDS read and its first MFMA (1..3)
#   rdoff    MFMA of a row block behind which the read is issued (0..7)
#   slab0    preferred first MFMA and stride of the 12 slab operations of step 0
#   slab1    the same for step 1 (they end before the barrier, which sits just
#            before the first operand read from the next slab)
#   b0, b1   preferred MFMAs of the weight (and scale) loads of steps 0 and 1
OPT = {"ahead": 2, "rdoff": 0, "slab0": (2, 5), "slab1": (1, 3.5), "b0": (52, 58), "b1": (52, 56, 60)}

RB = 8
PLANE = 128 * 16
STEP_BYTES = 4 * PLANE + 128
SLAB_BYTES = 2 * STEP_BYTES           # 16640 = 65 * 256
assert SLAB_BYTES % 256 == 0


def W(b, o): return 32 * b + 4 * o
def AF(x): return 64 + 4 * x
def AREG(i): return 80 + 4 * i
def BQ(u, r): return 112 + 16 * u + 4 * r
def SREG(u): return 144 + 4 * u
def ALANE(i): return 152 + i
VBOFF, VSOFF, VRD, VWR = 160, 161, 162, 163
WT = (164, 165)
VEX, VNEG72, VSWAP = 166, 167, 168
N_VGPR = 169
RA, RB_, RS = 40, 44, 48
S_BEGIN, S_END, S_STAGES, S_BROW, S_N2 = 52, 53, 54, 55, 56
S_CS, S_SG2, S_SOFFA, S_SOFFB, S_SOFFS, S_FULL = 57, 58, 59, 60, 61, 62
S_LOMASK, S_HIMASK, S_NEG1032, S_SIXTEENTH, S_TMP = 63, 64, 65, 66, 67


def q(base): return f"v[{base}:{base + 3}]"
def aq(base): return f"a[{base}:{base + 3}]"
def sq(base): return f"s[{base}:{base + 3}]"


class Emitter:
    """Collects instructions and works out the s_waitcnt immediates.

    Loads and LDS operations complete in order of issue, each kind on its own
    counter.  wait_vm(reg) / wait_lgkm(reg) emit a wait that lets exactly the
    operations issued after the one that last wrote `reg` stay in flight.  The
    caller emits the first turn of the loop as a copy of its own, so that the
    loop's body finds a turn of the same order of issue before it."""

    def __init__(self):
        self.lines = []
        self.vm = []      # destination base registers of loads, in issue order
        self.lgkm = []    # destination base register (reads) or None (writes)

    def emit(self, text):
        self.lines.append(text)

    def load(self, dst, voff, rsrc, soff):
        self.emit(f"buffer_load_dwordx4 {q(dst)}, v{voff}, {sq(rsrc)}, s{soff} offen")
        self.vm.append(dst)

    def lds_read(self, dst, off):
        assert 0 <= off < 65536
        self.emit(f"ds_read_b128 {q(dst)}, v{VRD} offset:{off}")
        self.lgkm.append(dst)

    def lds_write2(self, d0, d1, off0, off1):
        assert 0 <= off0 < 256 and 0 <= off1 < 256
        self.emit(f"ds_write2st64_b32 v{VWR}, v{d0}, v{d1} offset0:{off0} offset1:{off1}")
        self.lgkm.append(None)

    @staticmethod
    def _pending_after(queue, reg):
        for back, r in enumerate(reversed(queue)):
            if r == reg:
                return back
        return None  # written before anything tracked: it has landed

    def wait(self, vm_regs=(), lgkm_regs=()):
        vm = min([n for n in (self._pending_after(self.vm, r) for r in vm_regs) if n is not None],
                 default=None)
        lg = min([n for n in (self._pending_after(self.lgkm, r) for r in lgkm_regs)
                  if n is not None], default=None)
        parts = []
        if vm is not None:
            parts.append(f"vmcnt({min(vm, 63)})")
        if lg is not None:
            parts.append(f"lgkmcnt({min(lg, 15)})")
        if parts:
            self.emit("s_waitcnt " + " ".join(parts))

    def drained(self, vm=False, lgkm=False):
        """everything of that kind has completed (after an s_waitcnt ...(0))"""
        if vm:
            self.vm = []
        if lgkm:
            self.lgkm = []


def unpack_op(e, group, buf, u, rows, j, op, r):
    """operation `op` of the unpack of word j of packed row rows[r] of stage
    parity u into dwords 2r, 2r+1 of operands 2j, 2j+1 of buffer buf"""
    if True:
        src = BQ(u, rows[r]) + j
        lo, hi = W(buf, 2 * j), W(buf, 2 * j + 1)
        wt = WT[r]
        if op == 0:
            e.emit(f"v_lshrrev_b32 v{wt}, 8, v{src}")
        elif op == 1:
            e.emit(f"v_and_or_b32 v{lo + 2 * r}, v{src}, s{S_LOMASK}, v{VEX}")
        elif op == 2:
            e.emit(f"v_and_or_b32 v{lo + 2 * r + 1}, v{src}, s{S_HIMASK}, v{VEX}")
        elif op == 3:
            e.emit(f"v_and_or_b32 v{hi + 2 * r}, v{wt}, s{S_LOMASK}, v{VEX}")
        elif op == 4:
            e.emit(f"v_and_or_b32 v{hi + 2 * r + 1}, v{wt}, s{S_HIMASK}, v{VEX}")
        elif op in (5, 7):
            d = (lo if op == 5 else hi) + 2 * r
            e.emit(f"v_pk_add_f16 v{d}, v{d}, s{S_NEG1032} op_sel_hi:[1,0]")
        elif op in (6, 8):
            d = (lo if op == 6 else hi) + 2 * r + 1
            e.emit(f"v_pk_fma_f16 v{d}, v{d}, s{S_SIXTEENTH}, v{VNEG72} op_sel_hi:[1,0,0]")
        else:
            assert group
            sc = SREG(u) + j
            if op in (9, 10):    # columns c: the scale in the low half
                d = lo + 2 * r + (op - 9)
                e.emit(f"v_pk_mul_f16 v{d}, v{sc}, v{d} op_sel_hi:[0,1]")
            else:                # columns c+8: the scale in the high half
                d = hi + 2 * r + (op - 11)
                e.emit(f"v_pk_mul_f16 v{d}, v{sc}, v{d} op_sel:[1,0] op_sel_hi:[1,1]")


def stage_scalars(e, ahead):
    """SALU: validity and offsets of the stage `ahead` stages after s57"""
    e.emit(f"s_add_i32 s{S_SG2}, s{S_CS}, {ahead}")
    e.emit(f"s_add_i32 s{S_SG2}, s{S_SG2}, s{S_BEGIN}")
    # a stage past the end of this k half reads zeros for A: empty buffer
    e.emit(f"s_cmp_lt_i32 s{S_SG2}, s{S_END}")
    e.emit(f"s_cselect_b32 s{RA + 2}, s{S_FULL}, 0")
    e.emit(f"s_lshl_b32 s{S_SOFFA}, s{S_SG2}, 7")
    e.emit(f"s_lshl_b32 s{S_TMP}, s{S_SG2}, 2")
    e.emit(f"s_mul_i32 s{S_SOFFB}, s{S_TMP}, s{S_BROW}")
    e.emit(f"s_lshr_b32 s{S_TMP}, s{S_SG2}, 1")
    e.emit(f"s_mul_i32 s{S_SOFFS}, s{S_TMP}, s{S_N2}")


def load_b(e, u, r):
    """row r of the stage that stage_scalars addressed (rows in order 0..3)"""
    e.load(BQ(u, r), VBOFF, RB_, S_SOFFB)
    e.emit(f"s_add_i32 s{S_SOFFB}, s{S_SOFFB}, s{S_BROW}")


def slab_op(e, slab, x, first_i):
    """x-th of the 12 slab operations of a step: per staging register two
    ds_write2st64_b32 into LDS slab `slab`, then its reload for the stage that
    stage_scalars addressed"""
    i, g = first_i + x // 3, x % 3
    if g < 2:
        if g == 0:
            e.wait(vm_regs=[AREG(i)])
        unit = slab * (SLAB_BYTES // 256) + 16 * g + i
        e.lds_write2(AREG(i) + 2 * g, AREG(i) + 2 * g + 1, unit, unit + 8)
    else:
        e.load(AREG(i), ALANE(i), RA, S_SOFFA)


def mfma(e, i, o, buf, x):
    acc = 32 * i + 4 * o
    e.emit(f"v_mfma_f32_16x16x32_f16 {aq(acc)}, {q(W(buf, o))}, {q(AF(x))}, {aq(acc)}")


def assign_slots(prefs):
    """distinct MFMA slots 0..63 for operations with preferred slots `prefs`
    (ascending): each gets its preference or the next free slot after the one
    before it; if they run past the end, the tail is pushed back"""
    slots, last = [], -1
    for pr in prefs:
        last = max(last + 1, int(pr))
        slots.append(last)
    over = slots[-1] - 63 if slots else 0
    if over > 0:
        for k in range(len(slots) - 1, -1, -1):
            cap = 63 - (len(slots) - 1 - k)
            if slots[k] <= cap:
                break
            slots[k] = cap
    assert len(set(slots)) == len(slots) and all(0 <= x < 64 for x in slots), slots
    return slots


def step(e, group, h, slab_cur, mem_ops, unpack_u, unpack_rows):
    """64 MFMAs on buffer h and LDS step (slab_cur, h), while the next step's
    weights (rows unpack_rows of stage parity unpack_u) are unpacked into buffer
    h^1 and the memory operations mem_ops -- (preferred slot, emit function),
    the step's operand reads are added here -- are issued.

    A memory instruction and unpack arithmetic behind the same MFMA cost about
    a whole MFMA time more than either alone (measured: MFMAs with the unpack
    16.2 cycles per MFMA, with the memory operations 17.7, with both dealt out
    regardless 23.0), so every memory operation gets an MFMA of its own, and
    the unpack goes behind the others, two operations each and three where
    that is not enough."""
    ops_per_word = 13 if group else 9
    cur = slab_cur * SLAB_BYTES + h * STEP_BYTES
    nxt = (slab_cur * SLAB_BYTES + STEP_BYTES) if h == 0 else (slab_cur ^ 1) * SLAB_BYTES
    ahead = OPT["ahead"]
    ops = list(mem_ops)
    for i in range(RB):
        tgt = i + ahead
        off = (cur + tgt * 256) if tgt < RB else (nxt + (tgt - RB) * 256)
        ops.append((8 * i + OPT["rdoff"], lambda e, tgt=tgt, off=off: e.lds_read(AF(tgt & 3), off)))
    ops.sort(key=lambda x: x[0])
    slots = assign_slots([pr for pr, _ in ops])
    mem_at = dict(zip(slots, (fn for _, fn in ops)))
    # the unpack: 8 words x ops_per_word operations, rows in lockstep
    todo = [(t // ops_per_word, t % ops_per_word, r) for t in range(4 * ops_per_word)
            for r in (0, 1)]
    free = [m for m in range(64) if m not in mem_at]
    per = [2] * len(free)
    short = len(todo) - 2 * len(free)
    k = 0
    while short > 0:      # a third operation behind evenly spaced MFMAs
        per[(k * len(free)) // max(1, len(todo) - 2 * len(free))] += 1
        k += 1
        short -= 1
    valu_at = dict(zip(free, per))
    for i in range(RB):
        e.wait(lgkm_regs=[AF(i & 3)])
        for o in range(8):
            m = 8 * i + o
            mfma(e, i, o, h, i & 3)
            if m in mem_at:
                mem_at[m](e)
            n = min(valu_at.get(m, 0), len(todo))
            if n and len(todo) == 8 * ops_per_word:
                # the packed rows (and scales) of the step being unpacked
                regs = [BQ(unpack_u, unpack_rows[0]), BQ(unpack_u, unpack_rows[1])]
                if group:
                    regs.append(SREG(unpack_u))
                e.wait(vm_regs=regs)
            for _ in range(n):
                j, op, r = todo.pop(0)
                unpack_op(e, group, h ^ 1, unpack_u, unpack_rows, j, op, r)
    assert not todo


def stage(e, group, u):
    """One 64-deep stage cs of parity u.  Step 0: rows 2, 3 of this stage are
    unpacked, staging registers 0..3 go to LDS slab u^1 (stage cs+1) and are
    requested again for stage cs+2, rows 0, 1 of stage cs+2 are requested.
    Step 1: rows 0, 1 of stage cs+1 are unpacked, staging registers 4..7 go to
    LDS; then the one barrier of the stage -- after it nobody reads slab u
    again, so the next stage may overwrite it, and slab u^1 is complete --
    before the first operands of stage cs+1 are read; rows 2, 3 and the scales
    of stage cs+2 are requested."""
    stage_scalars(e, 2 + u)  # s57 counts the turn's first stage

    def barrier(e):
        e.emit("s_waitcnt lgkmcnt(0)")
        e.drained(lgkm=True)
        e.emit("s_barrier")

    a, st = OPT["slab0"]
    ops0 = [(a + st * x, lambda e, x=x: slab_op(e, u ^ 1, x, 0)) for x in range(12)]
    ops0 += [(OPT["b0"][r], lambda e, r=r: load_b(e, u, r)) for r in (0, 1)]
    a, st = OPT["slab1"]
    bar = 8 * (RB - OPT["ahead"]) + OPT["rdoff"] - 0.5  # just before the first read of the next slab
    ops1 = [(min(a + st * x, bar - 0.75), lambda e, x=x: slab_op(e, u ^ 1, x, 4)) for x in range(12)]
    ops1 += [(bar, barrier)]
    ops1 += [(OPT["b1"][r], lambda e, r=r: load_b(e, u, 2 + r)) for r in (0, 1)]
    if group:
        ops1 += [(OPT["b1"][2], lambda e: e.load(SREG(u), VSOFF, RS, S_SOFFS))]
    step(e, group, 0, u, ops0, u, (2, 3))
    step(e, group, 1, u, ops1, u ^ 1, (0, 1))


def prologue(e, group):
    e.emit(f"s_mov_b32 s{S_FULL}, s{RA + 2}")
    e.emit(f"s_mov_b32 s{S_CS}, 0")
    e.emit(f"s_mov_b32 s{S_LOMASK}, 0x000f000f")
    e.emit(f"s_mov_b32 s{S_HIMASK}, 0x00f000f0")
    e.emit(f"s_mov_b32 s{S_NEG1032}, 0xe408")      # fp16 -1032
    e.emit(f"s_mov_b32 s{S_SIXTEENTH}, 0x2c00")    # fp16 1/16
    e.emit(f"v_mov_b32 v{VEX}, 0x64006400")
    e.emit(f"v_mov_b32 v{VNEG72}, 0xd480")         # fp16 -72
    for st in (0, 1):
        stage_scalars(e, st)
        for r in range(4):
            load_b(e, st, r)
        if group:
            e.load(SREG(st), VSOFF, RS, S_SOFFS)
        if st == 0:
            for i in range(RB):
                e.load(AREG(i), ALANE(i), RA, S_SOFFA)
            # the accumulators start at zero
            for n in range(256):
                e.emit(f"v_accvgpr_write_b32 a{n}, 0")
        else:
            # slab 0 to LDS, its registers requested again for stage 1
            for i in range(RB):
                for x in range(3):
                    slab_op(e, 0, 3 * i + x, 0)
    # first k step's weights
    regs = [BQ(0, 0), BQ(0, 1)] + ([SREG(0)] if group else [])
    e.wait(vm_regs=regs)
    for j in range(4):
        for op in range(13 if group else 9):
            for r in (0, 1):
                unpack_op(e, group, 0, 0, (0, 1), j, op, r)
    # slab 0 is in LDS for everybody; the requests of stage 1 stay in flight
    # (the first turn of the loop has waits of its own, computed from the order
    # of issue above)
    e.emit("s_waitcnt lgkmcnt(0)")
    e.drained(lgkm=True)
    e.emit("s_barrier")
    for x in range(OPT["ahead"]):
        e.lds_read(AF(x), x * 256)


def epilogue(e):
    # the last MFMAs' results are not readable for 18 cycles, and the hardware
    # does not interlock that for what follows
    e.emit("s_nop 15")
    e.emit("s_nop 15")
    e.emit("s_waitcnt vmcnt(0) lgkmcnt(0)")
    e.emit("s_barrier")          # every wave is done with the slabs
    for i in range(4, RB):
        for o in range(8):
            e.emit(f"ds_write_b128 v{VSWAP}, {aq(32 * i + 4 * o)} offset:{((i - 4) * 8 + o) * 1024}")
    for n in range(128):
        e.emit(f"v_accvgpr_read_b32 v{n}, a{n}")
    e.emit("s_waitcnt lgkmcnt(0)")


def turn(e, group, label, back):
    """two stages; leaves to .Lwd_done when the stages run out, else goes (or
    falls through) to the steady loop"""
    if label:
        e.emit(f"{label}:")
    stage(e, group, 0)
    e.emit(f"s_add_i32 s{S_TMP}, s{S_CS}, 1")
    e.emit(f"s_cmp_ge_i32 s{S_TMP}, s{S_STAGES}")
    e.emit("s_cbranch_scc1 .Lwd_done_%=")
    stage(e, group, 1)
    e.emit(f"s_add_i32 s{S_CS}, s{S_CS}, 2")
    if back:
        e.emit(f"s_cmp_lt_i32 s{S_CS}, s{S_STAGES}")
        e.emit("s_cbranch_scc1 .Lwd_loop_%=")
    else:
        e.emit(f"s_cmp_ge_i32 s{S_CS}, s{S_STAGES}")
        e.emit("s_cbranch_scc1 .Lwd_done_%=")


def generate(group):
    e = Emitter()
    prologue(e, group)
    # The first turn is a copy of the loop's body with waits of its own: what is
    # in flight when it starts was issued by the prologue, in another order
    # than a turn of the loop leaves behind.  The loop's body follows; its
    # waits see the first turn as the turn before, which issues exactly like
    # the body itself.
    turn(e, group, None, back=False)
    turn(e, group, ".Lwd_loop_%=", back=True)
    e.emit(".Lwd_done_%=:")
    epilogue(e)
    return e.lines


def statement(group):
    lines = generate(group)
    out = ["// generated by gen_prefill_wide.py -- do not edit", "asm volatile("]
    out += [f'    "{l}\\n\\t"' for l in lines]
    outs = [f'"={{v[{32 * i + 4 * o}:{32 * i + 4 * o + 3}]}}"(fin[{i}][{o}])'
            for i in range(4) for o in range(8)]
    outs.append(f'"+{{s[{RA}:{RA + 3}]}}"(ra_words)')
    out.append("    : " + ",\n      ".join(outs))
    ins = [f'"{{s[{RB_}:{RB_ + 3}]}}"(rb_words)',
           f'"{{s[{RS}:{RS + 3}]}}"(rs_words)',
           f'"{{s{S_BEGIN}}}"(s_begin)', f'"{{s{S_END}}}"(s_end)', f'"{{s{S_STAGES}}}"(stages)',
           f'"{{s{S_BROW}}}"(b_row)', f'"{{s{S_N2}}}"(s_row)']
    ins += [f'"{{v{ALANE(i)}}}"(a_lane[{i}])' for i in range(RB)]
    ins += [f'"{{v{VBOFF}}}"(b_lane)', f'"{{v{VSOFF}}}"(s_lane)', f'"{{v{VRD}}}"(lds_rd)',
            f'"{{v{VWR}}}"(lds_wr)', f'"{{v{VSWAP}}}"(lds_swap)']
    out.append("    : " + ",\n      ".join(ins))
    clob = [f'"v{n}"' for n in range(128, 152)] + [f'"v{n}"' for n in (164, 165, 166, 167)]
    clob += [f'"a{n}"' for n in range(256)]
    clob += [f'"s{n}"' for n in range(S_CS, S_TMP + 1)] + ['"scc"', '"memory"']
    out.append("    : " + ", ".join(clob) + ");")
    return "\n".join(out) + "\n"


if __name__ == "__main__":
    outdir = sys.argv[1] if len(sys.argv) > 1 else "."
    for arg in sys.argv[2:]:
        key, val = arg.split("=")
        OPT[key] = tuple(float(x) for x in val.split(",")) if "," in val else int(val)
    for group, name in ((True, "group"), (False, "chan")):
        with open(f"{outdir}/w4a16_prefill_wide_{name}.inc", "w") as f:
            f.write(statement(group))
