#!/usr/bin/env python3
"""Writes gemm_wide_gfx950.inc: the 256 x 256 Matmul tile on four waves, one per SIMD, each with a
128 x 128 block of C in 256 accumulation registers; k loop and epilogue in gfx950 assembly.

Why this shape.  Measured on the matrix cores of an MI355X: about two other instructions of a
SIMD's waves issue for free under 16 cycles of MFMA work, every further one delays the next MFMA by
about four cycles, whichever wave it comes from.  So the k loop wants as few instructions per MFMA
cycle as it can get: the largest block of C per wave (an operand read from LDS once serves eight
MFMAs) and one wave per SIMD (no per-wave bookkeeping twice).

Why MFMAs of 16 x 16 x 64 bytes (v_mfma_i32_16x16x64_i8, v_mfma_f32_16x16x32_bf16) and not of
32 x 32 x 32: the board is power-limited, and on operands distributed like a benchmark's the
16 x 16 form sustains 4000 TOPS int8 / 2070 TFLOPS bf16 where the 32 x 32 form sustains 3360 /
1840 (back-to-back MFMAs on register operands, all SIMDs): it updates an accumulator once per 64
multiply-adds instead of once per 32.  The same k loop with either form: 65.1 against 70.6 us at
4096^3 int8, 798 against 842 us at 8192^3 bf16, same box.

One k step (tile kt, 128 bytes of K) is two slabs of 64 bytes; a slab is 8 x 8 MFMAs, block row
tm outermost.  Per slab a wave reads 8 A operands (ds_read_b128: lane (l % 16, l / 16) takes row
l % 16 of the block row and the l / 16-th 16 bytes of the slab) and 8 B operands (two transposing
ds_read_b64_tr each: the 16-lane group l / 16 takes the same 16 k of the slab for the block's 16
columns).  The k index of an MFMA is a contraction index: which 16 bytes of K a lane group holds is
free as long as both operands agree, and here both hold bytes 16 g .. 16 g + 15 of the slab.
  * A operands have ONE register set: block row tm's operand is used by eight MFMAs in a row and
    is dead after them, so the next slab's goes into the same registers right behind its last use,
    56 MFMAs before its first.  B operands are used all through a slab and have two sets.
  * A of tile kt + 1 goes from a register set to its LDS stage (xor 0x80 on the way for a u8
    operand: a - 128, once per byte) and the set is refilled with tile kt + 3 from global memory:
    two register sets, two LDS stages;
  * B of tile kt + 2 is requested straight into the third of three LDS slots
    (global_load_lds_dwordx4; one M0 per step, the instructions' immediate offsets, added to both
    addresses, tell the pieces apart);
  * the column sums of B that the u8 correction needs are added up from the B operand registers
    (xor 0x80, sum of unsigned bytes: b + 128; the dot-product instructions hold up the MFMAs
    behind them); the two wave rows share the columns and take half of them each -- in the code
    it is block columns 0 .. 3 for every wave, and the kernel numbers the lower wave row's block
    columns from the fifth on, so that all four waves run the same instructions;
  * one barrier, three quarters through the step, preceded by the step's wait for memory:
    everything requested before this step began has landed; the next tile's first operands are
    read behind it;
  * an accumulating Spec loads C's old values during the first eight steps, a block row a step,
    and adds them to the blocks' accumulators a step later, clear of the blocks' own MFMAs, so
    that the epilogue only stores.  These steps are unrolled (the additions name their
    accumulators); the rest is a loop of six steps.  All of it together must stay well inside the
    64 KB instruction cache: a body that does not fit is fetched anew by every launch, which cost
    100 to 350 cycles a step when the unrolled steps numbered eighteen.

Register map (all named in the clobber list of the asm statement):
  a[0:255]    accumulators, block (tm, tn) at 4 * (8 * tm + tn); register i of lane l holds row
              4 * (l / 16) + i, column l % 16 of the block
  v[0:63]     A staging, set p chunk i at 32 * p + 4 * i; after the loop: values on their way to C
  v[64:95]    A operands, block row tm at 64 + 4 * tm; after the loop: the column sums' partials
  v[96:159]   B operands, set b block column tn at 96 + 32 * b + 4 * tn; after the loop: partials
  v[160:167]  LDS address of the lane's B operand, per tn, in the third slot (the first two are
              reached from the kernel's %[b_rd] with the instruction's offset)
  v[168:175]  column sums of B (u8 correction), one per tn; after the loop: 128 * column sum
  v[176:177]  scratch
  v[180:211]  old values of a block row of C
  s[60:61] A tile pointer   s[62:63] B tile pointer   s64 loop counter   s67 index of the next
  A tile to fetch, s68 of the next B tile   s[72:73] C block row pointer   s74 0x80808080   s69, s[78:79] scratch
"""
import os
import sys

A_STAGE = 32768
B_SLOT = 32768
B_BASE = 2 * A_STAGE
SLAB_BYTES = 16384  # one 64-byte slab of K in a B slot: its k rows x 256 (i8) / 512 (bf16) bytes
HI_BYTES = 2048     # second transposing read of an operand: 8 (i8) / 4 (bf16) k rows on
TM, TN = 8, 8       # MFMA blocks per wave
MF = TM * TN        # MFMAs per slab
SLABS = 2
GAPS = SLABS * MF   # MFMAs per k step
BARRIER_AT = 96     # the step's barrier comes before this MFMA (88, 100, 104: the same; 80: 1-2 % slower)
GAP_SLOTS = 2       # instructions placed behind one MFMA before the next is due (2: 63.7 us at 4096^3 int8, 3: 64.5, 4: 65)
VALU_SLOTS = 2      # of which vector instructions
C_STEPS = 8         # k steps that carry the loads of C's old values: a block row (32 registers) a step


def acc(tm, tn):
    b = 4 * (TN * tm + tn)
    return f"a[{b}:{b + 3}]"


def areg(p, i, w=None):
    b = 32 * p + 4 * i
    return f"v[{b}:{b + 3}]" if w is None else f"v{b + w}"


def af(tm):
    b = 64 + 4 * tm
    return f"v[{b}:{b + 3}]"


def bf(buf, tn, half=None, w=None):
    b = 96 + 32 * buf + 4 * tn
    if w is not None:
        return f"v{b + w}"
    if half is None:
        return f"v[{b}:{b + 3}]"
    return f"v[{b + 2 * half}:{b + 2 * half + 1}]"


B_ADDR = 160    # v[160:167]
COL_SUM = 168   # v[168:175]
TMP0, TMP1 = 176, 177
C_TMP = (177, 178, 179)   # temporaries of the additions of C's old values
OLD_C = 180     # v[180:211]: the old values of one block row of C


class Emitter:
    """Collects instructions; derives s_waitcnt from the order of LDS and vector memory operations."""

    def __init__(self):
        self.lines = []
        self.lds_issued = 0
        self.lds_done = 0
        self.producer = {}      # register name -> index of the LDS read that fills it
        self.vm_issued = 0
        self.vm_done = 0        # vector memory operations with index < vm_done are known complete
        self.vm_producer = {}

    def emit(self, text):
        self.lines.append(text)

    def lds_read(self, dst, text):
        self.producer[dst] = self.lds_issued
        self.lds_issued += 1
        self.emit(text)

    def lds_write(self, text):
        self.lds_issued += 1
        self.emit(text)

    def need(self, *regs):
        idx = max((self.producer.get(r, -1) for r in regs), default=-1)
        if idx >= self.lds_done:
            allowed = self.lds_issued - idx - 1
            self.emit(f"s_waitcnt lgkmcnt({min(allowed, 15)})")
            self.lds_done = idx + 1 if allowed <= 15 else self.lds_issued - 15

    def all_lds_done(self):
        self.lds_done = self.lds_issued

    def vm(self, text, dst=None):
        if dst is not None:
            self.vm_producer[dst] = self.vm_issued
        self.vm_issued += 1
        self.emit(text)

    def vm_wait_index(self, idx):
        """Every vector memory operation up to and including index idx has completed."""
        if idx >= self.vm_done:
            allowed = min(self.vm_issued - idx - 1, 63)   # the counter holds 63 at most
            self.emit(f"s_waitcnt vmcnt({allowed})")
            self.vm_done = self.vm_issued - allowed

    def vm_need(self, reg):
        self.vm_wait_index(self.vm_producer.get(reg, -1))


# Instructions of each class for issue-cost experiments (timing only: v176 is the column sums' temporary).
FILLERS = {
    "valu": "v_mov_b32 v176, v176",
    "salu": "s_mov_b32 s90, s69",
    "nop": "s_nop 0",
    "lds": "ds_read_b32 v176, %[a_rd0]",
    "vmem": "global_load_dword v176, %[a_off0], s[60:61]",
    "wait": "s_waitcnt lgkmcnt(15)",
}


class Item:
    """A piece of work to place behind some MFMA of a step: fn emits it, cost is its instruction
    count, earliest / latest the gaps (MFMA indices) it may go to, after an Item it follows.
    Measured on the bare loop (MFMAs and the barrier only): two vector instructions behind every
    MFMA cost half a cycle each, a third one four cycles; two scalar instructions cost nothing."""

    def __init__(self, fn, cost, earliest=0, latest=GAPS - 1, after=None, valu=0):
        self.fn, self.cost, self.earliest, self.latest, self.after = fn, cost, earliest, latest, after
        self.valu = valu     # how many of its instructions go to the vector unit (the matrix core's own port)
        self.gap = None


def gen(kind, accum, opts=None, gap=0):
    """kind: 'u8' (A unsigned bytes), 'i8', 'bf16'.
    accum: the Spec accumulates into C (its old contents are read).
    gap: k steps of the loop run between two steps that load C's old values (0: those steps follow
    one another).

    Tried instead of loading C at all: the epilogue's stores as atomic additions that return nothing
    (global_atomic_add / _f32, one per element, so the sums are the same).  Bit-exact, and the loop
    is the plain one, but the additions leave a wave at a twelfth of the stores' rate (95 K cycles
    for a wave's 256 instead of 8 K; bf16 8192^3 accumulating 980 us against 790)."""
    opts = opts or {}     # experiment switches; the shipped loops are generated with none
    # Experiment (atomic_c): an accumulating variant as the plain loop with the epilogue's stores
    # turned into atomic additions (see above); results are the same, the launch is slower.
    add_in_memory = bool(accum and opts.get("atomic_c"))
    if add_in_memory:
        accum, gap = False, 0
    unsigned = kind == "u8" and not opts.get("no_valu")
    is_float = kind == "bf16"
    mfma = "v_mfma_f32_16x16x32_bf16" if is_float else "v_mfma_i32_16x16x64_i8"
    tr = "ds_read_b64_tr_b16" if is_float else "ds_read_b64_tr_b8"
    e = Emitter()
    E = e.emit

    trace = bool(opts.get("trace"))
    # Experiment (c_load_nt): C's old values, read once, loaded with the non-temporal hint.
    c_load_hint = " nt" if opts.get("c_load_nt") else ""

    def stamp(pair):
        """Timing build only: the shader clock counter into s[pair:pair+1] (read after the next
        wait for lgkmcnt(0))."""
        if trace:
            E(f"s_memtime s[{pair}:{pair + 1}]")

    if trace:
        # s80..s95: s[80:81] start, s82 loop start, s83 end of the unrolled steps, s[84:89] a step's
        # three stamps, s90 scratch, s91 cycles waited for memory before barriers, s92 cycles in
        # barriers, s93 end of loop, s94 last stamp before a barrier, s95 real-time clock at start
        stamp(80)
        E("s_memrealtime s[86:87]")
        E("s_mov_b32 s91, 0")
        E("s_mov_b32 s92, 0")
        E("s_mov_b32 s88, 0")
        E("s_mov_b32 s94, 0")
        E("s_waitcnt lgkmcnt(0)")
        E("s_mov_b32 s95, s86")

    def advance(ptr_lo, ptr_hi, idx, step, tmp):
        """Next tile: one k step on; past the last tile the pointer stays (that tile is fetched
        again, into places nobody reads).  In one piece: the carry and the comparison's result
        live in SCC."""
        E(f"s_add_u32 {idx}, {idx}, 1")
        E(f"s_cmp_lt_u32 {idx}, %[nk]")
        E(f"s_cselect_b32 {tmp}, {step}, 0")
        E(f"s_add_u32 {ptr_lo}, {ptr_lo}, {tmp}")
        E(f"s_addc_u32 {ptr_hi}, {ptr_hi}, 0")

    def advance_a():
        advance("s60", "s61", "s67", "128", "s69")

    def advance_b():
        advance("s62", "s63", "s68", "%[bstep]", "s69")

    def load_a(p, i):
        if opts.get("no_stage") or step_no[0] > int(opts.get("stage_until", 1 << 30)):
            return
        e.vm(f"global_load_dwordx4 {areg(p, i)}, %[a_off{i}], s[60:61]", dst=areg(p, i))

    def flip_a(p, i, words):
        """u8 -> i8 (a - 128) of two of the chunk's four registers."""
        if opts.get("no_stage") or step_no[0] > int(opts.get("stage_until", 1 << 30)):
            return
        e.vm_need(areg(p, i))
        for w in words:
            E(f"v_xor_b32 {areg(p, i, w)}, s74, {areg(p, i, w)}")

    def store_a(p, i, stage, flip=True):
        if opts.get("no_stage") or step_no[0] > int(opts.get("stage_until", 1 << 30)):
            return
        e.vm_need(areg(p, i))
        if unsigned and flip:
            for w in range(4):
                E(f"v_xor_b32 {areg(p, i, w)}, s74, {areg(p, i, w)}")
        e.lds_write(f"ds_write_b128 %[a_wr], {areg(p, i)} offset:{stage * A_STAGE + i * 4096}")

    def set_m0(slot):
        E(f"s_add_u32 m0, %[dma_base], {slot * B_SLOT + 4096}")   # the immediate offsets run from -4096 to 3072
        E("s_nop 0")                                                # one wait state before M0 is read

    step_no = [0]        # steps written so far (the rolled loop counts as late)

    def dma_b(j):
        if opts.get("no_dma") or step_no[0] > int(opts.get("dma_until", 1 << 30)):
            return
        e.vm(f"global_load_lds_dwordx4 %[b_off{j}], s[62:63] offset:{j * 1024 - 4096}")

    def a_read(stage, slab, tm):
        if opts.get("no_reads"):
            return lambda: None
        return lambda: e.lds_read(af(tm), f"ds_read_b128 {af(tm)}, %[a_rd{slab}] offset:{stage * A_STAGE + tm * 2048}")

    def b_read(slot, slab, buf, tn, half):
        """The slot is known when the code is written (the loop body is six steps long: two A
        stages x three B slots), so the whole address is a register plus an immediate: %[b_rd] is
        the lane's address in slot 0 and reaches slot 1 with the 16-bit offset, v[160:167] the
        same in slot 2."""
        reg = bf(buf, tn, half)
        if opts.get("no_reads"):
            return lambda: None
        base = f"%[b_rd{tn}]" if slot < 2 else f"v{B_ADDR + tn}"
        off = (slot % 2) * B_SLOT + slab * SLAB_BYTES + half * HI_BYTES
        return lambda: e.lds_read(reg, f"{tr} {reg}, {base} offset:{off}")

    # ---- prologue -------------------------------------------------------------------------
    E("s_mov_b32 s74, 0x80808080")      # in a register: a literal would double the size of every xor
    E("s_mov_b64 s[60:61], %[abase]")
    E("s_mov_b64 s[62:63], %[bbase]")
    E("s_mov_b32 s67, 0")
    E("s_mov_b32 s68, 0")
    # A tiles 0 and 1 into the two register sets, B tiles 0 and 1 into slots 0 and 1
    for p in range(2):
        for i in range(8):
            load_a(p, i)
        advance_a()
    for slot in range(2):
        set_m0(slot)
        for j in range(8):
            dma_b(j)
        advance_b()
    for tn in range(TN):
        E(f"v_mov_b32 v{COL_SUM + tn}, 0")
    for i in range(8):
        store_a(0, i, 0)            # waits for A tile 0 only
    for i in range(8):
        load_a(0, i)                # A tile 2
    advance_a()
    e.vm_wait_index(e.vm_issued - 9)  # all but A tile 2: B tiles 0 and 1 have landed
    E("s_waitcnt lgkmcnt(0)")
    e.all_lds_done()
    E("s_barrier")
    for tn in range(TN):
        E(f"v_add_u32 v{B_ADDR + tn}, {2 * B_SLOT}, %[b_rd{tn}]")
    # What a step expects to find: slab 0's B operands in set 0 and its A operands but the last,
    # which every step reads behind its first MFMA.
    for tn in range(TN):
        b_read(0, 0, 0, tn, 0)()
        b_read(0, 0, 0, tn, 1)()
    for tm in range(TM - 1):
        a_read(0, 0, tm)()

    # ---- one k step ----------------------------------------------------------------------
    def step(kt, zero_first=False, extra=()):
        """kt: the step's position in the cycle of six (tile kt is in A stage kt % 2 and B slot
        kt % 3).  zero_first: the accumulators start from zero in this step.  extra: Items to place
        in the gaps besides the step's own."""
        cur, slot = kt % 2, kt % 3
        step_no[0] += 1
        p = cur ^ 1  # register set holding tile kt + 1 = LDS stage it goes to
        vm_before_step = e.vm_issued
        items = []

        def add(fn, cost, earliest, latest=GAPS - 1, after=None, valu=0):
            items.append(Item(fn, cost, earliest, latest, after, valu))
            return items[-1]

        # Operand reads: fixed places.  A's block row tm for the next slab right behind the last of
        # the eight MFMAs that use the current one (the last block row's lands in the next slab /
        # step); B's set for the next slab spread over the current one; what comes from the next
        # tile, behind the barrier.
        read_at = {}

        def at(g, r):
            read_at.setdefault(g, []).append(r)

        at(0, a_read(cur, 0, TM - 1))                       # this step's own: slab 0, last block row
        for tm in range(TM):
            at(8 * tm + 8, a_read(cur, 1, tm))              # slab 1 (tm = 7: behind slab 1's first MFMA)
        for tn in range(TN):                                 # slab 1's B operands into set 1
            at(2 + 6 * tn, b_read(slot, 1, 1, tn, 0))
            at(3 + 6 * tn, b_read(slot, 1, 1, tn, 1))
        for tn in range(TN):                                 # the next tile's slab 0 into set 0
            at(BARRIER_AT + 3 * tn, b_read((slot + 1) % 3, 0, 0, tn, 0))
            at(BARRIER_AT + 1 + 3 * tn, b_read((slot + 1) % 3, 0, 0, tn, 1))
        for tm in range(TM - 1):                             # and its A operands as theirs go dead
            at(max(MF + 8 * tm + 8, BARRIER_AT + 2 + 3 * tm), a_read(cur ^ 1, 0, tm))

        # The step's own work.  LDS writes must be out before the barrier.
        last_a = None
        for i, g in enumerate([1, 12, 23, 34, 45, 56, 67, 78]):
            if unsigned:   # in pieces that fit a gap
                last_a = add(lambda i=i: flip_a(p, i, (0, 1)), 2, g, BARRIER_AT - 4, after=last_a, valu=2)
                last_a = add(lambda i=i: flip_a(p, i, (2, 3)), 2, g, BARRIER_AT - 3, after=last_a, valu=2)
            last_a = add(lambda i=i: (store_a(p, i, cur ^ 1, flip=False), load_a(p, i)), 2, g, BARRIER_AT - 2, after=last_a)
        m0 = add(lambda: set_m0((slot + 2) % 3), 1, 0)   # tile kt + 2 goes where tile kt - 1 was
        last_b = m0
        for j, g in enumerate([6, 17, 28, 39, 50, 61, 72, 83]):
            last_b = add(lambda j=j: dma_b(j), 1, g, after=last_b)
        add(advance_a, 2, 84, after=last_a)          # scalar instructions: next to free
        add(advance_b, 2, 88, after=last_b)
        if unsigned:
            # Block columns 0 .. 3 of both slabs: the other wave row, whose block columns are the
            # same columns rotated by four, adds up the other half.
            for s in range(SLABS):
                for tn in range(TN // 2):
                    for w in range(4):
                        # after the first MFMA that waited for this operand, before the reads that overwrite it
                        add(lambda s=s, tn=tn, w=w: (e.need(bf(s, tn, w // 2)),
                                                      E(f"v_xor_b32 v{TMP0}, s74, {bf(s, tn, w=w)}"),
                                                      E(f"v_sad_u8 v{COL_SUM + tn}, v{TMP0}, 0, v{COL_SUM + tn}")),
                            2, MF * s + tn + 1, MF * s + MF - 1 if s == 0 else GAPS - 1, valu=2)
        for it in extra:
            items.append(it)
        # Place the items in the order given, each into the first gap from its earliest on with room
        # for it: GAP_SLOTS instructions behind an MFMA in all, VALU_SLOTS of them vector ones.
        slots, vslots = int(opts.get("slots", GAP_SLOTS)), int(opts.get("valu", VALU_SLOTS))
        room = [slots - len(read_at.get(g, [])) for g in range(GAPS)]
        vroom = [vslots] * GAPS
        room[BARRIER_AT - 1] -= 3              # the waits and the barrier
        placed = [[] for _ in range(GAPS)]
        for it in items:
            first = max(it.earliest, it.after.gap if it.after is not None else 0)
            last_gap = max(first, it.latest)
            g = first
            while g <= last_gap and (room[g] < it.cost or vroom[g] < it.valu):
                g += 1
            if g > last_gap:               # no gap has room: the emptiest one allowed
                g = max(range(first, last_gap + 1), key=lambda x: (min(room[x] - it.cost, vroom[x] - it.valu), -x))
            room[g] -= it.cost
            vroom[g] -= it.valu
            it.gap = g
            placed[g].append(it)
        if os.environ.get("WIDE_SHOW_GAPS"):
            sys.stderr.write("gaps " + " ".join(str(slots - r) for r in room) + "\n")

        def sync():
            # everything requested before this step has landed (B of tile kt + 1, A of tile kt + 2);
            # this wave's LDS writes are done and the operands of the rest of the step are in
            stamp(84)
            e.vm_wait_index(vm_before_step - 1)
            stamp(86)
            E("s_waitcnt lgkmcnt(0)")
            e.all_lds_done()
            if trace:
                E("s_sub_u32 s90, s88, s94")      # the previous step's barrier
                E("s_add_u32 s92, s92, s90")
                E("s_sub_u32 s90, s86, s84")      # this step's wait for memory
                E("s_add_u32 s91, s91, s90")
                E("s_mov_b32 s94, s86")
            E("s_barrier")
            stamp(88)

        n = 0
        for s in range(SLABS):
            for tm in range(TM):
                for tn in range(TN):
                    if n == BARRIER_AT:
                        sync()
                    e.need(af(tm), bf(s, tn, 0), bf(s, tn, 1))
                    src_c = "0" if (zero_first and s == 0) else acc(tm, tn)
                    E(f"{mfma} {acc(tm, tn)}, {af(tm)}, {bf(s, tn)}, {src_c}")
                    for r in read_at.get(n, []):
                        r()
                    for it in placed[n]:
                        it.fn()
                    for kind_, text in FILLERS.items():   # timing experiments: fill_<kind>=<per step>
                        per_step = int(opts.get("fill_" + kind_, 0))
                        if per_step and (n * per_step) // GAPS != ((n + 1) * per_step) // GAPS:
                            for _ in range(max(1, per_step // GAPS)):
                                E(text)
                    n += 1

    # ---- C: register q = 0..255: block q / 4 (tm = block / 8, tn = block % 8), register i = q % 4,
    # which holds row 4 * (lane / 16) + i of the block (%[c_lo i] / %[c_hi i]) and column lane % 16.
    ptr_tm = [None]

    def c_ptr(tm):
        """s[72:73] = the wave's corner of C + tm * 16 rows, if it is not that already."""
        if ptr_tm[0] == tm:
            return
        ptr_tm[0] = tm
        E("s_mov_b64 s[72:73], %[cbase]")
        if tm:
            E(f"s_mul_i32 s78, %[ldc16], {tm}")
            E(f"s_mul_hi_u32 s79, %[ldc16], {tm}")
            E("s_add_u32 s72, s72, s78")
            E("s_addc_u32 s73, s73, s79")

    def c_addr(tn, i):
        """The lane's byte offset of row i of a block in block column tn, less tn * 64: one set of
        registers for block columns 0 .. 3 and one for 4 .. 7 (they differ for a wave row whose
        block columns are rotated)."""
        return f"%[c_lo{i}]" if tn < TN // 2 else f"%[c_hi{i}]"

    def where(q):
        block = q // 4
        return block // TN, block % TN, q % 4

    def c_ops(j, spaced=False):
        """The j-th of the steps that carry C's old values (spaced: with steps of the loop between
        them, so that what one of them loaded has long landed when the next one adds it, and the
        additions go first in the step, the loads behind them with the rest of it to land in).
        Step j of an accumulating Spec: the old values of block row j - 1 (loaded a step ago) join
        their accumulators, and behind each addition the same register is loaded with block row
        j's.  An addition is three instructions (the accumulator out, the sum, back in); it keeps
        clear of the block's own MFMAs (8 (j - 1) + tn in either slab): an MFMA's result is read
        four MFMAs after it at the earliest, and a register written for the block's next MFMA has
        other instructions between the write and that MFMA.  Spread over the whole step, one
        every four MFMAs, its pieces behind three MFMAs in a row (three temporaries take turns)."""
        out, chain = [], []
        for r in range(32):
            tn, i = r // 4, r % 4
            reg = f"v{OLD_C + r}"
            g = 2 * r + 1 if spaced else 4 * r + 1
            add_item = None
            if 1 <= j <= C_STEPS:
                q = 4 * (TN * (j - 1) + tn) + i
                n0 = TN * (j - 1) + tn
                zones = [(n0 - 2, n0 + 3), (MF + n0 - 2, MF + n0 + 3)]
                for lo, hi in zones:               # three gaps in a row outside both zones
                    if lo - 2 <= g <= hi:
                        g = hi + 1
                if g + 2 > GAPS - 1:                  # the last block row's second zone reaches the step's end
                    g = zones[1][0] - 6
                latest = min([lo - 1 for lo, hi in zones if lo > g] + [GAPS - 1])

                tmp = f"v{C_TMP[r % len(C_TMP)]}"
                read = Item(lambda q=q, tmp=tmp: E(f"v_accvgpr_read_b32 {tmp}, a{q}"), 1, g, latest - 2,
                            after=chain[-len(C_TMP)] if len(chain) >= len(C_TMP) else None, valu=1)

                def add_old(tmp=tmp, reg=reg):
                    # its own wait: the loads of a step are 32 KiB in flight per compute unit, which at
                    # HBM's latency is all the chip can have of C, so the last of them arrive late
                    if not spaced:
                        e.vm_need(reg)
                    E(f"v_add_f32 {tmp}, {tmp}, {reg}" if is_float else f"v_add_u32 {tmp}, {tmp}, {reg}")
                add_item = Item(add_old, 1, g + 1, latest - 1, after=read, valu=1)
                write = Item(lambda q=q, tmp=tmp: E(f"v_accvgpr_write_b32 a{q}, {tmp}"), 1, g + 2, latest, after=add_item, valu=1)
                chain.append(write)     # the temporary is free again behind this
                out += [read, add_item, write]
            if j < C_STEPS:
                def ld(tn=tn, i=i, reg=reg):
                    c_ptr(j)
                    e.vm(f"global_load_dword {reg}, {c_addr(tn, i)}, s[72:73] offset:{tn * 64}{c_load_hint}", dst=reg)
                out.append(Item(ld, 1, g, GAPS - 1, after=add_item))
        return out

    def loop(first):
        """Six steps, left after any two of them when the tiles run out; entered at position
        `first` (the number of unrolled steps before it, modulo six)."""
        if first % 6:
            E(f"s_branch 1{first % 6}f")
        for pos in (0, 2, 4):
            E(f"1{pos}:")
            step(pos)
            step(pos + 1)
            E("s_sub_u32 s64, s64, 2")
            E("s_cmp_lg_u32 s64, 0")
            E("s_cbranch_scc1 10b" if pos == 4 else "s_cbranch_scc0 2f")

    def steady_state(kt):
        """The emitter's bookkeeping (which load or LDS read fills which register, what is known to
        have completed) as two ordinary steps before step kt leave it: code that is jumped to is
        written from this state, whatever precedes it in the text."""
        n0, saved = len(e.lines), step_no[0]
        step((kt - 2) % 6)
        step((kt - 1) % 6)
        del e.lines[n0:]
        step_no[0] = saved

    def loop_any(returns):
        """The loop of six steps as a subroutine: entered at any step (label 1<position>) with the
        number of steps to run in s64, left after any step; s75 says where to: one of the steps
        that carry C's old values (label 4<j>), or, zero, the epilogue."""
        steady_state(0)
        for pos in range(6):
            E(f"1{pos}:")
            step(pos)
            E("s_sub_u32 s64, s64, 1")
            E("s_cmp_eq_u32 s64, 0")
            E("s_cbranch_scc1 20f" if pos < 5 else "s_cbranch_scc0 10b")
        E("20:")
        for j in returns:
            E(f"s_cmp_eq_u32 s75, {j}")
            E(f"s_cbranch_scc1 4{j}b")

    # ---- the k loop ---------------------------------------------------------------------------------
    if trace:
        stamp(82)
        E("s_waitcnt lgkmcnt(0)")
        e.all_lds_done()
    early = int(opts.get("early_stores", 0))   # timing experiment (C2's 32 steps only): see below
    landing = min(int(opts.get("landing", 0)), max(gap - 1, 0))
    if accum and gap > 0:
        # C's old values at steps 0, gap + 1, 2 (gap + 1), ...: between them the loop runs `gap` steps.
        kt = 0
        for j in range(C_STEPS + 1):
            if j > 0:
                E(f"4{j}:")
                steady_state(kt)
            step(kt % 6, zero_first=(j == 0), extra=[] if opts.get("no_cops") else c_ops(j, spaced=True))
            kt += 1
            if j < C_STEPS:
                # Experiment (landing=N): N plain steps written here, behind the loads of C, so that
                # their waits count those loads exactly; the loop's waits are written for a queue
                # without them.  Measured the same as without: vector memory returns in order.
                for _ in range(landing):
                    step(kt % 6)
                    kt += 1
                E(f"s_mov_b32 s64, {gap - landing}")
                E(f"s_mov_b32 s75, {j + 1}")
                E(f"s_branch 1{kt % 6}f")
                kt += gap - landing
        if trace:
            stamp(84)
            E("s_waitcnt lgkmcnt(0)")
            e.all_lds_done()
            E("s_mov_b32 s83, s84")
        E("s_mov_b32 s75, 0")
        E(f"s_sub_u32 s64, %[nk], {kt}")
        E("s_cmp_eq_u32 s64, 0")
        E("s_cbranch_scc1 2f")
        E(f"s_branch 1{kt % 6}f")
        loop_any(range(1, C_STEPS + 1))
    else:
        unrolled = C_STEPS + 2 if accum else 2
        for j in range(unrolled):
            extra = c_ops(j) if accum and not opts.get("no_cops") else []
            step(j % 6, zero_first=(j == 0), extra=extra)
        if trace:
            stamp(84)
            E("s_waitcnt lgkmcnt(0)")
            e.all_lds_done()
            E("s_mov_b32 s83, s84")
        E(f"s_sub_u32 s64, %[nk], {unrolled + (2 if early else 0)}")
        E("s_cmp_eq_u32 s64, 0")
        E("s_cbranch_scc1 2f")
        loop(unrolled)
    E("2:")
    if early:
        # An upper bound for what any reordering of the last step could hide of the epilogue: the
        # first `early` stores of C go out spread over the last step's MFMAs, whether or not their
        # accumulators are final (they are not: the results are wrong).
        def early_store(q):
            tm, tn, i = where(q)
            c_ptr(tm)
            t = f"v{OLD_C + q % 32}"
            E(f"v_accvgpr_read_b32 {t}, a{q}")
            if unsigned:
                E(f"v_add_u32 {t}, {t}, v{COL_SUM + tn}")
            E(f"global_store_dword {c_addr(tn, i)}, {t}, s[72:73] offset:{tn * 64}")
        step(30 % 6)
        step(31 % 6, extra=[Item(lambda q=q: early_store(q), 3, (q * GAPS) // early, GAPS - 1, valu=2) for q in range(early)])
    # nothing may land in LDS once the epilogue reuses it; the last MFMAs must have written the
    # accumulators before they are read
    E("s_waitcnt vmcnt(0) lgkmcnt(0)")
    if trace:
        E("s_sub_u32 s90, s88, s94")
        E("s_add_u32 s92, s92, s90")
        stamp(84)
        E("s_waitcnt lgkmcnt(0)")
        E("s_mov_b32 s93, s84")
    E("s_barrier")

    # ---- epilogue -----------------------------------------------------------------------------------
    if unsigned:
        # Column sums: a wave holds, per lane group, the sums of b + 128 over a quarter of K for its
        # block columns 0 .. 3; the four groups' partials of every column meet in LDS, where each
        # wave finds those of all eight of its block columns (its own and the other wave row's).
        for tn in range(TN // 2):
            E(f"v_subrev_u32 v{COL_SUM + tn}, %[k32], v{COL_SUM + tn}")
            e.lds_write(f"ds_write_b32 %[part_wr], v{COL_SUM + tn} offset:{tn * 64}")
        E("s_waitcnt lgkmcnt(0)")
        e.all_lds_done()
        E("s_barrier")
        for tn in range(TN):
            for w in range(4):
                reg = f"v{64 + 4 * tn + w}"
                addr = "%[part_rd_lo]" if tn < TN // 2 else "%[part_rd_hi]"
                e.lds_read(reg, f"ds_read_b32 {reg}, {addr} offset:{w * 1024 + tn * 64}")
        for tn in range(TN):
            regs = [f"v{64 + 4 * tn + w}" for w in range(4)]
            e.need(*regs)
            E(f"v_add3_u32 v{COL_SUM + tn}, {regs[0]}, {regs[1]}, {regs[2]}")
            E(f"v_add_lshl_u32 v{COL_SUM + tn}, v{COL_SUM + tn}, {regs[3]}, 7")
    else:
        E("s_nop 15")
        E("s_nop 15")
    st_flags = opts.get("st_flags", "")
    if opts.get("no_epilogue"):
        pass
    else:
        for q in range(early, 256):
            tm, tn, i = where(q)
            c_ptr(tm)
            out = "global_store_dword"
            if add_in_memory:
                out = "global_atomic_add_f32" if is_float else "global_atomic_add"
            if not unsigned:
                E(f"{out} {c_addr(tn, i)}, a{q}, s[72:73] offset:{tn * 64}{st_flags}")
            else:
                t = f"v{16 + q % 32}"
                E(f"v_accvgpr_read_b32 {t}, a{q}")
                E(f"v_add_u32 {t}, {t}, v{COL_SUM + tn}")
                E(f"{out} {c_addr(tn, i)}, {t}, s[72:73] offset:{tn * 64}{st_flags}")
    if trace:
        # The stamps replace the first rows of the wave's block of C (a timing build: its results are
        # not looked at): value j at row j % 4, columns 16 * (j / 4) .. + 15 of the block.
        stamp(84)
        E("s_waitcnt vmcnt(0) lgkmcnt(0)")
        stamp(86)
        E("s_memrealtime s[88:89]")
        E("s_getreg_b32 s90, hwreg(HW_REG_HW_ID)")
        E("s_getreg_b32 s81, hwreg(HW_REG_XCC_ID)")
        E("s_waitcnt lgkmcnt(0)")
        ptr_tm[0] = None
        c_ptr(0)
        for j, sreg in enumerate(["s80", "s82", "s83", "s93", "s84", "s86", "s95", "s88", "s91", "s92", "s90",
                                   "s81"]):
            E(f"v_mov_b32 v{TMP0}, {sreg}")
            E(f"global_store_dword %[c_lo{j % 4}], v{TMP0}, s[72:73] offset:{(j // 4) * 64}")
            E("s_nop 1")
    return e.lines


MIN_STEPS = C_STEPS + 4   # k steps a problem needs: the steps that carry C's old values, then the loop


SPACED_GAPS = (2, 11)    # loop steps between the steps that carry C's old values, for K long enough


def spaced_min_steps(gap):
    """k steps a problem needs for the variant with `gap` loop steps between C's steps."""
    return C_STEPS * (gap + 1) + 2


def variants():
    for kind in ("u8", "i8", "bf16"):
        yield f"GEMM_WIDE_{kind.upper()}", kind, False, 0
        yield f"GEMM_WIDE_{kind.upper()}_ACC", kind, True, 0
        for gap in SPACED_GAPS:
            yield f"GEMM_WIDE_{kind.upper()}_ACC_G{gap}", kind, True, gap


def main():
    out_path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "gemm_wide_gfx950.inc")
    if len(sys.argv) > 1:
        out_path = sys.argv[1]
    # Experiment switches (timing builds with one ingredient left out, the cycle-stamp build, and the
    # two alternatives landing=N and atomic_c, whose results stay right): a comma-separated list in
    # MRL_WIDE_OPTS.  The library is built with none.
    opts = {o: True for o in os.environ.get("MRL_WIDE_OPTS", "").split(",") if o}
    for o in list(opts):
        if "=" in o:                  # fill_valu=32 and the like
            del opts[o]
            opts[o.split("=")[0]] = o.split("=")[1]
        elif o.startswith("st_"):       # st_nt, st_sc1, st_sc0_sc1: cache policy bits on the stores of C
            opts["st_flags"] = " " + " ".join(o.split("_")[1:])
    parts = ["// Generated by gen_gemm_wide.py -- do not edit; the generator documents the schedule.\n",
             f"#define GEMM_WIDE_MIN_STEPS {MIN_STEPS}\n"]
    for gap in SPACED_GAPS:
        parts.append(f"#define GEMM_WIDE_G{gap}_MIN_STEPS {spaced_min_steps(gap)}\n")
    for name, kind, accum, gap in variants():
        lines = gen(kind, accum, opts, gap)
        body = " \\\n".join('  "' + l + '\\n"' for l in lines)
        parts.append(f"#define {name} \\\n{body}\n")
    with open(out_path, "w") as f:
        f.write("\n".join(parts))
    print(f"wrote {out_path}")


if __name__ == "__main__":
    main()
