#!/usr/bin/env python3
"""Writes gemm_loop_gfx950.inc: the k loop of the 256 x 256 Matmul tile as gfx950 assembly.

The loop is the part of the kernel where the order of instructions decides the speed: MFMAs of two
waves per SIMD have to issue back to back while LDS reads, LDS writes, global loads and
direct-to-LDS loads for later tiles are slotted between them, each waiting exactly as long as its
own data needs.  A compiler schedules such a loop from its own cost model (and adds a full
memory wait before every barrier); here the order and every s_waitcnt are written down.

One k step of a wave (tile kt; 8 waves as 2 x 4, each 128 x 64 outputs = 4 x 2 MFMA blocks):
  * four 32-byte slabs of K, 8 MFMAs each; the operands of slab s+1 are read from LDS between
    the MFMAs of slab s (8 reads: 4 ds_read_b128 of A, 4 transposing ds_read_b64_tr of B);
  * A of tile kt+1 goes from a register set to its LDS stage (xor 0x80 on the way for a u8
    operand) and the set is refilled with tile kt+3 from global memory: two register sets, two
    LDS stages, so a global load has two k steps to land;
  * B of tile kt+2 is requested straight into the third of three LDS slots
    (global_load_lds_dwordx4), which costs neither registers nor LDS write instructions;
  * one barrier, before the MFMAs of the last slab, preceded by the only vmcnt wait of the step:
    everything requested before this step has landed.
Past the last tile the source pointers stop advancing: the last tile is fetched again into
places nobody reads, which keeps the loop free of branches.

Register map (fixed, named in the clobber list of the asm statement):
  v[0:127]    accumulators, block (tm, tn) at 16 * (2 * tm + tn)
  v[128:159]  A staging, set p chunk i at 128 + 16 * p + 4 * i
  v[160:191]  A operands, buffer b block tm at 160 + 16 * b + 4 * tm
  v[192:207]  B operands, buffer b block tn at 192 + 8 * b + 4 * tn
  v[208:209]  LDS address of the lane's B operand in the slot being read
  v[210:211]  column sums of B (u8 correction), one per tn
  s[60:61] A tile pointer   s[62:63] B tile pointer   s64 kt   s65, s66, s69, s70 scratch
  s67 / s68 index of the next A / B tile to fetch   s71 byte offset of tile kt's B slot
"""
import os
import sys

A_STAGE = 32768
B_SLOT = 32768
B_BASE = 2 * A_STAGE
SLAB_BYTES = 8192  # one 32-byte slab of K in a B slot: K_SLAB rows x row bytes, 8192 for i8 and bf16
HI_BYTES = 2048    # second transposing read of a slab: K_PER_READ rows further


def acc(tm, tn):
    b = 16 * (2 * tm + tn)
    return f"v[{b}:{b + 15}]"


def areg(p, i, w=None):
    b = 128 + 16 * p + 4 * i
    return f"v[{b}:{b + 3}]" if w is None else f"v{b + w}"


def af(buf, tm):
    b = 160 + 16 * buf + 4 * tm
    return f"v[{b}:{b + 3}]"


def bf(buf, tn, half=None, w=None):
    b = 192 + 8 * buf + 4 * tn
    if w is not None:
        return f"v{b + w}"
    if half is None:
        return f"v[{b}:{b + 3}]"
    return f"v[{b + 2 * half}:{b + 2 * half + 1}]"


class Emitter:
    """Collects instructions and derives each s_waitcnt lgkmcnt from the order of LDS operations."""

    def __init__(self):
        self.lines = []
        self.lds_issued = 0     # LDS operations issued so far
        self.lds_done = 0       # operations with index < lds_done are known to be complete
        self.producer = {}      # register tuple -> index of the LDS read that fills it

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
            outstanding_allowed = self.lds_issued - idx - 1
            self.emit(f"s_waitcnt lgkmcnt({min(outstanding_allowed, 15)})")
            self.lds_done = idx + 1 if outstanding_allowed <= 15 else self.lds_issued - 15

    def all_lds_done(self):
        self.lds_done = self.lds_issued


def gen(kind, wm, opts=None):
    """kind: 'u8' (A unsigned bytes), 'i8', 'bf16'.  wm: the wave row (which slabs' column sums it adds).
    opts: experiment switches (lab use); the shipped loops are generated with none."""
    opts = opts or {}
    unsigned = kind == "u8"
    mfma = "v_mfma_f32_32x32x16_bf16" if kind == "bf16" else "v_mfma_i32_32x32x32_i8"
    tr = "ds_read_b64_tr_b16" if kind == "bf16" else "ds_read_b64_tr_b8"
    e = Emitter()
    E = e.emit

    def advance(ptr_lo, ptr_hi, idx, step):
        E(f"s_add_u32 {idx}, {idx}, 1")
        E(f"s_cmp_lt_u32 {idx}, %[nk]")
        E(f"s_cselect_b32 s69, {step}, 0")
        E(f"s_add_u32 {ptr_lo}, {ptr_lo}, s69")
        E(f"s_addc_u32 {ptr_hi}, {ptr_hi}, 0")

    def load_a(p, i):
        E(f"global_load_dwordx4 {areg(p, i)}, %[a_off{i}], s[60:61]")

    def dma_b(slot_base_sgpr, i):
        # one wait state between the write of M0 and the direct-to-LDS load that reads it
        E(f"s_add_u32 m0, {slot_base_sgpr}, {i * 1024}")
        E("s_nop 0")
        E(f"global_load_lds_dwordx4 %[b_off{i}], s[62:63]")

    def store_a(p, i, stage):
        if unsigned:
            for w in range(4):
                E(f"v_xor_b32 {areg(p, i, w)}, 0x80808080, {areg(p, i, w)}")
        e.lds_write(f"ds_write_b128 %[a_wr], {areg(p, i)} offset:{stage * A_STAGE + i * 8192}")

    def reads(stage, slab, buf):
        """The 8 operand reads of one slab in the order the MFMAs want them, as closures."""
        def a_read(tm):
            return lambda: e.lds_read(af(buf, tm), f"ds_read_b128 {af(buf, tm)}, %[a_rd{slab}] offset:{stage * A_STAGE + tm * 4096}")

        def b_read(tn, half):
            reg = bf(buf, tn, half)
            return lambda: e.lds_read(reg, f"{tr} {reg}, v{208 + tn} offset:{slab * SLAB_BYTES + half * HI_BYTES}")
        return [[a_read(0)], [b_read(0, 0), b_read(0, 1)], [b_read(1, 0), b_read(1, 1)], [a_read(1)], [a_read(2)], [a_read(3)], [], []]

    def set_b_read_base(slot_off_sgpr):
        for tn in range(2):
            E(f"v_add_u32 v{208 + tn}, {slot_off_sgpr}, %[b_rd{tn}]")

    # ---- prologue -------------------------------------------------------------------------
    E("s_mov_b64 s[60:61], %[abase]")
    E("s_mov_b64 s[62:63], %[bbase]")
    E("s_mov_b32 s67, 0")
    E("s_mov_b32 s68, 0")
    E("s_mov_b32 s71, 0")
    E("s_mov_b32 s64, 0")
    for p in range(2):
        for i in range(4):
            load_a(p, i)
        advance("s60", "s61", "s67", "128")
    for slot in range(2):
        E(f"s_add_u32 s66, %[dma_base], {slot * B_SLOT}")
        for i in range(4):
            dma_b("s66", i)
        advance("s62", "s63", "s68", "%[bstep]")
    for r in range(128):
        E(f"v_mov_b32 v{r}, 0")
    E("v_mov_b32 v210, 0")
    E("v_mov_b32 v211, 0")
    E("s_waitcnt vmcnt(12)")           # A tile 0 is in
    for i in range(4):
        store_a(0, i, 0)
    for i in range(4):
        load_a(0, i)
    advance("s60", "s61", "s67", "128")
    E("s_waitcnt vmcnt(4) lgkmcnt(0)")  # all but A tile 2: B tiles 0 and 1 have landed
    e.all_lds_done()
    E("s_barrier")
    E(f"s_mov_b32 s65, {B_BASE}")
    set_b_read_base("s65")
    for group in reads(0, 0, 0):
        for r in group:
            r()

    # ---- one k step ----------------------------------------------------------------------
    def step(cur):
        p = cur ^ 1  # register set holding tile kt+1 = LDS stage it goes to
        # slot of tile kt+1 (for the reads after the barrier) and of tile kt+2 (direct-to-LDS target)
        E("s_add_u32 s69, s71, 0x8000")
        E("s_cmp_eq_u32 s69, 0x18000")
        E("s_cselect_b32 s69, 0, s69")
        E("s_sub_u32 s70, s71, 0x8000")
        E("s_cmp_eq_u32 s71, 0")
        E("s_cselect_b32 s70, 0x10000, s70")
        E("s_add_u32 s66, %[dma_base], s70")
        E(f"s_add_u32 s65, s69, {B_BASE}")
        E("s_mov_b32 s71, s69")
        for s in range(4):
            buf, nb = s & 1, (s & 1) ^ 1
            others = []
            chunks = opts.get("chunks", [[0], [1], [2, 3], []])[s]
            for i in chunks:
                others.append(lambda i=i: store_a(p, i, cur ^ 1))
                others.append(lambda i=i: load_a(p, i))
                others.append(lambda i=i: dma_b("s66", i))
            if s == 2:
                others.append(lambda: advance("s60", "s61", "s67", "128"))
                others.append(lambda: advance("s62", "s63", "s68", "%[bstep]"))
            if unsigned and s % 2 == wm and not opts.get("no_dot4"):
                for tn in range(2):
                    for w in range(4):
                        others.append(lambda tn=tn, w=w: (e.need(bf(buf, tn, w // 2)),
                                                          E(f"v_dot4c_i32_i8 v{210 + tn}, 0x1010101, {bf(buf, tn, w=w)}")))
            def sync():
                # everything requested before this step has landed (B of tile kt+1, A of tile kt+2);
                # this wave's LDS writes are done and the operands of this slab are in
                E("s_waitcnt vmcnt(8) lgkmcnt(0)")
                e.all_lds_done()
                if opts.get("trace"):
                    E("s_memtime s[72:73]")
                E("s_barrier")
                if opts.get("trace"):
                    E("s_memtime s[74:75]")
                    E("s_waitcnt lgkmcnt(0)")
                    E("s_sub_u32 s76, s74, s72")
                    E("s_add_u32 s77, s77, s76")
                set_b_read_base("s65")
            before_sync = opts.get("mfma_before_barrier", 0) if s == 3 else 0
            if s < 3:
                rd = reads(cur, s + 1, nb)
            else:
                if before_sync == 0:
                    sync()
                rd = reads(cur ^ 1, 0, nb)
                rd = [[] for _ in range(before_sync)] + [g for g in rd if g] + [[] for _ in range(8)]
                rd = rd[:8] if len([g for g in rd[8:] if g]) == 0 else None
            # spread the other work over the gaps behind the MFMAs, in order
            gaps = [[] for _ in range(8)]
            first = 1 if (unsigned and s % 2 == wm and not opts.get("no_dot4")) else 0  # dot4 needs both halves of B: not before MFMA 1
            for j, item in enumerate(others):
                gaps[min(7, first + j * (8 - first) // max(1, len(others)))].append(item)
            n = 0
            for tm in range(4):
                for tn in range(2):
                    e.need(af(buf, tm), bf(buf, tn, 0), bf(buf, tn, 1))
                    if opts.get("prio") and n == 0:
                        E("s_setprio 1")
                    E(f"{mfma} {acc(tm, tn)}, {af(buf, tm)}, {bf(buf, tn)}, {acc(tm, tn)}")
                    if opts.get("prio") and n == 7:
                        E("s_setprio 0")
                    if s == 3 and before_sync and n == before_sync - 1:
                        sync()
                    for r in rd[n]:
                        r()
                    for item in gaps[n]:
                        item()
                    n += 1

    if opts.get("trace"):
        E("s_mov_b32 s77, 0")
        E("s_memtime s[78:79]")
    E("1:")
    step(0)
    step(1)
    E("s_add_u32 s64, s64, 2")
    E("s_cmp_lt_u32 s64, %[nk]")
    E("s_cbranch_scc1 1b")
    # nothing may land in LDS once the epilogue reuses it; the last MFMAs must have written the
    # accumulators before compiler-scheduled code reads them
    E("s_waitcnt vmcnt(0) lgkmcnt(0)")
    if opts.get("trace"):
        E("s_memtime s[80:81]")
        E("s_waitcnt lgkmcnt(0)")
        E("s_sub_u32 s76, s80, s78")
        E("v_mov_b32 v208, s77")
        E("v_mov_b32 v209, s76")
    E("s_barrier")
    E("s_nop 15")
    E("s_nop 15")
    return e.lines


def main():
    out_path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "gemm_loop_gfx950.inc")
    if len(sys.argv) > 1:
        out_path = sys.argv[1]
    parts = ["// Generated by gen_gemm_loop.py -- do not edit; the generator documents the schedule.\n"]
    for kind, wms in (("u8", (0, 1)), ("i8", (0,)), ("bf16", (0,))):
        for wm in wms:
            name = f"GEMM_LOOP_{kind.upper()}_{wm}" if kind == "u8" else f"GEMM_LOOP_{kind.upper()}"
            lines = gen(kind, wm)
            body = " \\\n".join('  "' + l + '\\n"' for l in lines)
            parts.append(f"#define {name} \\\n{body}\n")
    with open(out_path, "w") as f:
        f.write("\n".join(parts))
    print(f"wrote {out_path}")


if __name__ == "__main__":
    main()
