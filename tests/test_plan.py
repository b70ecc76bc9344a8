"""The backend as a search target (morello/src/target/mod.rs:37-117): the target description, the
plan of a Spec (which kernels a run launches: Kernel::applies_to_logical_spec) and the cost model
over it (Kernel::main_cost / memory_allocated).  Planning is the run's own dispatch code with the
launches recorded instead of made, so everything except the last two tests runs without a GPU."""
import numpy as np
import pytest

import morello_amd as M
from morello_amd import synth

KT = M.layout(0, 2, 1)


def c1(): return M.MatmulAccum([1, 64, 64, 64], (M.f32, M.f32, M.f32))
def c2(): return M.MatmulAccum([1, 4096, 4096, 4096], (M.u8, M.i8, M.i32))
def c3(): return M.MatmulAccum([1, 8192, 8192, 8192], (M.bf16, M.bf16, M.f32))
def c4(): return M.Conv([32, 64, 64, 54, 54, 3, 3], (M.u8, M.i8, M.i32))
def c5(): return M.ComposeMSM(16, 2048, 128, 2048, 128, layouts=[None, None, KT, None])


def test_target_description():
    """The answers an `impl Target` forwards: four memories fastest first (MEMORY_COUNT,
    target/mod.rs:30-33), registers counted and not parallel-tiled, HBM the level a grid tiles
    (Memory trait, target/mod.rs:80-95)."""
    assert M.Target.target_id() == "Gfx950"
    assert M.Target.line_size() == 128
    assert M.Target.processors() == 256
    mems = M.Target.memories()
    assert [m.name for m in mems] == ["ACC", "VGPR", "LDS", "HBM"]
    assert [m.counts_registers for m in mems] == [True, True, False, False]
    assert [m.can_parallel_tile for m in mems] == [False, False, False, True]
    assert mems[1].vector_bytes == [4, 8, 16] and mems[0].has_layout is False
    assert mems[2].limit == 160 * 1024 and mems[3].limit == 288 << 30
    assert [m.cache_hit_cost for m in mems] == sorted(m.cache_hit_cost for m in mems)
    kernels = M.Target.kernels()
    assert len(kernels) == len(set(kernels)) and {"k_gemm", "k_conv_i8", "k_attn", "k_softmax_regs"} <= set(kernels)


def test_target_memories_and_layouts_for_search():
    """Target::default_memory, possible_destination_memories, all_layouts_for_shape
    (target/mod.rs:54-67), the last built as target/cpu.rs:317-398 builds it."""
    T = M.Target
    assert T.default_memory().name == "HBM"
    assert T.possible_destination_memories("HBM") == ["HBM", "LDS", "VGPR"]
    assert T.possible_destination_memories("LDS") == ["LDS", "VGPR"]
    assert T.possible_destination_memories("ACC") == ["ACC"]
    sq = [64, 64]
    layouts = T.all_layouts_for_shape(sq, M.f32)
    reprs = [repr(l) for l in layouts]
    assert layouts[0] == M.row_major(sq) and layouts[1] == M.col_major(sq) and len(set(reprs)) == len(reprs)
    # f32: Packed 2 and 4 (8 / 4 and 16 / 4 bytes), never of the innermost dim; OddEven 2, 4, 8, any dim.
    assert "layout![0, 1, 0 p(4)]" in reprs and "layout![1, 0, 1 p(2)]" in reprs
    assert not any(r.startswith("layout![0, 1, 1 p(") or r.startswith("layout![1, 0, 0 p(") for r in reprs)
    assert {r for r in reprs if "oe" in r and r.startswith("layout![0, 1,")} == {
        f"layout![0, 1, {d} oe({n})]" for d in (0, 1) for n in (2, 4, 8)}
    assert len(layouts) == 2 + 2 * 2 + 2 * 6
    # bytes pack up to 16; rank 3 adds the k-fastest order, rank 4 channels-last.
    assert "layout![0, 1, 2, 1 p(16)]" in [repr(l) for l in T.all_layouts_for_shape([4, 64, 32], M.u8)]
    assert T.all_layouts_for_shape([4, 64, 32], M.bf16)[1] == M.layout(0, 2, 1)
    assert T.all_layouts_for_shape([2, 16, 8, 8], M.u8)[1] == M.nhwc([2, 16, 8, 8])
    # Sizes that do not divide the dim are left out; every layout listed applies and can be moved to.
    for shape, dt in (([6, 10], M.f32), ([4, 64, 32], M.bf16), ([2, 16, 8, 8], M.u8), ([1, 1], M.f32), ([7], M.i32)):
        for l in T.all_layouts_for_shape(shape, dt):
            assert l.applies_to_shape(shape), (shape, l)
            assert M.Move(shape, (dt, dt), layouts=[M.row_major(shape), l]).plan().steps
    assert [repr(l) for l in T.all_layouts_for_shape([6, 10], M.f32) if "p(4)" in repr(l)] == []


def test_benchmark_configurations_pick_their_kernels():
    p = c1().plan()
    assert p.kernels == ["k_gemm"] and "T = F32" in p.steps[0].kernel and "Tile<64, 64, 128" in p.steps[0].kernel
    p = c2().plan()
    assert p.kernels == ["k_gemm_wide"] and p.scratch_bytes == 0
    assert "T = I8, A_UNSIGNED = true" in p.steps[0].kernel
    assert p.steps[0].grid == (256, 1, 1) and p.steps[0].block == (256, 1, 1) and p.steps[0].unit == "mfma_i8"
    assert p.steps[0].ops == 2 * 4096 ** 3 and p.steps[0].bytes == 2 * 4096 ** 2 + 2 * 4 * 4096 ** 2  # accumulating: C read too
    p = c3().plan()
    assert p.kernels == ["k_gemm_wide"] and "T = BF16" in p.steps[0].kernel and p.steps[0].grid == (1024, 1, 1)
    p = c4().plan()
    assert p.kernels == ["k_conv_i8"] and "SLABS = 9" in p.steps[0].kernel and p.steps[0].ops == 6879707136
    p = c5().plan()
    assert p.kernels == ["k_attn"] and "D = 128, RAGGED = false, KT_ROWS = false" in p.steps[0].kernel
    assert p.steps[0].grid == (256, 1, 1) and p.steps[0].lds_bytes > 64 * 1024
    p = M.Softmax([16, 2048, 2048], 2).plan()
    assert p.kernels == ["k_softmax_regs"] and p.steps[0].bytes == 2 * 4 * 16 * 2048 * 2048


def test_plans_follow_shape_dtype_and_layout():
    # The reference's default layouts: KT row-major, read in place by its own build of the kernel.
    assert "KT_ROWS = true" in M.ComposeMSM(16, 2048, 128, 2048, 128).plan().steps[0].kernel
    # Few queries, many keys: the keys are shared out, at most one workgroup per compute unit.
    p = M.ComposeMSM(16, 1, 128, 32768, 128, layouts=[None, None, KT, None]).plan()
    assert p.kernels == ["k_attn", "k_attn_merge"]
    gx, gy, _ = p.steps[0].grid
    assert gx == 16 and gy > 1 and gx * gy <= 256 and p.scratch_bytes >= 16 * gy * (128 + 4) * 4
    # Head dim 256: staged, P in bf16.
    p = M.ComposeMSM(16, 2048, 256, 2048, 256, layouts=[None, None, KT, None]).plan()
    assert p.kernels == ["k_gemm", "k_softmax_regs", "k_gemm_wide"] and "OUT_BF16 = true" in p.steps[1].kernel
    assert "B_KMAJOR = true" in p.steps[0].kernel
    # Ragged sizes: zero-padded copies of A and B, then the edge build of a small tile.
    p = M.Matmul([1, 1000, 1000, 1000], (M.u8, M.i8, M.i32)).plan()
    assert p.kernels == ["k_pad_rows_pair", "k_gemm"] and "EDGE = true" in p.steps[1].kernel   # both operands' padded copies in one launch
    # One row of A with a ragged K: padded, and still on the matrix cores.
    assert M.Matmul([4, 1, 3565, 256], (M.bf16, M.bf16, M.f32)).plan().kernels == ["k_pad_rows", "k_gemm"]
    # Matrix-vector with a k-fastest B: dot products, not the matrix cores.
    p = M.Matmul([1, 1, 2048, 16384], (M.bf16, M.bf16, M.f32), layouts=[None, KT, None]).plan()
    assert p.kernels == ["k_gemv"] and p.steps[0].unit == "hbm"
    # A dtype triple without an MFMA form, and a problem too small to pay for one.
    assert M.Matmul([1, 256, 256, 256], (M.i16, M.i16, M.i32)).plan().kernels == ["k_matmul_generic"]
    assert M.Matmul([1, 8, 8, 8], (M.f32, M.f32, M.f32)).plan().kernels == ["k_matmul_generic"]
    # Conv shapes beside the benchmark's: implicit Matmul; three channels: unfolded first.
    assert M.Conv([32, 128, 128, 26, 26, 3, 3], (M.bf16, M.bf16, M.f32)).plan().kernels == ["k_gemm"]
    assert "CONV = true" in M.Conv([32, 128, 128, 26, 26, 3, 3], (M.bf16, M.bf16, M.f32)).plan().steps[0].kernel
    assert M.Conv([8, 32, 3, 110, 110, 5, 5], (M.f32, M.f32, M.f32)).plan().kernels == ["k_conv_windows"]
    assert "k_unfold" in M.Conv([8, 32, 3, 110, 110, 11, 11], (M.f32, M.f32, M.f32)).plan().kernels   # windows of 1452 bytes
    # ... in int8 and bf16 with windows of up to 384 bytes: formed in LDS by the kernel that multiplies them.
    assert "KIND = 2" in M.Conv([8, 32, 3, 110, 110, 5, 5], (M.bf16, M.bf16, M.f32)).plan().steps[0].kernel
    first = M.Conv([32, 64, 3, 112, 112, 7, 7], (M.u8, M.i8, M.i32)).plan()
    assert first.kernels == ["k_conv_windows"] and "KS = 3" in first.steps[0].kernel and first.scratch_bytes == 0
    assert "k_unfold_gather" in M.Conv([32, 64, 3, 112, 112, 11, 11], (M.u8, M.i8, M.i32)).plan().kernels   # 363-byte windows
    # Softmax by row length and by which dim is scanned.
    assert M.Softmax([64, 100000], 1).plan().kernels == ["k_softmax_chunk_stats", "k_softmax_chunk_write"]
    assert M.Softmax([8192, 8192], 1).plan().kernels == ["k_softmax_block"]
    assert M.Softmax([16, 2048, 2048], 1).plan().kernels == ["k_softmax_cols"]
    # ... with too few columns for that, the scan dim is shared out over workgroups as well: a
    # launch for the pieces' (max, denominator) pairs, one that merges them and writes.
    p = M.Softmax([2048, 4096], 0).plan()
    assert p.kernels == ["k_softmax_cols", "k_softmax_cols"] and p.steps[0].grid == (64, 16, 1)
    assert p.steps[1].grid == (64, 16, 1) and p.steps[0].bytes == pytest.approx(5.2 * 2048 * 4096)
    assert p.scratch_bytes == 64 * 16 * 64 * 8
    # Fewer than 16 contiguous elements behind the scan dim: scan dim turned innermost and back.
    assert M.Softmax([45, 1963, 4], 1).plan().kernels[0].startswith("k_move") and len(M.Softmax([45, 1963, 4], 1).plan().kernels) == 4
    assert M.Softmax([100000, 67], 1).plan().kernels == ["k_softmax_short"]
    # Moves: transpose tiled through LDS, Packed destination gathered, plain copy.
    sq = [4096, 4096]
    transposed = [M.row_major(sq), M.col_major(sq)]
    assert M.Move(sq, (M.f32, M.f32), layouts=transposed).plan().kernels == ["k_move_tiled32"]
    assert M.Move(sq, (M.bf16, M.bf16), layouts=transposed).plan().kernels == ["k_move_tiled16v"]
    assert M.Move(sq, (M.u8, M.u8), layouts=transposed).plan().kernels == ["k_move_tiled8v"]
    odd8 = [4100, 4100]
    assert M.Move(odd8, (M.u8, M.u8), layouts=[M.row_major(odd8), M.col_major(odd8)]).plan().kernels == ["k_move_tiled_as"]
    assert M.Move(sq, (M.u8, M.f32), layouts=transposed).plan().kernels == ["k_move_tiled"]
    odd = [4098, 4098]
    assert M.Move(odd, (M.bf16, M.bf16), layouts=[M.row_major(odd), M.col_major(odd)]).plan().kernels == ["k_move_tiled16"]
    assert M.Move(sq, (M.f32, M.f32)).plan().kernels == ["k_copy16"]
    assert M.Move(sq, (M.bf16, M.f32)).plan().kernels == ["k_convert4"]


def test_scratch_of_a_plan_covers_the_staging_bytes():
    packed = M.layout(0, 2, 1, (2, M.Packed(16)))
    s = M.Matmul([1, 64, 64, 64], [M.f32] * 3, layouts=[None, packed, None])
    p = s.plan()
    assert s.workspace_bytes() == 64 * 64 * 4 and p.scratch_bytes >= s.workspace_bytes()
    assert p.kernels[0].startswith("k_move") and p.kernels[-1] in ("k_gemm", "k_gemm_big", "k_gemm_wide", "k_matmul_generic")
    for spec in (c1(), c2(), c4(), c5()):
        assert spec.plan().scratch_bytes == 0 == spec.workspace_bytes()


def test_every_planned_kernel_is_a_kernel_of_the_target():
    families = set(M.Target.kernels())
    specs = [c1(), c2(), c3(), c4(), c5(), M.Softmax([3, 7, 1001], 2), M.Softmax([5, 9, 64], 1),
             M.Matmul([2, 100, 70, 50], (M.i8, M.i8, M.i32)), M.Matmul([1, 300, 300, 300], (M.bf16, M.f32, M.f32)),
             M.Conv([2, 8, 8, 30, 30, 3, 3], (M.i16, M.i16, M.i32)), M.Conv([1, 4, 4, 3, 3, 2, 2], (M.f32, M.f32, M.f32)),
             M.Move([64, 48], (M.u8, M.u8), layouts=[M.row_major([64, 48]), M.layout(0, 1, (1, M.OddEven(16)))]),
             M.Fill([100, 100], M.f32, M.FillValue.NegInf), M.Max([64, 64], 1), M.Broadcast([4, 8], 1),
             M.SoftmaxDenominatorAndMax([16, 256], 1), M.DivideVecScalar([16, 256], 1), M.OnePrefix([4, 8])]
    for spec in specs:
        plan = spec.plan()
        assert plan.steps and set(plan.kernels) <= families, (spec, plan)
        assert plan.cost_ns >= 2000 * len(plan.steps) and abs(plan.cost_ns - sum(s.cost_ns for s in plan.steps)) < 1e-3


def test_target_kernel_list_is_the_kernels_in_the_sources():
    import glob, os, re
    root = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "morello_amd", "csrc")
    found = set()
    for path in glob.glob(os.path.join(root, "*.hip")) + glob.glob(os.path.join(root, "*.h")):
        found |= set(re.findall(r"__global__[^;{]*?void (k_\w+)\(", open(path).read(), flags=re.S))
    found.discard("k_mfma_rate")  # the rate measurement, not a Spec's kernel
    assert found == set(M.Target.kernels())


def test_cost_orders_what_search_has_to_order():
    """The model is only asked to rank alternatives (cost.rs:13-17 compares `main` first)."""
    mm = lambda n, dts: M.Matmul([1, n, n, n], dts).plan().cost_ns
    i8, bf, f32 = (M.u8, M.i8, M.i32), (M.bf16, M.bf16, M.f32), (M.f32, M.f32, M.f32)
    for dts in (i8, bf, f32):
        costs = [mm(n, dts) for n in (256, 1024, 2048, 4096, 8192)]
        assert costs == sorted(costs) and costs[-1] > 6 * costs[-2] > 18 * costs[-3]
    assert mm(4096, i8) < mm(4096, bf) < mm(4096, f32)
    # Fused attention beats the same Compose with its intermediates materialised (bufferize).
    staged = M.Compose([M.Matmul([16, 2048, 2048, 128], [M.f32, M.bf16, M.f32]), M.Softmax([16, 2048, 2048], 2),
                        M.Matmul([16, 2048, 128, 2048], [M.bf16, M.bf16, M.f32])], layouts=[None, None, KT, None])
    fused, unfused = staged.plan(), staged.bufferize(0).plan()
    assert fused.kernels == ["k_attn"] and len(unfused.steps) >= 3
    assert fused.cost_ns * 4 < unfused.cost_ns and unfused.scratch_bytes >= 16 * 2048 * 2048 * 4
    # A column-major A costs its transposing copy on top.
    a_t = M.Matmul([1, 4096, 4096, 4096], bf, layouts=[M.batched_col_major([1, 4096, 4096]), None, None]).plan()
    assert a_t.kernels[-1] == "k_gemm_wide" and len(a_t.steps) == 2 and a_t.cost_ns > mm(4096, bf)


def test_every_manual_schedule_has_its_plan():
    """`spec.tile_out([1, m, n]).split(k)` (scheduling_sugar.rs:37-132) plans the tile it names."""
    spec = M.Matmul([1, 2048, 2048, 2048], (M.bf16, M.bf16, M.f32))
    schedules = spec.available_schedules()
    assert len(schedules) == 8
    costs = {}
    for tm, tn, sk in schedules:
        plan = spec.tile_out([1, tm, tn]).split(sk).plan()
        if (tm, tn, sk * 2) == (256, 256, 128):     # the tile with the hand-scheduled k loop
            assert plan.kernels in (["k_gemm_big"], ["k_gemm_wide"])
        else:
            assert plan.kernels == ["k_gemm"] and f"Tile<{tm}, {tn}, {sk * 2}," in plan.steps[0].kernel   # split in bytes
        assert plan.steps[0].grid[0] == (2048 // tm) * (2048 // tn)
        costs[(tm, tn, sk)] = plan.cost_ns
    # 64 workgroups of 256 x 256 leave three quarters of the chip idle: never the cheapest here.
    assert min(costs, key=costs.get)[0] < 256


def test_schedule_search_returns_the_cheapest_plan():
    for dts, n in (((M.u8, M.i8, M.i32), 1024), ((M.bf16, M.bf16, M.f32), 4096), ((M.f32, M.f32, M.f32), 512)):
        spec = M.Matmul([1, n, n, n], dts)
        found = spec.search_schedule()
        costs = {s: spec.tile_out([1, s[0], s[1]]).split(s[2]).plan().cost_ns for s in spec.available_schedules()}
        assert (found.tile_m, found.tile_n, found.split_k) in costs
        assert found.plan().cost_ns == min(costs.values())
    assert M.Matmul([1, 4096, 4096, 4096], (M.u8, M.i8, M.i32)).search_schedule().tile_m == 256
    assert M.Matmul([1, 512, 1024, 512], (M.u8, M.i8, M.i32)).search_schedule().tile_m == 64
    with pytest.raises(M.MorelloError):
        M.Matmul([1, 64, 64, 64], (M.i16, M.i16, M.i32)).search_schedule()   # no matrix-core form


def test_plan_errors_are_the_run_errors():
    import ctypes as C
    from morello_amd import _binding as B
    bad = M.Matmul([1, 65536, 65536, 2], [M.u8, M.i8, M.i32])
    head = B.PlanC()
    assert B.load().mrl_spec_plan(C.byref(bad._c), C.byref(head), None, 0) == bad.check() != 0
    ok = c2()
    assert B.load().mrl_spec_plan(C.byref(ok._c), None, None, 0) != 0       # null plan
    assert B.load().mrl_spec_plan(C.byref(ok._c), C.byref(head), None, 0) == 0 and head.n_steps == 1  # count only


@pytest.mark.gpu
def test_planning_leaves_runs_alone(gpu):
    """A plan between two runs changes nothing: the recorder is per call and per thread."""
    from gpu_util import run_spec
    spec = M.Matmul([1, 96, 200, 72], (M.u8, M.i8, M.i32))
    a, b = synth.uniform_u8(501, 0, (1, 96, 200)), synth.uniform_i8(501, 1, (1, 200, 72))
    first = run_spec(spec, [a, b, np.zeros((1, 96, 72), np.int32)])
    assert spec.plan().steps
    second = run_spec(spec, [a, b, np.zeros((1, 96, 72), np.int32)])
    want = a.astype(np.int32)[0] @ b.astype(np.int32)[0]
    assert np.array_equal(first[0], want) and np.array_equal(second[0], want)


def _settle_clocks():
    """A GPU coming out of idle runs its first few hundred launches at changing clocks (fast, then
    40 % slower, then settling): timings taken for a comparison start after that."""
    spec = M.Matmul([1, 2048, 2048, 2048], (M.u8, M.i8, M.i32))
    bufs = [M.DeviceBuffer(spec.bytes_used(i)) for i in range(3)]
    spec.run_timed([b.ptr for b in bufs], 1500)
    for b in bufs:
        b.free()


def _median_ms(run, ptrs, launches=20, repeats=5):
    run.run_timed(ptrs, 3)
    return sorted(run.run_timed(ptrs, launches) for _ in range(repeats))[repeats // 2] / launches


@pytest.mark.gpu
def test_cost_model_against_measured_launches(gpu):
    """Predicted against measured per-launch time on benchmark-like operands for the kernels the
    benchmark configurations and their neighbours run, each timing the median of five bursts on
    settled clocks.  The ratios are printed (measured on the first ten: 0.80-1.21); the model, which
    ranks the lowerings that mrl_target_actions and mrl_matmul_search_schedule offer, is held to
    a factor of two either way for every kernel family here."""
    rng = np.random.default_rng(7)
    specs = [c2(), c4(), c5(), M.Matmul([1, 2048, 2048, 2048], (M.bf16, M.bf16, M.f32)),
             M.Matmul([1, 1024, 1024, 1024], (M.f32, M.f32, M.f32)), M.Softmax([16, 2048, 2048], 2),
             M.Softmax([64, 100000], 1), M.ComposeMSM(16, 1, 128, 32768, 128, layouts=[None, None, KT, None]),
             M.Matmul([1, 1, 2048, 16384], (M.bf16, M.bf16, M.f32), layouts=[None, KT, None]),
             M.Move([4096, 4096], (M.f32, M.f32), layouts=[M.row_major([4096, 4096]), M.col_major([4096, 4096])]),
             # a first-layer Conv (windows formed in LDS), a deep one on small images (windows shared out), a Softmax
             # over an outer dim of few columns (scan dim shared out)
             M.Conv([32, 64, 3, 112, 112, 7, 7], (M.u8, M.i8, M.i32)), M.Conv([32, 512, 512, 5, 5, 3, 3], (M.u8, M.i8, M.i32)),
             M.Softmax([2048, 4096], 0)]
    _settle_clocks()
    for spec in specs:
        bufs = []
        for i, dt in enumerate(spec.dtypes):
            n = spec.bytes_used(i)
            if dt == M.f32: arr = rng.standard_normal(n // 4, dtype=np.float32)
            elif dt == M.bf16: arr = (rng.standard_normal(n // 2, dtype=np.float32).view(np.uint32) >> 16).astype(np.uint16)
            else: arr = rng.integers(0, 256, n, dtype=np.uint8)
            bufs.append(M.DeviceBuffer.from_numpy(arr))
        ptrs = [b.ptr for b in bufs]
        measured_ns = _median_ms(spec, ptrs) * 1e6
        predicted_ns = spec.plan().cost_ns
        for b in bufs:
            b.free()
        print(f"cost model: {spec.plan().kernels} predicted {predicted_ns / 1e3:.1f} us measured {measured_ns / 1e3:.1f} us "
              f"ratio {predicted_ns / measured_ns:.2f}")
        assert 0.5 < predicted_ns / measured_ns < 2.0, (spec, predicted_ns, measured_ns)


@pytest.mark.gpu
def test_cost_model_ranks_manual_schedules(gpu):
    """What a search over tile_out / split needs from the model is an order.  Only quantities
    measured in this run, one after the other on settled clocks, are compared: where the model
    puts two schedules a factor of two or more apart, the measured order must not be the reverse
    by more than a quarter, and the schedule it calls cheapest runs within 2x of the fastest
    (measured: the fastest itself or within 1.15x; bf16 2048^3 1.4x)."""
    rng = np.random.default_rng(11)
    _settle_clocks()
    for dts in ((M.u8, M.i8, M.i32), (M.bf16, M.bf16, M.f32)):
        for m, k, n in ((512, 1024, 512), (2048, 2048, 2048), (4096, 4096, 4096), (1024, 8192, 1024)):
            spec = M.Matmul([1, m, k, n], dts)
            bufs = []
            for i, dt in enumerate(spec.dtypes):
                nbytes = spec.bytes_used(i)
                if dt == M.bf16: arr = (rng.standard_normal(nbytes // 2, dtype=np.float32).view(np.uint32) >> 16).astype(np.uint16)
                else: arr = rng.integers(0, 256, nbytes, dtype=np.uint8)
                bufs.append(M.DeviceBuffer.from_numpy(arr))
            ptrs = [b.ptr for b in bufs]
            measured, predicted = {}, {}
            for tm, tn, sk in spec.available_schedules():
                sched = spec.tile_out([1, tm, tn]).split(sk)
                measured[(tm, tn, sk)] = _median_ms(sched, ptrs)
                predicted[(tm, tn, sk)] = sched.plan().cost_ns
            for b in bufs:
                b.free()
            pick = min(predicted, key=predicted.get)
            assert measured[pick] <= 2.0 * min(measured.values()), (dts[0], m, k, n, pick, measured)
            for x in predicted:
                for y in predicted:
                    if predicted[x] * 2.0 <= predicted[y]:
                        assert measured[x] <= 1.25 * measured[y], (dts[0], m, k, n, x, y, measured, predicted)


def test_early_layer_convs_of_whole_chunk_pixels():
    """Host only: pixels of whole 16-byte chunks with windows of up to 320 bytes, at most 48 filters
    and filters x window bytes of at most 9216 go to the kernel that keeps the filters in
    registers (pixels of a single chunk included: the kernel that forms windows in LDS is for
    pixels that are not whole chunks); more filters, longer windows and small problems stay with
    the implicit Matmul."""
    kernels = lambda c, f, fs, dts, b=32: M.Conv([b, f, c, 112, 112, fs, fs], dts).plan().kernels
    i8, bf = (M.u8, M.i8, M.i32), (M.bf16, M.bf16, M.f32)
    assert kernels(16, 32, 3, i8) == ["k_conv_small"] and kernels(8, 32, 3, bf) == ["k_conv_small"]
    assert kernels(32, 32, 3, i8) == ["k_conv_small"] and kernels(16, 32, 3, bf) == ["k_conv_small"] and kernels(48, 48, 2, i8) == ["k_conv_small"]
    assert kernels(32, 64, 3, i8) == ["k_gemm"] and kernels(16, 32, 5, i8) == ["k_gemm"] and kernels(32, 32, 3, bf) == ["k_gemm"]
    assert kernels(32, 48, 3, i8) == ["k_gemm"]          # 48 filters of 288 bytes: more than the bank the rule allows
    assert kernels(32, 32, 3, i8, b=4) == ["k_gemm"]     # 50176 pixels: too few for a tile per wave to pay
    assert kernels(12, 32, 3, i8) == ["k_conv_windows"]  # pixels of 12 bytes are not whole chunks


def test_plans_of_the_softmax_primitives():
    """Host only: which kernel a primitive of the decomposition takes.  Contiguous lines of up to
    4096 elements in whole 16-byte vectors stay in a wavefront's registers; a scan dim that is
    not the innermost puts 16, 32 or 64 lines side by side in a workgroup, as many as still
    leave two workgroups per compute unit; anything else a wavefront per line.  Broadcast
    between row-major tensors moves 16-byte pieces."""
    kernel = lambda spec: (spec.plan().steps[0].family, spec.plan().steps[0].grid[:2])
    assert kernel(M.Max([16, 2048, 2048], 2)) == ("k_parts_rows", (8192, 1))
    assert kernel(M.SoftmaxComplete([7, 12], 1))[0] == "k_parts_rows"
    assert kernel(M.Max([4096, 4100], 1))[0] == "k_parts" and kernel(M.Max([7, 33], 1))[0] == "k_parts"
    assert kernel(M.Max([3, 4100], 1)) == ("k_parts_block", (3, 1))   # few long lines: a workgroup per line
    assert kernel(M.DivideVec([64, 64]))[0] == "k_parts_rows" and kernel(M.DivideVec([64, 66]))[0] == "k_parts"
    assert kernel(M.SoftmaxDenominatorAndMax([2048, 4096], 0)) == ("k_parts_cols", (256, 1))     # 16 lines each
    assert kernel(M.SoftmaxDenominatorAndMax([40, 20000], 0)) == ("k_parts_cols", (625, 1))      # 32
    assert kernel(M.SoftmaxDenominatorAndMax([40, 40000], 0)) == ("k_parts_cols", (625, 1))      # 64
    # lines of a handful of elements (the merge of a few tiles' pairs): a thread per line
    assert kernel(M.SoftmaxDenominatorAndMax([5, 20000], 0)) == ("k_parts_cols", (79, 1))
    assert kernel(M.SoftmaxDenominatorAndMaxFromParts([16, 2048, 2], 2)) == ("k_parts_cols", (128, 1))
    assert kernel(M.Max([5, 9, 4], 1))[0] == "k_parts"                                           # rows of 4 elements: not worth lining up
    # col-major: the lines are contiguous, each starting on any 4 bytes
    assert kernel(M.Max([33, 64], 0, layouts=[M.col_major([33, 64]), None]))[0] == "k_parts"
    one_read, two_reads = M.SoftmaxDenominatorAndUnscaled([64, 1024], 1).plan(), M.SoftmaxDenominatorAndUnscaled([1024, 64], 0).plan()
    assert one_read.steps[0].bytes == 2 * 4 * 65536 and two_reads.steps[0].bytes == 3 * 4 * 65536
    assert kernel(M.Broadcast([16, 2048, 2048], 2))[0] == "k_broadcast_fill_rows"
    assert kernel(M.Broadcast([2048, 4096], 0)) == ("k_broadcast_rows", (4, 512))
    assert kernel(M.Broadcast([4, 9], 1))[0] == "k_broadcast" and kernel(M.Broadcast([6, 32], 1, M.u8))[0] == "k_broadcast_fill_rows"
    assert kernel(M.Broadcast([4, 8, 64], 1, layouts=[None, M.layout(2, 1, 0)]))[0] == "k_broadcast"


def test_actions_of_a_softmax():
    """Host only: the Softmax stage of C5 on its own lists the fused kernels' choice, the two
    whole-row rewrites and the tiled one for every power-of-two tile count down to 64-element
    tiles, each priced; the fused kernel (8 bytes an element) is the cheapest."""
    K = M.ActionKind
    acts = M.Softmax([16, 2048, 2048], 2).actions()
    assert [a.kind for a in acts] == [K.Select, K.ToSoftmaxParts, K.ToSoftmaxPartsRecompute] + [K.ParallelSoftmax] * 5
    assert [a.parts for a in acts[3:]] == [2, 4, 8, 16, 32]
    assert acts[0].plan().kernels == ["k_softmax_regs"]
    # whole contiguous lines stay in a wavefront's registers; the merge of two tiles' pairs is a thread per line
    assert acts[1].plan().kernels == ["k_parts_rows"] * 2 and acts[3].plan().kernels == ["k_parts_rows", "k_parts_cols", "k_parts_rows"]
    assert all(a.cost_ns > acts[0].cost_ns for a in acts[1:])
    assert acts[1].scratch_bytes >= 16 * 2048 * 4 and acts[3].scratch_bytes >= 16 * 2048 * 4 * (2 + 2 * 2)
    # integers and other dtypes have no Softmax; a Matmul lists none of these
    assert not {K.ToSoftmaxParts, K.ParallelSoftmax} & {a.kind for a in c2().actions()}


def test_actions_of_the_benchmark_configurations():
    """Target::actions (target/mod.rs:69) for C2-C5, host only: every lowering the backend can run,
    priced; the dispatch rules' own choice (Select) is among the cheapest the model knows."""
    K = M.ActionKind
    rewrites = (K.ToAccum, K.MoveRelayout, K.Cast)     # last in every list, with children (tested below)
    every = c2().actions()
    # C2 accumulates and is row-major: of the general rewrites only the casts of its inputs to i32 apply.
    assert [(a.kind, a.tile_m, a.tile_n) for a in every if a.kind in rewrites] == [(K.Cast, 0, int(M.i32)), (K.Cast, 1, int(M.i32))]
    acts = [a for a in every if a.kind not in rewrites]
    assert every[:len(acts)] == acts
    tiles = {(a.tile_m, a.tile_n, a.split_k) for a in acts if a.kind == K.TileOutSplit}
    assert acts[0].kind == K.Select and tiles == set(c2().available_schedules()) and len(tiles) == 8
    assert all(a.n_steps == 1 and a.scratch_bytes == 0 and a.cost_ns > 20e3 for a in acts)
    assert acts[0].plan().kernels == ["k_gemm_wide"]
    # The move_param steps: the 256 x 256 tile under each staging is an action of its own kernel.
    staged = {a.staging: a for a in acts if a.kind == K.TileOutSplit and a.staging}
    assert {st: a.plan().kernels for st, a in staged.items()} == {
        M.Staging.Registers: ["k_gemm"], M.Staging.DirectB: ["k_gemm_big"], M.Staging.DirectBWide: ["k_gemm_wide"]}
    assert staged[M.Staging.DirectBWide].cost_ns == acts[0].cost_ns < staged[M.Staging.DirectB].cost_ns < staged[M.Staging.Registers].cost_ns
    assert len(c2().available_schedules(with_staging=True)) == 11
    # A staging the shape does not admit is no action: K = 1024 is too short for the four-wave kernel.
    short = M.MatmulAccum([1, 512, 1024, 512], (M.u8, M.i8, M.i32)).actions()
    assert {a.staging for a in short if a.kind == K.TileOutSplit} == {M.Staging.Default, M.Staging.Registers, M.Staging.DirectB}
    acts = c3().actions()
    assert len([a for a in acts if a.kind not in rewrites]) == 12 and acts[0].cost_ns == min(a.cost_ns for a in acts)
    # C4 overwrites its output and its tensors are channels-last: to_accum, a row-major copy of each parameter, two casts.
    assert [(a.kind, a.tile_m) for a in c4().actions() if a.kind in rewrites] == [
        (K.ToAccum, 0), (K.MoveRelayout, 0), (K.MoveRelayout, 1), (K.MoveRelayout, 2), (K.Cast, 0), (K.Cast, 1)]
    acts = {(a.kind, a.tile_m): a for a in c4().actions() if a.kind not in rewrites}
    assert set(acts) == {(K.Select, 0), (K.Fused, 0), (K.Fused, 54), (K.SpatialSplit, 64), (K.SpatialSplit, 128), (K.SpatialSplit, 256),
                         (K.Unfold, 0), (K.Generic, 0)}
    assert acts[(K.Fused, 0)].plan().kernels == ["k_conv_i8"] and acts[(K.Select, 0)].cost_ns == acts[(K.Fused, 0)].cost_ns
    # tile_out over whole output rows: two rows per workgroup, their four input rows (padded to 64 pixels) in LDS
    rows = acts[(K.Fused, 54)].plan().steps[0]
    assert rows.kernel.startswith("k_conv_rows_i8") and rows.grid == (864, 1, 1) and rows.block == (256, 1, 1)
    assert acts[(K.SpatialSplit, 128)].plan().kernels == ["k_gemm"] and "CONV = true" in acts[(K.SpatialSplit, 128)].plan().steps[0].kernel
    assert acts[(K.Unfold, 0)].plan().kernels == ["k_unfold", "k_gemm"] and acts[(K.Unfold, 0)].scratch_bytes > 50e6
    assert acts[(K.Generic, 0)].plan().kernels == ["k_conv_generic"]
    assert acts[(K.Fused, 0)].cost_ns < acts[(K.SpatialSplit, 64)].cost_ns < acts[(K.Unfold, 0)].cost_ns < acts[(K.Generic, 0)].cost_ns
    acts = c5().actions()
    # Fused: the keys in `parts` shares (parallel_softmax.rs) x 128 or 64 queries per workgroup (tile_out over the rows).
    assert [(a.parts, a.tile_m) for a in acts if a.kind == K.Fused] == [(p, r) for p in (1, 2, 4, 8, 16) for r in (128, 64)]
    assert acts[-1].kind == K.Bufferize and len(acts[-1].plan().steps) == 3
    fused = {a.parts: a for a in acts if a.kind == K.Fused and a.tile_m == 128}
    narrow = {a.parts: a for a in acts if a.kind == K.Fused and a.tile_m == 64}
    assert "QG = 4" in fused[1].plan().steps[0].kernel and fused[1].plan().steps[0].block == (512, 1, 1)
    assert "QG = 2" in narrow[1].plan().steps[0].kernel and narrow[1].plan().steps[0].block == (256, 1, 1)
    assert narrow[1].plan().steps[0].grid[0] == 2 * fused[1].plan().steps[0].grid[0]
    assert fused[1].scratch_bytes == 0 and fused[2].plan().kernels == ["k_attn", "k_attn_merge"]
    assert fused[2].scratch_bytes == 16 * 2048 * 2 * (128 + 4) * 4
    assert acts[0].cost_ns == fused[1].cost_ns == min(a.cost_ns for a in acts)
    # Specs with one lowering list it alone; what no kernel takes lists nothing it cannot run.
    assert [a.kind for a in M.Move([64, 64], (M.f32, M.f32)).actions()] == [K.Select]
    odd = M.Conv([2, 3, 5, 6, 6, 2, 2], (M.i16, M.i16, M.i32)).actions()
    assert {a.kind for a in odd} - set(rewrites) == {K.Select, K.Generic}
    assert [a.kind for a in M.ComposeMSM(2, 64, 256, 128, 256, layouts=[None, None, KT, None]).actions()] == [K.Select, K.Bufferize]


@pytest.mark.gpu
def test_a_run_launches_what_its_plan_lists(gpu):
    """The plan comes from the dispatch code itself; this holds the two against each other from
    outside: a run launches as many kernels as its plan has steps, for Specs of every kind and
    path (matrix cores, padded and transposed operands, slices of K, fused and staged Compose,
    split keys, every Softmax and Move kernel family, generic kernels)."""
    sq = [600, 520]
    specs = [
        c1(), M.Matmul([1, 1000, 1000, 1000], (M.u8, M.i8, M.i32)), M.Matmul([1, 512, 8192, 512], (M.bf16, M.bf16, M.f32)),
        M.Matmul([2, 100, 70, 50], (M.i16, M.i16, M.i32)), M.Matmul([1, 1, 2048, 4096], (M.bf16, M.bf16, M.f32), layouts=[None, KT, None]),
        M.Matmul([1, 300, 256, 200], (M.f32, M.f32, M.f32), layouts=[M.batched_col_major([1, 300, 256]), None, M.batched_col_major([1, 300, 200])]),
        M.Matmul([1, 64, 64, 64], [M.f32] * 3, layouts=[None, M.layout(0, 2, 1, (2, M.Packed(16))), None]),
        M.Conv([2, 64, 64, 20, 20, 3, 3], (M.u8, M.i8, M.i32)), M.Conv([2, 32, 16, 20, 20, 3, 3], (M.bf16, M.bf16, M.f32)),
        M.Conv([2, 16, 3, 30, 30, 5, 5], (M.u8, M.i8, M.i32)), M.Conv([1, 4, 4, 6, 6, 3, 3], (M.u16, M.u16, M.u32)),
        M.ComposeMSM(2, 256, 128, 512, 128, layouts=[None, None, KT, None]), M.ComposeMSM(2, 256, 128, 512, 128),
        M.ComposeMSM(2, 100, 96, 300, 72, layouts=[None, None, KT, None]), M.ComposeMSM(4, 1, 128, 8192, 128, layouts=[None, None, KT, None]),
        M.ComposeMSM(1, 200, 160, 1001, 160, layouts=[None, None, KT, None]),
        M.Compose([M.Matmul([2, 64, 96, 32], [M.f32, M.bf16, M.f32]), M.Softmax([2, 64, 96], 2),
                   M.Matmul([2, 64, 32, 96], [M.bf16, M.bf16, M.f32])], layouts=[None, None, KT, None]).bufferize(0),
        M.Softmax([64, 2048], 1), M.Softmax([1000, 67], 1), M.Softmax([300, 8192], 1), M.Softmax([40, 100000], 1),
        M.Softmax([600, 1001], 1), M.Softmax([2149, 172], 0), M.Softmax([600, 64, 300], 0), M.Softmax([6, 4], 0),
        M.Move(sq, (M.f32, M.f32), layouts=[M.row_major(sq), M.col_major(sq)]), M.Move(sq, (M.u8, M.u8), layouts=[M.row_major(sq), M.col_major(sq)]),
        M.Move(sq, (M.bf16, M.f32)), M.Move([96, 208, 64], (M.i32, M.i32), layouts=[M.layout(2, 1, 0), M.layout(1, 2, 0, (0, M.OddEven(16)))]),
        M.Move([64, 48], (M.u8, M.u8), layouts=[M.row_major([64, 48]), M.layout(0, 1, (1, M.OddEven(16)))]),
        M.Fill([100, 100], M.f32, M.FillValue.NegInf), M.Max([64, 64], 1), M.Broadcast([4, 8], 1), M.OnePrefix([4, 8]),
    ]
    for spec in specs:
        if isinstance(spec, M.Spec):
            sizes = [spec.bytes_used(i) for i in range(len(spec.dtypes))]
        else:  # a general Compose: dense row-major external parameters
            sizes = [int(np.prod(shape)) * dt.size for shape, dt in zip(spec.parameter_shapes(), spec.parameter_dtypes())]
        bufs = [M.DeviceBuffer(max(4, s)) for s in sizes]
        for b in bufs:
            b.zero()
        steps = len(spec.plan().steps)
        before = M.launch_count()
        spec.run_device([b.ptr for b in bufs])
        launched = M.launch_count() - before
        for b in bufs:
            b.free()
        assert launched == steps, (spec.plan(), launched)


def test_rewrite_actions_have_children_and_the_others_are_leaves():
    """mrl_action_apply: the Softmax rewrites and the Compose's bufferize hand out their sub-Specs
    (scheduling/to_softmax_parts.rs:33-181, parallel_softmax.rs:24-223, bufferize.rs:24-116) with
    the source of every parameter; what the library runs as one piece has none.  Each child is a
    Spec of its own with actions of its own: the recursion of a search."""
    K = M.ActionKind
    sm = M.Softmax([16, 2048, 2048], 2)
    by_kind = {}
    for a in sm.actions():
        by_kind.setdefault(a.kind, a)
    assert by_kind[K.Select].apply().is_leaf()
    rw = by_kind[K.ToSoftmaxParts].apply()
    assert [(s.kind, src) for s, src in rw.subspecs] == [(M.SpecKind.SoftmaxDenominatorAndUnscaled, [0, -1, 1]),
                                                         (M.SpecKind.DivideVecScalar, [1, -1])]
    assert rw.intermediate_bytes == [16 * 2048 * 4]
    rw = by_kind[K.ToSoftmaxPartsRecompute].apply()
    assert [(s.kind, src) for s, src in rw.subspecs] == [(M.SpecKind.SoftmaxDenominatorAndMax, [0, -1, -2]),
                                                         (M.SpecKind.SoftmaxComplete, [0, -1, -2, 1])]
    rw = by_kind[K.ParallelSoftmax].apply()      # parts = 2
    assert [(s.kind, s.spec_shape, src) for s, src in rw.subspecs] == [
        (M.SpecKind.SoftmaxDenominatorAndMax, [16, 2048, 2, 1024], [0, -3, -4]),
        (M.SpecKind.SoftmaxDenominatorAndMaxFromParts, [16, 2048, 2], [-3, -4, -1, -2]),
        (M.SpecKind.SoftmaxComplete, [16, 2048, 2048], [0, -1, -2, 1])]
    assert rw.intermediate_bytes == [16 * 2048 * 4] * 2 + [16 * 2048 * 2 * 4] * 2
    for sub, _ in rw.subspecs:
        assert sub.check() == 0 and sub.actions()[0].kind == K.Select and len(sub.plan().kernels) >= 1
    # The Compose: parameters V, Q, KT, out; S and P between the components as f32.
    KT = M.layout(0, 2, 1)
    c5 = M.ComposeMSM(16, 2048, 128, 2048, 128, layouts=[None, None, KT, None])
    buf = [a for a in c5.actions() if a.kind == K.Bufferize][0].apply()
    assert [(s.kind, s.spec_shape, list(s.dtypes), src) for s, src in buf.subspecs] == [
        (M.SpecKind.Matmul, [16, 2048, 128, 2048], [M.bf16, M.bf16, M.f32], [1, 2, -1]),
        (M.SpecKind.Softmax, [16, 2048, 2048], [M.f32, M.f32], [-1, -2]),
        (M.SpecKind.Matmul, [16, 2048, 2048, 128], [M.f32, M.bf16, M.f32], [-2, 0, 3])]
    assert buf.subspecs[0][0].layouts[1] == KT and buf.intermediate_bytes == [16 * 2048 * 2048 * 4] * 2
    assert len(buf.subspecs[1][0].actions()) > 3          # the Softmax child has the rewrites again
    assert all(a.apply().is_leaf() for a in c5.actions() if a.kind != K.Bufferize)
    general = (K.ToAccum, K.MoveRelayout, K.Cast)
    assert all(a.apply().is_leaf() for a in M.MatmulAccum([1, 512, 512, 512], (M.u8, M.i8, M.i32)).actions() if a.kind not in general)
    assert all(a.apply().is_leaf() for a in M.Conv([2, 64, 64, 10, 10, 3, 3], (M.u8, M.i8, M.i32)).actions() if a.kind not in general)
    # to_accum (to_accum.rs:12-60): Zero on the output, then the accumulating Spec.
    mm = M.Matmul([2, 100, 96, 70], (M.bf16, M.bf16, M.f32), layouts=[M.batched_col_major([2, 100, 96]), None, M.batched_col_major([2, 100, 70])])
    by = {(a.kind, a.tile_m): a.apply() for a in mm.actions() if a.kind in general}
    assert set(by) == {(K.ToAccum, 0), (K.MoveRelayout, 0), (K.MoveRelayout, 2), (K.Cast, 0), (K.Cast, 1)}
    zero, body = by[(K.ToAccum, 0)].subspecs
    assert (zero[0].kind, zero[0].spec_shape, zero[1]) == (M.SpecKind.Fill, [2, 100, 70], [2]) and zero[0].layouts[0] == mm.layouts[2]
    assert body[0].kind == M.SpecKind.Matmul and body[0].accum and body[1] == [0, 1, 2] and by[(K.ToAccum, 0)].intermediate_bytes == []
    # move_relayout (moves.rs:49-130) of an input: prologue Move, body on the row-major copy.
    pro, body = by[(K.MoveRelayout, 0)].subspecs
    assert pro[0].kind == M.SpecKind.Move and pro[0].layouts == [mm.layouts[0], M.row_major([2, 100, 96])] and pro[1] == [0, -1]
    assert body[0].layouts[0] == M.row_major([2, 100, 96]) and body[1] == [-1, 1, 2]
    assert by[(K.MoveRelayout, 0)].intermediate_bytes == [2 * 100 * 96 * 2]
    # ... of the output of a Spec that overwrites it: no prologue, an epilogue Move back.
    body, epi = by[(K.MoveRelayout, 2)].subspecs
    assert body[1] == [0, 1, -1] and epi[0].kind == M.SpecKind.Move and epi[1] == [-1, 2] and epi[0].layouts[1] == mm.layouts[2]
    acc = M.MatmulAccum([2, 100, 96, 70], (M.bf16, M.bf16, M.f32), layouts=[None, None, M.batched_col_major([2, 100, 70])])
    three = [a for a in acc.actions() if a.kind == K.MoveRelayout][0].apply().subspecs
    assert [s.kind for s, _ in three] == [M.SpecKind.Move, M.SpecKind.Matmul, M.SpecKind.Move]     # read and written
    # cast (moves.rs with another dtype): the input as the output's dtype, in its own layout.
    pro, body = by[(K.Cast, 0)].subspecs
    assert list(pro[0].dtypes) == [M.bf16, M.f32] and pro[0].layouts == [mm.layouts[0]] * 2 and list(body[0].dtypes) == [M.f32, M.bf16, M.f32]
    assert by[(K.Cast, 0)].intermediate_bytes == [2 * 100 * 96 * 4]
    # The rewrites of the Softmax primitives (to_max_and_denom.rs, to_max_and_unscaled.rs, broadcast_first.rs).
    dm = [a for a in M.SoftmaxDenominatorAndMax([6, 640], 1).actions() if a.kind == K.ToMaxAndDenominator][0].apply()
    assert [(s.kind, src) for s, src in dm.subspecs] == [(M.SpecKind.Max, [0, 1]), (M.SpecKind.SoftmaxDenominator, [0, 1, 2])]
    assert dm.intermediate_bytes == []
    du = [a for a in M.SoftmaxDenominatorAndUnscaled([6, 640], 1).actions() if a.kind == K.ToMaxAndUnscaled][0].apply()
    assert [(s.kind, src) for s, src in du.subspecs] == [(M.SpecKind.Max, [0, -1]),
                                                         (M.SpecKind.SoftmaxDenominatorAndUnscaledFromMax, [0, -1, 1, 2])]
    assert du.intermediate_bytes == [6 * 4]
    bf = [a for a in M.DivideVecScalar([6, 640], 1).actions() if a.kind == K.BroadcastFirst][0].apply()
    assert [(s.kind, s.parameter_shapes(), src) for s, src in bf.subspecs] == [
        (M.SpecKind.Broadcast, [[6, 1], [6, 640]], [1, -1]), (M.SpecKind.DivideVec, [[6, 640], [6, 640]], [0, -1])]
    assert bf.intermediate_bytes == [6 * 640 * 4]
