"""Every action Target::actions lists for a Spec (mrl_target_actions; target/mod.rs:69), run through
mrl_run_action and held against the CPU oracle: integer Specs bit for bit, the bf16 Compose within
its 1e-2.  Small shapes against the oracle itself; the benchmark configurations against the
result of the dispatch rules' own choice (which the other GPU tests hold against the oracle)."""
import numpy as np
import pytest

import morello_amd as M
import orc
from gpu_util import rel_err
from morello_amd import synth

pytestmark = pytest.mark.gpu
KT = M.layout(0, 2, 1)
KT_ORC = orc.make_layout([0, 2, 1])


def run_action(action, arrays):
    bufs = [M.DeviceBuffer.from_numpy(a) for a in arrays]
    action.run_device([b.ptr for b in bufs])
    out = bufs[-1].to_numpy(arrays[-1].dtype, arrays[-1].shape)
    for b in bufs:
        b.free()
    return out


def test_matmul_actions_against_the_oracle(gpu):
    for dts, np_out, odt in (((M.u8, M.i8, M.i32), np.int32, [orc.U8, orc.I8, orc.I32]),
                             ((M.bf16, M.bf16, M.f32), np.float32, [orc.BF16, orc.BF16, orc.F32])):
        m, k, n = 512, 2560, 256  # K long enough (20 steps of 128 bytes) for every staging of the 256 x 256 tile
        spec = M.MatmulAccum([1, m, k, n], dts)
        if dts[0] == M.u8:
            a, b = synth.uniform_u8(31, 0, (1, m, k)), synth.uniform_i8(31, 1, (1, k, n))
            c0 = synth.uniform_u8(31, 2, (1, m, n)).astype(np.int32) - 99
        else:
            a, b = synth.normal_bf16(31, 0, (1, m, k)), synth.normal_bf16(31, 1, (1, k, n))
            c0 = synth.normal_f32(31, 2, (1, m, n))
        want = orc.matmul([1, m, k, n], odt, a, b, c0.copy(), True)
        acts = spec.actions()
        assert len([a for a in acts if a.kind < M.ActionKind.ToAccum]) == 12 and {a.staging for a in acts} == set(M.Staging)
        for act in acts:
            got = run_action(act, [a, b, c0.copy()])
            if np_out == np.int32:
                assert np.array_equal(got, want), act
            else:
                assert rel_err(got, want) < 1e-4, act


def test_conv_actions_against_the_oracle(gpu):
    b, f, c, oh, ow, fh, fw = 2, 64, 64, 12, 10, 3, 3
    spec = M.Conv([b, f, c, oh, ow, fh, fw], (M.u8, M.i8, M.i32))
    img = synth.uniform_u8(32, 0, (b, oh + fh - 1, ow + fw - 1, c))
    filt = synth.uniform_i8(32, 1, (f, fh, fw, c))
    nhwc = orc.make_layout([0, 2, 3, 1])
    want = orc.conv([b, f, c, oh, ow, fh, fw], [orc.U8, orc.I8, orc.I32], img, filt, np.zeros((b, oh, ow, f), np.int32),
                    layouts=[nhwc, nhwc, nhwc])
    acts = spec.actions()
    assert {a.kind for a in acts if a.kind < M.ActionKind.ToAccum} == {
        M.ActionKind.Select, M.ActionKind.Fused, M.ActionKind.SpatialSplit, M.ActionKind.Unfold, M.ActionKind.Generic}
    # the fused kernel both ways: a wave per pixel tile, and whole output rows per workgroup
    assert [a.tile_m for a in acts if a.kind == M.ActionKind.Fused] == [0, ow]
    for act in acts:
        got = run_action(act, [img, filt, np.full((b, oh, ow, f), -7, np.int32)])
        assert np.array_equal(got, want), act


def test_compose_actions_against_the_oracle(gpu):
    b, m, k, n2, n = 2, 256, 64, 1024, 64
    spec = M.ComposeMSM(b, m, k, n2, n, layouts=[None, None, KT, None])
    v, q, kmat = (synth.normal_bf16(33, 2, (b, n2, n), 0.5), synth.normal_bf16(33, 0, (b, m, k), 0.5),
                  synth.normal_bf16(33, 1, (b, n2, k), 0.5))
    want = orc.compose_msm(b, m, k, n2, n, [7, 7, 7, 6], v, q, kmat, np.zeros((b, m, n), np.float32),
                           layouts=[None, None, KT_ORC, None])
    acts = spec.actions()
    assert [(a.parts, a.tile_m) for a in acts if a.kind == M.ActionKind.Fused] == [(p, r) for p in (1, 2, 4, 8) for r in (128, 64)]
    assert acts[-1].kind == M.ActionKind.Bufferize
    for act in acts:
        got = run_action(act, [v, q, kmat, np.zeros((b, m, n), np.float32)])
        assert rel_err(got, want) < 1e-2, act


@pytest.mark.parametrize("dims,accum", [((3, 64, 64, 5, 7, 3, 3), False), ((2, 128, 64, 54, 54, 3, 3), True), ((5, 64, 64, 1, 40, 1, 1), False),
                                        ((1, 64, 64, 9, 100, 2, 3), False), ((40, 64, 64, 2, 3, 3, 2), True), ((2, 192, 64, 6, 17, 1, 3), False)])
def test_conv_over_whole_output_rows(gpu, dims, accum):
    """The fused Conv kernel whose workgroups take runs of whole output rows (tile_out over rows; the
    rows' pixels shared through LDS, 16 filters per wave): runs that cross image boundaries, rows
    that are not whole tiles of 16 pixels, several groups of 64 filters, every tap count, u8 and i8
    images, accumulating or not, against the oracle."""
    b, f, c, oh, ow, fh, fw = dims
    for img_dt, img_code, gen in ((M.u8, orc.U8, synth.uniform_u8), (M.i8, orc.I8, synth.uniform_i8)):
        spec = M.Conv(list(dims), (img_dt, M.i8, M.i32), accum=accum)
        img = gen(37, 0, (b, oh + fh - 1, ow + fw - 1, c))
        filt = synth.uniform_i8(37, 1, (f, fh, fw, c))
        out0 = (synth.uniform_i8(37, 2, (b, oh, ow, f)).astype(np.int32) * 77) if accum else np.full((b, oh, ow, f), -3, np.int32)
        nhwc = orc.make_layout([0, 2, 3, 1])
        want = orc.conv(list(dims), [img_code, orc.I8, orc.I32], img, filt, out0.copy(), accum, layouts=[nhwc, nhwc, nhwc])
        rows = [a for a in spec.actions() if a.kind == M.ActionKind.Fused and a.tile_m == ow]
        assert len(rows) == 1 and rows[0].plan().kernels == ["k_conv_rows_i8"]
        assert np.array_equal(run_action(rows[0], [img, filt, out0.copy()]), want)


@pytest.mark.parametrize("shape,dim", [((64, 1024), 1), ((3, 50, 256), 2), ((7, 128, 33), 1), ((2, 4, 640, 5), 2), ((1000, 96), 1),
                                       ((4096, 8), 0)])
def test_softmax_actions_against_the_oracle(gpu, shape, dim):
    """The reference's Softmax rewrites as actions (scheduling_sugar.rs:69-95: to_softmax_parts,
    to_softmax_parts_recompute, and the latter with its first stage split along the scan dim,
    parallel_softmax.rs:24): each runs its stages as primitive Specs and must give the Softmax."""
    x = synth.normal_f32(35, 0, shape, 3.0)
    want = orc.softmax(list(shape), dim, x)
    spec = M.Softmax(list(shape), dim)
    acts = spec.actions()
    kinds = [a.kind for a in acts]
    assert kinds[:3] == [M.ActionKind.Select, M.ActionKind.ToSoftmaxParts, M.ActionKind.ToSoftmaxPartsRecompute]
    scan = shape[dim]
    assert [a.parts for a in acts[3:]] == [p for p in (2, 4, 8, 16, 32, 64) if scan % p == 0 and scan // p >= 64]
    assert all(a.kind == M.ActionKind.ParallelSoftmax for a in acts[3:])
    for act in acts:
        got = run_action(act, [x, np.full(shape, 9.0, np.float32)])
        assert np.abs(got - want).max() < 1e-5, act
        # one launch per stage: two stages, or three with the merge of the tiles' pairs
        if act.kind != M.ActionKind.Select:
            assert act.n_steps == (3 if act.kind == M.ActionKind.ParallelSoftmax else 2), act


@pytest.mark.parametrize("shape,dim", [((6, 640), 1), ((3, 256, 40), 1), ((128, 33), 0)])
def test_children_of_the_rewrites_compute_the_spec(gpu, shape, dim):
    """mrl_action_apply: a rewrite's sub-Specs, run one after the other with mrl_run on the buffers
    their sources name (the intermediates allocated by the caller), give the Softmax."""
    x = synth.normal_f32(37, 0, shape, 3.0)
    want = orc.softmax(list(shape), dim, x)
    rewrites = [a for a in M.Softmax(list(shape), dim).actions() if a.kind != M.ActionKind.Select]
    assert len(rewrites) >= 2
    for act in rewrites:
        rw = act.apply()
        assert not rw.is_leaf() and sum(rw.intermediate_bytes) <= act.scratch_bytes   # the arena rounds each to 256 bytes
        bufs = [M.DeviceBuffer.from_numpy(x), M.DeviceBuffer.from_numpy(np.full(shape, 9.0, np.float32))]
        rw.run_device([b.ptr for b in bufs])
        got = bufs[1].to_numpy(np.float32, shape)
        for b in bufs:
            b.free()
        assert np.abs(got - want).max() < 1e-5, act


@pytest.mark.parametrize("dts,codes", [((M.u8, M.i8, M.i32), [0, 1, 5]), ((M.bf16, M.bf16, M.f32), [7, 7, 6])])
@pytest.mark.parametrize("accum", [False, True])
def test_to_accum_move_relayout_and_cast(gpu, dts, codes, accum):
    """The rewrites any Spec may take (to_accum.rs:12-60, moves.rs:49-130), on a Matmul whose A and
    C are stored column-major: each as the library runs it (mrl_run_action) and as its children
    run one by one on caller-held copies (mrl_action_apply), against the oracle on an output
    that starts from a sentinel (overwritten) or from old values (accumulated)."""
    b, m, k, n = 2, 192, 128, 136
    gen = {M.u8: synth.uniform_u8, M.i8: synth.uniform_i8, M.bf16: synth.normal_bf16}
    A, Bm = gen[dts[0]](73, 0, (b, m, k)), gen[dts[1]](73, 1, (b, k, n))
    out_np = np.int32 if dts[2] == M.i32 else np.float32
    C0 = synth.uniform_u8(73, 2, (b, m, n)).astype(out_np) if accum else np.full((b, m, n), 5, out_np)
    want = orc.matmul([b, m, k, n], codes, A, Bm, C0.copy() if accum else np.zeros((b, m, n), out_np), accum)
    layouts = [M.batched_col_major([b, m, k]), None, M.batched_col_major([b, m, n])]
    spec = M.Matmul([b, m, k, n], dts, layouts=layouts, accum=accum)
    At, C0t = np.ascontiguousarray(A.transpose(0, 2, 1)), np.ascontiguousarray(C0.transpose(0, 2, 1))
    K = M.ActionKind
    acts = [a for a in spec.actions() if a.kind in (K.ToAccum, K.MoveRelayout, K.Cast)]
    assert [(a.kind, a.tile_m) for a in acts] == ([] if accum else [(K.ToAccum, 0)]) + [(K.MoveRelayout, 0), (K.MoveRelayout, 2),
                                                                                        (K.Cast, 0), (K.Cast, 1)]
    for act in acts:
        for how in ("library", "children"):
            bufs = [M.DeviceBuffer.from_numpy(x) for x in (At, Bm, C0t)]
            if how == "library":
                act.run_device([x.ptr for x in bufs])
            else:
                act.apply().run_device([x.ptr for x in bufs])
            got = bufs[2].to_numpy(out_np, (b, n, m)).transpose(0, 2, 1)
            for x in bufs:
                x.free()
            if dts[2] == M.i32:
                assert np.array_equal(got, want), (act, how)
            else:
                assert rel_err(got, want) < 1e-5, (act, how)


def test_rewrites_of_a_conv_and_a_softmax_in_other_layouts(gpu):
    """move_relayout of every parameter of a channels-last Conv (to NCHW / FCRS copies), its casts
    and to_accum; move_relayout of a column-major Softmax's input and output."""
    K = M.ActionKind
    b, f, c, oh, ow, fh, fw = 2, 64, 32, 9, 11, 3, 3
    spec = M.Conv([b, f, c, oh, ow, fh, fw], (M.u8, M.i8, M.i32))
    img, filt = synth.uniform_u8(74, 0, (b, oh + fh - 1, ow + fw - 1, c)), synth.uniform_i8(74, 1, (f, fh, fw, c))
    nhwc = orc.make_layout([0, 2, 3, 1])
    want = orc.conv([b, f, c, oh, ow, fh, fw], [orc.U8, orc.I8, orc.I32], img, filt, np.zeros((b, oh, ow, f), np.int32),
                    layouts=[nhwc, nhwc, nhwc])
    acts = [a for a in spec.actions() if a.kind in (K.ToAccum, K.MoveRelayout, K.Cast)]
    assert len(acts) == 6
    for act in acts:
        assert np.array_equal(run_action(act, [img, filt, np.full((b, oh, ow, f), -7, np.int32)]), want), act
        bufs = [M.DeviceBuffer.from_numpy(x) for x in (img, filt, np.full((b, oh, ow, f), -7, np.int32))]
        act.apply().run_device([x.ptr for x in bufs])
        got = bufs[2].to_numpy(np.int32, (b, oh, ow, f))
        for x in bufs:
            x.free()
        assert np.array_equal(got, want), act
    shape = (48, 320)
    x = synth.normal_f32(75, 0, shape, 2.0)
    cm = M.col_major(list(shape))
    sm = M.Softmax(list(shape), 1, layouts=[cm, cm])
    moves = [a for a in sm.actions() if a.kind == K.MoveRelayout]
    assert [a.tile_m for a in moves] == [0, 1]
    for act in moves:
        got = run_action(act, [np.ascontiguousarray(x.T), np.zeros((shape[1], shape[0]), np.float32)])
        assert np.abs(got.T - orc.softmax(list(shape), 1, x)).max() < 1e-5, act


def test_children_of_the_bufferized_compose_compute_it(gpu):
    """The Compose's bufferize as sub-Specs: Matmul, Softmax, Matmul with S and P in f32 buffers of
    the caller's; with f32 intermediates the result matches the oracle's closed form to 1e-5."""
    b, m, k, n2, n = 2, 200, 128, 330, 128
    spec = M.ComposeMSM(b, m, k, n2, n, layouts=[None, None, KT, None])
    v, q, kmat = (synth.normal_bf16(38, 2, (b, n2, n), 0.5), synth.normal_bf16(38, 0, (b, m, k), 0.5),
                  synth.normal_bf16(38, 1, (b, n2, k), 0.5))
    want = orc.compose_msm(b, m, k, n2, n, [7, 7, 7, 6], v, q, kmat, np.zeros((b, m, n), np.float32),
                           layouts=[None, None, KT_ORC, None])
    rw = [a for a in spec.actions() if a.kind == M.ActionKind.Bufferize][0].apply()
    bufs = [M.DeviceBuffer.from_numpy(a) for a in (v, q, kmat, np.full((b, m, n), 7.5, np.float32))]
    rw.run_device([x.ptr for x in bufs])
    got = bufs[3].to_numpy(np.float32, (b, m, n))
    for x in bufs:
        x.free()
    assert rel_err(got, want) < 1e-5


def test_softmax_actions_keep_the_parameters_layouts(gpu):
    """Input and output in another layout than row-major: the whole-tensor rewrites take them as
    they are, the tiled one (which reads the scan dim as two dims of the same buffer) declines."""
    shape = (48, 320)
    x = synth.normal_f32(36, 0, shape, 2.0)
    want = orc.softmax(list(shape), 1, x)
    cm = M.col_major(list(shape))
    spec = M.Softmax(list(shape), 1, layouts=[cm, cm])
    acts = spec.actions()
    assert [a.kind for a in acts] == [M.ActionKind.Select, M.ActionKind.ToSoftmaxParts, M.ActionKind.ToSoftmaxPartsRecompute,
                                      M.ActionKind.MoveRelayout, M.ActionKind.MoveRelayout]
    for act in acts:
        got = run_action(act, [np.ascontiguousarray(x.T), np.zeros((shape[1], shape[0]), np.float32)])
        assert np.abs(got.T - want).max() < 1e-5, act


@pytest.mark.parametrize("dims", [(1, 136, 128, 1000, 128), (3, 200, 128, 70, 128), (2, 1, 128, 1, 128), (1, 257, 64, 65, 64),
                                  (2, 300, 32, 129, 32), (2, 70, 96, 333, 40)])
def test_compose_query_blocks_on_ragged_shapes(gpu, dims):
    """Both query-block sizes of the fused kernel (tile_out over the Compose's rows: 128 or 64
    queries per workgroup) and every key share count, on sequence lengths that are multiples of
    neither, head dims the kernel has and one it pads: against the oracle."""
    b, m, k, n2, n = dims
    spec = M.ComposeMSM(b, m, k, n2, n, layouts=[None, None, KT, None])
    v, q, kmat = (synth.normal_bf16(34, 2, (b, n2, n), 0.5), synth.normal_bf16(34, 0, (b, m, k), 0.5),
                  synth.normal_bf16(34, 1, (b, n2, k), 0.5))
    want = orc.compose_msm(b, m, k, n2, n, [7, 7, 7, 6], v, q, kmat, np.zeros((b, m, n), np.float32),
                           layouts=[None, None, KT_ORC, None])
    fused = [a for a in spec.actions() if a.kind == M.ActionKind.Fused]
    assert {a.tile_m for a in fused} == {64, 128}
    for act in fused:
        sentinel = np.full((b, m, n), 7.5, np.float32)
        assert rel_err(run_action(act, [v, q, kmat, sentinel]), want) < 1e-2, act


def test_actions_of_the_benchmark_configurations_agree(gpu):
    """C2, C4, C5 at full size: every action gives what Select gives (bit for bit for the integer
    Specs; C3's eight tiles take seconds each on the slower ones and are covered by the 512 x 384 x 256 case)."""
    a, b = synth.uniform_u8(2, 0, (1, 4096, 4096)), synth.uniform_i8(2, 1, (1, 4096, 4096))
    acts = M.MatmulAccum([1, 4096, 4096, 4096], (M.u8, M.i8, M.i32)).actions()
    ref = run_action(acts[0], [a, b, np.ones((1, 4096, 4096), np.int32)])
    for act in acts[1:]:
        assert np.array_equal(run_action(act, [a, b, np.ones((1, 4096, 4096), np.int32)]), ref), act
    img, filt = synth.uniform_u8(4, 0, (32, 56, 56, 64)), synth.uniform_i8(4, 1, (64, 3, 3, 64))
    acts = M.Conv([32, 64, 64, 54, 54, 3, 3], (M.u8, M.i8, M.i32)).actions()
    ref = run_action(acts[0], [img, filt, np.zeros((32, 54, 54, 64), np.int32)])
    for act in acts[1:]:
        if act.kind != M.ActionKind.Generic:     # 2.3 ms a launch, and held against the oracle above
            assert np.array_equal(run_action(act, [img, filt, np.zeros((32, 54, 54, 64), np.int32)]), ref), act
    v, q, kmat = (synth.normal_bf16(5, 2, (16, 2048, 128), 0.5), synth.normal_bf16(5, 0, (16, 2048, 128), 0.5),
                  synth.normal_bf16(5, 1, (16, 2048, 128), 0.5))
    acts = M.ComposeMSM(16, 2048, 128, 2048, 128, layouts=[None, None, KT, None]).actions()
    ref = run_action(acts[0], [v, q, kmat, np.zeros((16, 2048, 128), np.float32)])
    for act in acts[1:]:
        assert rel_err(run_action(act, [v, q, kmat, np.zeros((16, 2048, 128), np.float32)]), ref) < 1e-2, act
