"""Conv Spec on the MI355X against the CPU oracle (bit exact), through the C ABI."""
import numpy as np
import pytest

import morello_amd as M
import orc
from gpu_util import run_spec
from morello_amd import synth

pytestmark = pytest.mark.gpu

NHWC = orc.make_layout([0, 2, 3, 1])


def nhwc_inputs(seed, b, f, c, oh, ow, fh, fw, dt_img=M.u8):
    gen = synth.uniform_u8 if dt_img == M.u8 else synth.uniform_i8
    img = gen(seed, 0, (b, oh + fh - 1, ow + fw - 1, c))      # NHWC buffer
    filt = synth.uniform_i8(seed, 1, (f, fh, fw, c))          # KRSC buffer
    return img, filt


@pytest.mark.parametrize("dt_img", [M.u8, M.i8])
@pytest.mark.parametrize("shape,accum", [
    ((1, 64, 64, 6, 6, 3, 3), False),
    ((2, 64, 64, 9, 11, 3, 3), True),
    ((1, 8, 8, 1, 1, 3, 3), False),      # examples/simple_conv_x86.rs shape
    ((2, 5, 7, 4, 3, 2, 3), True),       # ragged channels: generic kernel
    ((3, 64, 64, 54, 54, 3, 3), False),  # benchmark configuration 4 at batch 3
    ((1, 64, 64, 5, 5, 1, 1), False),    # 1x1 filter
    ((2, 128, 64, 9, 11, 3, 3), True),   # two groups of 64 filters on the fused kernel
    ((1, 192, 128, 7, 7, 1, 1), False),  # three groups, two 64-channel slabs
    ((2, 64, 256, 5, 6, 1, 1), True),    # four slabs
    ((1, 128, 64, 6, 6, 3, 1), False),   # three slabs (3x1 filter)
    ((1, 64, 128, 6, 5, 1, 3), True),    # six slabs (1x3 filter over 128 channels)
])
def test_conv_nhwc_bit_exact(gpu, dt_img, shape, accum):
    b, f, c, oh, ow, fh, fw = shape
    img, filt = nhwc_inputs(101, *shape, dt_img=dt_img)
    out0 = (synth.uniform_u8(101, 2, (b, oh, ow, f)).astype(np.int32) - 50) if accum else np.zeros((b, oh, ow, f), np.int32)
    dts = (dt_img, M.i8, M.i32)
    got = run_spec(M.Conv(shape, dts, accum=accum), [img, filt, out0])
    want = orc.conv(list(shape), [int(d) for d in dts], img, filt, out0.copy(), accum, layouts=[NHWC] * 3)
    assert np.array_equal(got, want)


def test_conv_nchw_layout_generic(gpu):
    shape = (2, 6, 5, 4, 4, 3, 3)
    b, f, c, oh, ow, fh, fw = shape
    img = synth.uniform_u8(111, 0, (b, c, oh + 2, ow + 2))
    filt = synth.uniform_i8(111, 1, (f, c, fh, fw))
    rm = [M.row_major(s) for s in M.Conv(shape, (M.u8, M.i8, M.i32)).parameter_shapes()]
    got = run_spec(M.Conv(shape, (M.u8, M.i8, M.i32), layouts=rm), [img, filt, np.zeros((b, f, oh, ow), np.int32)])
    want = orc.conv(list(shape), [0, 1, 5], img, filt, np.zeros((b, f, oh, ow), np.int32))
    assert np.array_equal(got, want)


@pytest.mark.parametrize("accum", [False, True])
def test_conv_nchw_layout_on_the_matrix_cores(gpu, accum):
    """NCHW image and output, FCRS filters (all row-major) at a shape the matrix-core kernel
    takes: the tensors are moved to channels-last and back around it.  Mixed: only the output
    in NCHW."""
    shape = (3, 64, 64, 9, 11, 3, 3)
    b, f, c, oh, ow, fh, fw = shape
    img = synth.uniform_u8(112, 0, (b, c, oh + 2, ow + 2))
    filt = synth.uniform_i8(112, 1, (f, c, fh, fw))
    out0 = synth.uniform_u8(112, 2, (b, f, oh, ow)).astype(np.int32) if accum else np.zeros((b, f, oh, ow), np.int32)
    want = orc.conv(list(shape), [0, 1, 5], img, filt, out0.copy(), accum)
    rm = [M.row_major(s) for s in M.Conv(shape, (M.u8, M.i8, M.i32)).parameter_shapes()]
    got = run_spec(M.Conv(shape, (M.u8, M.i8, M.i32), layouts=rm, accum=accum), [img, filt, out0.copy()])
    assert np.array_equal(got, want)
    nhwc_img = np.ascontiguousarray(img.transpose(0, 2, 3, 1))
    krsc = np.ascontiguousarray(filt.transpose(0, 2, 3, 1))
    got = run_spec(M.Conv(shape, (M.u8, M.i8, M.i32), layouts=[None, None, rm[2]], accum=accum),
                   [nhwc_img, krsc, out0.copy()])
    assert np.array_equal(got, want)


@pytest.mark.parametrize("shape,accum", [((3, 64, 64, 9, 11, 3, 3), True), ((2, 128, 64, 13, 7, 2, 2), False),
                                         ((5, 192, 128, 6, 6, 1, 2), True), ((1, 64, 64, 54, 54, 3, 3), False)])
@pytest.mark.parametrize("img_dt,img_code,gen", [(M.u8, 0, synth.uniform_u8), (M.i8, 1, synth.uniform_i8)])
def test_fused_conv_writes_a_row_major_output_in_place(gpu, shape, accum, img_dt, img_code, gen):
    """A dense NCHW output of a shape the fused kernel takes: the kernel writes the planes of
    filters itself (16 consecutive pixels of a plane per lane group, tiles that cross from one
    image into the next included), no Move of the output remains in the plan; bit for bit, with
    old values when accumulating and a sentinel otherwise."""
    b, f, c, oh, ow, fh, fw = shape
    img = gen(113, 0, (b, oh + fh - 1, ow + fw - 1, c))
    filt = synth.uniform_i8(113, 1, (f, fh, fw, c))
    out0 = (synth.uniform_i8(113, 2, (b, f, oh, ow)).astype(np.int32) * 999) if accum else np.full((b, f, oh, ow), -5, np.int32)
    spec = M.Conv(list(shape), (img_dt, M.i8, M.i32), layouts=[None, None, M.row_major([b, f, oh, ow])], accum=accum)
    assert spec.plan().kernels == ["k_conv_i8"]
    want = orc.conv(list(shape), [img_code, 1, 5], img, filt, out0.copy(), accum, layouts=[NHWC, NHWC, None])
    assert np.array_equal(run_spec(spec, [img, filt, out0.copy()]), want)


@pytest.mark.parametrize("dts,codes", [((M.u8, M.i8, M.i32), [0, 1, 5]), ((M.i8, M.i8, M.i32), [1, 1, 5]),
                                        ((M.bf16, M.bf16, M.f32), [7, 7, 6]), ((M.f32, M.f32, M.f32), [6, 6, 6])])
@pytest.mark.parametrize("shape,accum", [((2, 64, 3, 20, 37, 5, 5), False), ((3, 32, 3, 9, 50, 3, 3), True),
                                         ((2, 80, 5, 17, 15, 2, 3), True), ((1, 16, 1, 33, 33, 3, 3), False)])
@pytest.mark.parametrize("which", ["all", "image", "output"])
def test_first_layer_conv_on_row_major_tensors(gpu, dts, codes, shape, accum, which):
    """A first layer on NCHW tensors: the kernel that forms its windows in LDS fetches a patch's
    bytes from planes of channels as well as from channels-last pixels, and writes planes of
    filters from its accumulators; only the (small) filters are moved.  All three tensors
    row-major, or the image alone, or the output alone."""
    b, f, c, oh, ow, fh, fw = shape
    gen = {M.u8: synth.uniform_u8, M.i8: synth.uniform_i8, M.bf16: synth.normal_bf16, M.f32: synth.normal_f32}
    img = gen[dts[0]](114, 0, (b, c, oh + fh - 1, ow + fw - 1))
    filt = gen[dts[1]](114, 1, (f, c, fh, fw))
    floats = dts[2] == M.f32
    out0 = synth.uniform_u8(114, 2, (b, f, oh, ow)).astype(np.float32 if floats else np.int32) - 90
    want = orc.conv(list(shape), codes, img, filt, out0.copy(), accum)     # everything row-major
    spec0 = M.Conv(list(shape), dts)
    rm = [M.row_major(s) for s in spec0.parameter_shapes()]
    cl = lambda a: np.ascontiguousarray(a.transpose(0, 2, 3, 1))
    if which == "all":
        layouts, bufs, back = rm, [img, filt, out0.copy()], lambda a: a
    elif which == "image":
        layouts, bufs, back = [rm[0], None, None], [img, cl(filt), cl(out0)], lambda a: a.transpose(0, 3, 1, 2)
    else:
        layouts, bufs, back = [None, None, rm[2]], [cl(img), cl(filt), out0.copy()], lambda a: a
    spec = M.Conv(list(shape), dts, layouts=layouts, accum=accum)
    # (filters of one channel are channels-last as they stand)
    assert spec.plan().kernels == (["k_move_rows", "k_conv_windows"] if which == "all" and c > 1 else ["k_conv_windows"]), spec.plan()
    got = back(run_spec(spec, bufs))
    if floats:
        assert float(np.abs(got.astype(np.float64) - want).max() / np.abs(want).max()) < 1e-5
    else:
        assert np.array_equal(got, want)


CONV_GEN = {M.u8: synth.uniform_u8, M.i8: synth.uniform_i8, M.bf16: synth.normal_bf16, M.f32: synth.uniform_f32}


@pytest.mark.parametrize("dts,codes", [((M.u8, M.i8, M.i32), [0, 1, 5]), ((M.i8, M.i8, M.i32), [1, 1, 5]),
                                        ((M.bf16, M.bf16, M.f32), [7, 7, 6]), ((M.f32, M.f32, M.f32), [6, 6, 6])])
@pytest.mark.parametrize("shape,accum", [
    ((2, 48, 24, 20, 17, 3, 3), True),     # window of 216 elements: rows padded to whole chunks
    ((1, 32, 3, 40, 40, 7, 7), False),     # three channels: the window is gathered element by element
    ((3, 128, 128, 9, 9, 1, 1), True),     # 1x1 filter: the image is the left operand as it lies
    ((2, 64, 32, 12, 12, 5, 5), False),    # 64 filters but not the fused kernel's channel count
    ((1, 7, 20, 30, 30, 2, 4), True),      # few filters, uneven window
    ((5, 96, 64, 14, 14, 3, 3), False),    # 64 channels but not the fused kernel's filter count
    ((2, 130, 128, 17, 19, 3, 3), True),   # implicit for every dtype: 18 slabs of 64 channels, ragged everywhere
    ((1, 64, 16, 70, 70, 5, 5), False),    # 16 channels: implicit for int8 too, windows of 400 elements
    ((3, 256, 32, 9, 9, 2, 2), True),
])
def test_conv_as_matmul(gpu, dts, codes, shape, accum):
    """Shapes outside the fused kernel's run as a Matmul on the matrix cores, for every dtype triple
    those take: implicitly (the kernel reads the windows where they lie) when a pixel's channels
    are whole 16-byte chunks, through windows unfolded into rows otherwise."""
    b, f, c, oh, ow, fh, fw = shape
    img = CONV_GEN[dts[0]](131, 0, (b, oh + fh - 1, ow + fw - 1, c))
    filt = CONV_GEN[dts[1]](131, 1, (f, fh, fw, c))
    out_np = np.int32 if dts[2] == M.i32 else np.float32
    out0 = synth.uniform_u8(131, 2, (b, oh, ow, f)).astype(out_np) if accum else np.zeros((b, oh, ow, f), out_np)
    got = run_spec(M.Conv(shape, dts, accum=accum), [img, filt, out0.copy()])
    want = orc.conv(list(shape), codes, img, filt, out0.copy(), accum, layouts=[NHWC] * 3)
    if dts[2] == M.i32:
        assert np.array_equal(got, want)
    else:
        err = float(np.abs(got.astype(np.float64) - want).max() / np.abs(want).max())
        assert err < 1e-5


@pytest.mark.parametrize("dts,codes", [((M.u8, M.i8, M.i32), [0, 1, 5]), ((M.i8, M.i8, M.i32), [1, 1, 5]),
                                        ((M.bf16, M.bf16, M.f32), [7, 7, 6]), ((M.f32, M.f32, M.f32), [6, 6, 6])])
@pytest.mark.parametrize("shape,accum", [((8, 512, 512, 5, 5, 3, 3), False), ((8, 512, 512, 5, 5, 3, 3), True),
                                         ((3, 200, 256, 6, 7, 4, 4), True)])
def test_deep_conv_on_small_images_shares_its_windows_out(gpu, dts, codes, shape, accum):
    """Few output tiles and windows of thousands of elements: the implicit Matmul runs over
    slices of the window as batch entries whose partial results are then summed in slice order
    (exact for integers), into an output that may hold old values."""
    b, f, c, oh, ow, fh, fw = shape
    plan = M.Conv(shape, dts, accum=accum).plan()
    assert plan.kernels == ["k_gemm", "k_sum_splits"] and plan.steps[0].grid[1] > 1
    img = CONV_GEN[dts[0]](133, 0, (b, oh + fh - 1, ow + fw - 1, c))
    filt = CONV_GEN[dts[1]](133, 1, (f, fh, fw, c))
    out_np = np.int32 if dts[2] == M.i32 else np.float32
    out0 = synth.uniform_u8(133, 2, (b, oh, ow, f)).astype(out_np) if accum else np.zeros((b, oh, ow, f), out_np)
    got = run_spec(M.Conv(shape, dts, accum=accum), [img, filt, out0.copy()])
    want = orc.conv(list(shape), codes, img, filt, out0.copy(), accum, layouts=[NHWC] * 3)
    if dts[2] == M.i32:
        assert np.array_equal(got, want)
    else:
        err = float(np.abs(got.astype(np.float64) - want).max() / np.abs(want).max())
        assert err < 1e-5


@pytest.mark.parametrize("shape,accum", [
    ((2, 64, 3, 20, 37, 7, 7), False),    # a first layer: three k steps, ragged tiles both ways
    ((4, 16, 1, 30, 30, 3, 3), True),     # one channel, one k step, sixteen filters
    ((3, 48, 4, 8, 33, 3, 3), False),     # runs that are whole dwords
    ((2, 80, 3, 17, 15, 5, 5), True),     # two groups of filters, the second of sixteen; two k steps
    ((1, 128, 24, 5, 50, 3, 3), False),   # 24 channels: runs of 72 bytes, four k steps
    ((64, 32, 2, 1, 3, 2, 9), True),      # three output pixels per image
    ((1, 64, 5, 30, 30, 1, 1), False),    # 1 x 1 filters
    ((2, 32, 3, 11, 40, 9, 3), False),    # tall filters
    ((3, 32, 20, 20, 33, 3, 3), True),    # pixels of a chunk and a quarter, windows of 180 bytes
    ((2, 16, 10, 9, 40, 2, 5), False),    # two runs of 50 bytes
])
@pytest.mark.parametrize("img_dt,img_code,gen", [(M.u8, 0, synth.uniform_u8), (M.i8, 1, synth.uniform_i8)])
def test_conv_with_few_channels_forms_its_windows_in_lds(gpu, shape, accum, img_dt, img_code, gen):
    """Pixels that are not whole 16-byte chunks, windows of at most 384 bytes (runs padded to
    dwords), filters in 16s: one kernel forms the windows in LDS and multiplies them.  Against
    the oracle, bit for bit, with old values in the output when accumulating and a sentinel
    otherwise; once more with the image and the filters at addresses that are not 16-byte aligned."""
    b, f, c, oh, ow, fh, fw = shape
    spec = M.Conv(list(shape), (img_dt, M.i8, M.i32), accum=accum)
    assert spec.plan().kernels == ["k_conv_windows"]
    img = gen(134, 0, (b, oh + fh - 1, ow + fw - 1, c))
    filt = synth.uniform_i8(134, 1, (f, fh, fw, c))
    out0 = (synth.uniform_i8(134, 2, (b, oh, ow, f)).astype(np.int32) * 1001) if accum else np.full((b, oh, ow, f), -5, np.int32)
    want = orc.conv(list(shape), [img_code, 1, 5], img, filt, out0.copy(), accum, layouts=[NHWC] * 3)
    assert np.array_equal(run_spec(spec, [img, filt, out0.copy()]), want)
    # the same from unaligned addresses: the operands 3 and 5 bytes into their buffers
    pad_img, pad_filt = np.zeros(img.size + 16, img.dtype), np.zeros(filt.size + 16, np.int8)
    pad_img[3:3 + img.size], pad_filt[5:5 + filt.size] = img.reshape(-1), filt.reshape(-1)
    bufs = [M.DeviceBuffer.from_numpy(x) for x in (pad_img, pad_filt, out0)]
    spec.run_device([bufs[0].ptr + 3, bufs[1].ptr + 5, bufs[2].ptr])
    got = bufs[2].to_numpy(np.int32, (b, oh, ow, f))
    for x in bufs:
        x.free()
    assert np.array_equal(got, want)


@pytest.mark.parametrize("shape,accum", [
    ((41, 32, 32, 40, 41, 3, 3), False),  # 32 channels, 3 x 3: 288 bytes, the last k step half empty
    ((30, 32, 16, 50, 45, 4, 4), True),   # 16 channels (pixels of one chunk), 4 x 4: four whole k steps
    ((71, 48, 48, 30, 31, 2, 2), False),  # 48 channels: runs of 96 bytes, k steps across runs; three tiles of filters
    ((11, 16, 32, 90, 70, 2, 5), True),   # 320 bytes, five k steps
    ((4, 16, 64, 130, 129, 2, 2), False), # 64 channels under 2 x 2 with 16 filters (the 64-channel kernel wants filters in 64s)
])
@pytest.mark.parametrize("dts,codes", [((M.u8, M.i8, M.i32), [0, 1, 5]), ((M.i8, M.i8, M.i32), [1, 1, 5]), ((M.bf16, M.bf16, M.f32), [7, 7, 6])])
def test_early_layer_conv_with_the_filters_in_registers(gpu, shape, accum, dts, codes):
    """Pixels of whole 16-byte chunks, windows of up to 320 bytes, up to 48 filters (and 9216 bytes of
    filters times window), 65536 pixels or more: the kernel that keeps the filter bank in registers.  Integers bit for bit, bf16 to 1e-5
    of the oracle; an infinity in a bf16 image reaches the outputs whose windows hold it as an
    infinity (the chunks past the window's end are zero on both sides)."""
    b, f, c, oh, ow, fh, fw = shape
    if dts[0] == M.bf16:
        c //= 2   # the same bytes per pixel
    shape = (b, f, c, oh, ow, fh, fw)
    spec = M.Conv(list(shape), dts, accum=accum)
    assert spec.plan().kernels == ["k_conv_small"], spec.plan()
    floats = dts[0] == M.bf16
    gen = {M.u8: synth.uniform_u8, M.i8: synth.uniform_i8, M.bf16: synth.normal_bf16}
    img, filt = gen[dts[0]](138, 0, (b, oh + fh - 1, ow + fw - 1, c)), gen[dts[1]](138, 1, (f, fh, fw, c))
    out0 = synth.uniform_u8(138, 2, (b, oh, ow, f)).astype(np.float32 if floats else np.int32) - 100
    want = orc.conv(list(shape), codes, img, filt, out0.copy(), accum, layouts=[NHWC] * 3)
    got = run_spec(spec, [img, filt, out0.copy()])
    if not floats:
        assert np.array_equal(got, want)
        return
    assert float(np.abs(got.astype(np.float64) - want).max() / np.abs(want).max()) < 1e-5
    img = img.copy()
    img[b - 1, oh + fh - 2, ow + fw - 2, c - 1] = 0x7f80       # +inf in the last pixel's last channel
    want = orc.conv(list(shape), codes, img, filt, out0.copy(), accum, layouts=[NHWC] * 3)
    got = run_spec(spec, [img, filt, out0.copy()])
    assert np.array_equal(np.isnan(got), np.isnan(want)) and np.array_equal(np.isinf(got), np.isinf(want))


@pytest.mark.parametrize("shape,accum", [
    ((2, 64, 3, 20, 37, 5, 5), False),    # runs of 60 bytes, five k steps
    ((4, 16, 1, 30, 30, 3, 3), True),     # runs of 12 bytes
    ((2, 80, 3, 17, 15, 3, 3), True),     # two groups of filters
    ((1, 64, 5, 30, 30, 1, 1), False),    # 1 x 1 filters, runs of 20 bytes
    ((2, 32, 6, 9, 21, 3, 3), False),     # 24 bytes a pixel
    ((3, 48, 2, 33, 5, 9, 2), True),      # tall filters, ragged tiles
])
def test_f32_conv_with_few_channels_forms_its_windows_in_lds(gpu, shape, accum):
    """The same kernel on f32 operands: four MFMAs of k = 4 per 64 bytes of window, windows of up
    to 640 bytes.  To 1e-5 of the oracle (f32 sums in another order), and NaN and infinity reach
    exactly the outputs whose windows hold them."""
    b, f, c, oh, ow, fh, fw = shape
    spec = M.Conv(list(shape), (M.f32, M.f32, M.f32), accum=accum)
    assert spec.plan().kernels == ["k_conv_windows"] and "KIND = 3" in spec.plan().steps[0].kernel
    img = synth.normal_f32(136, 0, (b, oh + fh - 1, ow + fw - 1, c))
    filt = synth.normal_f32(136, 1, (f, fh, fw, c))
    out0 = synth.uniform_u8(136, 2, (b, oh, ow, f)).astype(np.float32) if accum else np.full((b, oh, ow, f), 7, np.float32)
    want = orc.conv(list(shape), [6, 6, 6], img, filt, out0.copy(), accum, layouts=[NHWC] * 3)
    got = run_spec(spec, [img, filt, out0.copy()])
    assert float(np.abs(got.astype(np.float64) - want).max() / np.abs(want).max()) < 1e-5
    img = img.copy()
    img[0, 0, 0, 0] = np.nan
    img[b - 1, oh + fh - 2, ow + fw - 2, c - 1] = np.inf
    want = orc.conv(list(shape), [6, 6, 6], img, filt, out0.copy(), accum, layouts=[NHWC] * 3)
    got = run_spec(spec, [img, filt, out0.copy()])
    assert np.array_equal(np.isfinite(got), np.isfinite(want))
    ok = np.isfinite(want)
    assert float(np.abs(got[ok].astype(np.float64) - want[ok]).max() / np.abs(want[ok]).max()) < 1e-5


def test_f32_first_layer_conv_at_its_longest_window(gpu):
    """3 channels, 7 x 7 filters: runs of 84 bytes, 588 bytes a window, ten k steps of 64."""
    shape = (2, 64, 3, 20, 37, 7, 7)
    spec = M.Conv(list(shape), (M.f32, M.f32, M.f32))
    assert spec.plan().kernels == ["k_conv_windows"] and "KS = 10" in spec.plan().steps[0].kernel
    img, filt = synth.normal_f32(137, 0, (2, 26, 43, 3)), synth.normal_f32(137, 1, (64, 7, 7, 3))
    out0 = np.full((2, 20, 37, 64), 7, np.float32)
    want = orc.conv(list(shape), [6, 6, 6], img, filt, out0.copy(), False, layouts=[NHWC] * 3)
    got = run_spec(spec, [img, filt, out0])
    assert float(np.abs(got.astype(np.float64) - want).max() / np.abs(want).max()) < 1e-5


@pytest.mark.parametrize("shape,accum", [
    ((2, 64, 3, 20, 37, 7, 7), False),    # a first layer in bf16: runs of 42 bytes padded to 44, five k steps
    ((4, 16, 1, 30, 30, 3, 3), True),     # runs of 6 bytes
    ((2, 80, 3, 17, 15, 5, 5), True),     # two groups of filters
    ((1, 64, 5, 30, 30, 1, 1), False),    # 1 x 1 filters, runs of 10 bytes
    ((2, 32, 12, 9, 21, 3, 3), False),    # 24 bytes a pixel
    ((2, 32, 10, 9, 21, 3, 3), True),     # 20 bytes a pixel, windows of 180 bytes
])
def test_bf16_conv_with_few_channels_forms_its_windows_in_lds(gpu, shape, accum):
    """The same kernel on bf16 operands (f32 sums, as a bf16 Matmul's).  An image that holds a NaN
    and an infinity: they reach exactly the outputs whose windows contain them, not their
    neighbours through the padding of the windows' runs."""
    b, f, c, oh, ow, fh, fw = shape
    spec = M.Conv(list(shape), (M.bf16, M.bf16, M.f32), accum=accum)
    assert spec.plan().kernels == ["k_conv_windows"] and "KIND = 2" in spec.plan().steps[0].kernel
    img = synth.normal_bf16(135, 0, (b, oh + fh - 1, ow + fw - 1, c))
    filt = synth.normal_bf16(135, 1, (f, fh, fw, c))
    out0 = synth.uniform_u8(135, 2, (b, oh, ow, f)).astype(np.float32) if accum else np.full((b, oh, ow, f), 7, np.float32)
    want = orc.conv(list(shape), [7, 7, 6], img, filt, out0.copy(), accum, layouts=[NHWC] * 3)
    got = run_spec(spec, [img, filt, out0.copy()])
    assert float(np.abs(got.astype(np.float64) - want).max() / np.abs(want).max()) < 1e-5
    img = img.copy()
    img[0, 0, 0, 0] = 0x7fc0                                   # NaN in the first pixel's first channel
    img[b - 1, oh + fh - 2, ow + fw - 2, c - 1] = 0x7f80       # +inf in the last pixel's last channel
    want = orc.conv(list(shape), [7, 7, 6], img, filt, out0.copy(), accum, layouts=[NHWC] * 3)
    got = run_spec(spec, [img, filt, out0.copy()])
    assert np.array_equal(np.isfinite(got), np.isfinite(want))
    ok = np.isfinite(want)
    assert float(np.abs(got[ok].astype(np.float64) - want[ok]).max() / np.abs(want[ok]).max()) < 1e-5


def test_conv_as_matmul_from_nchw(gpu):
    """Row-major (NCHW / FCRS) tensors at a shape the unfolded path takes: moved to channels-last
    and back around it."""
    shape = (2, 40, 12, 18, 21, 3, 2)
    b, f, c, oh, ow, fh, fw = shape
    img = synth.uniform_u8(132, 0, (b, c, oh + fh - 1, ow + fw - 1))
    filt = synth.uniform_i8(132, 1, (f, c, fh, fw))
    out0 = synth.uniform_u8(132, 2, (b, f, oh, ow)).astype(np.int32)
    rm = [M.row_major(s) for s in M.Conv(shape, (M.u8, M.i8, M.i32)).parameter_shapes()]
    got = run_spec(M.Conv(shape, (M.u8, M.i8, M.i32), layouts=rm, accum=True), [img, filt, out0.copy()])
    assert np.array_equal(got, orc.conv(list(shape), [0, 1, 5], img, filt, out0.copy(), True))


def test_conv_as_matmul_in_several_passes(gpu):
    """Three channels (windows are unfolded into rows) and more windows than one pass unfolds
    (1 GiB of rows): the batch is cut into passes.  Checked on the first, a middle and the last
    image and through the per-image checksum."""
    # 62 500 windows of 147 bytes padded to 160 per image: 107 images per pass, so passes of 107 and 3
    b, f, c, oh, ow, fh, fw = shape = (110, 8, 3, 250, 250, 7, 7)
    img = synth.uniform_u8(133, 0, (b, oh + fh - 1, ow + fw - 1, c))
    filt = synth.uniform_i8(133, 1, (f, fh, fw, c))
    got = run_spec(M.Conv(shape, (M.u8, M.i8, M.i32)), [img, filt, np.zeros((b, oh, ow, f), np.int32)])
    for bi in (0, 106, 107, 109):
        sub = (1,) + shape[1:]
        want = orc.conv(list(sub), [0, 1, 5], img[bi:bi + 1], filt, np.zeros((1, oh, ow, f), np.int32), layouts=[NHWC] * 3)
        assert np.array_equal(got[bi:bi + 1], want)
    fsum = filt.astype(np.int64).sum(axis=0)  # [r,s,c]
    for bi in range(b):
        im = img[bi].astype(np.int64)
        total = 0
        for r in range(fh):
            for s in range(fw):
                total += int((im[r:r + oh, s:s + ow, :].sum(axis=(0, 1)) * fsum[r, s]).sum())
        assert int(got[bi].astype(np.int64).sum()) == total


def test_implicit_conv_at_a_large_image_count(gpu):
    """The implicit Matmul form at 2.3 million windows (row offsets of the left operand up to
    150 MB into the image): first and last image against the oracle, all through the checksum."""
    b, f, c, oh, ow, fh, fw = shape = (36, 8, 64, 250, 250, 4, 4)
    img = synth.uniform_u8(134, 0, (b, oh + fh - 1, ow + fw - 1, c))
    filt = synth.uniform_i8(134, 1, (f, fh, fw, c))
    got = run_spec(M.Conv(shape, (M.u8, M.i8, M.i32)), [img, filt, np.zeros((b, oh, ow, f), np.int32)])
    for bi in (0, 35):
        sub = (1,) + shape[1:]
        want = orc.conv(list(sub), [0, 1, 5], img[bi:bi + 1], filt, np.zeros((1, oh, ow, f), np.int32), layouts=[NHWC] * 3)
        assert np.array_equal(got[bi:bi + 1], want)
    fsum = filt.astype(np.int64).sum(axis=0)
    for bi in range(b):
        im = img[bi].astype(np.int64)
        total = 0
        for r in range(fh):
            for s in range(fw):
                total += int((im[r:r + oh, s:s + ow, :].sum(axis=(0, 1)) * fsum[r, s]).sum())
        assert int(got[bi].astype(np.int64).sum()) == total


def test_conv_full_size_properties(gpu):
    """benchmark configuration 4 (32x56x56x64 -> 64, 3x3): a few images against the oracle, every
    image through a checksum (sum over filters and pixels, computed in int64 from box sums),
    and the extreme-value bound 576*255*128."""
    shape = (32, 64, 64, 54, 54, 3, 3)
    b, f, c, oh, ow, fh, fw = shape
    img, filt = nhwc_inputs(121, *shape)
    got = run_spec(M.Conv(shape, (M.u8, M.i8, M.i32)), [img, filt, np.zeros((b, oh, ow, f), np.int32)])
    for bi in (0, 17, 31):
        sub = (1,) + shape[1:]
        want = orc.conv(list(sub), [0, 1, 5], img[bi:bi + 1], filt, np.zeros((1, oh, ow, f), np.int32), layouts=[NHWC] * 3)
        assert np.array_equal(got[bi:bi + 1], want)
    # sum_{y,x,f} out = sum_{r,s,c} (sum_f filt[f,r,s,c]) * (sum of the image window shifted by r,s)
    fsum = filt.astype(np.int64).sum(axis=0)  # [r,s,c]
    for bi in range(b):
        im = img[bi].astype(np.int64)
        total = 0
        for r in range(fh):
            for s in range(fw):
                total += int((im[r:r + oh, s:s + ow, :].sum(axis=(0, 1)) * fsum[r, s]).sum())
        assert int(got[bi].astype(np.int64).sum()) == total
    img[:] = 255
    filt[:] = -128
    got = run_spec(M.Conv((1,) + shape[1:], (M.u8, M.i8, M.i32)), [img[:1], filt, np.zeros((1, oh, ow, f), np.int32)])
    assert (got == -18800640).all()


@pytest.mark.parametrize("accum", [False, True])
def test_conv_with_bf16_output(gpu, accum):
    """Conv bf16 x bf16 -> bf16 (NHWC / KRSC buffers): f32 sums, one rounding (see
    test_matmul_with_bf16_output)."""
    b, f, c, oh, ow, fh, fw = 2, 24, 40, 9, 11, 3, 2
    img = synth.normal_bf16(78, 0, (b, oh + fh - 1, ow + fw - 1, c), 0.5)
    filt = synth.normal_bf16(78, 1, (f, fh, fw, c), 0.5)
    out0 = synth.normal_bf16(78, 2, (b, oh, ow, f), 2.0) if accum else np.zeros((b, oh, ow, f), np.uint16)
    want = synth.bf16_bits_to_f32(orc.conv([b, f, c, oh, ow, fh, fw], [7, 7, 7], img, filt, out0.copy(), accum=accum,
                                           layouts=[NHWC, NHWC, NHWC]))
    got = synth.bf16_bits_to_f32(run_spec(M.Conv([b, f, c, oh, ow, fh, fw], (M.bf16, M.bf16, M.bf16), accum=accum),
                                          [img, filt, out0.copy()]))
    assert (got == want).mean() > 0.97
    assert np.all(np.abs(got - want) <= 2.0 ** -7 * np.maximum(np.abs(want), 2.0 ** -10 * np.abs(want).max()))
