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
