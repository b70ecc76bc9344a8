"""Pins the CPU oracle (oracle/morello_oracle.c) before anything is compared against it.

Every check here uses something the oracle did not produce: numpy/scipy library routines,
closed forms, brute force in Python integers, or C that the reference itself holds (the
emitted kernel quoted in examples/simple_matmul_x86.rs and the x86 partials), compiled into
oracle/_ref when the reference checkout is present.  No GPU needed.
"""
import ctypes as C

import numpy as np
import pytest
import scipy.signal
import scipy.special

import orc
from morello_amd import synth

INT_DTYPES = [orc.U8, orc.I8, orc.U16, orc.I16, orc.U32, orc.I32]


def rand_ints(dt, seed, tid, shape):
    raw = synth.raw_u64(seed, tid, int(np.prod(shape)))
    return raw.astype(np.uint64).astype(orc.NP[dt] if orc.NP[dt]().itemsize == 8 else np.uint64).astype(orc.NP[dt]).reshape(shape)


def np_matmul_mod(a, b, c0, out_dt):
    """Independent integer Matmul: cast inputs to the output dtype (wrapping), multiply in
    Python-sized integers via int64 on small shapes, wrap to the output dtype."""
    t = orc.NP[out_dt]
    a64 = a.astype(t).astype(np.int64)
    b64 = b.astype(t).astype(np.int64)
    bits = t().itemsize * 8
    # keep products small enough for int64: reduce inputs modulo 2^bits first (done above)
    acc = c0.astype(np.int64).astype(object) + np.matmul(a64.astype(object), b64.astype(object))
    mod = 1 << bits
    wrapped = np.vectorize(lambda v: int(v) % mod, otypes=[object])(acc)
    return np.array(wrapped, dtype=np.uint64).astype(np.dtype(f"u{bits // 8}")).view(t)


@pytest.mark.parametrize("da,db,dc", [(orc.U8, orc.I8, orc.I32), (orc.I8, orc.I8, orc.I32),
                                      (orc.U8, orc.U8, orc.U32), (orc.U8, orc.I8, orc.I16),
                                      (orc.I16, orc.U16, orc.I32), (orc.U32, orc.U32, orc.U32),
                                      (orc.I8, orc.U8, orc.U8)])
@pytest.mark.parametrize("accum", [False, True])
def test_matmul_int_vs_numpy(da, db, dc, accum):
    b, m, k, n = 2, 7, 13, 5
    A = rand_ints(da, 1, 0, (b, m, k))
    Bm = rand_ints(db, 1, 1, (b, k, n))
    C0 = rand_ints(dc, 1, 2, (b, m, n))
    got = orc.matmul([b, m, k, n], [da, db, dc], A, Bm, C0.copy(), accum)
    want = np_matmul_mod(A, Bm, C0 if accum else np.zeros_like(C0), dc)
    assert np.array_equal(got, want)


def test_matmul_identity_and_ones():
    n = 16
    A = synth.uniform_u8(2, 0, (1, n, n))
    eye = np.eye(n, dtype=np.int8).reshape(1, n, n)
    out = orc.matmul([1, n, n, n], [orc.U8, orc.I8, orc.I32], A, eye, np.zeros((1, n, n), np.int32))
    assert np.array_equal(out, A.astype(np.int32))
    ones = np.ones((1, n, n), np.int8)
    out = orc.matmul([1, n, n, n], [orc.U8, orc.I8, orc.I32], A, ones, np.zeros((1, n, n), np.int32))
    assert np.array_equal(out[0, :, 0], A[0].astype(np.int64).sum(axis=1))


def test_matmul_extremes_reach_the_stated_bound():
    """u8=255 times i8=-128 over K=4096: |C| = 133 693 440 < 2^31, the no-overflow bound."""
    k = 4096
    A = np.full((1, 1, k), 255, np.uint8)
    Bm = np.full((1, k, 1), -128, np.int8)
    out = orc.matmul([1, 1, k, 1], [orc.U8, orc.I8, orc.I32], A, Bm, np.zeros((1, 1, 1), np.int32))
    assert int(out[0, 0, 0]) == -133693440


def test_matmul_reference_check_pattern_known_answer():
    """Inputs as verification.rs:893-952 makes them (counting ints; the output buffer is
    filled too); expected values by exact integer arithmetic."""
    b, m, k, n = 1, 5, 300, 6
    A = orc.check_pattern(orc.U8, b * m * k).reshape(b, m, k)
    Bm = orc.check_pattern(orc.I8, b * k * n).reshape(b, k, n)
    C0 = orc.check_pattern(orc.I32, b * m * n).reshape(b, m, n)
    assert A.flat[255] == 255 and A.flat[256] == 0 and Bm.flat[0] == -128 and Bm.flat[255] == 127
    assert C0.flat[0] == -2**31 and np.array_equal(A.reshape(-1), synth.check_pattern("u8", A.size))
    assert np.array_equal(Bm.reshape(-1), synth.check_pattern("i8", Bm.size))
    want = np.matmul(A.astype(np.int64), Bm.astype(np.int64))
    got = orc.matmul([b, m, k, n], [orc.U8, orc.I8, orc.I32], A, Bm, C0.copy(), accum=False)
    assert np.array_equal(got, want)
    got = orc.matmul([b, m, k, n], [orc.U8, orc.I8, orc.I32], A, Bm, C0.copy(), accum=True)
    assert np.array_equal(got.astype(np.int64), ((want + C0.astype(np.int64) + 2**31) % 2**32) - 2**31)


def test_matmul_f32_pattern_is_exact_and_random_is_close():
    b, m, k, n = 1, 64, 64, 64
    A = orc.check_pattern(orc.F32, m * k).reshape(b, m, k)
    Bm = orc.check_pattern(orc.F32, k * n).reshape(b, k, n)
    got = orc.matmul([b, m, k, n], [orc.F32] * 3, A, Bm, np.zeros((b, m, n), np.float32))
    want = np.matmul(A.astype(np.int64), Bm.astype(np.int64))
    assert np.array_equal(got, want.astype(np.float32))  # integer-valued: bit exact
    A = synth.uniform_f32(3, 0, (b, m, k))
    Bm = synth.uniform_f32(3, 1, (b, k, n))
    got = orc.matmul([b, m, k, n], [orc.F32] * 3, A, Bm, np.zeros((b, m, n), np.float32))
    want = np.matmul(A.astype(np.float64), Bm.astype(np.float64))
    assert np.abs(got - want).max() < 1e-5


def test_matmul_rows_subset_matches_full():
    b, m, k, n = 2, 12, 9, 5
    A, Bm = synth.uniform_u8(4, 0, (b, m, k)), synth.uniform_i8(4, 1, (b, k, n))
    full = orc.matmul([b, m, k, n], [0, 1, 5], A, Bm, np.zeros((b, m, n), np.int32))
    part = np.full((b, m, n), 77, np.int32)
    orc.matmul([b, m, k, n], [0, 1, 5], A, Bm, part, rows=(3, 8))
    assert np.array_equal(part[:, 3:8], full[:, 3:8]) and (part[:, :3] == 77).all() and (part[:, 8:] == 77).all()


# ---- the reference's own emitted kernel (examples/simple_matmul_x86.rs:144-178) ----------

def test_against_reference_emitted_kernel_u32():
    ref = orc.ref_lib("libref_simple_matmul.so")
    if ref is None:
        pytest.skip("oracle/_ref not built (reference checkout absent)")
    A = rand_ints(orc.U32, 5, 0, (1, 64, 64))
    Bm = rand_ints(orc.U32, 5, 1, (1, 64, 64))
    out = np.full((1, 64, 64), 123, np.uint32)  # the emitted kernel zeroes C itself
    ref.ref_simple_matmul_u32(A.ctypes.data_as(C.c_void_p), Bm.ctypes.data_as(C.c_void_p),
                              out.ctypes.data_as(C.c_void_p))
    got = orc.matmul([1, 64, 64, 64], [orc.U32] * 3, A, Bm, np.zeros((1, 64, 64), np.uint32))
    assert np.array_equal(got, out)


def test_against_reference_emitted_kernel_f32():
    ref = orc.ref_lib("libref_simple_matmul.so")
    if ref is None:
        pytest.skip("oracle/_ref not built (reference checkout absent)")
    for A, Bm, tol in [
        (orc.check_pattern(orc.F32, 4096).reshape(1, 64, 64), orc.check_pattern(orc.F32, 4096).reshape(1, 64, 64), 0.0),
        (synth.uniform_f32(6, 0, (1, 64, 64)), synth.uniform_f32(6, 1, (1, 64, 64)), 1e-5),
    ]:
        out = np.empty((1, 64, 64), np.float32)
        ref.ref_simple_matmul_f32(A.ctypes.data_as(C.c_void_p), Bm.ctypes.data_as(C.c_void_p),
                                  out.ctypes.data_as(C.c_void_p))
        got = orc.matmul([1, 64, 64, 64], [orc.F32] * 3, A, Bm, np.zeros((1, 64, 64), np.float32))
        assert np.abs(got - out).max() <= tol


# ---- bf16 ------------------------------------------------------------------------------

def test_bf16_conversions():
    lib = orc.lib()
    # exact widening = shift by 16; against the reference's cvtbf16_fp32 partial when built
    bits = np.array([0x3F80, 0x4049, 0xC000, 0x0001, 0x7F7F, 0x8000, 0x3DCD, 0x4300], np.uint16)
    ours = np.array([lib.orc_bf16_to_f32(int(b)) for b in bits], np.float32)
    assert np.array_equal(ours.view(np.uint32), bits.astype(np.uint32) << 16)
    assert np.array_equal(synth.bf16_bits_to_f32(bits), ours)
    ref = orc.ref_lib("libref_partials.so")
    if ref is not None:
        out = np.empty(8, np.float32)
        ref.ref_cvtbf16_fp32(bits.ctypes.data_as(C.c_void_p), out.ctypes.data_as(C.c_void_p))
        assert np.array_equal(out.view(np.uint32), ours.view(np.uint32))
    # narrowing is round-to-nearest-even: ties go to the even mantissa
    cases = {1.0: 0x3F80, 1.00390625: 0x3F80, 1.01171875: 0x3F82, 1.005: 0x3F81, -2.5: 0xC020,
             3.0e38: 0x7F62}
    for f, want in cases.items():
        assert lib.orc_f32_to_bf16(f) == want, f
        assert int(synth.f32_to_bf16_bits(np.array([f], np.float32))[0]) == want
    x = synth.normal_f32(7, 0, (4096,))
    assert np.array_equal(synth.f32_to_bf16_bits(x),
                          np.array([lib.orc_f32_to_bf16(float(v)) for v in x], np.uint16))


def test_matmul_bf16_vs_float64():
    b, m, k, n = 1, 9, 50, 7
    A, Bm = synth.normal_bf16(8, 0, (b, m, k)), synth.normal_bf16(8, 1, (b, k, n))
    got = orc.matmul([b, m, k, n], [orc.BF16, orc.BF16, orc.F32], A, Bm, np.zeros((b, m, n), np.float32))
    want = np.matmul(synth.bf16_bits_to_f32(A).astype(np.float64), synth.bf16_bits_to_f32(Bm).astype(np.float64))
    assert np.abs(got - want).max() / np.abs(want).max() < 1e-6
    # 0..3 pattern: exact (verification.rs:933-935)
    A = orc.check_pattern(orc.BF16, m * k).reshape(b, m, k)
    Bm = orc.check_pattern(orc.BF16, k * n).reshape(b, k, n)
    got = orc.matmul([b, m, k, n], [orc.BF16, orc.BF16, orc.F32], A, Bm, np.zeros((b, m, n), np.float32))
    want = np.matmul(synth.bf16_bits_to_f32(A).astype(np.int64), synth.bf16_bits_to_f32(Bm).astype(np.int64))
    assert np.array_equal(got, want.astype(np.float32))


# ---- conv ------------------------------------------------------------------------------

def np_conv(img, filt):
    """Cross-correlation, valid, via scipy (a library routine, not the oracle's loops)."""
    b, c, h, w = img.shape
    f, _, fh, fw = filt.shape
    out = np.zeros((b, f, h - fh + 1, w - fw + 1), np.int64)
    for bi in range(b):
        for fi in range(f):
            for ci in range(c):
                out[bi, fi] += scipy.signal.correlate2d(img[bi, ci].astype(np.int64),
                                                        filt[fi, ci].astype(np.int64), mode="valid")
    return out


@pytest.mark.parametrize("accum", [False, True])
def test_conv_vs_scipy(accum):
    b, f, c, oh, ow, fh, fw = 2, 3, 4, 5, 6, 3, 2
    img = synth.uniform_u8(9, 0, (b, c, oh + fh - 1, ow + fw - 1))
    filt = synth.uniform_i8(9, 1, (f, c, fh, fw))
    out0 = (synth.uniform_u8(9, 2, (b, f, oh, ow)).astype(np.int32) - 100)
    got = orc.conv([b, f, c, oh, ow, fh, fw], [orc.U8, orc.I8, orc.I32], img, filt, out0.copy(), accum)
    want = np_conv(img, filt) + (out0 if accum else 0)
    assert np.array_equal(got, want)


@pytest.mark.parametrize("in_dtype", ["f32", "bf16"])
def test_conv_float_vs_scipy(in_dtype):
    """The float branch of the Conv oracle (bf16 or f32 operands, f32 result) against scipy's
    correlate2d in float64; bf16 operands widen exactly, so only the f32 sum's rounding is left."""
    b, f, c, oh, ow, fh, fw = 2, 3, 5, 4, 6, 3, 2
    img = synth.normal_f32(21, 0, (b, c, oh + fh - 1, ow + fw - 1))
    filt = synth.normal_f32(21, 1, (f, c, fh, fw))
    if in_dtype == "bf16":
        img_b, filt_b = synth.f32_to_bf16_bits(img), synth.f32_to_bf16_bits(filt)
        img, filt = synth.bf16_bits_to_f32(img_b), synth.bf16_bits_to_f32(filt_b)
        dts, args = [orc.BF16, orc.BF16, orc.F32], (img_b, filt_b)
    else:
        dts, args = [orc.F32, orc.F32, orc.F32], (img, filt)
    out0 = synth.normal_f32(21, 2, (b, f, oh, ow))
    want = np.zeros((b, f, oh, ow), np.float64)
    for bi in range(b):
        for fi in range(f):
            for ci in range(c):
                want[bi, fi] += scipy.signal.correlate2d(img[bi, ci].astype(np.float64),
                                                         filt[fi, ci].astype(np.float64), mode="valid")
    for accum in (False, True):
        got = orc.conv([b, f, c, oh, ow, fh, fw], dts, args[0], args[1], out0.copy(), accum)
        ref = want + (out0 if accum else 0)
        assert np.abs(got - ref).max() <= 1e-5 * np.abs(ref).max()
    # a dropped tap or a flipped filter would be far outside: the asymmetric-filter case in floats
    one = np.zeros((1, 1, 2, 2), np.float32)
    one[0, 0, 0, 1] = 1.0
    ramp = np.arange(9, dtype=np.float32).reshape(1, 1, 3, 3)
    got = orc.conv([1, 1, 1, 2, 2, 2, 2], [orc.F32, orc.F32, orc.F32], ramp, one, np.zeros((1, 1, 2, 2), np.float32))
    assert np.array_equal(got.reshape(2, 2), [[1, 2], [4, 5]])


def test_float_operands_saturate_at_the_output_dtype():
    """verification.rs:547-569 casts operands with Rust `as` into the output dtype: floats saturate
    at the bounds of the dtype they are cast to.  Expected values computed by hand from that rule."""
    a = np.array([[300.0, -200.0, -5.0, 70000.0, np.nan, 2.9]], np.float32)
    b = np.eye(6, dtype=np.float32)
    for dt, np_dt, want in ((orc.I8, np.int8, [127, -128, -5, 127, 0, 2]),
                            (orc.U8, np.uint8, [255, 0, 0, 255, 0, 2]),
                            (orc.U16, np.uint16, [300, 0, 0, 65535, 0, 2]),
                            (orc.I16, np.int16, [300, -200, -5, 32767, 0, 2]),
                            (orc.I32, np.int32, [300, -200, -5, 70000, 0, 2]),
                            (orc.U32, np.uint32, [300, 0, 0, 70000, 0, 2])):
        got = orc.matmul([1, 1, 6, 6], [orc.F32, orc.F32, dt], a, b, np.zeros((1, 6), np_dt))
        assert got.reshape(-1).tolist() == want, dt
    # and the product wraps in the output dtype like any integer product: 127 * 127 as i8
    big = np.array([[300.0]], np.float32)
    got = orc.matmul([1, 1, 1, 1], [orc.F32, orc.F32, orc.I8], big, big, np.zeros((1, 1), np.int8))
    assert int(got[0, 0]) == np.int8((127 * 127) & 0xff)


def test_bf16_outputs_round_once():
    """A bf16 output (spec.rs:3663-3698): both inputs cast to bf16 first (verification.rs:629-631),
    products summed in f32, the sum rounded to bf16 once, to nearest even.  Expected values worked out
    by hand: small integers are exact in bf16, so products and short sums are, and the first sums that
    are not (257, 259: ties between neighbours 2 apart) show the rounding."""
    bf = synth.f32_to_bf16_bits
    val = synth.bf16_bits_to_f32
    a = bf(np.array([[[1, 2, 3], [4, 5, 6]]], np.float32))                 # [1, 2, 3]
    b = bf(np.array([[[1, 0, 16], [0, 1, 32], [1, 1, 64]]], np.float32))   # [1, 3, 3]
    got = orc.matmul([1, 2, 3, 3], [orc.BF16] * 3, a, b, np.zeros((1, 2, 3), np.uint16))
    # row 0: [1+3, 2+3, 16+64+192] = [4, 5, 272]; row 1: [4+6, 5+6, 64+160+384] = [10, 11, 608]
    assert val(got).tolist() == [[[4, 5, 272], [10, 11, 608]]]
    ones = bf(np.ones((1, 1, 257), np.float32))
    col = bf(np.ones((1, 257, 1), np.float32))
    assert val(orc.matmul([1, 1, 257, 1], [orc.BF16] * 3, ones, col, np.zeros((1, 1, 1), np.uint16)))[0, 0, 0] == 256.0  # 257: tie, to even
    ones, col = bf(np.ones((1, 1, 259), np.float32)), bf(np.ones((1, 259, 1), np.float32))
    assert val(orc.matmul([1, 1, 259, 1], [orc.BF16] * 3, ones, col, np.zeros((1, 1, 1), np.uint16)))[0, 0, 0] == 260.0  # 259: tie, to even
    # accumulating: the old output joins the f32 sum before the rounding: 256 + 1 -> 257 -> 256, 256 + 3 -> 259 -> 260
    c = bf(np.array([[[256.0, 256.0]]], np.float32))
    got = orc.matmul([1, 1, 1, 2], [orc.BF16] * 3, bf(np.ones((1, 1, 1), np.float32)), bf(np.array([[[1.0, 3.0]]], np.float32)), c, accum=True)
    assert val(got).tolist() == [[[256.0, 260.0]]]
    # f32 inputs are cast to bf16 first: 1 + 2^-8 is a tie and becomes 1, 1 + 3 * 2^-8 becomes 1 + 2^-6
    af = np.array([[[1 + 2.0 ** -8, 1 + 3 * 2.0 ** -8]]], np.float32)
    eye = np.eye(2, dtype=np.float32)[None]
    got = orc.matmul([1, 1, 2, 2], [orc.F32, orc.F32, orc.BF16], af, eye, np.zeros((1, 1, 2), np.uint16))
    assert val(got).tolist() == [[[1.0, 1 + 2.0 ** -6]]]
    # Conv takes the same road: a 1x1 filter over small integers is the exact integer result
    img = bf(np.arange(2 * 3 * 2 * 2, dtype=np.float32).reshape(2, 3, 2, 2) % 5)
    filt = bf(np.array([[[[1]], [[2]], [[3]]], [[[0]], [[1]], [[0]]]], np.float32))
    got = orc.conv([2, 2, 3, 2, 2, 1, 1], [orc.BF16] * 3, img, filt, np.zeros((2, 2, 2, 2), np.uint16))
    want = np.einsum("bchw,fc->bfhw", val(img), val(filt)[:, :, 0, 0])
    assert np.array_equal(val(got), want)


def test_conv_degenerate_cases():
    # 1x1 filter == Matmul [1, B*H*W, C, F] (scheduling/spatial_split.rs:73-102)
    b, f, c, h, w = 2, 5, 7, 3, 4
    img = synth.uniform_u8(10, 0, (b, c, h, w))
    filt = synth.uniform_i8(10, 1, (f, c, 1, 1))
    got = orc.conv([b, f, c, h, w, 1, 1], [0, 1, 5], img, filt, np.zeros((b, f, h, w), np.int32))
    mm = np.einsum("bchw,fc->bfhw", img.astype(np.int64), filt[:, :, 0, 0].astype(np.int64))
    assert np.array_equal(got, mm)
    # oh = ow = 1 == one dot product per (b, f): the examples/simple_conv_x86.rs shape
    img = synth.uniform_u8(11, 0, (1, 8, 3, 3))
    filt = synth.uniform_i8(11, 1, (8, 8, 3, 3))
    got = orc.conv([1, 8, 8, 1, 1, 3, 3], [0, 1, 5], img, filt, np.zeros((1, 8, 1, 1), np.int32))
    want = np.einsum("chw,fchw->f", img[0].astype(np.int64), filt.astype(np.int64))
    assert np.array_equal(got.reshape(-1), want)
    # not a flipped-kernel convolution: an asymmetric filter tells them apart
    img = np.arange(9, dtype=np.uint8).reshape(1, 1, 3, 3)
    filt = np.array([1, 0, 0, 0], np.int8).reshape(1, 1, 2, 2)
    got = orc.conv([1, 1, 1, 2, 2, 2, 2], [0, 1, 5], img, filt, np.zeros((1, 1, 2, 2), np.int32))
    assert np.array_equal(got.reshape(2, 2), [[0, 1], [3, 4]])


def test_conv_nhwc_krsc_layout_equals_nchw():
    b, f, c, oh, ow, fh, fw = 2, 4, 3, 4, 5, 3, 3
    img = synth.uniform_u8(12, 0, (b, c, oh + 2, ow + 2))
    filt = synth.uniform_i8(12, 1, (f, c, fh, fw))
    want = orc.conv([b, f, c, oh, ow, fh, fw], [0, 1, 5], img, filt, np.zeros((b, f, oh, ow), np.int32))
    nhwc = orc.make_layout([0, 2, 3, 1])
    img_l = np.ascontiguousarray(img.transpose(0, 2, 3, 1))
    filt_l = np.ascontiguousarray(filt.transpose(0, 2, 3, 1))
    out_l = np.zeros((b, oh, ow, f), np.int32)
    orc.conv([b, f, c, oh, ow, fh, fw], [0, 1, 5], img_l, filt_l, out_l, layouts=[nhwc, nhwc, nhwc])
    assert np.array_equal(out_l.transpose(0, 3, 1, 2), want)


# ---- softmax ---------------------------------------------------------------------------

@pytest.mark.parametrize("shape,dim", [((4, 33), 1), ((3, 5, 7), 1), ((2, 3, 8), 2), ((6, 4), 0)])
def test_softmax_vs_scipy(shape, dim):
    x = synth.normal_f32(13, 0, shape, std=3.0)
    got = orc.softmax(list(shape), dim, x)
    want = scipy.special.softmax(x.astype(np.float64), axis=dim)
    assert np.abs(got - want).max() <= 1e-6
    assert np.abs(got.sum(axis=dim) - 1).max() < 1e-5
    shifted = orc.softmax(list(shape), dim, (x + np.float32(4.0)))
    assert np.abs(shifted - got).max() < 1e-5  # shift invariance up to input rounding
    const = orc.softmax([3, 10], 1, np.full((3, 10), 2.5, np.float32))
    assert np.array_equal(const, np.full((3, 10), np.float32(1.0) / np.float32(10.0), np.float32))


def test_online_merge_formula_equals_two_pass():
    """spec.rs:116-123: new = max(a,b); d = d_a*exp(a-new) + d_b*exp(b-new)."""
    x = synth.normal_f32(14, 0, (1000,), std=4.0).astype(np.float64)
    mx, den = -np.inf, 0.0
    for chunk in np.split(x, 10):
        cm = chunk.max()
        cd = np.exp(chunk - cm).sum()
        nm = max(mx, cm)
        den = den * np.exp(mx - nm) + cd * np.exp(cm - nm)
        mx = nm
    got = orc.softmax([1, 1000], 1, x.astype(np.float32).reshape(1, 1000))
    assert np.abs(np.exp(x - mx) / den - got[0]).max() < 1e-6


def test_reference_vector_exp_is_within_softmax_tolerance():
    """The reference's vector kernels use a degree-4 polynomial exp (partials/x86/
    expf_avx2.c).  It differs from libm expf by a few 1e-6 relative: inside the 1e-5 Softmax
    tolerance, so matching the closed form also matches what emitted vector code prints."""
    ref = orc.ref_lib("libref_partials.so")
    if ref is None:
        pytest.skip("oracle/_ref not built (reference checkout absent)")
    x = -np.abs(synth.normal_f32(15, 0, (4096,), std=5.0))  # softmax arguments are <= 0
    out = np.empty_like(x)
    ref.ref_exp256(x.ctypes.data_as(C.c_void_p), out.ctypes.data_as(C.c_void_p), x.size)
    want = np.exp(x.astype(np.float64))
    assert (np.abs(out - want) / want).max() < 1e-5
    v = synth.uniform_f32(16, 0, (8,))
    assert abs(ref_f(ref.ref_sum8, v) - float(v.astype(np.float64).sum())) < 1e-6
    # The reference's 8-wide horizontal max (partials/x86/max8.c) overwrites its vector with
    # the shuffled copy before the last max, so it returns the max of elements {2,3,6,7}
    # only.  Softmax is shift-invariant, so emitted code using it still computes the same
    # function as long as nothing overflows; the oracle uses the true max.
    assert ref_f(ref.ref_max8, v) == float(v[[2, 3, 6, 7]].max())
    assert ref_f(ref.ref_max4, v[:4]) == float(v[:4].max())


def ref_f(fn, arr):
    fn.restype = C.c_float
    return float(fn(arr.ctypes.data_as(C.c_void_p)))


# ---- compose ---------------------------------------------------------------------------

def test_compose_msm_vs_float64():
    b, m, k, n2, n = 2, 9, 16, 21, 5
    q = synth.normal_bf16(17, 0, (b, m, k), 0.5)
    kmat = synth.normal_bf16(17, 1, (b, n2, k), 0.5)       # K stored row-major
    v = synth.normal_bf16(17, 2, (b, n2, n), 0.5)
    qf, kf, vf = (synth.bf16_bits_to_f32(t).astype(np.float64) for t in (q, kmat, v))
    want = scipy.special.softmax(qf @ kf.transpose(0, 2, 1), axis=2) @ vf
    out = np.zeros((b, m, n), np.float32)
    # KT logical [b,k,n2] stored k-fastest == layout![0,2,1]
    kt_layout = orc.make_layout([0, 2, 1])
    orc.compose_msm(b, m, k, n2, n, [orc.BF16, orc.BF16, orc.BF16, orc.F32], v, q, kmat, out,
                    layouts=[None, None, kt_layout, None])
    assert np.abs(out - want).max() / np.abs(want).max() < 1e-5
    # and with KT materialised row-major
    kt = np.ascontiguousarray(kmat.transpose(0, 2, 1))
    out2 = np.zeros((b, m, n), np.float32)
    orc.compose_msm(b, m, k, n2, n, [orc.BF16, orc.BF16, orc.BF16, orc.F32], v, q, kt, out2)
    assert np.array_equal(out, out2)


# ---- move ------------------------------------------------------------------------------

def test_move_casts_vs_numpy_and_known_answers():
    shape = [3, 37]
    n = 3 * 37
    # int -> int wraps, int -> float converts: numpy astype does the same
    for sdt, ddt in [(orc.I32, orc.U8), (orc.U8, orc.I8), (orc.I16, orc.U32), (orc.U32, orc.I16),
                     (orc.I8, orc.F32), (orc.U32, orc.F32), (orc.I16, orc.I16)]:
        x = rand_ints(sdt, 21, 0, shape)
        got = orc.move(shape, [sdt, ddt], x, np.zeros(shape, orc.NP[ddt]))
        assert np.array_equal(got, x.astype(orc.NP[ddt])), (sdt, ddt)
    # float -> int saturates at the destination's bounds, NaN -> 0 (Rust `as`)
    x = np.array([300.7, -5.2, 127.9, -128.5, np.nan, 1e20, -1e20, 0.99], np.float32).reshape(1, 8)
    assert list(orc.move([1, 8], [orc.F32, orc.U8], x, np.zeros((1, 8), np.uint8))[0]) == [255, 0, 127, 0, 0, 255, 0, 0]
    assert list(orc.move([1, 8], [orc.F32, orc.I8], x, np.zeros((1, 8), np.int8))[0]) == [127, -5, 127, -128, 0, 127, -128, 0]
    assert list(orc.move([1, 8], [orc.F32, orc.I32], x, np.zeros((1, 8), np.int32))[0]) == \
        [300, -5, 127, -128, 0, 2**31 - 1, -2**31, 0]
    # f32 -> bf16 rounds to nearest even; bf16 -> f32 is exact
    f = synth.normal_f32(22, 0, (n,)).reshape(shape)
    b = orc.move(shape, [orc.F32, orc.BF16], f, np.zeros(shape, np.uint16))
    assert np.array_equal(b, synth.f32_to_bf16_bits(f))
    assert np.array_equal(orc.move(shape, [orc.BF16, orc.F32], b, np.zeros(shape, np.float32)),
                          synth.bf16_bits_to_f32(b))


def test_move_relayout_round_trip():
    shape = [4, 6, 8]
    x = synth.uniform_u8(23, 0, shape)
    packed = orc.make_layout([0, 2, 1, (2, 1, 4)])      # layout![0,2,1,2 p(4)]
    mid = orc.move(shape, [orc.U8, orc.U8], x, np.zeros(x.size, np.uint8), layouts=[None, packed])
    for pt in [(0, 0, 0), (1, 2, 3), (3, 5, 7)]:
        assert mid[orc.buffer_index(packed, shape, list(pt))] == x[pt]
    back = orc.move(shape, [orc.U8, orc.U8], mid, np.zeros(shape, np.uint8), layouts=[packed, None])
    assert np.array_equal(back, x)
    col = orc.make_layout([2, 1, 0])
    t = orc.move(shape, [orc.U8, orc.U8], x, np.zeros(x.size, np.uint8), layouts=[None, col])
    assert np.array_equal(t.reshape(8, 6, 4), x.transpose(2, 1, 0))
