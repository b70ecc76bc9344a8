"""GPU parity of the primitives Softmax decomposes into, Broadcast, Fill and OnePrefix, run
through the C ABI and checked against the CPU oracle.  Floating point to 1e-5 (the oracle
updates a line element by element, the GPU reduces a line in parallel; max is exact),
copies and fills bit-exact."""
import numpy as np
import pytest

import morello_amd as M
import orc
from gpu_util import run_spec

pytestmark = pytest.mark.gpu

RNG = np.random.default_rng(77)
SHAPES = [((7, 33), 1), ((5, 9, 4), 1), ((3, 4, 130), 2), ((6, 5), 0), ((2, 3, 4, 5), 2),
          ((64, 2048), 1), ((1, 1, 1), 1), ((4, 1, 300), 2),
          # contiguous lines of whole 16-byte vectors: register-resident (4, 8, 16 vectors a lane)
          ((33, 1024), 1), ((5, 12), 1), ((7, 3, 2048), 2), ((9, 4096), 1), ((3, 4100), 1),
          # few long lines that are not whole vectors: a workgroup per line
          ((5, 9001), 1), ((2, 2, 4099), 2),
          # the scan dim is not the innermost: lines side by side, 16, 32 or 64 to a workgroup
          ((37, 70), 0), ((3, 50, 33), 1), ((2, 300, 64), 1), ((40, 20000), 0), ((24, 40000), 0), ((1, 18), 0),
          # lines of a handful of elements: a thread per line
          ((5, 20000), 0), ((3000, 8), 1), ((40, 50, 2), 2)]
TOL = dict(rtol=1e-5, atol=1e-7)


def tol(shape, dim):
    """1e-5, loosened for long lines: the oracle adds a line's terms one by one in f32 as
    the reference's scalar kernels do, so its own rounding grows with the line length
    (observed 1.1e-5 at 2048 terms); the GPU's tree reduction is the more accurate side."""
    return dict(rtol=1e-5 if shape[dim] <= 512 else 5e-5, atol=1e-7)


def reduced(shape, dim):
    s = list(shape)
    s[dim] = 1
    return tuple(s)


def rnd(shape, scale=3.0):
    return (RNG.standard_normal(shape) * scale).astype(np.float32)


def run_all(spec, arrays):
    """Runs `spec` on the device and returns every parameter as it is afterwards."""
    bufs = [M.DeviceBuffer.from_numpy(a) for a in arrays]
    spec.run_device([b.ptr for b in bufs])
    res = [b.to_numpy(a.dtype, a.shape) for a, b in zip(arrays, bufs)]
    for b in bufs:
        b.free()
    return res


@pytest.mark.parametrize("shape,dim", SHAPES)
@pytest.mark.parametrize("accum", [False, True])
def test_max(gpu, shape, dim, accum):
    x, out = rnd(shape), rnd(reduced(shape, dim))
    got = run_all(M.Max(shape, dim, accum=accum), [x, out])[1]
    want = orc.softmax_part(orc.PART_MAX, shape, dim, [x, out.copy()], accum)[1]
    assert np.array_equal(got, want)


@pytest.mark.parametrize("shape,dim", SHAPES)
@pytest.mark.parametrize("accum", [False, True])
def test_softmax_denominator(gpu, shape, dim, accum):
    x = rnd(shape)
    mx = x.max(axis=dim, keepdims=True)
    dn = np.abs(rnd(reduced(shape, dim)))
    got = run_all(M.SoftmaxDenominator(shape, dim, accum=accum), [x, mx, dn])
    want = orc.softmax_part(orc.PART_DENOM, shape, dim, [x, mx, dn.copy()], accum)
    assert np.array_equal(got[0], x) and np.array_equal(got[1], mx)
    np.testing.assert_allclose(got[2], want[2], **tol(shape, dim))


@pytest.mark.parametrize("shape,dim", SHAPES)
@pytest.mark.parametrize("accum", [False, True])
def test_softmax_denominator_and_max(gpu, shape, dim, accum):
    x = rnd(shape)
    # A previous (max, denominator) pair as an earlier tile would have left it.
    prev = rnd(shape, 5.0)
    mx, dn = np.zeros(reduced(shape, dim), np.float32), np.zeros(reduced(shape, dim), np.float32)
    orc.softmax_part(orc.PART_DENOM_MAX, shape, dim, [prev, mx, dn])
    got = run_all(M.SoftmaxDenominatorAndMax(shape, dim, accum=accum), [x, mx, dn])
    want = orc.softmax_part(orc.PART_DENOM_MAX, shape, dim, [x, mx.copy(), dn.copy()], accum)
    assert np.array_equal(got[1], want[1])
    np.testing.assert_allclose(got[2], want[2], **tol(shape, dim))


@pytest.mark.parametrize("shape,dim", [((9, 130), 1), ((6, 1024), 1), ((300, 40), 0), ((5, 20000), 0)])
def test_softmax_denominator_and_max_of_masked_lines(gpu, shape, dim):
    """Lines with elements of -inf (masked positions), at their start too, and one line that is
    -inf throughout: the pair is the closed form's -- max over the line, sum of exp(x - max), a
    masked element adding exp(-inf) = 0 -- on every kernel that takes these Specs (a wavefront
    per line, the register-resident form, lines side by side); the line of nothing but -inf has
    max -inf and a denominator of NaN (every term is exp(-inf - -inf)), as the reference's
    recurrence gives it (codegen/cpu.rs:1360-1389).  The reference's recurrence, fed -inf before
    the first finite element, turns the whole line's denominator into NaN; that is not copied."""
    x = rnd(shape)
    mask = RNG.random(shape) < 0.3
    lead = [slice(None)] * len(shape)
    lead[dim] = slice(0, min(11, shape[dim] - 1))
    mask[tuple(lead)] = True
    x[mask] = -np.inf
    whole = [0] * len(shape)
    whole[dim] = slice(None)
    x[tuple(whole)] = -np.inf
    mx, dn = np.zeros(reduced(shape, dim), np.float32), np.zeros(reduced(shape, dim), np.float32)
    got = run_all(M.SoftmaxDenominatorAndMax(shape, dim), [x, mx, dn])
    x64 = x.astype(np.float64)
    m = x64.max(axis=dim, keepdims=True)
    with np.errstate(invalid="ignore"):
        d = np.exp(x64 - m).sum(axis=dim, keepdims=True)
    assert np.array_equal(got[1], m.astype(np.float32))
    first = tuple(0 for _ in shape)
    assert np.isnan(got[2][first]) and np.isnan(d[first])
    keep = np.ones(d.shape, bool)
    keep[first] = False
    np.testing.assert_allclose(got[2][keep], d[keep], rtol=2e-5)
    # the two-step forms agree: Max, then SoftmaxDenominator against it
    got_m = run_all(M.Max(shape, dim), [x, mx])[1]
    got_d = run_all(M.SoftmaxDenominator(shape, dim), [x, got_m, dn])[2]
    assert np.array_equal(got_m, got[1])
    np.testing.assert_allclose(got_d[keep], got[2][keep], rtol=2e-5)


@pytest.mark.parametrize("shape,dim", [((6, 5), 1), ((3, 9, 4), 1), ((4, 70), 1), ((8, 3), 0), ((40, 33), 0), ((3, 20, 64), 1),
                                       ((16, 300, 2), 2), ((2000, 7), 1)])
@pytest.mark.parametrize("accum", [False, True])
def test_softmax_denominator_and_max_from_parts(gpu, shape, dim, accum):
    tmax, tden = rnd(shape, 4.0), np.abs(rnd(shape)) + np.float32(1.0)
    omax, oden = rnd(reduced(shape, dim), 4.0), np.abs(rnd(reduced(shape, dim))) + np.float32(1.0)
    got = run_all(M.SoftmaxDenominatorAndMaxFromParts(shape, dim, accum=accum), [tmax, tden, omax, oden])
    want = orc.softmax_part(orc.PART_FROM_PARTS, shape, dim, [tmax, tden, omax.copy(), oden.copy()], accum)
    assert np.array_equal(got[2], want[2])
    np.testing.assert_allclose(got[3], want[3], **TOL)


@pytest.mark.parametrize("shape,dim", SHAPES)
def test_softmax_denominator_and_unscaled(gpu, shape, dim):
    x = rnd(shape)
    dn, un = np.zeros(reduced(shape, dim), np.float32), np.zeros(shape, np.float32)
    got = run_all(M.SoftmaxDenominatorAndUnscaled(shape, dim), [x, dn, un])
    want = orc.softmax_part(orc.PART_UNSCALED, shape, dim, [x, dn.copy(), un.copy()])
    np.testing.assert_allclose(got[1], want[1], **tol(shape, dim))
    np.testing.assert_allclose(got[2], want[2], **tol(shape, dim))


@pytest.mark.parametrize("shape,dim", SHAPES)
@pytest.mark.parametrize("accum", [False, True])
def test_softmax_denominator_and_unscaled_from_max(gpu, shape, dim, accum):
    x = rnd(shape)
    mx = x.max(axis=dim, keepdims=True)
    dn, un = np.abs(rnd(reduced(shape, dim))), np.zeros(shape, np.float32)
    got = run_all(M.SoftmaxDenominatorAndUnscaledFromMax(shape, dim, accum=accum), [x, mx, dn, un])
    want = orc.softmax_part(orc.PART_UNSCALED_FROM_MAX, shape, dim, [x, mx, dn.copy(), un.copy()], accum)
    np.testing.assert_allclose(got[2], want[2], **tol(shape, dim))
    np.testing.assert_allclose(got[3], want[3], **tol(shape, dim))


@pytest.mark.parametrize("shape,dim", SHAPES)
def test_softmax_complete(gpu, shape, dim):
    x = rnd(shape)
    mx = x.max(axis=dim, keepdims=True)
    dn = np.exp(x - mx).sum(axis=dim, keepdims=True).astype(np.float32)
    got = run_all(M.SoftmaxComplete(shape, dim), [x, mx, dn, np.zeros(shape, np.float32)])[3]
    want = orc.softmax_part(orc.PART_COMPLETE, shape, dim, [x, mx, dn, np.zeros(shape, np.float32)])[3]
    np.testing.assert_allclose(got, want, **TOL)


@pytest.mark.parametrize("shape,dim", SHAPES)
def test_divide_vec_and_scalar(gpu, shape, dim):
    a, b = rnd(shape), np.abs(rnd(shape)) + np.float32(0.5)
    got = run_all(M.DivideVec(shape), [a, b])
    assert np.array_equal(got[0], a / b) and np.array_equal(got[1], b)
    bs = np.abs(rnd(reduced(shape, dim))) + np.float32(0.5)
    got = run_all(M.DivideVecScalar(shape, dim), [a, bs])
    want = orc.softmax_part(orc.PART_DIVIDE_VEC_SCALAR, shape, dim, [a.copy(), bs])[0]
    assert np.array_equal(got[0], want)


def _both_ways(action, arrays):
    """Every parameter after the action ran as the library runs it, and after its children ran one
    by one on caller-held intermediates (mrl_action_apply)."""
    out = []
    for how in ("library", "children"):
        bufs = [M.DeviceBuffer.from_numpy(a) for a in arrays]
        (action if how == "library" else action.apply()).run_device([b.ptr for b in bufs])
        out.append([b.to_numpy(a.dtype, a.shape) for a, b in zip(arrays, bufs)])
        for b in bufs:
            b.free()
    return out


@pytest.mark.parametrize("shape,dim", SHAPES)
def test_rewrites_of_the_softmax_primitives(gpu, shape, dim):
    """to_max_and_denominator on SoftmaxDenominatorAndMax (to_max_and_denom.rs:13-72),
    to_max_and_unscaled on SoftmaxDenominatorAndUnscaled (to_max_and_unscaled.rs:30-110),
    broadcast_first on DivideVecScalar (broadcast_first.rs:24-130): each gives what the Spec
    gives, as an action and as its children."""
    K = M.ActionKind
    x = rnd(shape)
    red = reduced(shape, dim)
    spec = M.SoftmaxDenominatorAndMax(shape, dim)
    act = [a for a in spec.actions() if a.kind == K.ToMaxAndDenominator]
    assert len(act) == 1 and [s.kind for s, _ in act[0].apply().subspecs] == [M.SpecKind.Max, M.SpecKind.SoftmaxDenominator]
    want = orc.softmax_part(orc.PART_DENOM_MAX, shape, dim, [x, np.zeros(red, np.float32), np.zeros(red, np.float32)])
    for got in _both_ways(act[0], [x, np.full(red, 7, np.float32), np.full(red, 7, np.float32)]):
        assert np.array_equal(got[1], want[1])
        np.testing.assert_allclose(got[2], want[2], **tol(shape, dim))
    assert not [a for a in M.SoftmaxDenominatorAndMax(shape, dim, accum=True).actions() if a.kind == K.ToMaxAndDenominator]

    spec = M.SoftmaxDenominatorAndUnscaled(shape, dim)
    act = [a for a in spec.actions() if a.kind == K.ToMaxAndUnscaled]
    assert len(act) == 1 and act[0].apply().intermediate_bytes == [4 * int(np.prod(red))]
    want = orc.softmax_part(orc.PART_UNSCALED, shape, dim, [x, np.zeros(red, np.float32), np.zeros(shape, np.float32)])
    for got in _both_ways(act[0], [x, np.full(red, 7, np.float32), np.full(shape, 7, np.float32)]):
        np.testing.assert_allclose(got[1], want[1], **tol(shape, dim))
        np.testing.assert_allclose(got[2], want[2], **tol(shape, dim))

    a, bs = rnd(shape), np.abs(rnd(red)) + np.float32(0.5)
    spec = M.DivideVecScalar(shape, dim)
    act = [a_ for a_ in spec.actions() if a_.kind == K.BroadcastFirst]
    assert len(act) == 1 and [s.kind for s, _ in act[0].apply().subspecs] == [M.SpecKind.Broadcast, M.SpecKind.DivideVec]
    want = orc.softmax_part(orc.PART_DIVIDE_VEC_SCALAR, shape, dim, [a.copy(), bs])[0]
    for got in _both_ways(act[0], [a, bs]):
        assert np.array_equal(got[0], want) and np.array_equal(got[1], bs)


def test_decomposed_softmax_matches_the_fused_spec(gpu):
    """Max -> DenominatorAndUnscaledFromMax -> DivideVecScalar, as Softmax is scheduled by
    hand in the reference, equals the Softmax Spec on the same input."""
    shape, dim = (16, 8, 200), 2
    x = rnd(shape, 4.0)
    red = reduced(shape, dim)
    bx, bmx, bdn, bun, bout = (M.DeviceBuffer.from_numpy(a) for a in
                               (x, np.zeros(red, np.float32), np.zeros(red, np.float32),
                                np.zeros(shape, np.float32), np.zeros(shape, np.float32)))
    M.Max(shape, dim).run_device([bx.ptr, bmx.ptr])
    M.SoftmaxDenominatorAndUnscaledFromMax(shape, dim).run_device([bx.ptr, bmx.ptr, bdn.ptr, bun.ptr])
    M.DivideVecScalar(shape, dim).run_device([bun.ptr, bdn.ptr])
    M.Softmax(list(shape), dim).run_device([bx.ptr, bout.ptr])
    got, fused = bun.to_numpy(np.float32, shape), bout.to_numpy(np.float32, shape)
    np.testing.assert_allclose(got, fused, rtol=1e-5, atol=1e-8)
    np.testing.assert_allclose(got, orc.softmax(list(shape), dim, x), rtol=1e-5, atol=1e-8)


def test_parts_through_non_row_major_layouts(gpu):
    """A column-major input and a packed output go through the relayout staging."""
    shape, dim = (12, 16), 1
    x = rnd(shape)
    cm = M.col_major(list(shape))
    packed = M.layout(0, 1, (1, M.Packed(4)))
    spec = M.SoftmaxDenominatorAndUnscaled(shape, dim, layouts=[cm, None, packed])
    x_cm = np.ascontiguousarray(x.T)  # column-major buffer of x
    got = run_all(spec, [x_cm, np.zeros((12, 1), np.float32), np.zeros(shape, np.float32)])
    want = orc.softmax_part(orc.PART_UNSCALED, shape, dim,
                            [x, np.zeros((12, 1), np.float32), np.zeros(shape, np.float32)])
    np.testing.assert_allclose(got[1], want[1], **TOL)
    # [0, 1, (1, Packed 4)] over [12, 16]: buffer [12][4][4] in the same element order as row-major.
    np.testing.assert_allclose(got[2].reshape(shape), want[2], **TOL)


@pytest.mark.parametrize("shape,dim", [((70, 48), 1), ((48, 70), 0), ((64, 1024), 0), ((130, 20), 1)])
def test_parts_of_column_major_tensors(gpu, shape, dim):
    """Column-major parameters are strided tensors to these kernels: scanned along dim 0 their
    lines are contiguous (the register-resident form where they are whole vectors), scanned
    along dim 1 consecutive lines are neighbours in memory (the side-by-side form)."""
    x = rnd(shape)
    cm, cm_red = M.col_major(list(shape)), M.col_major(list(reduced(shape, dim)))
    stored = lambda a: np.ascontiguousarray(a.T)
    mx, dn = np.zeros(reduced(shape, dim), np.float32), np.zeros(reduced(shape, dim), np.float32)
    got = run_all(M.SoftmaxDenominatorAndMax(shape, dim, layouts=[cm, cm_red, cm_red]), [stored(x), stored(mx), stored(dn)])
    want = orc.softmax_part(orc.PART_DENOM_MAX, shape, dim, [x, mx.copy(), dn.copy()])
    assert np.array_equal(got[1], stored(want[1]))
    np.testing.assert_allclose(got[2], stored(want[2]), **tol(shape, dim))
    out = np.zeros(shape, np.float32)
    got = run_all(M.SoftmaxComplete(shape, dim, layouts=[cm, cm_red, cm_red, cm]), [stored(x), stored(want[1]), stored(want[2]), stored(out)])
    want_y = orc.softmax_part(orc.PART_COMPLETE, shape, dim, [x, want[1], want[2], out])[3]
    np.testing.assert_allclose(got[3], stored(want_y), **tol(shape, dim))


def test_one_prefix_of_a_large_tensor_is_a_copy(gpu):
    shape = (1024, 1000)
    x = rnd(shape)
    spec = M.OnePrefix(shape)
    assert spec.plan().kernels == ["k_copy16"]
    assert np.array_equal(run_all(spec, [x, np.zeros((1,) + shape, np.float32)])[1][0], x)
    spec = M.OnePrefix(shape, layouts=[None, M.layout(0, 2, 1)])
    assert "k_move_generic" not in spec.plan().kernels
    assert np.array_equal(run_all(spec, [x, np.zeros((1, 1000, 1024), np.float32)])[1][0], x.T)


@pytest.mark.parametrize("dtype,np_dtype", [(M.u8, np.uint8), (M.bf16, np.uint16), (M.f32, np.float32)])
@pytest.mark.parametrize("count", [1, 15, 16, 185, 4099])
def test_fill_stays_inside_its_tensor(gpu, dtype, np_dtype, count):
    """The 16-byte stores cover the whole units of the tensor and single elements the rest;
    nothing behind the tensor changes."""
    whole = np.full(count + 64, 0x55, np_dtype)
    buf = M.DeviceBuffer.from_numpy(whole)
    M.Fill([count], dtype, M.FillValue.Min).run_device([buf.ptr])
    back = buf.to_numpy(np_dtype, whole.shape)
    buf.free()
    want = orc.fill({M.u8: orc.U8, M.bf16: orc.BF16, M.f32: orc.F32}[dtype], int(M.FillValue.Min), count)
    assert np.array_equal(back[:count].view(np.uint8), want.view(np.uint8))
    assert np.all(back[count:] == 0x55)


@pytest.mark.parametrize("dtype,np_dtype,code", [(M.u8, np.uint8, orc.U8), (M.i8, np.int8, orc.I8),
                                                  (M.i16, np.int16, orc.I16), (M.u32, np.uint32, orc.U32),
                                                  (M.i32, np.int32, orc.I32), (M.f32, np.float32, orc.F32),
                                                  (M.bf16, np.uint16, orc.BF16)])
@pytest.mark.parametrize("value", [M.FillValue.Zero, M.FillValue.NegInf, M.FillValue.Min])
def test_fill(gpu, dtype, np_dtype, code, value):
    shape = (5, 37)
    spec = M.Fill(shape, dtype, value)
    if value == M.FillValue.NegInf and dtype not in (M.f32, M.bf16):
        assert spec.check() == 3  # MRL_ERR_BAD_SPEC: no -inf among the integers
        return
    got = run_all(spec, [np.full(shape, 0x55, np_dtype)])[0]
    want = orc.fill(code, int(value), 5 * 37).reshape(shape)
    assert np.array_equal(got.view(np.uint8), want.view(np.uint8))


@pytest.mark.parametrize("shape,dim", [((4, 9), 0), ((4, 9), 1), ((3, 5, 7), 1), ((2, 3, 4, 5), 3),
                                       # whole 16-byte pieces behind the dim, or of the innermost dim itself
                                       ((4, 8, 64), 1), ((70, 16), 0), ((300, 3, 48), 1), ((16, 256), 1), ((1000, 32), 1),
                                       ((5, 6, 16), 2), ((3, 40, 20), 1)])
@pytest.mark.parametrize("dtype,np_dtype", [(M.f32, np.float32), (M.u8, np.uint8), (M.bf16, np.uint16)])
def test_broadcast(gpu, shape, dim, dtype, np_dtype):
    x = RNG.integers(0, 250, size=reduced(shape, dim)).astype(np_dtype)
    got = run_all(M.Broadcast(shape, dim, dtype), [x, np.zeros(shape, np_dtype)])[1]
    assert np.array_equal(got, orc.broadcast(shape, dim, x))
    assert np.array_equal(got, np.broadcast_to(x, shape))


def test_one_prefix(gpu):
    shape = (6, 10)
    x = rnd(shape)
    spec = M.OnePrefix(shape)
    assert spec.parameter_shapes() == [[6, 10], [1, 6, 10]]
    got = run_all(spec, [x, np.zeros((1,) + shape, np.float32)])[1]
    assert np.array_equal(got[0], x)
    # Column-major output under the unit prefix.
    spec = M.OnePrefix(shape, layouts=[None, M.layout(0, 2, 1)])
    got = run_all(spec, [x, np.zeros((1, 10, 6), np.float32)])[1]
    assert np.array_equal(got[0], x.T)
