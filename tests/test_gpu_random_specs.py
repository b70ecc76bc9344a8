"""Differential test over seeded random Specs: random shapes (through and around the
matrix-core kernels' thresholds), dtype triples, accumulation and per-parameter layouts
(random permutations of the logical dims, optionally with a Packed or OddEven dim), run through
the C ABI and compared with the CPU oracle on the very same parameter buffers.  Integers must
match bit for bit, floating point to 1e-5 (norm-wise)."""
import numpy as np
import pytest

import morello_amd as M
import orc
from gpu_util import rel_err, run_spec
from morello_amd import synth

pytestmark = pytest.mark.gpu

SIZES = list(range(1, 20)) + [24, 31, 32, 33, 48, 63, 64, 65, 72, 96, 100, 128, 136, 200, 264]
NP = {M.u8: np.uint8, M.i8: np.int8, M.u16: np.uint16, M.i16: np.int16, M.u32: np.uint32, M.i32: np.int32,
      M.f32: np.float32, M.bf16: np.uint16}


def random_layout(rng, shape):
    """-> (M.Layout, orc layout) over `shape`: a random order of the dims, and sometimes one dim
    split off as a trailing Packed(n) / OddEven(n) dim (n divides the dim, layout.rs:769-810)."""
    rank = len(shape)
    order = list(rng.permutation(rank))
    m_dims, o_dims = [int(d) for d in order], [int(d) for d in order]
    if rng.random() < 0.35:
        d = int(rng.integers(rank))
        divisors = [n for n in (2, 4, 8, 16) if shape[d] % n == 0 and shape[d] > n]
        if divisors:
            n = int(rng.choice(divisors))
            if rng.random() < 0.7:
                m_dims.append((d, M.Packed(n)))
                o_dims.append((d, 1, n))
            else:
                m_dims.append((d, M.OddEven(n)))
                o_dims.append((d, 2, n))
    return M.layout(*m_dims), orc.make_layout(o_dims)


def random_values(rng, dtype, shape, seed):
    if dtype == M.f32:
        return synth.normal_f32(seed, 0, shape)
    if dtype == M.bf16:
        return synth.normal_bf16(seed, 1, shape)
    return synth.raw_u64(seed, 2, int(np.prod(shape))).astype(NP[dtype]).reshape(shape)


def compare(got, want, dtype, what):
    if dtype in (M.f32, M.bf16):
        assert rel_err(got, want) < 1e-5, what
    else:
        assert np.array_equal(got, want), what


MATMUL_DTYPES = [(M.u8, M.i8, M.i32), (M.i8, M.i8, M.i32), (M.bf16, M.bf16, M.f32), (M.f32, M.f32, M.f32),
                 (M.f32, M.bf16, M.f32), (M.u16, M.u16, M.u32), (M.u8, M.u8, M.u8), (M.i8, M.u8, M.f32),
                 (M.i16, M.i8, M.i32)]


@pytest.mark.parametrize("seed", range(120))
def test_random_matmul(gpu, seed):
    rng = np.random.default_rng(7000 + seed)
    b = int(rng.choice([1, 1, 2, 3]))
    # Half of the cases at sizes the matrix-core kernels take (every dim >= 64).
    sizes = [64, 65, 72, 96, 100, 128, 136, 200, 264, 300] if rng.random() < 0.5 else SIZES
    m, k, n = (int(rng.choice(sizes)) for _ in range(3))
    dts = MATMUL_DTYPES[int(rng.integers(len(MATMUL_DTYPES)))]
    accum = bool(rng.integers(2))
    shape = [b, m, k, n]
    pshapes = [[b, m, k], [b, k, n], [b, m, n]]
    lay = [random_layout(rng, s) for s in pshapes]
    bufs = [random_values(rng, dt, s, 7000 + seed * 3 + i) for i, (dt, s) in enumerate(zip(dts, pshapes))]
    if not accum:
        bufs[2] = np.zeros(pshapes[2], NP[dts[2]])
    spec = M.Matmul(shape, dts, layouts=[l[0] for l in lay], accum=accum)
    got = run_spec(spec, bufs)
    want = orc.matmul(shape, [int(d) for d in dts], bufs[0], bufs[1], bufs[2].copy(), accum,
                      layouts=[l[1] for l in lay])
    compare(got, want, dts[2], (shape, dts, accum, [repr(l[0]) for l in lay]))


MOVE_DTYPES = [M.u8, M.i8, M.u16, M.i16, M.u32, M.i32, M.f32, M.bf16]


@pytest.mark.parametrize("seed", range(60))
def test_random_move(gpu, seed):
    rng = np.random.default_rng(8000 + seed)
    rank = int(rng.integers(1, 5))
    shape = [int(rng.choice(SIZES)) for _ in range(rank)]
    sdt, ddt = (MOVE_DTYPES[int(rng.integers(8))] for _ in range(2))
    (ls, lso), (ld, ldo) = random_layout(rng, shape), random_layout(rng, shape)
    x = random_values(rng, sdt, shape, 8000 + seed)
    if sdt == M.f32:
        x = (x * 300).astype(np.float32)
    got = run_spec(M.Move(shape, (sdt, ddt), layouts=[ls, ld]), [x, np.zeros(shape, NP[ddt])])
    want = orc.move(shape, [int(sdt), int(ddt)], x, np.zeros(shape, NP[ddt]), layouts=[lso, ldo])
    assert np.array_equal(got.view(np.uint8), want.view(np.uint8)), (shape, sdt, ddt, repr(ls), repr(ld))


@pytest.mark.parametrize("seed", range(40))
def test_random_softmax(gpu, seed):
    rng = np.random.default_rng(9000 + seed)
    rank = int(rng.integers(1, 5))
    shape = [int(rng.choice(SIZES)) for _ in range(rank)]
    dim = int(rng.integers(rank))
    (li, lio), (lo, loo) = random_layout(rng, shape), random_layout(rng, shape)
    x = (synth.normal_f32(9000 + seed, 0, shape) * 4).astype(np.float32)
    got = run_spec(M.Softmax(shape, dim, layouts=[li, lo]), [x, np.zeros(shape, np.float32)])
    want = orc.softmax(shape, dim, x, np.zeros(shape, np.float32), layouts=[lio, loo])
    np.testing.assert_allclose(got, want, rtol=1e-5, atol=1e-8, err_msg=str((shape, dim, repr(li), repr(lo))))


CONV_DTYPES = [(M.u8, M.i8, M.i32), (M.i8, M.i8, M.i32), (M.f32, M.f32, M.f32), (M.u8, M.u8, M.u16)]


@pytest.mark.parametrize("seed", range(40))
def test_random_conv(gpu, seed):
    rng = np.random.default_rng(9500 + seed)
    big = rng.random() < 0.4  # shapes the matrix-core kernel takes
    b = int(rng.integers(1, 3))
    f = 64 if big else int(rng.integers(1, 9))
    c = 64 if big else int(rng.integers(1, 9))
    oh, ow = int(rng.integers(1, 7)), int(rng.integers(1, 7))
    fh, fw = ((3, 3) if rng.random() < 0.6 else (1, 1)) if big else (int(rng.integers(1, 4)), int(rng.integers(1, 4)))
    dts = CONV_DTYPES[int(rng.integers(2 if big else 4))]
    accum = bool(rng.integers(2))
    shape = [b, f, c, oh, ow, fh, fw]
    pshapes = [[b, c, oh + fh - 1, ow + fw - 1], [f, c, fh, fw], [b, f, oh, ow]]
    lay = [random_layout(rng, s) for s in pshapes]
    bufs = [random_values(rng, dt, s, 9500 + seed * 3 + i) for i, (dt, s) in enumerate(zip(dts, pshapes))]
    if not accum:
        bufs[2] = np.zeros(pshapes[2], NP[dts[2]])
    got = run_spec(M.Conv(shape, dts, layouts=[l[0] for l in lay], accum=accum), bufs)
    want = orc.conv(shape, [int(d) for d in dts], bufs[0], bufs[1], bufs[2].copy(), accum,
                    layouts=[l[1] for l in lay])
    compare(got, want, dts[2], (shape, dts, accum, [repr(l[0]) for l in lay]))


MFMA_DTYPES = [(M.u8, M.i8, M.i32), (M.i8, M.i8, M.i32), (M.bf16, M.bf16, M.f32), (M.f32, M.f32, M.f32),
               (M.bf16, M.f32, M.f32)]


@pytest.mark.parametrize("seed", range(60))
def test_random_matmul_mid_sizes(gpu, seed):
    """Sizes where the library's own choices change: which tile (64 / 128 / 256), padded copies
    for rows that are not whole 16-byte chunks, the matrix-vector kernel (few rows, k-fastest B),
    column-major operands made row-major; dims drawn so that the product stays below 2e8."""
    rng = np.random.default_rng(7500 + seed)
    b = int(rng.choice([1, 1, 1, 2]))
    pool = [1, 2, 3, 5, 8, 9, 16, 40, 64, 100, 128, 129, 255, 256, 257, 300, 384, 500, 512, 513, 640, 777, 1000, 1024, 1100]
    while True:
        m, k, n = (int(rng.choice(pool)) for _ in range(3))
        if b * m * k * n <= 2e8:
            break
    dts = MFMA_DTYPES[int(rng.integers(len(MFMA_DTYPES)))]
    accum = bool(rng.integers(2))
    shape = [b, m, k, n]
    pshapes = [[b, m, k], [b, k, n], [b, m, n]]
    # Row-major mostly; B k-fastest in a third of the cases; now and then any layout.
    lay = []
    for i, s in enumerate(pshapes):
        roll = rng.random()
        if i == 1 and roll < 0.35:
            lay.append((M.layout(0, 2, 1), orc.make_layout([0, 2, 1])))
        elif roll < 0.8:
            lay.append((M.row_major(s), orc.make_layout([0, 1, 2])))
        else:
            lay.append(random_layout(rng, s))
    bufs = [random_values(rng, dt, s, 7500 + seed * 3 + i) for i, (dt, s) in enumerate(zip(dts, pshapes))]
    if not accum:
        bufs[2] = np.zeros(pshapes[2], NP[dts[2]])
    spec = M.Matmul(shape, dts, layouts=[l[0] for l in lay], accum=accum)
    got = run_spec(spec, bufs)
    want = orc.matmul(shape, [int(d) for d in dts], bufs[0], bufs[1], bufs[2].copy(), accum,
                      layouts=[l[1] for l in lay])
    compare(got, want, dts[2], (shape, dts, accum, [repr(l[0]) for l in lay]))


@pytest.mark.parametrize("seed", range(40))
def test_random_conv_mid_sizes(gpu, seed):
    """Conv shapes the unfolded (Conv as Matmul) path takes, next to the fused kernel's and the
    generic kernel's: channel counts that are and are not whole dwords / 16-byte chunks, filters
    from 1x1 to 5x5, every Matmul dtype triple, random layouts now and then."""
    rng = np.random.default_rng(9700 + seed)
    b = int(rng.integers(1, 4))
    f = int(rng.choice([1, 8, 24, 64, 65, 100]))
    c = int(rng.choice([1, 3, 4, 16, 24, 64, 128]))
    oh, ow = int(rng.integers(1, 21)), int(rng.integers(1, 21))
    fh, fw = int(rng.integers(1, 6)), int(rng.integers(1, 6))
    dts = [(M.u8, M.i8, M.i32), (M.i8, M.i8, M.i32), (M.bf16, M.bf16, M.f32), (M.f32, M.f32, M.f32)][int(rng.integers(4))]
    accum = bool(rng.integers(2))
    shape = [b, f, c, oh, ow, fh, fw]
    pshapes = [[b, c, oh + fh - 1, ow + fw - 1], [f, c, fh, fw], [b, f, oh, ow]]
    nhwc = (lambda s: (M.nhwc(s), orc.make_layout([0, 2, 3, 1])))
    lay = [nhwc(s) if rng.random() < 0.75 else random_layout(rng, s) for s in pshapes]
    bufs = [random_values(rng, dt, s, 9700 + seed * 3 + i) for i, (dt, s) in enumerate(zip(dts, pshapes))]
    if not accum:
        bufs[2] = np.zeros(pshapes[2], NP[dts[2]])
    got = run_spec(M.Conv(shape, dts, layouts=[l[0] for l in lay], accum=accum), bufs)
    want = orc.conv(shape, [int(d) for d in dts], bufs[0], bufs[1], bufs[2].copy(), accum,
                    layouts=[l[1] for l in lay])
    compare(got, want, dts[2], (shape, dts, accum, [repr(l[0]) for l in lay]))


@pytest.mark.parametrize("seed", range(48))
def test_random_compose_msm(gpu, seed):
    """Matmul -> Softmax -> Matmul over random shapes: sequence lengths around the fused kernel's
    blocks (128 or 64 queries, 2 x 64 keys), head dims it is built for and ones it pads, the two
    head dims equal or not, KT k-fastest (layout![0,2,1]) or in the reference's default order,
    scores of random spread.  The dispatch rules' own choice and every fused action (both query
    blocks, every key share count) against the oracle: norm-wise 1e-2, and element-wise against
    a floor of the result's rms (bf16 rounding of P bounds the error per output, not per digit)."""
    from gpu_util import elem_err
    rng = np.random.default_rng(9900 + seed)
    b = int(rng.integers(1, 5))
    m = int(rng.choice([1, 2, 17, 31, 32, 33, 63, 64, 65, 100, 127, 128, 129, 200, 256, 300]))
    n2 = int(rng.choice([1, 7, 8, 63, 64, 65, 127, 128, 129, 200, 256, 264, 500, 777, 1024, 1500]))
    k = int(rng.choice([8, 16, 24, 32, 40, 64, 96, 128]))
    n = k if rng.random() < 0.6 else int(rng.choice([2, 8, 32, 48, 64, 100, 128]))
    kt_fastest = rng.random() < 0.6
    spread = float(rng.choice([0.2, 0.5, 1.0, 1.5]))
    q = synth.normal_bf16(9900 + seed, 0, (b, m, k), spread)
    v = synth.normal_bf16(9900 + seed, 2, (b, n2, n), 0.5)
    if kt_fastest:
        kmat = synth.normal_bf16(9900 + seed, 1, (b, n2, k), spread)   # K row-major == KT as layout![0,2,1]
        lay, olay = [None, None, M.layout(0, 2, 1), None], [None, None, orc.make_layout([0, 2, 1]), None]
    else:
        kmat = synth.normal_bf16(9900 + seed, 1, (b, k, n2), spread)   # KT row-major, n2 fastest
        lay, olay = None, None
    spec = M.ComposeMSM(b, m, k, n2, n, layouts=lay)
    want = orc.compose_msm(b, m, k, n2, n, [7, 7, 7, 6], v, q, kmat, np.zeros((b, m, n), np.float32), layouts=olay)
    what = (b, m, k, n2, n, kt_fastest, spread)

    def run(target):
        bufs = [M.DeviceBuffer.from_numpy(a) for a in (v, q, kmat, np.full((b, m, n), 7.5, np.float32))]
        target.run_device([x.ptr for x in bufs])
        out = bufs[-1].to_numpy(np.float32, (b, m, n))
        for x in bufs:
            x.free()
        return out

    for target in [spec] + [a for a in spec.actions() if a.kind == M.ActionKind.Fused]:
        got = run(target)
        assert np.isfinite(got).all(), (what, target)
        assert rel_err(got, want) < 1e-2, (what, target)
        assert elem_err(got, want, floor_frac=1.0) < 2e-2, (what, target)


PART_SPECS = [  # (constructor, oracle kind, which parameters span the scan dim, takes accum)
    (M.Max, orc.PART_MAX, (True, False), True),
    (M.SoftmaxDenominator, orc.PART_DENOM, (True, False, False), True),
    (M.SoftmaxDenominatorAndMax, orc.PART_DENOM_MAX, (True, False, False), True),
    (M.SoftmaxDenominatorAndMaxFromParts, orc.PART_FROM_PARTS, (True, True, False, False), True),
    (M.SoftmaxDenominatorAndUnscaled, orc.PART_UNSCALED, (True, False, True), False),
    (M.SoftmaxDenominatorAndUnscaledFromMax, orc.PART_UNSCALED_FROM_MAX, (True, False, False, True), True),
    (M.SoftmaxComplete, orc.PART_COMPLETE, (True, False, False, True), False),
    (M.DivideVecScalar, orc.PART_DIVIDE_VEC_SCALAR, (True, False), False),
]


@pytest.mark.parametrize("seed", range(96))
def test_random_softmax_primitives(gpu, seed):
    """The primitives of the Softmax decomposition over random shapes (one dim sometimes long, so
    that every way of sharing out the lines is met: a wavefront per line, register-resident lines,
    lines side by side), scan dims, accumulation and a random order of the dims per parameter;
    every parameter as it stands afterwards against the oracle's."""
    rng = np.random.default_rng(9300 + seed)
    ctor, kind, full, takes_accum = PART_SPECS[seed % len(PART_SPECS)]
    rank = int(rng.integers(1, 5))
    shape = [int(rng.choice(SIZES[:24])) for _ in range(rank)]
    if rng.random() < 0.6:
        shape[int(rng.integers(rank))] = int(rng.choice([256, 1000, 1024, 2048, 4096, 4100, 20000]))
    while int(np.prod(shape)) > (1 << 21):   # drop the smallest dim that is not 1 yet
        shape[min((d for d in range(rank) if shape[d] > 1), key=lambda d: shape[d])] = 1
    dim = int(rng.integers(rank))
    accum = takes_accum and bool(rng.integers(2))
    red = list(shape)
    red[dim] = 1
    x = (synth.normal_f32(9300 + seed, 0, shape) * 3).astype(np.float32)
    mx = x.max(axis=dim, keepdims=True) + np.float32(rng.integers(0, 2))
    positive = lambda i, s: np.abs(synth.normal_f32(9300 + seed, i, s)) + np.float32(0.5)
    if kind == orc.PART_MAX:
        params = [x, synth.normal_f32(9300 + seed, 1, red)]
    elif kind in (orc.PART_DENOM, orc.PART_DENOM_MAX):
        params = [x, mx if kind == orc.PART_DENOM else synth.normal_f32(9300 + seed, 1, red), positive(2, red)]
    elif kind == orc.PART_FROM_PARTS:
        params = [x, positive(1, shape), synth.normal_f32(9300 + seed, 2, red), positive(3, red)]
    elif kind == orc.PART_UNSCALED:
        params = [x, positive(1, red), np.zeros(shape, np.float32)]
    elif kind == orc.PART_UNSCALED_FROM_MAX:
        params = [x, mx, positive(2, red), np.zeros(shape, np.float32)]
    elif kind == orc.PART_COMPLETE:
        params = [x, mx, positive(2, red), np.zeros(shape, np.float32)]
    else:
        params = [x, positive(1, red)]
    perms = [tuple(int(d) for d in rng.permutation(rank)) for _ in params]
    stored = [np.ascontiguousarray(p.transpose(perm)) for p, perm in zip(params, perms)]
    kwargs = dict(accum=accum) if takes_accum else {}
    spec = ctor(shape, dim, layouts=[M.layout(*perm) for perm in perms], **kwargs)
    bufs = [M.DeviceBuffer.from_numpy(a) for a in stored]
    spec.run_device([b.ptr for b in bufs])
    got = [b.to_numpy(np.float32, a.shape) for a, b in zip(stored, bufs)]
    for b in bufs:
        b.free()
    want = orc.softmax_part(kind, shape, dim, [p.copy() for p in params], accum)
    what = (ctor.__name__, shape, dim, accum, perms, spec.plan().kernels)
    for g, w, perm in zip(got, want, perms):
        np.testing.assert_allclose(g, w.transpose(perm), rtol=1e-4 if shape[dim] > 512 else 2e-5, atol=1e-7, err_msg=str(what))


@pytest.mark.parametrize("seed", range(48))
def test_random_broadcast_and_fill(gpu, seed):
    rng = np.random.default_rng(9400 + seed)
    rank = int(rng.integers(1, 5))
    shape = [int(rng.choice(SIZES)) for _ in range(rank)]
    dim = int(rng.integers(rank))
    dtype = [M.u8, M.bf16, M.f32, M.i16, M.u32][seed % 5]
    red = list(shape)
    red[dim] = 1
    x = random_values(rng, dtype, red, 9400 + seed)
    lay = random_layout(rng, shape)[0] if rng.random() < 0.3 else None
    if lay is None:
        got = run_spec(M.Broadcast(shape, dim, dtype), [x, np.zeros(shape, NP[dtype])])
        assert np.array_equal(got, np.broadcast_to(x, shape)), (shape, dim, dtype)
    count = int(np.prod(shape))
    value = M.FillValue.NegInf if dtype in (M.bf16, M.f32) and seed % 2 else M.FillValue.Min
    whole = np.full(count + 40, 0x55, NP[dtype])
    buf = M.DeviceBuffer.from_numpy(whole)
    M.Fill(shape, dtype, value, layout=lay).run_device([buf.ptr])
    back = buf.to_numpy(NP[dtype], whole.shape)
    buf.free()
    codes = {M.u8: orc.U8, M.bf16: orc.BF16, M.f32: orc.F32, M.i16: orc.I16, M.u32: orc.U32}
    assert np.array_equal(back[:count].view(np.uint8), orc.fill(codes[dtype], int(value), count).view(np.uint8))
    assert np.all(back[count:] == 0x55)
