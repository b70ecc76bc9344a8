"""Move Spec on the MI355X against the CPU oracle (bit exact), through the C ABI."""
import numpy as np
import pytest

import morello_amd as M
import orc
from gpu_util import run_spec
from morello_amd import synth

pytestmark = pytest.mark.gpu


def test_move_plain_copy(gpu):
    for shape, dt in [((1024, 1024), M.f32), ((3, 5, 7), M.u8), ((1,), M.i32), ((4097,), M.i16)]:
        x = synth.raw_u64(401, 0, int(np.prod(shape))).astype(dt.numpy).reshape(shape)
        got = run_spec(M.Move(list(shape), (dt, dt)), [x, np.zeros(shape, dt.numpy)])
        assert np.array_equal(got, x)


@pytest.mark.parametrize("sdt,ddt", [(M.i32, M.u8), (M.u8, M.i32), (M.u8, M.f32), (M.f32, M.i8), (M.f32, M.u16),
                                     (M.f32, M.bf16), (M.bf16, M.f32), (M.i8, M.bf16), (M.bf16, M.i32)])
@pytest.mark.parametrize("shape", [[5, 129], [3, 4099]])   # the second: four elements per thread plus a tail
def test_move_casts(gpu, sdt, ddt, shape):
    if sdt == M.f32:
        x = (synth.normal_f32(402, 0, shape) * 200).astype(np.float32)
        x[0, :4] = [np.nan, 1e20, -1e20, 0.5]
    elif sdt == M.bf16:
        x = synth.f32_to_bf16_bits(synth.normal_f32(402, 0, shape) * 200)
    else:
        x = synth.raw_u64(402, 0, shape[0] * shape[1]).astype(sdt.numpy).reshape(shape)
    got = run_spec(M.Move(shape, (sdt, ddt)), [x, np.zeros(shape, ddt.numpy)])
    want = orc.move(shape, [int(sdt), int(ddt)], x, np.zeros(shape, ddt.numpy))
    assert np.array_equal(got, want)


def test_move_relayout(gpu):
    """The relayouts of examples/matmul_x86.rs:34-53 (layout![0,2,1,2 p(16)]) and NHWC."""
    shape = [2, 32, 48]
    x = synth.uniform_i8(403, 0, shape)
    packed = M.layout(0, 2, 1, (2, M.Packed(16)))
    got = run_spec(M.Move(shape, (M.i8, M.i8), layouts=[None, packed]), [x, np.zeros(x.size, np.int8)])
    want = orc.move(shape, [1, 1], x, np.zeros(x.size, np.int8),
                    layouts=[None, orc.make_layout([0, 2, 1, (2, 1, 16)])])
    assert np.array_equal(got, want)
    back = run_spec(M.Move(shape, (M.i8, M.i8), layouts=[packed, None]), [got, np.zeros(shape, np.int8)])
    assert np.array_equal(back, x)
    img = synth.uniform_u8(404, 0, (2, 3, 5, 7))
    got = run_spec(M.Move([2, 3, 5, 7], (M.u8, M.u8), layouts=[None, M.nhwc([2, 3, 5, 7])]),
                   [img, np.zeros((2, 5, 7, 3), np.uint8)])
    assert np.array_equal(got, img.transpose(0, 2, 3, 1))
    oe = M.layout(0, 1, (1, M.OddEven(8)))
    y = synth.uniform_u8(405, 0, (3, 16))
    got = run_spec(M.Move([3, 16], (M.u8, M.u8), layouts=[None, oe]), [y, np.zeros(48, np.uint8)])
    want = orc.move([3, 16], [0, 0], y, np.zeros(48, np.uint8), layouts=[None, orc.make_layout([0, 1, (1, 2, 8)])])
    assert np.array_equal(got, want)


def test_async_launches_on_two_streams(gpu):
    """Independent Specs enqueued on two streams (mrl_run_async), including one that stages a
    packed layout through the stream-ordered scratch allocation, then a dependent Spec on the
    first stream: results equal the synchronous ones."""
    s1, s2 = M.Stream(), M.Stream()
    b, m, k, n = 1, 256, 128, 256
    A, Bm = synth.uniform_u8(801, 0, (b, m, k)), synth.uniform_i8(801, 1, (b, k, n))
    x = synth.normal_f32(801, 2, (64, 96))
    da, db, dc = (M.DeviceBuffer.from_numpy(t) for t in (A, Bm, np.zeros((b, m, n), np.int32)))
    dx, dy = M.DeviceBuffer.from_numpy(x), M.DeviceBuffer.from_numpy(np.zeros((64, 96), np.float32))
    mm = M.MatmulAccum([b, m, k, n], (M.u8, M.i8, M.i32))
    sm = M.Softmax([64, 96], 1, layouts=[None, M.layout(0, 1, (1, M.Packed(8)))])
    for _ in range(3):
        mm.run_async([da.ptr, db.ptr, dc.ptr], s1)   # accumulates three times, in stream order
        sm.run_async([dx.ptr, dy.ptr], s2)
    s1.synchronize()
    s2.synchronize()
    want = orc.matmul([b, m, k, n], [0, 1, 5], A, Bm, np.zeros((b, m, n), np.int32))
    assert np.array_equal(dc.to_numpy(np.int32, (b, m, n)), 3 * want)
    # [0, 1, (1, Packed 8)] over [64, 96] keeps the row-major element order.
    got = dy.to_numpy(np.float32, (64, 96))
    assert np.abs(got - orc.softmax([64, 96], 1, x)).max() < 1e-6
    s1.destroy()
    s2.destroy()


def test_releasing_a_streams_arena(gpu):
    """mrl_stream_release: a Spec that stages operands (ragged K and N) runs on a stream, the
    stream's scratch arena is given back while the stream lives on, and the next call on the same
    stream (it starts a new arena) still accumulates onto the first one's result."""
    stream = M.Stream()
    b, m, k, n = 1, 300, 270, 290
    A, Bm = synth.uniform_u8(830, 0, (b, m, k)), synth.uniform_i8(830, 1, (b, k, n))
    bufs = [M.DeviceBuffer.from_numpy(x) for x in (A, Bm, np.zeros((b, m, n), np.int32))]
    spec = M.MatmulAccum([b, m, k, n], (M.u8, M.i8, M.i32))
    want = orc.matmul([b, m, k, n], [0, 1, 5], A, Bm, np.zeros((b, m, n), np.int32))
    free0 = M.device_free_bytes()
    spec.run_async([x.ptr for x in bufs], stream)
    stream.synchronize()
    held = free0 - M.device_free_bytes()
    M.release_stream(stream)  # waits for the work, then frees
    assert np.array_equal(bufs[2].to_numpy(np.int32, (b, m, n)), want)
    assert held >= 64 << 20 and M.device_free_bytes() >= free0 - (8 << 20)
    spec.run_async([x.ptr for x in bufs], stream)
    stream.synchronize()
    assert np.array_equal(bufs[2].to_numpy(np.int32, (b, m, n)), 2 * want)
    M.release_stream(None)  # the default stream: nothing kept, nothing to free, still fine
    stream.destroy()


def test_host_threads_share_a_stream_and_its_scratch(gpu):
    """Four host threads enqueue Matmuls that need scratch memory (K and N are not whole 16-byte
    chunks, so A and B are copied into padded rows) onto one stream, each thread several times
    with its own operands.  The stream's scratch arena is handed from call to call, so every
    result must still be its own thread's."""
    import threading
    stream = M.Stream()
    shapes = [(1, 300, 270, 290), (2, 257, 333, 201), (1, 400, 250, 310), (1, 260, 267, 500)]
    jobs = []
    for t, (b, m, k, n) in enumerate(shapes):
        A, Bm = synth.uniform_u8(820 + t, 0, (b, m, k)), synth.uniform_i8(820 + t, 1, (b, k, n))
        bufs = [M.DeviceBuffer.from_numpy(x) for x in (A, Bm, np.zeros((b, m, n), np.int32))]
        want = orc.matmul([b, m, k, n], [0, 1, 5], A, Bm, np.zeros((b, m, n), np.int32))
        jobs.append((M.MatmulAccum([b, m, k, n], (M.u8, M.i8, M.i32)), bufs, want, (b, m, n)))
    rounds, errors = 5, []

    def work(spec, bufs):
        try:
            for _ in range(rounds):
                spec.run_async([x.ptr for x in bufs], stream)
        except Exception as e:  # surfaced below: a thread's exception is otherwise lost
            errors.append(e)

    threads = [threading.Thread(target=work, args=(spec, bufs)) for spec, bufs, _, _ in jobs]
    for th in threads:
        th.start()
    for th in threads:
        th.join()
    stream.synchronize()
    assert not errors, errors
    for spec, bufs, want, shape in jobs:
        assert np.array_equal(bufs[2].to_numpy(np.int32, shape), rounds * want)
    stream.destroy()


@pytest.mark.parametrize("dt", [M.bf16, M.i16, M.u16])
@pytest.mark.parametrize("shape", [(2, 200, 136), (1, 130, 258), (3, 64, 64), (1, 1000, 2), (2, 33, 64), (1, 2048, 128),
                                   (1, 264, 520), (2, 136, 72), (1, 1030, 8)])
def test_transpose_of_16_bit_elements(gpu, dt, shape):
    """Row-major <-> batched column-major of 16-bit elements: eight elements per lane on the
    source side where its rows are whole 16-byte vectors, two per lane on both sides where the
    extents are even, one where they are not; whole and ragged 128 x 128 tiles."""
    x = synth.raw_u64(830, 0, int(np.prod(shape))).astype(np.uint16).reshape(shape)
    cm = M.batched_col_major(list(shape))
    got = run_spec(M.Move(list(shape), (dt, dt), layouts=[None, cm]), [x, np.zeros((shape[0], shape[2], shape[1]), np.uint16)])
    assert np.array_equal(got, x.transpose(0, 2, 1))
    back = run_spec(M.Move(list(shape), (dt, dt), layouts=[cm, None]), [got, np.zeros(shape, np.uint16)])
    assert np.array_equal(back, x)


@pytest.mark.parametrize("dt,npd", [(M.f32, np.float32), (M.i32, np.int32), (M.u32, np.uint32)])
@pytest.mark.parametrize("shape", [(2, 200, 136), (1, 132, 260), (3, 64, 64), (1, 1000, 4), (2, 33, 64), (1, 2048, 128),
                                   (1, 130, 258)])
def test_transpose_of_32_bit_elements(gpu, dt, npd, shape):
    """The same for 32-bit elements: four per lane on both sides where both extents are multiples
    of 4, one per lane otherwise; tiles in diagonal order."""
    x = synth.raw_u64(831, 0, int(np.prod(shape))).astype(np.uint32).view(npd).reshape(shape)
    cm = M.batched_col_major(list(shape))
    got = run_spec(M.Move(list(shape), (dt, dt), layouts=[None, cm]), [x, np.zeros((shape[0], shape[2], shape[1]), npd)])
    assert np.array_equal(got.view(np.uint32), x.transpose(0, 2, 1).view(np.uint32))
    back = run_spec(M.Move(list(shape), (dt, dt), layouts=[cm, None]), [got, np.zeros(shape, npd)])
    assert np.array_equal(back.view(np.uint32), x.view(np.uint32))


def _both(*dims):
    """A layout for the library and the same for the oracle: ints are Dynamic dims, (d, 'p', n) a
    Packed(n) dim and (d, 'oe', n) an OddEven(n) dim of logical dim d."""
    m, o = [], []
    for d in dims:
        if isinstance(d, tuple):
            m.append((d[0], M.Packed(d[2]) if d[1] == "p" else M.OddEven(d[2])))
            o.append((d[0], 1 if d[1] == "p" else 2, d[2]))
        else:
            m.append(d)
            o.append(d)
    return M.layout(*m), orc.make_layout(o)


GATHER_CASES = [
    (M.u8, M.u8, [40, 32, 96, 224], (3, 2, 1, 0), (1, 0, 3, 2, (3, "p", 8))),          # bytes in runs of four
    (M.u8, M.u8, [328, 640, 48], (1, 0, 2, (1, "oe", 4)), (1, 0, 2)),
    (M.i32, M.i32, [96, 208, 64], (2, 1, 0), (1, 2, 0, (0, "oe", 16))),                 # a digit covered in part
    (M.bf16, M.bf16, [16, 512, 64, 32], (3, 1, 2, 0, (3, "oe", 4)), (1, 0, 2, 3)),
    (M.u16, M.u16, [1152, 16, 32, 64], (2, 0, 3, 1), (1, 0, 2, 3)),                     # 16-bit runs
    (M.bf16, M.f32, [16, 280, 4, 504], (0, 2, 1, 3), (1, 2, 3, 0)),                     # converting, 2 -> 4 bytes
    (M.f32, M.bf16, [160, 35, 1024], (2, 0, 1, (2, "p", 8)), (0, 2, 1)),
    (M.i32, M.u8, [192, 35, 752], (0, 2, 1, (2, "oe", 8)), (0, 1, 2)),
    (M.u8, M.i32, [227, 35, 192], (0, 1, 2), (2, 0, 1, (2, "oe", 4))),
    (M.f32, M.f32, [12, 6, 20, 30, 40], (4, 3, 1, 2, 0), (0, 2, 1, 3, 4)),              # five digits
]


@pytest.mark.parametrize("sdt,ddt,shape,src,dst", GATHER_CASES)
def test_move_through_the_gather_kernel(gpu, sdt, ddt, shape, src, dst):
    """Layout pairs with neither a shared contiguous run nor two long contiguous dims, above the
    million elements up to which an element per thread serves: the tile kernel with runs of
    elements of every size, with and without conversion, with three to five digits in its tile."""
    NP = {M.u8: np.uint8, M.u16: np.uint16, M.i32: np.int32, M.f32: np.float32, M.bf16: np.uint16}
    (ls, lso), (ld, ldo) = _both(*src), _both(*dst)
    spec = M.Move(shape, (sdt, ddt), layouts=[ls, ld])
    assert spec.plan().kernels == ["k_move_gather"]
    if sdt == M.f32:
        x = (synth.normal_f32(840, 0, shape) * 300).astype(np.float32)
    elif sdt == M.bf16:
        x = synth.normal_bf16(840, 1, shape, 100.0)
    else:
        x = synth.raw_u64(840, 2, int(np.prod(shape))).astype(NP[sdt]).reshape(shape)
    got = run_spec(spec, [x, np.zeros(shape, NP[ddt])])
    want = orc.move(shape, [int(sdt), int(ddt)], x, np.zeros(shape, NP[ddt]), layouts=[lso, ldo])
    assert np.array_equal(got.view(np.uint8), want.view(np.uint8))


@pytest.mark.parametrize("dt,npd", [(M.u8, np.uint8), (M.i8, np.int8)])
@pytest.mark.parametrize("shape", [(2, 208, 144), (1, 132, 272), (3, 64, 64), (1, 1000, 16), (2, 36, 64), (1, 2048, 128),
                                   (1, 130, 258), (1, 400, 4000)])
def test_transpose_of_8_bit_elements(gpu, dt, npd, shape):
    """Bytes: sixteen per lane on the source side and a 4 x 4 byte transpose in registers where
    the source rows are whole 16-byte vectors and the destination rows whole dwords (whole and
    ragged 128 x 128 tiles, either direction), one byte per lane otherwise."""
    x = synth.raw_u64(832, 0, int(np.prod(shape))).astype(np.uint8).view(npd).reshape(shape)
    cm = M.batched_col_major(list(shape))
    spec = M.Move(list(shape), (dt, dt), layouts=[None, cm])
    if shape[2] % 16 == 0 and shape[1] % 4 == 0 and shape[1] * shape[2] * shape[0] > 65536:
        assert spec.plan().kernels == ["k_move_tiled8v"]
    got = run_spec(spec, [x, np.zeros((shape[0], shape[2], shape[1]), npd)])
    assert np.array_equal(got, x.transpose(0, 2, 1))
    back = run_spec(M.Move(list(shape), (dt, dt), layouts=[cm, None]), [got, np.zeros(shape, npd)])
    assert np.array_equal(back, x)
