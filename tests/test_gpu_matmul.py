"""Matmul Spec on the MI355X against the CPU oracle, through the C ABI.

Integer Specs must match bit for bit; bf16-in/f32-accumulate within 1e-2 relative (measured
far tighter); f32 within 1e-5 relative, and exactly on the reference's integer-valued check
inputs (verification.rs:893-952).
"""
import numpy as np
import pytest

import morello_amd as M
import orc
from gpu_util import elem_err, rel_err, run_spec
from morello_amd import synth

pytestmark = pytest.mark.gpu

GEN = {M.u8: synth.uniform_u8, M.i8: synth.uniform_i8}


def int_inputs(seed, dts, b, m, k, n, accum):
    A = GEN[dts[0]](seed, 0, (b, m, k))
    Bm = GEN[dts[1]](seed, 1, (b, k, n))
    C0 = (synth.uniform_u8(seed, 2, (b, m, n)).astype(np.int32) * 1000 - 99) if accum else np.zeros((b, m, n), np.int32)
    return A, Bm, C0


@pytest.mark.parametrize("dts", [(M.u8, M.i8, M.i32), (M.i8, M.i8, M.i32)])
@pytest.mark.parametrize("shape,accum", [
    ((1, 64, 64, 64), False),       # one 64 x 64 tile
    ((1, 256, 128, 256), False),    # exactly one MFMA tile, one k step
    ((1, 256, 256, 256), True),
    ((1, 512, 384, 768), False),    # several tiles, odd tile counts
    ((3, 256, 256, 512), True),     # batched
    ((1, 1024, 1024, 1024), True),
    ((1, 100, 37, 51), True),       # ragged, rows not whole 16-byte chunks: generic kernel
    ((1, 300, 208, 272), True),     # ragged, whole chunks: MFMA kernel with masked borders
    ((2, 257, 144, 1040), False),
    ((1, 1000, 1008, 1024), True),
    ((1, 64, 4096, 64), False),     # one sliver of a tile, long K
    ((1, 1, 1, 1), False),
])
def test_int8_matmul_bit_exact(gpu, dts, shape, accum):
    b, m, k, n = shape
    A, Bm, C0 = int_inputs(11, dts, b, m, k, n, accum)
    got = run_spec(M.Matmul(shape, dts, accum=accum), [A, Bm, C0])
    want = orc.matmul(list(shape), [int(d) for d in dts], A, Bm, C0.copy(), accum)
    assert np.array_equal(got, want)


def test_int8_matmul_extremes(gpu):
    """All-255 times all-(-128): every partial sum sits on the no-overflow bound, and the
    u8 -> signed correction term is at its largest."""
    m, k, n = 256, 4096, 256
    A = np.full((1, m, k), 255, np.uint8)
    Bm = np.full((1, k, n), -128, np.int8)
    got = run_spec(M.Matmul([1, m, k, n], (M.u8, M.i8, M.i32)), [A, Bm, np.zeros((1, m, n), np.int32)])
    assert (got == -133693440).all()
    Bm = np.full((1, k, n), 127, np.int8)
    got = run_spec(M.Matmul([1, m, k, n], (M.u8, M.i8, M.i32)), [A, Bm, np.zeros((1, m, n), np.int32)])
    assert (got == 255 * 127 * k).all()


def test_int8_matmul_reference_check_pattern(gpu):
    """The reference's own check inputs: counting ints in every parameter, output included."""
    b, m, k, n = 1, 256, 256, 256
    A = synth.check_pattern("u8", (b, m, k))
    Bm = synth.check_pattern("i8", (b, k, n))
    C0 = synth.check_pattern("i32", (b, m, n))
    want = np.matmul(A.astype(np.int64), Bm.astype(np.int64))
    got = run_spec(M.Matmul([b, m, k, n], (M.u8, M.i8, M.i32)), [A, Bm, C0])
    assert np.array_equal(got, want)
    got = run_spec(M.MatmulAccum([b, m, k, n], (M.u8, M.i8, M.i32)), [A, Bm, C0])
    assert np.array_equal(got.astype(np.int64), (want + C0 + 2**31) % 2**32 - 2**31)


def test_int8_matmul_full_size_properties(gpu):
    """benchmark configuration 2 (4096^3) through size-independent checks: a band of rows against
    the oracle, every row/column against checksums computed in int64, and accumulation
    across two calls (the reference's bench loop accumulates the same way)."""
    m = k = n = 4096
    A = synth.uniform_u8(21, 0, (1, m, k))
    Bm = synth.uniform_i8(21, 1, (1, k, n))
    spec = M.MatmulAccum([1, m, k, n], (M.u8, M.i8, M.i32))
    dA, dB = M.DeviceBuffer.from_numpy(A), M.DeviceBuffer.from_numpy(Bm)
    dC = M.DeviceBuffer(m * n * 4)
    dC.zero()
    spec.run_device([dA.ptr, dB.ptr, dC.ptr])
    got = dC.to_numpy(np.int32, (m, n))
    for lo in (0, 2017, 4064):
        want = np.zeros((1, m, n), np.int32)
        orc.matmul([1, m, k, n], [0, 1, 5], A, Bm, want, True, rows=(lo, lo + 32))
        assert np.array_equal(got[lo:lo + 32], want[0, lo:lo + 32])
    a64, b64 = A[0].astype(np.int64), Bm[0].astype(np.int64)
    assert np.array_equal(got.astype(np.int64).sum(axis=1), a64 @ b64.sum(axis=1))   # row checksums
    assert np.array_equal(got.astype(np.int64).sum(axis=0), a64.sum(axis=0) @ b64)   # column checksums
    spec.run_device([dA.ptr, dB.ptr, dC.ptr])
    assert np.array_equal(dC.to_numpy(np.int32, (m, n)), got * 2)


@pytest.mark.parametrize("da,db,dc", [(M.u8, M.u8, M.u32), (M.u8, M.i8, M.i16), (M.i16, M.u16, M.i32),
                                      (M.u32, M.u32, M.u32), (M.i8, M.u8, M.u8), (M.u8, M.i8, M.f32)])
def test_other_dtype_combinations_generic(gpu, da, db, dc):
    b, m, k, n = 2, 33, 70, 45
    raw = lambda t, d: synth.raw_u64(31, t, int(np.prod(d))).astype(np.uint64)
    A = raw(0, (b, m, k)).astype(da.numpy).reshape(b, m, k)
    Bm = raw(1, (b, k, n)).astype(db.numpy).reshape(b, k, n)
    C0 = np.zeros((b, m, n), dc.numpy)
    got = run_spec(M.Matmul([b, m, k, n], (da, db, dc)), [A, Bm, C0])
    want = orc.matmul([b, m, k, n], [int(da), int(db), int(dc)], A, Bm, C0.copy())
    if dc == M.f32:
        assert rel_err(got, want) < 1e-6
    else:
        assert np.array_equal(got, want)


def test_f32_matmul_plumbing_config(gpu):
    """benchmark configuration 1: f32 64^3, uniform[-1,1), accumulate into a zeroed C."""
    shape = [1, 64, 64, 64]
    A, Bm = synth.uniform_f32(41, 0, (1, 64, 64)), synth.uniform_f32(41, 1, (1, 64, 64))
    got = run_spec(M.MatmulAccum(shape, [M.f32] * 3), [A, Bm, np.zeros((1, 64, 64), np.float32)])
    want = orc.matmul(shape, [6, 6, 6], A, Bm, np.zeros((1, 64, 64), np.float32), True)
    assert rel_err(got, want) < 1e-5
    # the reference's check inputs are integer valued: exact
    A = synth.check_pattern("f32", (1, 64, 64))
    C0 = synth.check_pattern("f32", (1, 64, 64))
    got = run_spec(M.MatmulAccum(shape, [M.f32] * 3), [A, A.copy(), C0])
    want = np.matmul(A.astype(np.int64), A.astype(np.int64)) + C0.astype(np.int64)
    assert np.array_equal(got, want.astype(np.float32))


@pytest.mark.parametrize("shape,accum", [((1, 256, 64, 256), False), ((1, 512, 512, 512), True),
                                         ((2, 256, 192, 256), False), ((1, 60, 100, 36), False),
                                         ((1, 300, 200, 264), True), ((2, 129, 72, 520), False)])
def test_bf16_matmul(gpu, shape, accum):
    b, m, k, n = shape
    A, Bm = synth.normal_bf16(51, 0, (b, m, k)), synth.normal_bf16(51, 1, (b, k, n))
    C0 = synth.normal_f32(51, 2, (b, m, n)) if accum else np.zeros((b, m, n), np.float32)
    got = run_spec(M.Matmul(shape, (M.bf16, M.bf16, M.f32), accum=accum), [A, Bm, C0])
    want = orc.matmul(list(shape), [7, 7, 6], A, Bm, C0.copy(), accum)
    assert rel_err(got, want) < 1e-2  # stated tolerance
    assert rel_err(got, want) < 1e-5  # what f32 accumulation actually delivers at these K


@pytest.mark.parametrize("shape,accum", [((1, 256, 32, 256), False), ((1, 512, 512, 512), True),
                                         ((2, 256, 96, 256), False), ((1, 300, 100, 264), True),
                                         ((2, 129, 68, 516), False), ((1, 64, 64, 64), True)])
def test_f32_matmul_on_the_matrix_cores(gpu, shape, accum):
    """f32 x f32 -> f32 from 64 x 64 x 64 up runs on v_mfma_f32_32x32x2_f32: whole tiles,
    ragged borders (rows of whole 16-byte chunks), batches, accumulation."""
    b, m, k, n = shape
    A, Bm = synth.uniform_f32(61, 0, (b, m, k)), synth.uniform_f32(61, 1, (b, k, n))
    C0 = synth.normal_f32(61, 2, (b, m, n)) if accum else np.zeros((b, m, n), np.float32)
    got = run_spec(M.Matmul(shape, [M.f32] * 3, accum=accum), [A, Bm, C0])
    want = np.matmul(A.astype(np.float64), Bm.astype(np.float64)) + (C0 if accum else 0)
    assert rel_err(got, want) < 1e-5
    assert rel_err(got, orc.matmul(list(shape), [6, 6, 6], A, Bm, C0.copy(), accum)) < 1e-5
    # Integer-valued inputs (the reference's 0..3 pattern): every partial sum is exact.
    A, Bm = synth.check_pattern("f32", (b, m, k)), synth.check_pattern("f32", (b, k, n))
    got = run_spec(M.Matmul(shape, [M.f32] * 3), [A, Bm, np.zeros((b, m, n), np.float32)])
    assert np.array_equal(got, np.matmul(A.astype(np.int64), Bm.astype(np.int64)).astype(np.float32))


@pytest.mark.parametrize("dts,codes", [((M.u8, M.i8, M.i32), [0, 1, 5]), ((M.i8, M.i8, M.i32), [1, 1, 5]),
                                        ((M.bf16, M.bf16, M.f32), [7, 7, 6]), ((M.f32, M.f32, M.f32), [6, 6, 6])])
@pytest.mark.parametrize("shape,accum", [((1, 256, 256, 256), False), ((2, 300, 136, 200), True),
                                         ((1, 64, 64, 70), False), ((3, 512, 128, 256), True)])
def test_matmul_with_k_fastest_b(gpu, dts, codes, shape, accum):
    """B stored with k fastest (batched_col_major, layout.rs:1255-1271) runs on the matrix cores
    with its tile staged like A's: whole tiles, ragged borders (any N), batches, accumulation."""
    b, m, k, n = shape
    gen = {M.u8: synth.uniform_u8, M.i8: synth.uniform_i8, M.bf16: synth.normal_bf16, M.f32: synth.uniform_f32}
    A, Bm = gen[dts[0]](71, 0, (b, m, k)), gen[dts[1]](71, 1, (b, k, n))
    out_np = np.int32 if dts[2] == M.i32 else np.float32
    C0 = (synth.uniform_u8(71, 2, (b, m, n)).astype(out_np) if accum else np.zeros((b, m, n), out_np))
    layouts = [None, M.batched_col_major([b, k, n]), None]
    Bt = np.ascontiguousarray(Bm.transpose(0, 2, 1))  # the buffer a k-fastest layout describes
    got = run_spec(M.Matmul(shape, dts, layouts=layouts, accum=accum), [A, Bt, C0])
    want = orc.matmul(list(shape), codes, A, Bm, C0.copy(), accum)
    if dts[2] == M.i32:
        assert np.array_equal(got, want)
    else:
        assert rel_err(got, want) < 1e-5


@pytest.mark.parametrize("b_k_fastest", [False, True])
@pytest.mark.parametrize("dts,codes", [((M.u8, M.i8, M.i32), [0, 1, 5]), ((M.i8, M.i8, M.i32), [1, 1, 5]),
                                        ((M.bf16, M.bf16, M.f32), [7, 7, 6]), ((M.f32, M.f32, M.f32), [6, 6, 6])])
@pytest.mark.parametrize("shape,accum", [
    ((1, 1, 256, 512), False),      # a single row: the 64 x 64 tile with 63 rows out of range
    ((1, 16, 64, 16), True),        # less than one small tile in every direction
    ((3, 40, 48, 80), True),
    ((1, 768, 64, 704), False),     # 132 tiles of 64 x 64
    ((2, 1500, 32, 1296), True),    # int8 / bf16: 128 x 128 tiles (1008 small ones would be too many)
    ((1, 2900, 48, 2832), False),   # 144 tiles of 256 x 256, ragged on both borders and in K
    ((1, 3840, 32, 3600), True),    # 225 tiles: the 256 x 256 tile for f32 too
    ((2, 333, 77, 515), True),      # rows that are not whole 16-byte chunks: zero-padded copies
    ((1, 1000, 1001, 999), False),
    ((1, 1, 4099, 4101), True),
])
def test_matmul_every_tile_choice(gpu, dts, codes, shape, accum, b_k_fastest):
    """The library picks the workgroup tile (64, 128 or 256 square) from the problem size; each
    choice, with B stored n-fastest and k-fastest, against the oracle."""
    b, m, k, n = shape
    gen = {M.u8: synth.uniform_u8, M.i8: synth.uniform_i8, M.bf16: synth.normal_bf16, M.f32: synth.uniform_f32}
    A, Bm = gen[dts[0]](73, 0, (b, m, k)), gen[dts[1]](73, 1, (b, k, n))
    out_np = np.int32 if dts[2] == M.i32 else np.float32
    C0 = (synth.uniform_u8(73, 2, (b, m, n)).astype(out_np) if accum else np.zeros((b, m, n), out_np))
    layouts = [None, M.batched_col_major([b, k, n]), None] if b_k_fastest else None
    Bbuf = np.ascontiguousarray(Bm.transpose(0, 2, 1)) if b_k_fastest else Bm
    got = run_spec(M.Matmul(shape, dts, layouts=layouts, accum=accum), [A, Bbuf, C0])
    want = orc.matmul(list(shape), codes, A, Bm, C0.copy(), accum)
    if dts[2] == M.i32:
        assert np.array_equal(got, want)
    else:
        assert rel_err(got, want) < 1e-5


@pytest.mark.parametrize("dts,codes", [((M.u8, M.i8, M.i32), [0, 1, 5]), ((M.i8, M.i8, M.i32), [1, 1, 5]),
                                        ((M.bf16, M.bf16, M.f32), [7, 7, 6]), ((M.f32, M.f32, M.f32), [6, 6, 6])])
@pytest.mark.parametrize("shape,accum", [
    ((1, 1, 2048, 16384), False),   # examples/matvec_gemma_x86_bf16f32.rs:24-37
    ((1, 1, 1024, 70), True),       # columns that do not fill the last wavefront
    ((3, 2, 4096, 129), True),      # batched, two rows
    ((2, 3, 1040, 256), False),     # three rows on the four-row build, K not a multiple of a wave's stride
    ((1, 4, 8192, 64), True),
    ((2, 7, 2064, 100), True),      # seven rows on the eight-row build
    ((1, 8, 1024, 1000), False),
    ((1, 1, 300, 4096), False),     # row-major B: one slice of K that is not whole steps of 64
    ((2, 3, 1000, 8192), True),
    ((1, 4, 2048, 4112), True),
    ((4, 1, 3565, 256), False),     # one row whose K is not whole 16-byte chunks: the padded copy keeps its stride
    ((2, 1, 1001, 300), True),
])
@pytest.mark.parametrize("b_k_fastest", [True, False])
def test_matrix_vector_shapes(gpu, dts, codes, shape, accum, b_k_fastest):
    """Up to eight rows of A against a k-fastest B run as dot products that stream B once instead
    of on the matrix cores; the same shapes with a row-major B stay on the 64 x 64 MFMA tile.
    Same results as any other Matmul."""
    b, m, k, n = shape
    gen = {M.u8: synth.uniform_u8, M.i8: synth.uniform_i8, M.bf16: synth.normal_bf16, M.f32: synth.uniform_f32}
    A, Bm = gen[dts[0]](75, 0, (b, m, k)), gen[dts[1]](75, 1, (b, k, n))
    out_np = np.int32 if dts[2] == M.i32 else np.float32
    C0 = (synth.uniform_u8(75, 2, (b, m, n)).astype(out_np) if accum else np.zeros((b, m, n), out_np))
    Bbuf = np.ascontiguousarray(Bm.transpose(0, 2, 1)) if b_k_fastest else Bm
    spec = M.Matmul(shape, dts, layouts=[None, M.layout(0, 2, 1) if b_k_fastest else None, None], accum=accum)
    got = run_spec(spec, [A, Bbuf, C0])
    want = orc.matmul(list(shape), codes, A, Bm, C0.copy(), accum)
    if dts[2] == M.i32:
        assert np.array_equal(got, want)
    else:
        assert rel_err(got, want) < 1e-5


@pytest.mark.parametrize("dts,codes,shape,accum", [((M.bf16, M.bf16, M.f32), [7, 7, 6], (1, 1, 4096, 32768), True),
                                                    ((M.u8, M.i8, M.i32), [0, 1, 5], (1, 1, 8192, 32770), False)])
def test_matrix_vector_against_a_very_large_b(gpu, dts, codes, shape, accum):
    """One row of A against a k-fastest B of 200 MB and more: a row of B per wavefront (the
    smaller ones take two).  Same results as any other Matmul; the second shape's last
    workgroup holds two columns of its four."""
    b, m, k, n = shape
    gen = {M.u8: synth.uniform_u8, M.i8: synth.uniform_i8, M.bf16: synth.normal_bf16}
    A, Bm = gen[dts[0]](76, 0, (b, m, k)), gen[dts[1]](76, 1, (b, k, n))
    Bt = np.ascontiguousarray(Bm.transpose(0, 2, 1))   # B as stored: [n][k]
    out_np = np.int32 if dts[2] == M.i32 else np.float32
    C0 = synth.uniform_u8(76, 2, (b, m, n)).astype(out_np) if accum else np.zeros((b, m, n), out_np)
    spec = M.Matmul(shape, dts, layouts=[None, M.layout(0, 2, 1), None], accum=accum)
    assert spec.plan().kernels == ["k_gemv"] and "COLS = 1" in spec.plan().steps[0].kernel
    got = run_spec(spec, [A, Bt, C0])
    want = orc.matmul(list(shape), codes, A, Bm, C0.copy(), accum)
    if dts[2] == M.i32:
        assert np.array_equal(got, want)
    else:
        assert rel_err(got, want) < 1e-5


@pytest.mark.parametrize("dts,codes", [((M.u8, M.i8, M.i32), [0, 1, 5]), ((M.i8, M.i8, M.i32), [1, 1, 5]),
                                       ((M.bf16, M.bf16, M.f32), [7, 7, 6]), ((M.f32, M.f32, M.f32), [6, 6, 6])])
@pytest.mark.parametrize("shape,accum", [((1, 512, 8192, 512), False), ((1, 256, 16384, 192), True),
                                         ((1, 100, 4096, 300), True), ((1, 32, 4096, 1000), False),
                                         ((1, 130, 2048, 70), False),
                                         # K is no whole number of equal slices: a shorter one behind them
                                         ((1, 300, 30000, 300), True), ((1, 64, 16256, 128), False), ((1, 96, 5008, 40), False)])
@pytest.mark.parametrize("b_k_fastest", [True, False])
def test_matmul_with_k_shared_out_over_workgroups(gpu, dts, codes, shape, accum, b_k_fastest):
    """Few output tiles and a long K: slices of K run as batch entries and their partial results
    are summed in slice order (exact for integers, the f32 sum in another association for floats).
    Whole and ragged M and N, accumulation into C, both B orientations, every dtype kind; a K of
    127 steps (no divisor), of 234 steps and 48 bytes, of 39 steps and 16 bytes."""
    b, m, k, n = shape
    if dts[0] == M.f32:
        k //= 2  # the same number of 128-byte k steps at twice the element size would take twice as long on the oracle
    shape = (b, m, k, n)
    gen = {M.u8: synth.uniform_u8, M.i8: synth.uniform_i8, M.bf16: synth.normal_bf16, M.f32: synth.uniform_f32}
    A, Bm = gen[dts[0]](76, 0, (b, m, k)), gen[dts[1]](76, 1, (b, k, n))
    out_np = np.int32 if dts[2] == M.i32 else np.float32
    C0 = (synth.uniform_u8(76, 2, (b, m, n)).astype(out_np) if accum else np.zeros((b, m, n), out_np))
    Bbuf = np.ascontiguousarray(Bm.transpose(0, 2, 1)) if b_k_fastest else Bm
    spec = M.Matmul(list(shape), dts, layouts=[None, M.layout(0, 2, 1) if b_k_fastest else None, None], accum=accum)
    assert "k_sum_splits" in spec.plan().kernels
    got = run_spec(spec, [A, Bbuf, C0])
    want = orc.matmul(list(shape), codes, A, Bm, C0.copy(), accum)
    if dts[2] == M.i32:
        assert np.array_equal(got, want)
    else:
        assert rel_err(got, want) < (1e-2 if dts[0] == M.bf16 else 1e-5)


@pytest.mark.parametrize("dts,codes", [((M.f32, M.bf16, M.f32), [6, 7, 6]), ((M.bf16, M.f32, M.f32), [7, 6, 6])])
def test_mixed_bf16_f32_matmul(gpu, dts, codes):
    """One bf16 and one f32 input with an f32 output: both are taken to f32 before the product,
    as the reference's interpreter does (verification.rs:115-134)."""
    b, m, k, n = 2, 192, 136, 264
    gen = {M.bf16: synth.normal_bf16, M.f32: synth.uniform_f32}
    A, Bm = gen[dts[0]](81, 0, (b, m, k)), gen[dts[1]](81, 1, (b, k, n))
    C0 = synth.normal_f32(81, 2, (b, m, n))
    got = run_spec(M.MatmulAccum([b, m, k, n], dts), [A, Bm, C0])
    assert rel_err(got, orc.matmul([b, m, k, n], codes, A, Bm, C0.copy(), True)) < 1e-5


@pytest.mark.parametrize("dts,codes", [((M.u8, M.i8, M.i32), [0, 1, 5]), ((M.bf16, M.bf16, M.f32), [7, 7, 6]),
                                        ((M.f32, M.bf16, M.f32), [6, 7, 6])])
@pytest.mark.parametrize("accum", [False, True])
def test_matmul_with_column_major_a_and_c(gpu, dts, codes, accum):
    """A and C stored column-major (m fastest): brought to row-major with the strided Move,
    multiplied on the matrix cores, and C moved back."""
    b, m, k, n = 2, 192, 128, 136
    gen = {M.u8: synth.uniform_u8, M.i8: synth.uniform_i8, M.bf16: synth.normal_bf16, M.f32: synth.uniform_f32}
    A, Bm = gen[dts[0]](72, 0, (b, m, k)), gen[dts[1]](72, 1, (b, k, n))
    out_np = np.int32 if dts[2] == M.i32 else np.float32
    C0 = synth.uniform_u8(72, 2, (b, m, n)).astype(out_np) if accum else np.zeros((b, m, n), out_np)
    layouts = [M.batched_col_major([b, m, k]), None, M.batched_col_major([b, m, n])]
    At = np.ascontiguousarray(A.transpose(0, 2, 1))
    C0t = np.ascontiguousarray(C0.transpose(0, 2, 1))
    got_t = run_spec(M.Matmul([b, m, k, n], dts, layouts=layouts, accum=accum), [At, Bm, C0t])
    want = orc.matmul([b, m, k, n], codes, A, Bm, C0.copy(), accum)
    got = got_t.transpose(0, 2, 1)
    if dts[2] == M.i32:
        assert np.array_equal(got, want)
    else:
        assert rel_err(got, want) < 1e-5


def test_bf16_matmul_pattern_exact(gpu):
    """0..3 inputs (verification.rs:933-935): every partial sum is an exact integer."""
    b, m, k, n = 1, 256, 256, 256
    A = synth.check_pattern("bf16", (b, m, k))
    Bm = synth.check_pattern("bf16", (b, k, n))
    got = run_spec(M.Matmul([b, m, k, n], (M.bf16, M.bf16, M.f32)), [A, Bm, np.zeros((b, m, n), np.float32)])
    want = np.matmul(synth.bf16_bits_to_f32(A).astype(np.int64), synth.bf16_bits_to_f32(Bm).astype(np.int64))
    assert np.array_equal(got, want.astype(np.float32))


def test_bf16_matmul_full_size_sample(gpu):
    """benchmark configuration 3 (8192^3): sampled rows against the oracle, plus linearity."""
    m = k = n = 8192
    A, Bm = synth.normal_bf16(61, 0, (1, m, k)), synth.normal_bf16(61, 1, (1, k, n))
    dA, dB = M.DeviceBuffer.from_numpy(A), M.DeviceBuffer.from_numpy(Bm)
    dC = M.DeviceBuffer(m * n * 4)
    spec = M.Matmul([1, m, k, n], (M.bf16, M.bf16, M.f32))
    spec.run_device([dA.ptr, dB.ptr, dC.ptr])
    got = dC.to_numpy(np.float32, (m, n))
    for lo in (0, 5000, 8184):
        want = np.zeros((1, m, n), np.float32)
        orc.matmul([1, m, k, n], [7, 7, 6], A, Bm, want, False, rows=(lo, lo + 8))
        # stated tolerance 1e-2; what f32 accumulation in another order gives is far inside it, norm-wise
        # and element by element (|r| floored at 1 % of the RMS result)
        assert rel_err(got[lo:lo + 8], want[0, lo:lo + 8]) < 1e-4
        assert elem_err(got[lo:lo + 8], want[0, lo:lo + 8]) < 1e-3
    spec_acc = M.MatmulAccum([1, m, k, n], (M.bf16, M.bf16, M.f32))
    spec_acc.run_device([dA.ptr, dB.ptr, dC.ptr])
    # the old value of an element enters its sum first or last depending on the kernel: one rounding apart
    assert rel_err(dC.to_numpy(np.float32, (m, n)), got * 2) < 1e-5
    # The accumulating Spec on a C that is neither zero nor the product: bands against the oracle.
    C0 = synth.normal_f32(61, 2, (1, m, n), 100.0)
    dC.free()
    dC = M.DeviceBuffer.from_numpy(C0)
    spec_acc.run_device([dA.ptr, dB.ptr, dC.ptr])
    got = dC.to_numpy(np.float32, (m, n))
    for lo in (0, 2600, 8184):
        want = C0.copy()
        orc.matmul([1, m, k, n], [7, 7, 6], A, Bm, want, True, rows=(lo, lo + 8))
        assert rel_err(got[lo:lo + 8], want[0, lo:lo + 8]) < 1e-4
        assert elem_err(got[lo:lo + 8], want[0, lo:lo + 8]) < 1e-3


def test_matmul_layouts(gpu):
    """Column-major and packed parameter layouts (layout.rs:1249, examples/matmul_x86.rs
    relayouts) give the same logical result as row-major."""
    b, m, k, n = 1, 64, 48, 32
    A, Bm = synth.uniform_u8(71, 0, (b, m, k)), synth.uniform_i8(71, 1, (b, k, n))
    want = orc.matmul([b, m, k, n], [0, 1, 5], A, Bm, np.zeros((b, m, n), np.int32))
    # B column-major: buffer holds B transposed
    spec = M.Matmul([b, m, k, n], (M.u8, M.i8, M.i32), layouts=[None, M.col_major([b, k, n]), None])
    got = run_spec(spec, [A, np.ascontiguousarray(Bm.transpose(0, 2, 1)), np.zeros((b, m, n), np.int32)])
    assert np.array_equal(got, want)
    # B packed [0,2,1,2 p(16)] and C column-major
    packed = M.layout(0, 2, 1, (2, M.Packed(16)))
    Bp = np.zeros(b * k * n, np.int8)
    for kk in range(k):
        for nn in range(n):
            Bp[packed.buffer_index([b, k, n], [0, kk, nn])] = Bm[0, kk, nn]
    spec = M.Matmul([b, m, k, n], (M.u8, M.i8, M.i32), layouts=[None, packed, M.col_major([b, m, n])])
    got = run_spec(spec, [A, Bp, np.zeros((b, n, m), np.int32)])
    assert np.array_equal(got.transpose(0, 2, 1), want)
    # Packed dims that spell row-major order (read in place), on A and on the output
    same_a, same_c = M.layout(0, 1, 2, (2, M.Packed(16))), M.layout(0, 1, 2, (2, M.Packed(8)))
    spec = M.Matmul([b, m, k, n], (M.u8, M.i8, M.i32), layouts=[same_a, None, same_c])
    assert np.array_equal(run_spec(spec, [A, Bm, np.zeros((b, m, n), np.int32)]), want)
    # OddEven on K of A, Packed on N of B: staged through the layouts' common strided view
    oe, pk = M.layout(0, 1, 2, (2, M.OddEven(8))), M.layout(0, 1, 2, (1, M.Packed(4)))
    Ao, Bk = np.zeros(b * m * k, np.uint8), np.zeros(b * k * n, np.int8)
    for i in range(m):
        for kk in range(k):
            Ao[oe.buffer_index([b, m, k], [0, i, kk])] = A[0, i, kk]
    for kk in range(k):
        for nn in range(n):
            Bk[pk.buffer_index([b, k, n], [0, kk, nn])] = Bm[0, kk, nn]
    spec = M.Matmul([b, m, k, n], (M.u8, M.i8, M.i32), layouts=[oe, pk, None])
    assert np.array_equal(run_spec(spec, [Ao, Bk, np.zeros((b, m, n), np.int32)]), want)


def test_run_host_entry_point(gpu):
    """mrl_run_host: the stand-in for calling the emitted kernel with host pointers."""
    b, m, k, n = 1, 256, 128, 256
    A, Bm = synth.uniform_u8(81, 0, (b, m, k)), synth.uniform_i8(81, 1, (b, k, n))
    C1 = np.full((b, m, n), 5, np.int32)
    M.MatmulAccum([b, m, k, n], (M.u8, M.i8, M.i32)).run_host(A, Bm, C1)
    want = orc.matmul([b, m, k, n], [0, 1, 5], A, Bm, np.full((b, m, n), 5, np.int32), True)
    assert np.array_equal(C1, want)


def test_manual_schedules_give_identical_results(gpu):
    """Every tile_out/split schedule the kernel is built for computes the same Spec: bit for
    bit for the integer Spec, and to f32 rounding for bf16 (the k loop order changes)."""
    b, m, k, n = 2, 512, 384, 768
    A, Bm = synth.uniform_u8(91, 0, (b, m, k)), synth.uniform_i8(91, 1, (b, k, n))
    C0 = synth.uniform_u8(91, 2, (b, m, n)).astype(np.int32)
    spec = M.MatmulAccum([b, m, k, n], (M.u8, M.i8, M.i32))
    want = orc.matmul([b, m, k, n], [0, 1, 5], A, Bm, C0.copy(), True)
    scheds = spec.available_schedules()
    assert (256, 256, 128) in scheds and len(scheds) >= 4
    for tm, tn, sk in scheds:
        bufs = [M.DeviceBuffer.from_numpy(x) for x in (A, Bm, C0)]
        spec.tile_out([1, tm, tn]).split(sk).run_device([x.ptr for x in bufs])
        assert np.array_equal(bufs[2].to_numpy(np.int32, (b, m, n)), want), (tm, tn, sk)
    # ragged problem under a small-tile schedule
    b, m, k, n = 1, 200, 144, 336
    A, Bm = synth.uniform_i8(92, 0, (b, m, k)), synth.uniform_i8(92, 1, (b, k, n))
    spec = M.Matmul([b, m, k, n], (M.i8, M.i8, M.i32))
    want = orc.matmul([b, m, k, n], [1, 1, 5], A, Bm, np.zeros((b, m, n), np.int32))
    bufs = [M.DeviceBuffer.from_numpy(x) for x in (A, Bm, np.zeros((b, m, n), np.int32))]
    spec.tile_out([1, 128, 128]).split(64).run_device([x.ptr for x in bufs])
    assert np.array_equal(bufs[2].to_numpy(np.int32, (b, m, n)), want)
    # bf16: split counted in elements (32 bf16 = 64 bytes)
    b, m, k, n = 1, 256, 256, 512
    A, Bm = synth.normal_bf16(93, 0, (b, m, k)), synth.normal_bf16(93, 1, (b, k, n))
    spec = M.Matmul([b, m, k, n], (M.bf16, M.bf16, M.f32))
    want = orc.matmul([b, m, k, n], [7, 7, 6], A, Bm, np.zeros((b, m, n), np.float32))
    for tm, tn, sk in spec.available_schedules():
        bufs = [M.DeviceBuffer.from_numpy(x) for x in (A, Bm, np.zeros((b, m, n), np.float32))]
        spec.tile_out([1, tm, tn]).split(sk).run_device([x.ptr for x in bufs])
        assert rel_err(bufs[2].to_numpy(np.float32, (b, m, n)), want) < 1e-5, (tm, tn, sk)
    # f32: split counted in elements (16 f32 = 64 bytes)
    b, m, k, n = 1, 320, 136, 264
    A, Bm = synth.uniform_f32(94, 0, (b, m, k)), synth.uniform_f32(94, 1, (b, k, n))
    fspec = M.Matmul([b, m, k, n], [M.f32] * 3)
    want = np.matmul(A.astype(np.float64), Bm.astype(np.float64))
    assert (256, 256, 32) in fspec.available_schedules() and (128, 128, 16) in fspec.available_schedules()
    for tm, tn, sk in fspec.available_schedules():
        fb = [M.DeviceBuffer.from_numpy(x) for x in (A, Bm, np.zeros((b, m, n), np.float32))]
        fspec.tile_out([1, tm, tn]).split(sk).run_device([x.ptr for x in fb])
        assert rel_err(fb[2].to_numpy(np.float32, (b, m, n)), want) < 1e-5, (tm, tn, sk)
    # a schedule that is not built, and a Spec without a matrix-core kernel
    with pytest.raises(M.MorelloError) as e:
        spec.tile_out([1, 32, 32]).split(32).run_device([x.ptr for x in bufs])
    assert e.value.status == 1
    assert M.Matmul([1, 64, 64, 64], [M.u32] * 3).available_schedules() == []


def test_matmul_output_beyond_4_gib(gpu):
    """Near the largest output the Spec surface admits (volume < 2^31 elements,
    tensorspec.rs:180-182): C is 8.5 GB, so byte offsets pass 2^32 and 2^33 is near.  Bands of rows at the
    start, across the 4 GiB and 6 GiB marks and at the end, bit-exact against the oracle;
    the rows between must have been written too (a sentinel would survive otherwise)."""
    import ctypes as C
    from morello_amd import _binding as B
    m, k, n = 1 << 20, 64, 2040
    A = synth.uniform_u8(99, 0, (1, m, k))
    Bm = synth.uniform_i8(99, 1, (1, k, n))
    spec = M.Matmul([1, m, k, n], (M.u8, M.i8, M.i32))
    assert spec.check() == 0 and spec.bytes_used(2) == m * n * 4 > (1 << 32)
    da, db = M.DeviceBuffer.from_numpy(A), M.DeviceBuffer.from_numpy(Bm)
    dc = M.DeviceBuffer(m * n * 4)
    assert B.load().mrl_memset(dc.ptr, 0x5a, m * n * 4) == 0
    spec.run_device([da.ptr, db.ptr, dc.ptr])
    row_bytes = n * 4
    for r0 in (0, (1 << 32) // row_bytes - 2, (3 << 31) // row_bytes - 2, m // 3, m - 4):
        got = np.empty((4, n), np.int32)
        assert B.load().mrl_memcpy_d2h(got.ctypes.data_as(C.c_void_p), C.c_void_p(dc.ptr + r0 * row_bytes),
                                       4 * row_bytes) == 0
        want = A[0, r0:r0 + 4].astype(np.int32) @ Bm[0].astype(np.int32)
        assert np.array_equal(got, want), r0
    for buf in (da, db, dc):
        buf.free()


def test_generic_matmul_with_a_million_rows(gpu):
    """A dtype triple without a matrix-core kernel at 2^20 + 5 rows: the generic kernel's tile
    numbering must not depend on the 65535 limit of the second grid dimension."""
    m, k, n = (1 << 20) + 5, 3, 20
    A = synth.check_pattern("u16", (1, m, k))
    Bm = synth.check_pattern("u16", (1, k, n))
    got = run_spec(M.Matmul([1, m, k, n], (M.u16, M.u16, M.u32)), [A, Bm, np.zeros((1, m, n), np.uint32)])
    want = (A[0].astype(np.uint64) @ Bm[0].astype(np.uint64)).astype(np.uint32)
    assert np.array_equal(got[0], want)


def test_float_operands_saturate_at_the_output_dtype(gpu):
    """Operands are cast to the output dtype with Rust `as` (verification.rs:547-569): a float
    saturates at that dtype's own bounds.  Hand-computed: 300.0 as i8 = 127, -200.0 as i8 = -128,
    -5.0 as u8 = 0, 70000.0 as u16 = 65535, NaN = 0."""
    a = np.array([[300.0, -200.0, -5.0, 70000.0, np.nan, 2.9]], np.float32)        # 1 x 6
    b = np.eye(6, dtype=np.float32)
    for dt, np_dt, want in ((M.i8, np.int8, [127, -128, -5, 127, 0, 2]),
                            (M.u8, np.uint8, [255, 0, 0, 255, 0, 2]),
                            (M.u16, np.uint16, [300, 0, 0, 65535, 0, 2]),
                            (M.i16, np.int16, [300, -200, -5, 32767, 0, 2])):
        got = run_spec(M.Matmul([1, 1, 6, 6], (M.f32, M.f32, dt)), [a, b, np.zeros((1, 6), np_dt)])
        assert got.reshape(-1).tolist() == want, (dt, got)
        orc_dt = {M.i8: orc.I8, M.u8: orc.U8, M.u16: orc.U16, M.i16: orc.I16}[dt]
        ref = orc.matmul([1, 1, 6, 6], [orc.F32, orc.F32, orc_dt], a, b, np.zeros((1, 6), np_dt))
        assert np.array_equal(got, ref)


@pytest.mark.parametrize("dts,codes", [((M.bf16, M.bf16, M.bf16), [7, 7, 7]), ((M.f32, M.f32, M.bf16), [6, 6, 7]),
                                       ((M.bf16, M.f32, M.bf16), [7, 6, 7]), ((M.u8, M.i8, M.bf16), [0, 1, 7])])
@pytest.mark.parametrize("accum", [False, True])
def test_matmul_with_bf16_output(gpu, dts, codes, accum):
    """bf16 outputs (spec.rs:3663-3698): inputs cast to bf16, f32 sums on the matrix cores, one
    rounding to bf16 (old output included for the accumulating form).  The oracle sums in k order,
    the kernel in its own, so sums may round to neighbouring bf16 values: nearly all elements are
    bit-identical and none is further than one rounding step (2^-8 relative) apart.  The reference
    itself has no comparison for bf16 (verification.rs:597)."""
    b, m, k, n = 2, 200, 384, 136
    def operand(dt, tid, shape):
        return {M.bf16: lambda: synth.normal_bf16(77, tid, shape, 0.5), M.f32: lambda: synth.normal_f32(77, tid, shape, 0.5),
                M.u8: lambda: synth.uniform_u8(77, tid, shape), M.i8: lambda: synth.uniform_i8(77, tid, shape)}[dt]()
    a, bm = operand(dts[0], 0, (b, m, k)), operand(dts[1], 1, (b, k, n))
    c0 = synth.normal_bf16(77, 2, (b, m, n), 3.0) if accum else np.zeros((b, m, n), np.uint16)
    want = synth.bf16_bits_to_f32(orc.matmul([b, m, k, n], codes, a, bm, c0.copy(), accum))
    got = synth.bf16_bits_to_f32(run_spec(M.Matmul([b, m, k, n], dts, accum=accum), [a, bm, c0.copy()]))
    assert np.isfinite(got).all()
    assert (got == want).mean() > 0.97
    assert np.all(np.abs(got - want) <= 2.0 ** -7 * np.maximum(np.abs(want), 2.0 ** -10 * np.abs(want).max()))
    # A column-major output and a packed input keep working through the same road.
    if dts == (M.bf16, M.bf16, M.bf16) and not accum:
        spec = M.Matmul([b, m, k, n], dts, layouts=[None, None, M.batched_col_major([b, m, n])])
        got_t = synth.bf16_bits_to_f32(run_spec(spec, [a, bm, np.zeros((b, n, m), np.uint16)]))
        assert np.array_equal(got_t.transpose(0, 2, 1), got)


@pytest.mark.parametrize("dts,codes", [((M.u8, M.i8, M.i32), [0, 1, 5]), ((M.i8, M.i8, M.i32), [1, 1, 5]),
                                       ((M.bf16, M.bf16, M.f32), [7, 7, 6])])
@pytest.mark.parametrize("shape", [(1, 256, 20, 256), (2, 512, 22, 256), (1, 256, 36, 768), (1, 768, 52, 512)])
@pytest.mark.parametrize("accum", [False, True])
def test_the_four_wave_kernel_on_its_shapes(gpu, dts, codes, shape, accum):
    """k_gemm_wide (256 x 256 tiles on four waves, MFMAs of 16 x 16) named through its schedule:
    one and several tiles each way, batch entries, every length of the unrolled prologue
    (accumulating Specs read C's old values during the first sixteen k steps) and of the rolled
    loop behind it, all three operand types; K in steps of 128 bytes.  Integers bit for bit."""
    b, m, steps, n = shape
    es = 2 if dts[0] == M.bf16 else 1
    k = steps * 128 // es
    if dts[0] == M.bf16:
        A, Bm = synth.normal_bf16(95, 0, (b, m, k)), synth.normal_bf16(95, 1, (b, k, n))
        C0 = synth.normal_f32(95, 2, (b, m, n)) if accum else np.zeros((b, m, n), np.float32)
    else:
        A = synth.uniform_u8(95, 0, (b, m, k)) if dts[0] == M.u8 else synth.uniform_i8(95, 0, (b, m, k))
        Bm = synth.uniform_i8(95, 1, (b, k, n))
        C0 = (synth.uniform_u8(95, 2, (b, m, n)).astype(np.int32) * 1000003 - 77) if accum else np.zeros((b, m, n), np.int32)
    spec = M.Matmul([b, m, k, n], dts, accum=accum)
    sched = spec.tile_out([1, 256, 256]).split(128 // es).staged(M.Staging.DirectBWide)
    assert sched.plan().kernels == ["k_gemm_wide"]
    bufs = [M.DeviceBuffer.from_numpy(x) for x in (A, Bm, C0)]
    sched.run_device([x.ptr for x in bufs])
    got = bufs[2].to_numpy(C0.dtype, (b, m, n))
    for x in bufs:
        x.free()
    want = orc.matmul([b, m, k, n], codes, A, Bm, C0.copy(), accum)
    if dts[2] == M.i32:
        assert np.array_equal(got, want)
    else:
        assert rel_err(got, want) < 1e-5


def test_the_four_wave_kernel_turns_down_other_shapes(gpu):
    spec = M.Matmul([1, 256, 2432, 256], (M.u8, M.i8, M.i32))     # 19 steps: an odd number, and too few
    with pytest.raises(M.MorelloError) as e:
        spec.tile_out([1, 256, 256]).split(128).staged(M.Staging.DirectBWide).plan()
    assert e.value.status == 1


@pytest.mark.parametrize("dts,codes", [((M.u8, M.i8, M.i32), [0, 1, 5]), ((M.bf16, M.bf16, M.f32), [7, 7, 6])])
@pytest.mark.parametrize("steps", [4, 6, 10])
def test_the_four_wave_kernel_on_a_short_k(gpu, dts, codes, steps):
    """A Spec that does not accumulate needs none of the eight k steps that carry C's old values:
    the kernel takes it from four steps of 128 bytes on (the dispatch rules' own choice where the
    tiles run in one round); an accumulating Spec that short is turned down."""
    b, m, n = 1, 512, 768
    es = 2 if dts[0] == M.bf16 else 1
    k = steps * 128 // es
    if dts[0] == M.bf16:
        A, Bm = synth.normal_bf16(96, 0, (b, m, k)), synth.normal_bf16(96, 1, (b, k, n))
    else:
        A, Bm = synth.uniform_u8(96, 0, (b, m, k)), synth.uniform_i8(96, 1, (b, k, n))
    C0 = np.full((b, m, n), 7, np.float32 if dts[2] == M.f32 else np.int32)   # overwritten, not added to
    spec = M.Matmul([b, m, k, n], dts)
    assert M.Matmul([1, 4096, k, 4096], dts).plan().kernels == ["k_gemm_wide"]       # 256 tiles: one round
    assert M.Matmul([1, 8192, k, 8192], dts).plan().kernels == ["k_gemm_big"]        # four rounds
    sched = spec.tile_out([1, 256, 256]).split(128 // es).staged(M.Staging.DirectBWide)
    assert sched.plan().kernels == ["k_gemm_wide"]
    want = orc.matmul([b, m, k, n], codes, A, Bm, np.zeros_like(C0), False)
    bufs = [M.DeviceBuffer.from_numpy(x) for x in (A, Bm, C0)]
    sched.run_device([x.ptr for x in bufs])
    got = bufs[2].to_numpy(C0.dtype, (b, m, n))
    for x in bufs:
        x.free()
    if dts[2] == M.i32:
        assert np.array_equal(got, want)
    else:
        assert rel_err(got, want) < 1e-5
    with pytest.raises(M.MorelloError) as e:
        M.MatmulAccum([b, m, k, n], dts).tile_out([1, 256, 256]).split(128 // es).staged(M.Staging.DirectBWide).plan()
    assert e.value.status == 1


@pytest.mark.gpu
@pytest.mark.parametrize("dts,codes", [((M.u8, M.i8, M.i32), [0, 1, 5]), ((M.i8, M.i8, M.i32), [1, 1, 5]),
                                       ((M.bf16, M.bf16, M.f32), [7, 7, 6])])
@pytest.mark.parametrize("steps", [20, 26])
def test_the_four_wave_kernel_accumulating_over_several_rounds_of_tiles(gpu, dts, codes, steps):
    """More tiles than compute units (workgroups that start while others are in their loops or
    storing), on a C that is not zero, with a K that takes the variant with two loop steps between
    the steps that carry C's old values (26 steps) and the consecutive one (20)."""
    b, m, n = 33, 512, 1024         # 264 tiles
    es = 2 if dts[0] == M.bf16 else 1
    k = steps * 128 // es
    if dts[0] == M.bf16:
        A, Bm = synth.normal_bf16(98, 0, (b, m, k)), synth.normal_bf16(98, 1, (b, k, n))
        C0 = synth.normal_f32(98, 2, (b, m, n), 30.0)
    else:
        A = synth.uniform_u8(98, 0, (b, m, k)) if dts[0] == M.u8 else synth.uniform_i8(98, 0, (b, m, k))
        Bm = synth.uniform_i8(98, 1, (b, k, n))
        C0 = (synth.uniform_i8(98, 2, (b, m, n)).astype(np.int32) * 1000003)
    spec = M.MatmulAccum([b, m, k, n], dts)
    assert spec.plan().kernels == ["k_gemm_wide"]
    want = orc.matmul([b, m, k, n], codes, A, Bm, C0.copy(), True)
    bufs = [M.DeviceBuffer.from_numpy(x) for x in (A, Bm, C0)]
    spec.run_device([x.ptr for x in bufs])
    got = bufs[2].to_numpy(C0.dtype, (b, m, n))
    for x in bufs:
        x.free()
    if dts[2] == M.i32:
        assert np.array_equal(got, want)
    else:
        assert rel_err(got, want) < 1e-5


@pytest.mark.parametrize("dts,codes", [((M.u8, M.i8, M.i32), [0, 1, 5]), ((M.bf16, M.bf16, M.f32), [7, 7, 6])])
@pytest.mark.parametrize("steps", [12, 14, 16, 18, 20, 22, 24, 26, 28, 30, 32, 98, 100, 102])
def test_the_four_wave_kernel_accumulating_over_every_loop_exit(gpu, dts, codes, steps):
    """An accumulating Spec runs ten unrolled steps (the first eight load C's old values) and then a
    loop of six that is entered at its fifth step and left after any two; from 26 and from 98
    steps on, the steps with C's old values have two / eleven steps of the loop between them and
    the loop is left after any step: every number of steps modulo six for each of the three,
    from the shortest K the kernel takes, against the oracle on a C that is not zero."""
    b, m, n = 2, 256, 512
    es = 2 if dts[0] == M.bf16 else 1
    k = steps * 128 // es
    if dts[0] == M.bf16:
        A, Bm = synth.normal_bf16(97, 0, (b, m, k)), synth.normal_bf16(97, 1, (b, k, n))
        C0 = synth.normal_f32(97, 2, (b, m, n), 30.0)
    else:
        A, Bm = synth.uniform_u8(97, 0, (b, m, k)), synth.uniform_i8(97, 1, (b, k, n))
        C0 = (synth.uniform_i8(97, 2, (b, m, n)).astype(np.int32) * 1000003)
    sched = M.MatmulAccum([b, m, k, n], dts).tile_out([1, 256, 256]).split(128 // es).staged(M.Staging.DirectBWide)
    assert sched.plan().kernels == ["k_gemm_wide"]
    want = orc.matmul([b, m, k, n], codes, A, Bm, C0.copy(), True)
    bufs = [M.DeviceBuffer.from_numpy(x) for x in (A, Bm, C0)]
    sched.run_device([x.ptr for x in bufs])
    got = bufs[2].to_numpy(C0.dtype, (b, m, n))
    for x in bufs:
        x.free()
    if dts[2] == M.i32:
        assert np.array_equal(got, want)
    else:
        assert rel_err(got, want) < 1e-5
