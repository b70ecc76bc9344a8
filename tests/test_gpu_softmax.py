"""Softmax Spec and the Matmul->Softmax->Matmul Compose on the MI355X vs the CPU oracle."""
import numpy as np
import pytest

import morello_amd as M
import orc
from gpu_util import elem_err, rel_err, run_spec
from morello_amd import synth

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("shape,dim", [((8, 2048), 1), ((5, 33), 1), ((3, 7, 1000), 2), ((2, 64, 4096), 2),
                                       ((2, 3, 5000), 2), ((4, 9, 16), 1), ((6, 4), 0), ((16, 1), 1),
                                       ((2, 128, 1), 1)])
def test_softmax_within_1e5(gpu, shape, dim):
    x = synth.normal_f32(201, 0, shape, std=3.0)
    got = run_spec(M.Softmax(list(shape), dim), [x, np.zeros(shape, np.float32)])
    want = orc.softmax(list(shape), dim, x)
    # stated tolerance: 1e-5 relative, element-wise with a floor for denormal-small outputs
    assert (np.abs(got - want) <= 1e-5 * np.abs(want) + 1e-12).all()
    assert np.abs(got.sum(axis=dim) - 1).max() < 1e-5


def test_softmax_edge_values(gpu):
    x = np.zeros((4, 256), np.float32)
    x[0] = 2.5                                  # constant row -> exactly 1/n
    x[1, 7] = 1e4                               # one dominant element
    x[2] = -1e30                                # huge negatives, still finite
    x[3] = synth.normal_f32(202, 0, (256,)) + np.float32(80.0)  # exp(x) alone would overflow
    got = run_spec(M.Softmax([4, 256], 1), [x, np.zeros_like(x)])
    want = orc.softmax([4, 256], 1, x)
    assert np.array_equal(got[0], np.full(256, np.float32(1) / np.float32(256)))
    assert got[1, 7] == 1.0 and got[1].sum() == 1.0
    assert np.isfinite(got).all() and (np.abs(got - want) <= 1e-5 * np.abs(want) + 1e-12).all()


@pytest.mark.parametrize("shape,dim", [((64, 100000), 1), ((3, 4097), 1), ((5, 20000), 1), ((2, 8192), 1),
                                       ((1, 1 << 20), 1), ((300, 4100), 1), ((2, 3, 12290), 2), ((256, 8192), 1),
                                       ((300, 16384), 1), ((260, 4100), 1), ((257, 12292), 1), ((134, 2350), 1),
                                       ((7, 3, 1001), 2), ((4000, 258), 1)])
def test_softmax_long_rows(gpu, shape, dim):
    """Rows beyond the register kernel's 4096 columns: a workgroup per 4096-element chunk, the
    chunks' (max, denominator) pairs merged per row.  Column counts that are and are not
    multiples of 4 (vector and scalar loads), whole and ragged last chunks, one row.  With 256
    rows or more of up to 16384 columns a workgroup keeps its whole row in registers instead."""
    x = synth.normal_f32(204, 0, shape, std=3.0)
    got = run_spec(M.Softmax(list(shape), dim), [x, np.zeros(shape, np.float32)])
    want = orc.softmax(list(shape), dim, x)
    # The oracle sums a row's exponentials one after another in f32, as the reference's
    # interpreter does (verification.rs:166-184); over 1e5 terms that sum is itself 1.3e-4 away
    # from the exact value.  So: 1e-5 against the value computed in f64, and against the oracle
    # 1e-5 plus the oracle's own distance from it.
    x64 = x.astype(np.float64)
    e = np.exp(x64 - x64.max(axis=dim, keepdims=True))
    exact = e / e.sum(axis=dim, keepdims=True)
    assert (np.abs(got - exact) <= 1e-5 * exact + 1e-12).all()
    oracle_off = (np.abs(want - exact) / np.maximum(exact, 1e-30)).max()
    assert (np.abs(got - want) <= (1e-5 + oracle_off) * np.abs(want) + 1e-12).all()
    assert np.abs(got.sum(axis=dim, dtype=np.float64) - 1).max() < 1e-5


def test_softmax_long_rows_edge_values(gpu):
    """The chunked path's edges: the maximum in one chunk and everything else far below it, a
    chunk of f32::MIN, a NaN (the whole row becomes NaN, other rows do not)."""
    x = synth.normal_f32(205, 0, (4, 9000))
    x[0, 8999] = 1e4
    x[1, :4096] = np.finfo(np.float32).min
    x[2, 5000] = np.nan
    got = run_spec(M.Softmax([4, 9000], 1), [x, np.zeros_like(x)])
    want = orc.softmax([3, 9000], 1, np.ascontiguousarray(x[[0, 1, 3]]))
    assert got[0, 8999] == 1.0 and got[0].sum() == 1.0
    assert (got[1, :4096] == 0).all()
    assert np.isnan(got[2]).all()
    assert (np.abs(got[[0, 1, 3]] - want) <= 1e-5 * np.abs(want) + 1e-12).all()


@pytest.mark.parametrize("shape,dim", [((100000, 3), 1), ((5000, 67), 1), ((1000, 5, 12), 2), ((4097, 255), 1), ((3, 256), 1),
                                       ((7, 1), 1), ((300, 584, 5), 2), ((1, 129), 1), ((65, 33), 1), ((4, 9, 16), 2)])
def test_softmax_short_rows(gpu, shape, dim):
    """Rows of up to 256 elements: 1 to 32 lanes per row, several rows per wavefront (every lane
    count, row counts that leave a wavefront partly empty, a NaN confined to its row)."""
    x = synth.normal_f32(207, 0, shape, std=3.0)
    got = run_spec(M.Softmax(list(shape), dim), [x, np.zeros(shape, np.float32)])
    want = orc.softmax(list(shape), dim, x)
    assert (np.abs(got - want) <= 1e-5 * np.abs(want) + 1e-12).all()
    flat = x.reshape(-1, shape[-1]).copy()
    flat[0, 0] = np.nan
    if flat.shape[0] > 1:
        flat[1, :] = -np.inf
    got = run_spec(M.Softmax(list(flat.shape), 1), [flat, np.zeros_like(flat)])
    assert np.isnan(got[0]).all() and not np.isnan(got[2:]).any()
    want = orc.softmax(list(flat.shape), 1, flat)
    assert np.array_equal(np.isnan(got), np.isnan(want))
    assert (np.abs(got[2:] - want[2:]) <= 1e-5 * np.abs(want[2:]) + 1e-12).all()


@pytest.mark.parametrize("shape,dim", [((2048, 4096), 0), ((600, 70), 0), ((3, 1000, 130), 1), ((513, 64), 0),
                                       ((7, 16), 0), ((2, 5000, 17), 1)])
def test_softmax_over_an_outer_dim(gpu, shape, dim):
    _softmax_outer(shape, dim)


@pytest.mark.parametrize("shape,dim", [((8, 70000), 0), ((3, 5, 300, 100), 1), ((2, 16, 40000), 1), ((1, 70001), 0)])
def test_softmax_over_a_short_outer_dim(gpu, shape, dim):
    """A scan dim of at most 16 elements beside 65536 columns or more: a thread per column."""
    assert M.Softmax(list(shape), dim).plan().kernels == ["k_softmax_cols_short"]
    _softmax_outer(shape, dim)


@pytest.mark.parametrize("shape,dim", [((600, 64, 300), 0), ((100, 64, 300), 0), ((3, 520, 20000), 1)])
def test_softmax_over_an_outer_dim_in_one_kernel(gpu, shape, dim):
    """Enough columns for 256 workgroups of 64: the kernel that walks the scan dim itself, on 16
    waves (scan dims from 512) and on 4."""
    assert M.Softmax(list(shape), dim).plan().kernels == ["k_softmax_cols"]
    _softmax_outer(shape, dim)


@pytest.mark.parametrize("shape,dim,grid", [((2048, 4096), 0, (64, 16, 1)), ((2149, 172), 0, (3, 67, 1)),
                                            ((100000, 64), 0, (1, 256, 1)), ((5, 1000, 130), 1, (15, 31, 1)),
                                            ((3, 129, 8, 16), 1, (6, 4, 1))])
def test_softmax_over_an_outer_dim_of_few_columns(gpu, shape, dim, grid):
    """Fewer column tiles than compute units: the scan dim is cut into pieces as well (ragged last
    pieces, ragged column tiles, dims before and behind the scan dim), one launch leaves the
    pieces' (max, denominator) pairs and a second merges them (spec.rs:107-132) and writes.  A
    column with a NaN is NaN throughout, one of -inf only too, one with a single +inf as the
    reference's interpreter has it; the others are untouched by them."""
    plan = M.Softmax(list(shape), dim).plan()
    assert plan.kernels == ["k_softmax_cols", "k_softmax_cols"] and plan.steps[0].grid == grid
    _softmax_outer(shape, dim)
    x = synth.normal_f32(207, 0, shape, std=3.0)
    xs = np.moveaxis(x, dim, -1).copy()
    flat = xs.reshape(-1, shape[dim])
    flat[0, shape[dim] // 2] = np.nan
    flat[1, :] = -np.inf
    flat[2, shape[dim] - 1] = np.inf
    x = np.ascontiguousarray(np.moveaxis(xs, -1, dim))
    got = run_spec(M.Softmax(list(shape), dim), [x, np.zeros(shape, np.float32)])
    want = orc.softmax(list(shape), dim, x)
    assert np.array_equal(np.isnan(got), np.isnan(want))
    ok = ~np.isnan(want)
    tol = 1e-5 if shape[dim] <= 4096 else 2e-4      # the oracle's own f32 sum, as above
    assert (np.abs(got[ok] - want[ok]) <= tol * np.abs(want[ok]) + 1e-12).all()


def _softmax_outer(shape, dim):
    """The scan dim is not the contiguous one: 64 columns per workgroup, the scan dim split over
    its 4 or 16 waves (short and long scan dims, ragged column tiles and scan lengths).  1e-5
    against the value computed in f64, and against the oracle 1e-5 plus the oracle's own distance
    from it (its one-by-one f32 sum over 1e5 terms is 1e-4 off by itself)."""
    x = synth.normal_f32(206, 0, shape, std=3.0)
    got = run_spec(M.Softmax(list(shape), dim), [x, np.zeros(shape, np.float32)])
    want = orc.softmax(list(shape), dim, x)
    x64 = x.astype(np.float64)
    e = np.exp(x64 - x64.max(axis=dim, keepdims=True))
    exact = e / e.sum(axis=dim, keepdims=True)
    assert (np.abs(got - exact) <= 1e-5 * exact + 1e-12).all()
    oracle_off = (np.abs(want - exact) / np.maximum(exact, 1e-30)).max()
    assert (np.abs(got - want) <= (1e-5 + oracle_off) * np.abs(want) + 1e-12).all()


@pytest.mark.parametrize("shape,perm,dim", [((300, 200), (1, 0), 0), ((300, 200), (1, 0), 1), ((70, 4096), (1, 0), 1),
                                            ((8, 300, 64), (2, 1, 0), 0), ((8, 300, 64), (2, 1, 0), 1), ((8, 300, 64), (2, 1, 0), 2),
                                            ((6, 40, 500), (1, 0, 2), 2), ((6, 40, 500), (0, 2, 1), 2), ((5, 1, 260), (2, 1, 0), 0)])
def test_softmax_of_tensors_stored_in_another_order(gpu, shape, perm, dim):
    """Both tensors in the same permuted order (column-major, say): the dispatch goes by the order
    the dims are stored in, so a column-major matrix scanned along dim 0 takes the row kernels
    and one scanned along dim 1 the column kernels.  With only one of the two permuted the
    strided kernel runs."""
    lay = M.layout(*perm)
    x = (synth.normal_f32(31, 0, shape) * 3).astype(np.float32)
    want = orc.softmax(list(shape), dim, x)
    stored = lambda a: np.ascontiguousarray(a.transpose(perm))
    spec = M.Softmax(list(shape), dim, layouts=[lay, lay])
    # stored order [.., scan, after]: the column kernels want 16 contiguous elements behind the scan dim
    behind = int(np.prod([shape[d] for d in perm[perm.index(dim) + 1:]]))
    if behind == 1 or behind >= 16:
        assert spec.plan().kernels[0] in ("k_softmax_regs", "k_softmax_short", "k_softmax_block", "k_softmax_cols"), spec.plan()
    got = run_spec(spec, [stored(x), np.zeros(stored(x).shape, np.float32)])
    np.testing.assert_allclose(got, stored(want), rtol=2e-5, atol=1e-8)
    got = run_spec(M.Softmax(list(shape), dim, layouts=[lay, None]), [stored(x), np.zeros(shape, np.float32)])
    np.testing.assert_allclose(got, want, rtol=2e-5, atol=1e-8)


def test_softmax_full_size(gpu):
    """The Softmax stage of benchmark configuration 5 alone: 16x2048 rows of 2048."""
    shape = (16, 2048, 2048)
    x = synth.normal_f32(203, 0, shape, std=2.0)
    got = run_spec(M.Softmax(list(shape), 2), [x, np.zeros((1,), np.float32).repeat(x.size).reshape(shape)])
    want = orc.softmax(list(shape), 2, x)
    assert (np.abs(got - want) <= 1e-5 * np.abs(want) + 1e-12).all()


def msm_inputs(seed, b, m, k, n2, n):
    q = synth.normal_bf16(seed, 0, (b, m, k), 0.5)
    kmat = synth.normal_bf16(seed, 1, (b, n2, k), 0.5)   # K row-major == KT with layout![0,2,1]
    v = synth.normal_bf16(seed, 2, (b, n2, n), 0.5)
    return q, kmat, v


KT_LAYOUT = M.layout(0, 2, 1)
KT_ORC = orc.make_layout([0, 2, 1])


@pytest.mark.parametrize("dims", [(1, 64, 128, 64, 128), (2, 256, 128, 512, 128), (1, 128, 64, 256, 64),
                                  (3, 50, 24, 70, 10), (1, 2048, 128, 2048, 128), (2, 256, 64, 512, 64),
                                  (4, 128, 32, 256, 32), (2, 1024, 64, 1024, 64)])
def test_compose_msm(gpu, dims):
    b, m, k, n2, n = dims
    q, kmat, v = msm_inputs(301, *dims)
    spec = M.ComposeMSM(b, m, k, n2, n, layouts=[None, None, KT_LAYOUT, None])
    got = run_spec(spec, [v, q, kmat, np.zeros((b, m, n), np.float32)])
    want = orc.compose_msm(b, m, k, n2, n, [7, 7, 7, 6], v, q, kmat, np.zeros((b, m, n), np.float32),
                           layouts=[None, None, KT_ORC, None])
    assert rel_err(got, want) < 1e-2  # stated tolerance for the composed pipeline


@pytest.mark.parametrize("dims", [(2, 200, 160, 328, 160), (1, 136, 136, 1000, 96), (2, 256, 192, 192, 72),
                                  (1, 512, 256, 1024, 256),
                                  # every Softmax kernel that writes P as bf16: rows that are not whole
                                  # vectors (many, few), a workgroup per row, short rows, rows in chunks
                                  (1, 600, 160, 1001, 160), (1, 100, 160, 1001, 160), (1, 300, 160, 2048, 160),
                                  (2, 130, 160, 67, 160), (1, 40, 160, 9000, 160)])
def test_compose_msm_staged_on_the_matrix_cores(gpu, dims):
    """Head dims beyond 128, which the fused kernel does not take: Q.KT runs as a bf16 Matmul with
    a k-fastest B, Softmax over f32 rows writes P rounded to bf16 (as the fused kernel does), and
    P.V runs as a bf16 Matmul: within the Compose's 1e-2.  The same pipeline with its
    intermediates materialised (f32, as the reference keeps them) agrees with the oracle to 1e-5."""
    b, m, k, n2, n = dims
    q, kmat, v = msm_inputs(303, *dims)
    spec = M.ComposeMSM(b, m, k, n2, n, layouts=[None, None, KT_LAYOUT, None])
    got = run_spec(spec, [v, q, kmat, np.zeros((b, m, n), np.float32)])
    want = orc.compose_msm(b, m, k, n2, n, [7, 7, 7, 6], v, q, kmat, np.zeros((b, m, n), np.float32),
                           layouts=[None, None, KT_ORC, None])
    assert rel_err(got, want) < 1e-2
    staged = run_spec(M.Compose([M.Matmul([b, m, n2, n], [M.f32, M.bf16, M.f32]), M.Softmax([b, m, n2], 2),
                                 M.Matmul([b, m, k, n2], [M.bf16, M.bf16, M.f32])],
                                layouts=[None, None, KT_LAYOUT, None]).bufferize(0),
                      [v, q, kmat, np.zeros((b, m, n), np.float32)])
    # Sums of 9000 f32 terms: the oracle adds them one after another, the kernels in trees; the two
    # associations differ by more than 1e-5 of the largest output at that length.
    assert rel_err(staged, want) < (1e-5 if n2 <= 4096 else 5e-5)


@pytest.mark.parametrize("trend", ["rising", "falling", "spike"])
@pytest.mark.parametrize("dims", [(2, 256, 128, 1024, 128), (1, 130, 64, 700, 64)])
def test_compose_msm_scores_that_outgrow_the_reference(gpu, dims, trend):
    """The fused kernel takes its exponentials against a reference it sets from the first block of
    keys and moves only when a block's sum shows a score more than 2^40 above it.  Keys whose
    magnitude rises along the sequence (scores from ~1 to ~100: the reference must move, more than
    once), falls (everything after the first blocks underflows towards zero), or spikes in one
    late block, against the oracle and against the staged pipeline."""
    b, m, k, n2, n = dims
    q, kmat, v = msm_inputs(311, *dims)
    pos = np.arange(n2, dtype=np.float32) / n2
    scale = {"rising": 0.05 + 12.0 * pos ** 2, "falling": 12.0 * (1 - pos) ** 2 + 0.05,
             "spike": np.where((pos > 0.7) & (pos < 0.75), 15.0, 0.2)}[trend]
    kf = synth.bf16_bits_to_f32(kmat) * scale[None, :, None]
    kmat = synth.f32_to_bf16_bits(kf.astype(np.float32))
    spec = M.ComposeMSM(b, m, k, n2, n, layouts=[None, None, KT_LAYOUT, None])
    got = run_spec(spec, [v, q, kmat, np.zeros((b, m, n), np.float32)])
    want = orc.compose_msm(b, m, k, n2, n, [7, 7, 7, 6], v, q, kmat, np.zeros((b, m, n), np.float32),
                           layouts=[None, None, KT_ORC, None])
    assert np.isfinite(got).all()
    assert rel_err(got, want) < 1e-2
    assert elem_err(got, want, floor_frac=1.0) < 2e-2


@pytest.mark.parametrize("dims", [(1, 136, 128, 1000, 128), (2, 1, 128, 1, 128), (1, 130, 128, 64, 128),
                                  (3, 200, 128, 70, 128), (1, 128, 128, 2049, 128), (2, 300, 128, 129, 128),
                                  (1, 257, 128, 65, 128), (2, 384, 128, 192, 128),
                                  (1, 136, 64, 1000, 64), (2, 1, 64, 1, 64), (2, 200, 64, 328, 64),
                                  (1, 257, 64, 65, 64), (3, 200, 32, 70, 32), (2, 300, 32, 129, 32),
                                  (1, 1, 32, 2049, 32)])
def test_compose_msm_fused_ragged(gpu, dims):
    """Sequence lengths that are not multiples of the fused kernel's blocks (128 queries,
    2 x 64 keys): clamped rows, masked keys, uneven split of the key blocks over the two
    halves (down to one key, where the second half has no block at all).  The rows past m must
    stay untouched: the output buffer is exactly m rows."""
    b, m, k, n2, n = dims
    q, kmat, v = msm_inputs(304, *dims)
    spec = M.ComposeMSM(b, m, k, n2, n, layouts=[None, None, KT_LAYOUT, None])
    sentinel = np.full((b, m, n), 7.5, np.float32)
    got = run_spec(spec, [v, q, kmat, sentinel])
    want = orc.compose_msm(b, m, k, n2, n, [7, 7, 7, 6], v, q, kmat, np.zeros((b, m, n), np.float32),
                           layouts=[None, None, KT_ORC, None])
    assert rel_err(got, want) < 1e-2
    # The same Spec with the intermediates materialised agrees with the oracle to 1e-5, and the
    # fused result with it to the bf16 rounding of P.
    staged = run_spec(M.Compose([M.Matmul([b, m, n2, n], [M.f32, M.bf16, M.f32]), M.Softmax([b, m, n2], 2),
                                 M.Matmul([b, m, k, n2], [M.bf16, M.bf16, M.f32])],
                                layouts=[None, None, KT_LAYOUT, None]).bufferize(0),
                      [v, q, kmat, np.zeros((b, m, n), np.float32)])
    assert rel_err(staged, want) < 1e-5
    assert rel_err(got, staged) < 1e-2


@pytest.mark.parametrize("dims", [(2, 200, 48, 328, 48), (1, 136, 96, 1000, 96), (2, 256, 96, 192, 72),
                                  (1, 128, 64, 256, 128), (3, 50, 24, 70, 10), (1, 77, 100, 130, 30),
                                  (2, 128, 128, 256, 2), (1, 64, 8, 64, 128)])
def test_compose_msm_fused_with_padded_head_dims(gpu, dims):
    """Head dims up to 128 other than 32 / 64 / 128, and different ones for the two products: Q, K
    and V are zero-padded to the next size the fused kernel is built for and only the n real
    columns of the result are stored (the buffer is exactly b x m x n)."""
    b, m, k, n2, n = dims
    q, kmat, v = msm_inputs(305, *dims)
    spec = M.ComposeMSM(b, m, k, n2, n, layouts=[None, None, KT_LAYOUT, None])
    got = run_spec(spec, [v, q, kmat, np.full((b, m, n), 7.5, np.float32)])
    want = orc.compose_msm(b, m, k, n2, n, [7, 7, 7, 6], v, q, kmat, np.zeros((b, m, n), np.float32),
                           layouts=[None, None, KT_ORC, None])
    assert rel_err(got, want) < 1e-2


@pytest.mark.parametrize("dims", [(16, 1, 128, 2048, 128), (2, 1, 128, 32768, 128), (4, 16, 64, 8200, 64),
                                  (3, 130, 32, 1100, 32), (2, 5, 96, 3000, 72), (1, 1, 128, 257, 128),
                                  (5, 3, 64, 640, 64)])
def test_compose_msm_few_queries_many_keys(gpu, dims):
    """Few (entry, query block) pairs and many keys: the keys are shared out over several
    workgroups per query block and the partial (max, denominator, O) triples merged afterwards.
    Covers splits that end up without a key block, ragged key counts, padded head dims, and both
    KT orders."""
    b, m, k, n2, n = dims
    q, kmat, v = msm_inputs(307, *dims)
    want = orc.compose_msm(b, m, k, n2, n, [7, 7, 7, 6], v, q, kmat, np.zeros((b, m, n), np.float32),
                           layouts=[None, None, KT_ORC, None])
    spec = M.ComposeMSM(b, m, k, n2, n, layouts=[None, None, KT_LAYOUT, None])
    got = run_spec(spec, [v, q, kmat, np.full((b, m, n), 7.5, np.float32)])
    assert rel_err(got, want) < 1e-2
    if n2 % 8 == 0:
        kt = np.ascontiguousarray(kmat.transpose(0, 2, 1))
        got = run_spec(M.ComposeMSM(b, m, k, n2, n), [v, q, kt, np.full((b, m, n), 7.5, np.float32)])
        assert rel_err(got, want) < 1e-2


def test_compose_msm_f32_inputs_stay_staged(gpu):
    """f32 inputs run on the staged (unfused) path, exact to 1e-5: nothing is rounded to bf16."""
    b, m, k, n2, n = 2, 40, 32, 48, 24
    q, kmat, v = msm_inputs(302, b, m, k, n2, n)
    kt = np.ascontiguousarray(kmat.transpose(0, 2, 1))
    want = orc.compose_msm(b, m, k, n2, n, [7, 7, 7, 6], v, q, kt, np.zeros((b, m, n), np.float32))
    qf, ktf, vf = (synth.bf16_bits_to_f32(t) for t in (q, kt, v))
    got = run_spec(M.ComposeMSM(b, m, k, n2, n, dtypes=(M.f32, M.f32, M.f32, M.f32)),
                   [vf, qf, ktf, np.zeros((b, m, n), np.float32)])
    assert rel_err(got, want) < 1e-5


@pytest.mark.parametrize("dims", [(2, 40, 32, 48, 24), (2, 256, 128, 384, 128), (1, 200, 64, 130, 64),
                                  (1, 128, 64, 256, 64), (2, 136, 128, 1000, 128), (1, 77, 32, 72, 32),
                                  (3, 128, 32, 128, 32), (1, 300, 64, 2056, 64), (1, 64, 128, 8, 128)])
def test_compose_msm_fused_from_other_layouts(gpu, dims):
    """The reference's default layouts (everything row-major, KT as [b, k, n2] with n2 fastest,
    examples/matmul_chain.rs:26-57), a batched column-major Q, a V with a Packed dim and a batched column-major
    result.  A row-major KT whose n2 is a multiple of 8 is read in place by the kernel's build for
    it (whole and ragged sequence lengths, head dims 32 / 64 / 128); everything else is brought
    to the order the fused kernel reads (one copy) and the result moved out.  Within the composed
    pipeline's tolerance."""
    b, m, k, n2, n = dims
    q, kmat, v = msm_inputs(306, *dims)
    kt = np.ascontiguousarray(kmat.transpose(0, 2, 1))                       # [b, k, n2] row-major
    want = orc.compose_msm(b, m, k, n2, n, [7, 7, 7, 6], v, q, kt, np.zeros((b, m, n), np.float32))
    got = run_spec(M.ComposeMSM(b, m, k, n2, n), [v, q, kt, np.zeros((b, m, n), np.float32)])
    assert rel_err(got, want) < 1e-2
    layouts = [M.layout(0, 1, 2, (1, M.Packed(2))), M.batched_col_major([b, m, k]), None, M.batched_col_major([b, m, n])]
    vp = np.ascontiguousarray(v.reshape(b, n2 // 2, 2, n).transpose(0, 1, 3, 2))      # [b, n2/2, n, 2]
    qc = np.ascontiguousarray(q.transpose(0, 2, 1))
    got = run_spec(M.ComposeMSM(b, m, k, n2, n, layouts=layouts), [vp, qc, kt, np.zeros((b, n, m), np.float32)])
    assert rel_err(got.transpose(0, 2, 1), want) < 1e-2


def test_compose_msm_full_size(gpu):
    """benchmark configuration 5: 16 heads of 2048x128; four heads against the oracle, all heads
    through the row-stochastic property: with V = ones, out must be all ones."""
    b, m, k, n2, n = 16, 2048, 128, 2048, 128
    q, kmat, v = msm_inputs(303, b, m, k, n2, n)
    spec = M.ComposeMSM(b, m, k, n2, n, layouts=[None, None, KT_LAYOUT, None])
    got = run_spec(spec, [v, q, kmat, np.zeros((b, m, n), np.float32)])
    for h in (0, 5, 10, 15):
        want = orc.compose_msm(1, m, k, n2, n, [7, 7, 7, 6], v[h:h + 1], q[h:h + 1], kmat[h:h + 1],
                               np.zeros((1, m, n), np.float32), layouts=[None, None, KT_ORC, None])
        # Stated tolerance 1e-2, norm-wise (measured 1e-3).  Element by element: an output is a sum of
        # 2048 signed terms p * v whose P factors are rounded to bf16 for the second product (half an
        # ulp, 2^-9, each), so its error is bounded by 2^-9 * sum p |v|, about 1.3e-2 of the RMS
        # output for these inputs, whatever the element's own value where the terms cancel.  With |r|
        # floored at that RMS the worst of 262144 elements measures 1.2e-2; the gate of 2e-2 is what
        # a kernel wrong on small outputs (a dropped key block, a stale row) cannot pass.
        assert rel_err(got[h:h + 1], want) < 1e-2
        assert elem_err(got[h:h + 1], want, floor_frac=1.0) < 2e-2
    ones = synth.f32_to_bf16_bits(np.ones((b, n2, n), np.float32))
    got = run_spec(spec, [ones, q, kmat, np.zeros((b, m, n), np.float32)])
    assert np.abs(got - 1).max() < 1e-2


def test_softmax_tensor_beyond_4_gib(gpu):
    """2^19 rows of 4092 f32 = 8.6 GB in, 8.6 GB out: the largest tensor the Spec surface admits, byte
    offsets up to 2^33.  Rows at the start, near the 4 GiB and 6 GiB marks and at the end, each within 1e-5
    of the oracle; the input is one 64 MiB pattern repeated, uploaded piecewise."""
    import ctypes as C
    from morello_amd import _binding as B
    rows, cols = 1 << 19, 4092
    spec = M.Softmax([rows, cols], 1)
    assert spec.check() == 0 and spec.bytes_used(0) > (1 << 32)
    lib = B.load()
    din, dout = M.DeviceBuffer(rows * cols * 4), M.DeviceBuffer(rows * cols * 4)
    piece_rows = 4096
    piece = synth.normal_f32(77, 0, (piece_rows, cols), 3.0)
    for r0 in range(0, rows, piece_rows):
        assert lib.mrl_memcpy_h2d(C.c_void_p(din.ptr + r0 * cols * 4), piece.ctypes.data_as(C.c_void_p),
                                  piece.nbytes) == 0
    spec.run_device([din.ptr, dout.ptr])
    want = orc.softmax([8, cols], 1, piece[:8].copy())
    row_bytes = cols * 4
    for r0 in (0, ((1 << 32) // row_bytes // piece_rows) * piece_rows, ((3 << 31) // row_bytes // piece_rows) * piece_rows,
               rows - piece_rows):
        got = np.empty((8, cols), np.float32)
        assert lib.mrl_memcpy_d2h(got.ctypes.data_as(C.c_void_p), C.c_void_p(dout.ptr + r0 * row_bytes),
                                  8 * row_bytes) == 0
        np.testing.assert_allclose(got, want, rtol=1e-5, atol=1e-9)
    # The row that straddles the 4 GiB mark, whatever its place in the pattern.
    r = (1 << 32) // row_bytes
    got = np.empty((1, cols), np.float32)
    assert lib.mrl_memcpy_d2h(got.ctypes.data_as(C.c_void_p), C.c_void_p(dout.ptr + r * row_bytes), row_bytes) == 0
    np.testing.assert_allclose(got, orc.softmax([1, cols], 1, piece[r % piece_rows:r % piece_rows + 1].copy()),
                               rtol=1e-5, atol=1e-9)
    din.free()
    dout.free()


@pytest.mark.parametrize("shape,dim", [((6, 256), 1), ((6, 2048), 1), ((6, 4100), 1), ((6, 9000), 1), ((6, 40000), 1),
                                       ((6, 33), 1), ((6, 5), 1), ((300, 6, 12), 2), ((6, 700, 8), 1), ((3, 2, 1100), 2),
                                       ((6, 70000), 0)])
def test_softmax_infinities_follow_the_reference(gpu, shape, dim):
    """Rows with infinities and NaNs on every Softmax kernel (rows in registers, short rows, a
    workgroup per row, rows in chunks, a scan dim that is not the innermost, a thread per column), as the reference's
    interpreter treats them (verification.rs:166-184 with the NaN-propagating max that starts
    from f32::MIN, :842-861): -inf among finite scores gives exact zeros; a row that is all
    -inf, or holds +inf or a NaN, is NaN throughout; the other rows are untouched by it."""
    x = synth.normal_f32(206, 0, shape)
    lines = np.moveaxis(x, dim, -1).reshape(-1, shape[dim])   # a copy: one row per softmax
    n = lines.shape[1]
    lines[0, ::2] = -np.inf          # finite scores between -inf
    lines[1, :] = -np.inf            # nothing but -inf
    lines[2, n // 2] = np.inf        # one +inf
    lines[3, n - 1] = np.nan         # a NaN in the last place
    lines[4, 0] = -np.inf            # a single -inf
    moved = np.moveaxis(x, dim, -1)
    x = np.ascontiguousarray(np.moveaxis(lines.reshape(moved.shape), -1, dim))
    got = run_spec(M.Softmax(list(shape), dim), [x, np.zeros_like(x)])
    want = orc.softmax(list(shape), dim, x)
    g = np.moveaxis(got, dim, -1).reshape(-1, n)
    w = np.moveaxis(want, dim, -1).reshape(-1, n)
    assert np.isnan(w[1]).all() and np.isnan(w[2]).all() and np.isnan(w[3]).all()   # the oracle itself
    assert np.array_equal(np.isnan(g), np.isnan(w))
    assert (g[0, ::2] == 0).all() and g[4, 0] == 0
    ok = ~np.isnan(w)
    assert (np.abs(g[ok] - w[ok]) <= 1e-5 * np.abs(w[ok]) + 1e-12).all()


@pytest.mark.parametrize("dims,where", [((2, 200, 64, 300, 64), 150), ((1, 130, 128, 700, 128), 5), ((1, 64, 32, 1100, 32), 1099)])
def test_compose_msm_with_an_infinite_key(gpu, dims, where):
    """One +inf in K: a query whose product with it is +inf has a NaN row (inf - inf in the
    softmax, verification.rs:166-184), one whose product is -inf gives that key weight zero and
    is otherwise unchanged.  On the fused kernel the infinity arrives in the first key block or
    in a later one, where the running reference has to move to it; every fused action agrees."""
    b, m, k, n2, n = dims
    q, kmat, v = msm_inputs(312, *dims)
    kf = synth.bf16_bits_to_f32(kmat)
    kf[0, where, 3] = np.inf
    kmat = synth.f32_to_bf16_bits(kf)
    spec = M.ComposeMSM(b, m, k, n2, n, layouts=[None, None, KT_LAYOUT, None])
    want = orc.compose_msm(b, m, k, n2, n, [7, 7, 7, 6], v, q, kmat, np.zeros((b, m, n), np.float32),
                           layouts=[None, None, KT_ORC, None])
    nan_rows = np.isnan(want).all(axis=2)
    assert nan_rows[0].any() and not nan_rows[0].all() and np.array_equal(np.isnan(want).any(axis=2), nan_rows)
    for target in [spec] + [a for a in spec.actions() if a.kind == M.ActionKind.Fused]:
        bufs = [M.DeviceBuffer.from_numpy(a) for a in (v, q, kmat, np.zeros((b, m, n), np.float32))]
        target.run_device([x.ptr for x in bufs])
        got = bufs[-1].to_numpy(np.float32, (b, m, n))
        for x in bufs:
            x.free()
        assert np.array_equal(np.isnan(got), np.isnan(want)), target
        ok = ~np.isnan(want)
        assert np.abs(got[ok] - want[ok]).max() / np.abs(want[ok]).max() < 1e-2, target
