"""Pins the oracle's restatement of the primitives Softmax decomposes into against what the
mathematics fixes (float64 numpy / scipy), not against a retyped formula:
max == np.max, denominators == exp(logsumexp - max), Complete == scipy softmax, merging
per-tile pairs == the whole-row pair, accumulating == the plain form over the concatenation."""
import numpy as np
import pytest
from scipy.special import logsumexp, softmax as sp_softmax

import orc

RNG = np.random.default_rng(20240)
SHAPES = [((7, 33), 1), ((5, 9, 4), 1), ((3, 4, 130), 2), ((6, 5), 0), ((2, 3, 4, 5), 2)]


def reduced(shape, dim):
    s = list(shape)
    s[dim] = 1
    return tuple(s)


def rnd(shape, scale=3.0):
    return (RNG.standard_normal(shape) * scale).astype(np.float32)


@pytest.mark.parametrize("shape,dim", SHAPES)
def test_max_is_numpy_max(shape, dim):
    x = rnd(shape)
    out = np.zeros(reduced(shape, dim), np.float32)
    orc.softmax_part(orc.PART_MAX, shape, dim, [x, out])
    assert np.array_equal(out, x.max(axis=dim, keepdims=True))
    # Accumulating: the old value takes part.
    out2 = np.full(reduced(shape, dim), 1.25, np.float32)
    orc.softmax_part(orc.PART_MAX, shape, dim, [x, out2], accum=True)
    assert np.array_equal(out2, np.maximum(x.max(axis=dim, keepdims=True), np.float32(1.25)))


@pytest.mark.parametrize("shape,dim", SHAPES)
def test_denominator_and_max_is_logsumexp(shape, dim):
    x = rnd(shape)
    mx = np.zeros(reduced(shape, dim), np.float32)
    dn = np.zeros(reduced(shape, dim), np.float32)
    orc.softmax_part(orc.PART_DENOM_MAX, shape, dim, [x, mx, dn])
    x64 = x.astype(np.float64)
    assert np.array_equal(mx, x.max(axis=dim, keepdims=True))
    want = np.exp(logsumexp(x64, axis=dim, keepdims=True) - x64.max(axis=dim, keepdims=True))
    np.testing.assert_allclose(dn, want, rtol=2e-6)


@pytest.mark.parametrize("shape,dim", SHAPES)
def test_accumulating_equals_concatenation(shape, dim):
    """Running the accumulating form on two halves equals the plain form on their
    concatenation (the property the Spec's split-over-scan-dim schedules rely on)."""
    x1, x2 = rnd(shape), rnd(shape, 5.0)
    red = reduced(shape, dim)
    mx, dn = np.zeros(red, np.float32), np.zeros(red, np.float32)
    orc.softmax_part(orc.PART_DENOM_MAX, shape, dim, [x1, mx, dn])
    orc.softmax_part(orc.PART_DENOM_MAX, shape, dim, [x2, mx, dn], accum=True)
    both = np.concatenate([x1, x2], axis=dim).astype(np.float64)
    assert np.array_equal(mx, both.max(axis=dim, keepdims=True).astype(np.float32))
    want = np.exp(logsumexp(both, axis=dim, keepdims=True) - both.max(axis=dim, keepdims=True))
    np.testing.assert_allclose(dn, want, rtol=3e-6)


@pytest.mark.parametrize("shape,dim", SHAPES)
def test_denominator_given_max(shape, dim):
    x = rnd(shape)
    red = reduced(shape, dim)
    mx = (x.max(axis=dim, keepdims=True) + np.float32(0.5)).astype(np.float32)  # any shift is legal
    dn = np.zeros(red, np.float32)
    orc.softmax_part(orc.PART_DENOM, shape, dim, [x, mx, dn])
    want = np.exp(x.astype(np.float64) - mx).sum(axis=dim, keepdims=True)
    np.testing.assert_allclose(dn, want, rtol=2e-6)
    dn2 = np.full(red, 2.0, np.float32)
    orc.softmax_part(orc.PART_DENOM, shape, dim, [x, mx, dn2], accum=True)
    np.testing.assert_allclose(dn2, want + 2.0, rtol=2e-6)


@pytest.mark.parametrize("tiles", [1, 2, 5])
def test_from_parts_merges_tiles_to_the_whole_row_pair(tiles):
    rows, per = 6, 17
    x = rnd((rows, tiles * per), 4.0)
    xt = x.reshape(rows, tiles, per).astype(np.float64)
    tmax = xt.max(axis=2).astype(np.float32)
    tden = np.exp(xt - xt.max(axis=2, keepdims=True)).sum(axis=2).astype(np.float32)
    omax, oden = np.zeros((rows, 1), np.float32), np.zeros((rows, 1), np.float32)
    orc.softmax_part(orc.PART_FROM_PARTS, (rows, tiles), 1, [tmax, tden, omax, oden])
    x64 = x.astype(np.float64)
    assert np.array_equal(omax[:, 0], x.max(axis=1))
    np.testing.assert_allclose(oden[:, 0], np.exp(logsumexp(x64, axis=1) - x64.max(axis=1)), rtol=3e-6)


@pytest.mark.parametrize("shape,dim", SHAPES)
def test_unscaled_forms_and_complete_rebuild_softmax(shape, dim):
    x = rnd(shape)
    red = reduced(shape, dim)
    want = sp_softmax(x.astype(np.float64), axis=dim)
    # DenominatorAndUnscaled, then DivideVecScalar == Softmax.
    dn, un = np.zeros(red, np.float32), np.zeros(shape, np.float32)
    orc.softmax_part(orc.PART_UNSCALED, shape, dim, [x, dn, un])
    np.testing.assert_allclose(un.sum(axis=dim, keepdims=True, dtype=np.float64), dn, rtol=2e-6)
    assert float(un.max()) == 1.0  # exp(max - max)
    orc.softmax_part(orc.PART_DIVIDE_VEC_SCALAR, shape, dim, [un, dn])
    np.testing.assert_allclose(un, want, rtol=3e-6, atol=1e-9)
    # Max, DenominatorAndUnscaledFromMax, DivideVec by the broadcast denominator == Softmax.
    mx, dn2, un2 = np.zeros(red, np.float32), np.zeros(red, np.float32), np.zeros(shape, np.float32)
    orc.softmax_part(orc.PART_MAX, shape, dim, [x, mx])
    orc.softmax_part(orc.PART_UNSCALED_FROM_MAX, shape, dim, [x, mx, dn2, un2])
    np.testing.assert_allclose(dn2, dn, rtol=1e-6)
    den_full = orc.broadcast(shape, dim, dn2)
    assert np.array_equal(den_full, np.broadcast_to(dn2, shape))
    orc.softmax_part(orc.PART_DIVIDE_VEC, shape, 0, [un2, den_full])
    np.testing.assert_allclose(un2, want, rtol=3e-6, atol=1e-9)
    # SoftmaxComplete from (max, denom) == Softmax, and equals the whole-Softmax oracle.
    out = np.zeros(shape, np.float32)
    orc.softmax_part(orc.PART_COMPLETE, shape, dim, [x, mx, dn2, out])
    np.testing.assert_allclose(out, want, rtol=3e-6, atol=1e-9)
    np.testing.assert_allclose(out, orc.softmax(list(shape), dim, x), rtol=1e-6, atol=1e-9)


def test_divide_is_true_division():
    a = np.array([[1.0, -3.0, 0.0, 5.0]], np.float32)
    b = np.array([[4.0, 2.0, 7.0, -0.5]], np.float32)
    orc.softmax_part(orc.PART_DIVIDE_VEC, (1, 4), 1, [a, b])
    assert a.tolist() == [[0.25, -1.5, 0.0, -10.0]]


def test_fill_values():
    assert np.array_equal(orc.fill(orc.I32, 0, 5), np.zeros(5, np.int32))
    assert np.array_equal(orc.fill(orc.I8, 2, 3), np.full(3, -128, np.int8))
    assert np.array_equal(orc.fill(orc.I16, 2, 3), np.full(3, -32768, np.int16))
    assert np.array_equal(orc.fill(orc.I32, 2, 3), np.full(3, -2**31, np.int32))
    assert np.array_equal(orc.fill(orc.U8, 2, 3), np.zeros(3, np.uint8))
    assert np.array_equal(orc.fill(orc.U32, 2, 3), np.zeros(3, np.uint32))
    assert np.array_equal(orc.fill(orc.F32, 2, 3), np.full(3, np.finfo(np.float32).min, np.float32))
    assert np.all(np.isneginf(orc.fill(orc.F32, 1, 4)))
    bf = orc.fill(orc.BF16, 1, 2)
    assert np.all(np.isneginf((bf.astype(np.uint32) << 16).view(np.float32)))
    # bf16::MIN is the most negative finite bf16: -(2 - 2^-7) * 2^127.
    bmin = (orc.fill(orc.BF16, 2, 1).astype(np.uint32) << 16).view(np.float32)[0]
    assert float(bmin) == -(2.0 - 2.0 ** -7) * 2.0 ** 127
