"""Layout arithmetic: the oracle and the library's host code against the expectations the
reference asserts in its own unit tests and book (no GPU needed).

Sources of the expected values: morello/src/layout.rs:1452-1551 (physical shapes),
:2391-2452 (index expressions, batched_col_major), book/src/data_layouts.md:59-99 (packed
layout worked example), morello/src/views.rs:1282-1347 (squeeze / one_prefix / transpose).
"""
import itertools

import numpy as np
import pytest

import morello_amd as M
import orc

P, OE = 1, 2  # kinds


def both(dims):
    """The same layout for the oracle and for the library."""
    lib_dims = [(d, M.Dynamic) if isinstance(d, int) else (d[0], M.PhysDim(d[1], d[2])) for d in dims]
    return orc.make_layout(dims), M.Layout(lib_dims)


PHYSICAL_SHAPES = [
    # layout, logical shape, expected physical shape (None = error)     layout.rs line
    ([0, 1, (0, P, 4)], [64, 64], [16, 64, 4]),                        # 1452
    ([0, (1, P, 2)], [2, 2], [2, 2]),                                   # 1461
    ([(0, P, 4), 1], [1, 64], [1, 64]),                                 # 1470
    ([(0, P, 2)], [6], None),                                           # 1480
    ([0, 1, (0, P, 4)], [2, 64], [1, 64, 2]),                           # 1490
    ([(0, P, 2)], [1], [1]),                                            # 1499
    ([(0, P, 4)], [2], [2]),                                            # 1507
    ([(0, OE, 4)], [1], [1]),                                           # 1507
    ([(0, OE, 4)], [2], None),                                          # 1507
    ([(0, P, 4), 1], [8, 64], None),                                    # 1520
    ([1, 0, (1, P, 8)], [10, 4], [1, 10, 4]),                           # 1530
    ([1, 0, (1, P, 4), (0, P, 2), (1, P, 4)], [10, 8], [1, 5, 2, 2, 4]),  # 1537
    ([1, 0, (1, P, 4), (0, P, 2), (1, P, 4)], [10, 6], None),           # 1544
]


@pytest.mark.parametrize("dims,shape,expected", PHYSICAL_SHAPES)
def test_physical_shape_known_answers(dims, shape, expected):
    o, l = both(dims)
    assert orc.physical_shape(o, shape) == expected
    if expected is None:
        assert not l.applies_to_shape(shape)
    else:
        assert l.physical_shape(shape) == expected


INDEX_EXPRS = [
    ([0, 1], [16, 4], lambda p: 4 * p[0] + p[1]),                                     # layout.rs:2391
    ([(0, OE, 8)], [8], lambda p: (p[0] % 8) // 2 + (p[0] % 2) * 4),                    # :2402
    ([0, (0, OE, 8)], [16], lambda p: (p[0] // 8) * 8 + (p[0] % 8) // 2 + (p[0] % 2) * 4),  # :2413
    ([0, (1, OE, 8)], [2, 8], lambda p: 8 * p[0] + (p[1] % 8) // 2 + (p[1] % 2) * 4),  # :2424
    ([1, 0, (1, P, 4)], [6, 8], lambda p: 24 * (p[1] // 4) + 4 * p[0] + p[1] % 4),     # data_layouts.md
    ([0, 2], [2, 1, 3], lambda p: 3 * p[0] + p[2]),                                   # views.rs:1282 (squeezed)
    ([1, 2], [1, 2, 3], lambda p: 3 * p[1] + p[2]),                                   # views.rs:1305 (one_prefix)
    ([1, 0], [3, 2], lambda p: 3 * p[1] + p[0]),                                      # views.rs:1328 (transpose)
]


@pytest.mark.parametrize("dims,shape,expr", INDEX_EXPRS)
def test_buffer_index_known_answers(dims, shape, expr):
    o, l = both(dims)
    for pt in itertools.product(*[range(s) for s in shape]):
        want = expr(pt)
        assert orc.buffer_index(o, shape, list(pt)) == want
        assert l.buffer_index(shape, list(pt)) == want


def test_constructors_match_reference():
    # layout.rs:1234-1279 and the expectation at :2441-2452.
    assert M.row_major([16, 4]).dims == [(0, M.Dynamic), (1, M.Dynamic)]
    assert M.row_major([1, 8, 1, 4]).dims == [(1, M.Dynamic), (3, M.Dynamic)]
    assert M.col_major([16, 4]).dims == [(1, M.Dynamic), (0, M.Dynamic)]
    assert M.batched_col_major([2, 2, 2, 2]).dims == [(0, M.Dynamic), (3, M.Dynamic), (2, M.Dynamic), (1, M.Dynamic)]
    assert M.batched_col_major([1, 4, 8]).dims == [(2, M.Dynamic), (1, M.Dynamic)]
    assert M.nhwc([2, 3, 4, 5]).dims == [(0, M.Dynamic), (2, M.Dynamic), (3, M.Dynamic), (1, M.Dynamic)]
    assert M.nhwc([1, 3, 4, 5]).dims == [(2, M.Dynamic), (3, M.Dynamic), (1, M.Dynamic)]


BIJECTION_CASES = [
    ([0, 1], [5, 7]),
    ([1, 0], [5, 7]),
    ([0, 2, 3, 1], [2, 3, 4, 5]),
    ([0, 2, 1], [3, 4, 6]),
    ([0, 1, (0, P, 4)], [8, 6]),
    ([1, 0, (1, P, 4)], [6, 8]),
    ([0, 2, 1, (2, P, 16)], [2, 4, 32]),
    ([0, 1, (1, OE, 8)], [3, 16]),
    ([1, 0, (1, P, 4), (0, P, 2), (1, P, 4)], [10, 16]),
    ([0, 1, (0, P, 4)], [2, 5]),  # smaller-remaining packed dim
]


@pytest.mark.parametrize("dims,shape", BIJECTION_CASES)
def test_layout_is_a_bijection(dims, shape):
    """book/src/data_layouts.md:12-13: distinct points never share a buffer offset, and the
    offsets fill [0, volume).  Also the oracle and the library agree everywhere."""
    o, l = both(dims)
    vol = int(np.prod(shape))
    seen = set()
    for pt in itertools.product(*[range(s) for s in shape]):
        a = orc.buffer_index(o, shape, list(pt))
        assert a == l.buffer_index(shape, list(pt))
        seen.add(a)
    assert seen == set(range(vol))


def test_dtype_table():
    # common.rs:30-36, :52-65
    names = ["u8", "i8", "u16", "i16", "u32", "i32", "f32", "bf16"]
    sizes = [1, 1, 2, 2, 4, 4, 4, 2]
    for i, (n, s) in enumerate(zip(names, sizes)):
        assert str(M.Dtype(i)) == n and M.Dtype(i).size == s
        assert orc.lib().orc_dtype_size(i) == s
