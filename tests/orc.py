"""ctypes view of the CPU oracle (oracle/libmorello_oracle.so).  Test infrastructure."""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
ORACLE_DIR = os.path.join(ROOT, "oracle")
LIB = os.path.join(ORACLE_DIR, "libmorello_oracle.so")
REF_DIR = os.path.join(ORACLE_DIR, "_ref")

U8, I8, U16, I16, U32, I32, F32, BF16 = range(8)
NP = {U8: np.uint8, I8: np.int8, U16: np.uint16, I16: np.int16, U32: np.uint32, I32: np.int32,
      F32: np.float32, BF16: np.uint16}
MAX_PHYS = 10


class PhysDim(C.Structure):
    _fields_ = [("logical_dim", C.c_uint8), ("kind", C.c_uint8), ("size", C.c_uint32)]


class Layout(C.Structure):
    _fields_ = [("ndims", C.c_uint32), ("dims", PhysDim * MAX_PHYS)]


def make_layout(dims) -> Layout:
    """dims: ints (Dynamic) or (logical_dim, kind, size) with kind 1 Packed, 2 OddEven."""
    l = Layout()
    l.ndims = len(dims)
    for i, d in enumerate(dims):
        if isinstance(d, int):
            l.dims[i].logical_dim, l.dims[i].kind, l.dims[i].size = d, 0, 0
        else:
            l.dims[i].logical_dim, l.dims[i].kind, l.dims[i].size = d
    return l


_lib = None


def lib() -> C.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(LIB):
            subprocess.run(["make", "-C", ORACLE_DIR, "libmorello_oracle.so"], check=True,
                           capture_output=True)
        _lib = C.CDLL(LIB)
        _lib.orc_layout_buffer_index.restype = C.c_int64
        _lib.orc_bf16_to_f32.restype = C.c_float
        _lib.orc_bf16_to_f32.argtypes = [C.c_uint16]
        _lib.orc_f32_to_bf16.restype = C.c_uint16
        _lib.orc_f32_to_bf16.argtypes = [C.c_float]
        _lib.orc_fill_check_pattern.argtypes = [C.c_int, C.c_void_p, C.c_size_t]
    return _lib


def _u32(vals):
    return (C.c_uint32 * len(vals))(*vals)


def _layouts(layouts, n):
    """None or a list of (None | Layout) -> C array of pointers (NULL = row-major)."""
    if layouts is None:
        return None, None
    keep = [l for l in layouts]
    arr = (C.POINTER(Layout) * n)()
    for i, l in enumerate(keep):
        arr[i] = C.pointer(l) if l is not None else None
    return arr, keep


def physical_shape(layout: Layout, shape):
    out = (C.c_uint32 * MAX_PHYS)()
    rc = lib().orc_layout_physical_shape(C.byref(layout), _u32(shape), len(shape), out)
    if rc != 0:
        return None
    return [int(out[i]) for i in range(layout.ndims)]


def buffer_index(layout: Layout, shape, point) -> int:
    return int(lib().orc_layout_buffer_index(C.byref(layout), _u32(shape), len(shape), _u32(point)))


def matmul(spec_shape, dtypes, a, b, c, accum=False, layouts=None, rows=None):
    """Runs the oracle Matmul in place on `c` (numpy arrays are raw parameter buffers)."""
    arr, keep = _layouts(layouts, 3)
    dt = (C.c_int * 3)(*dtypes)
    if rows is None:
        rc = lib().orc_matmul(_u32(spec_shape), dt, arr, int(accum), a.ctypes.data_as(C.c_void_p),
                              b.ctypes.data_as(C.c_void_p), c.ctypes.data_as(C.c_void_p))
    else:
        rc = lib().orc_matmul_rows(_u32(spec_shape), dt, arr, int(accum),
                                   a.ctypes.data_as(C.c_void_p), b.ctypes.data_as(C.c_void_p),
                                   c.ctypes.data_as(C.c_void_p), C.c_uint32(rows[0]), C.c_uint32(rows[1]))
    assert rc == 0, f"oracle matmul rc={rc}"
    return c


def conv(spec_shape, dtypes, image, filters, out, accum=False, layouts=None):
    arr, keep = _layouts(layouts, 3)
    rc = lib().orc_conv(_u32(spec_shape), (C.c_int * 3)(*dtypes), arr, int(accum),
                        image.ctypes.data_as(C.c_void_p), filters.ctypes.data_as(C.c_void_p),
                        out.ctypes.data_as(C.c_void_p))
    assert rc == 0, f"oracle conv rc={rc}"
    return out


def softmax(shape, scan_dim, x, out=None, layouts=None):
    arr, keep = _layouts(layouts, 2)
    if out is None:
        out = np.empty_like(x)
    rc = lib().orc_softmax(_u32(shape), len(shape), scan_dim, arr, x.ctypes.data_as(C.c_void_p),
                           out.ctypes.data_as(C.c_void_p))
    assert rc == 0, f"oracle softmax rc={rc}"
    return out


def compose_msm(b, m, k, n2, n, dtypes, v, q, kt, out, layouts=None):
    arr, keep = _layouts(layouts, 4)
    rc = lib().orc_compose_msm(b, m, k, n2, n, (C.c_int * 4)(*dtypes), arr,
                               v.ctypes.data_as(C.c_void_p), q.ctypes.data_as(C.c_void_p),
                               kt.ctypes.data_as(C.c_void_p), out.ctypes.data_as(C.c_void_p))
    assert rc == 0, f"oracle compose rc={rc}"
    return out


def move(shape, dtypes, x, out, layouts=None):
    arr, keep = _layouts(layouts, 2)
    rc = lib().orc_move(_u32(shape), len(shape), (C.c_int * 2)(*dtypes), arr,
                        x.ctypes.data_as(C.c_void_p), out.ctypes.data_as(C.c_void_p))
    assert rc == 0, f"oracle move rc={rc}"
    return out


def check_pattern(dtype, count):
    out = np.empty(count, dtype=NP[dtype])
    assert lib().orc_fill_check_pattern(dtype, out.ctypes.data_as(C.c_void_p), count) == 0
    return out


def ref_lib(name):
    """A library built from the reference's own C (oracle/_ref), or None when absent."""
    path = os.path.join(REF_DIR, name)
    return C.CDLL(path) if os.path.exists(path) else None


# Kind codes shared by the oracle and the GPU library's ABI.
PART_MAX, PART_DENOM, PART_DENOM_MAX, PART_FROM_PARTS, PART_UNSCALED, PART_UNSCALED_FROM_MAX, \
    PART_COMPLETE, PART_DIVIDE_VEC, PART_DIVIDE_VEC_SCALAR = range(6, 15)


def softmax_part(kind, shape, scan_dim, params, accum=False):
    """Runs one primitive of the Softmax decomposition in place on `params` (f32 arrays,
    dense row-major, Spec parameter order)."""
    ptrs = (C.c_void_p * 4)()
    for i, p in enumerate(params):
        assert p.dtype == np.float32 and p.flags["C_CONTIGUOUS"]
        ptrs[i] = p.ctypes.data
    rc = lib().orc_softmax_part(kind, int(accum), _u32(shape), len(shape), scan_dim, ptrs)
    assert rc == 0, f"oracle softmax_part rc={rc}"
    return params


def broadcast(shape, dim, x):
    out = np.empty(shape, dtype=x.dtype)
    rc = lib().orc_broadcast(_u32(shape), len(shape), dim, C.c_size_t(x.itemsize),
                             x.ctypes.data_as(C.c_void_p), out.ctypes.data_as(C.c_void_p))
    assert rc == 0
    return out


def fill(dtype, value, count):
    out = np.full(count, 0x55, dtype=NP[dtype])
    rc = lib().orc_fill(dtype, value, out.ctypes.data_as(C.c_void_p), C.c_size_t(count))
    assert rc == 0, f"oracle fill rc={rc}"
    return out
