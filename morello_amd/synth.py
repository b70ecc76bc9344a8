"""Seeded synthetic tensors for parity tests and the benchmark.

A counter-based generator: element ``i`` of tensor ``tensor_id`` under ``seed`` is a pure
function of ``(seed, tensor_id, i)`` (SplitMix64 finaliser), so any slice of any tensor can
be regenerated anywhere without shipping data.  The reference fills benchmark buffers with
``rand()`` (morello/src/codegen/c_utils.rs:193-252) and check-mode buffers with a counting
pattern (morello/src/verification.rs:893-952); :func:`check_pattern` reproduces the latter.
"""
from __future__ import annotations

import numpy as np

_GOLDEN = np.uint64(0x9E3779B97F4A7C15)


def _mix(z: np.ndarray) -> np.ndarray:
    z = (z ^ (z >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)
    z = (z ^ (z >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)
    return z ^ (z >> np.uint64(31))


def raw_u64(seed: int, tensor_id: int, count: int, start: int = 0) -> np.ndarray:
    """``count`` 64-bit words for flat logical indices ``start .. start+count``."""
    with np.errstate(over="ignore"):
        key = _mix(np.array([seed], dtype=np.uint64) * _GOLDEN + np.uint64(tensor_id + 1))
        idx = np.arange(start, start + count, dtype=np.uint64)
        return _mix((idx + np.uint64(1)) * _GOLDEN ^ key)


def uniform_u8(seed, tensor_id, shape):
    n = int(np.prod(shape))
    return (raw_u64(seed, tensor_id, n) >> np.uint64(56)).astype(np.uint8).reshape(shape)


def uniform_i8(seed, tensor_id, shape):
    return uniform_u8(seed, tensor_id, shape).view(np.int8)


def uniform_f32(seed, tensor_id, shape):
    """uniform[-1, 1): 24 random bits scaled by 2^-23, minus one."""
    n = int(np.prod(shape))
    u = (raw_u64(seed, tensor_id, n) >> np.uint64(40)).astype(np.float64)
    return (u * 2.0 ** -23 - 1.0).astype(np.float32).reshape(shape)


def normal_f32(seed, tensor_id, shape, std=1.0):
    """N(0, std^2) by Box-Muller in float64, rounded to float32."""
    n = int(np.prod(shape))
    r = raw_u64(seed, tensor_id, n)
    u1 = ((r >> np.uint64(32)).astype(np.float64) + 1.0) * 2.0 ** -32  # (0, 1]
    u2 = (r & np.uint64(0xFFFFFFFF)).astype(np.float64) * 2.0 ** -32  # [0, 1)
    z = np.sqrt(-2.0 * np.log(u1)) * np.cos(2.0 * np.pi * u2)
    return (z * std).astype(np.float32).reshape(shape)


def f32_to_bf16_bits(x: np.ndarray) -> np.ndarray:
    """Round-to-nearest-even narrowing, as `half::bf16::from_f32` and clang's __bf16 do."""
    bits = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32)
    lsb = (bits >> np.uint32(16)) & np.uint32(1)
    with np.errstate(over="ignore"):
        rounded = bits + np.uint32(0x7FFF) + lsb
    out = (rounded >> np.uint32(16)).astype(np.uint16)
    nan = (bits & np.uint32(0x7FFFFFFF)) > np.uint32(0x7F800000)
    out[nan] = ((bits[nan] >> np.uint32(16)) | np.uint32(0x40)).astype(np.uint16)
    return out


def bf16_bits_to_f32(b: np.ndarray) -> np.ndarray:
    """Exact widening: the 16 bits become the top half of a float32."""
    return (np.ascontiguousarray(b, dtype=np.uint16).astype(np.uint32) << np.uint32(16)).view(np.float32)


def normal_bf16(seed, tensor_id, shape, std=1.0):
    return f32_to_bf16_bits(normal_f32(seed, tensor_id, shape, std))


def check_pattern(dtype_name: str, shape):
    """The reference's check-mode inputs (verification.rs:893-952) in logical row-major
    order: integers count up from the dtype minimum and wrap; f32/bf16 cycle 0,1,2,3."""
    n = int(np.prod(shape))
    i = np.arange(n, dtype=np.uint64)
    if dtype_name == "u8":
        return i.astype(np.uint8).reshape(shape)
    if dtype_name == "i8":
        return (i + np.uint64(128)).astype(np.uint8).view(np.int8).reshape(shape)
    if dtype_name == "u16":
        return i.astype(np.uint16).reshape(shape)
    if dtype_name == "i16":
        return (i + np.uint64(32768)).astype(np.uint16).view(np.int16).reshape(shape)
    if dtype_name == "u32":
        return i.astype(np.uint32).reshape(shape)
    if dtype_name == "i32":
        return (i + np.uint64(1 << 31)).astype(np.uint32).view(np.int32).reshape(shape)
    if dtype_name == "f32":
        return (i & np.uint64(3)).astype(np.float32).reshape(shape)
    if dtype_name == "bf16":
        return f32_to_bf16_bits((i & np.uint64(3)).astype(np.float32)).reshape(shape)
    raise ValueError(dtype_name)
