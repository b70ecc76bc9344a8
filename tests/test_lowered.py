"""The hand-restated "Morello-lowered" C (oracle/lowered) against the closed-form oracle.
These kernels are the CPU baseline the benchmark times; they must compute the same thing.
No GPU needed."""
import ctypes as C
import os
import subprocess

import numpy as np
import pytest

import orc
from morello_amd import synth

LIB = os.path.join(orc.ORACLE_DIR, "liblowered.so")


@pytest.fixture(scope="module")
def low():
    if not os.path.exists(LIB):
        subprocess.run(["make", "-C", orc.ORACLE_DIR, "liblowered.so"], check=True, capture_output=True)
    return C.CDLL(LIB)


def p(a):
    return a.ctypes.data_as(C.c_void_p)


def test_c1_f32(low):
    m = k = n = 64
    A, Bm = synth.uniform_f32(1, 0, (1, m, k)), synth.uniform_f32(1, 1, (1, k, n))
    out = np.full((1, m, n), 9.0, np.float32)
    low.lowered_matmul_f32(p(A), p(Bm), p(out), m, k, n)
    want = orc.matmul([1, m, k, n], [6, 6, 6], A, Bm, np.zeros((1, m, n), np.float32))
    assert np.abs(out - want).max() < 1e-5
    ref = orc.ref_lib("libref_simple_matmul.so")
    if ref is not None:  # same loop nest as the reference's quoted kernel: same bits
        out2 = np.empty_like(out)
        ref.ref_simple_matmul_f32(p(A), p(Bm), p(out2))
        assert np.array_equal(out, out2)


@pytest.mark.parametrize("threads", [1, 0])
def test_c2_u8i8i32(low, threads):
    m, k, n = 24, 200, 48
    A, Bm = synth.uniform_u8(2, 0, (1, m, k)), synth.uniform_i8(2, 1, (1, k, n))
    C0 = synth.uniform_u8(2, 2, (1, m, n)).astype(np.int32)
    out = C0.copy()
    low.lowered_matmul_u8i8i32(p(A), p(Bm), p(out), m, k, n, 4, 20, threads)
    want = orc.matmul([1, m, k, n], [0, 1, 5], A, Bm, C0.copy(), True, rows=(4, 20))
    assert np.array_equal(out, want)


def test_c3_bf16(low):
    m, k, n = 8, 300, 32
    A, Bm = synth.normal_bf16(3, 0, (1, m, k)), synth.normal_bf16(3, 1, (1, k, n))
    out = np.zeros((1, m, n), np.float32)
    low.lowered_matmul_bf16f32(p(A), p(Bm), p(out), m, k, n, 0, m, 0)
    want = orc.matmul([1, m, k, n], [7, 7, 6], A, Bm, np.zeros((1, m, n), np.float32))
    assert np.abs(out - want).max() / np.abs(want).max() < 1e-6


def test_c4_conv(low):
    b, f, c, oh, ow, fh, fw = 3, 8, 16, 5, 6, 3, 3
    img = synth.uniform_u8(4, 0, (b, oh + 2, ow + 2, c))
    filt = synth.uniform_i8(4, 1, (f, fh, fw, c))
    out = np.full((b, oh, ow, f), 3, np.int32)
    low.lowered_conv_u8i8i32(p(img), p(filt), p(out), b, f, c, oh, ow, fh, fw, 0, b, 0)
    nhwc = orc.make_layout([0, 2, 3, 1])
    want = orc.conv([b, f, c, oh, ow, fh, fw], [0, 1, 5], img, filt, np.zeros((b, oh, ow, f), np.int32),
                    layouts=[nhwc] * 3)
    assert np.array_equal(out, want)


def test_c5_compose(low):
    b, m, k, n2, n = 2, 12, 16, 40, 8
    q = synth.normal_bf16(5, 0, (b, m, k), 0.5)
    kmat = synth.normal_bf16(5, 1, (b, n2, k), 0.5)
    v = synth.normal_bf16(5, 2, (b, n2, n), 0.5)
    out = np.zeros((b, m, n), np.float32)
    low.lowered_compose_msm(p(v), p(q), p(kmat), p(out), b, m, k, n2, n, 0, b, 0)
    want = orc.compose_msm(b, m, k, n2, n, [7, 7, 7, 6], v, q, kmat, np.zeros((b, m, n), np.float32),
                           layouts=[None, None, orc.make_layout([0, 2, 1]), None])
    assert np.abs(out - want).max() / np.abs(want).max() < 1e-5
