"""General Compose Specs: external parameter order and chain validation (host logic), and GPU
parity of whole pipelines against the oracle's components applied in execution order."""
import numpy as np
import pytest

import morello_amd as M
import orc
from morello_amd import synth


def test_parameter_order_of_the_reference_matmul_chain():
    # matmul_chain_test_data (spec.rs:4650-4700) and the expectation of
    # test_compose_parameters (spec.rs:3733-3785): [c0.rhs, c1.rhs, c2.lhs, c2.rhs, c0.out].
    c = M.Compose([M.Matmul([16, 128, 128, 128], [M.u8, M.u16, M.u32]),
                   M.Matmul([16, 128, 128, 128], [M.u32, M.u16, M.u8]),
                   M.Matmul([16, 128, 128, 128], [M.u8, M.u8, M.u32])])
    assert c.n_params == 5
    assert [c.parameter(i) for i in range(5)] == [(0, 1), (1, 1), (2, 0), (2, 1), (0, 2)]
    assert c.parameter_shapes() == [[16, 128, 128]] * 5
    assert c.parameter_dtypes() == [M.u16, M.u16, M.u8, M.u8, M.u32]


def test_parameter_order_of_the_attention_compose():
    # examples/matmul_chain.rs:26-57; spec.rs:3329-3365: [V, Q, KT, out].
    b, m, k, n2, n = 16, 2048, 128, 2048, 128
    c = M.Compose([M.Matmul([b, m, n2, n], [M.f32, M.bf16, M.f32]), M.Softmax([b, m, n2], 2),
                   M.Matmul([b, m, k, n2], [M.bf16, M.bf16, M.f32])])
    assert c.parameter_shapes() == M.ComposeMSM(b, m, k, n2, n).parameter_shapes()
    assert c.parameter_dtypes() == [M.bf16, M.bf16, M.bf16, M.f32]
    assert [c.parameter(i) for i in range(4)] == [(0, 1), (2, 0), (2, 1), (0, 2)]


def test_middle_components_contribute_their_extra_inputs():
    # SoftmaxComplete in the middle takes (max, denom) as extra inputs after its first.
    shape = [4, 6, 10]
    c = M.Compose([M.Matmul([4, 6, 10, 3], [M.f32] * 3), M.SoftmaxComplete(shape, 2),
                   M.Matmul([4, 6, 5, 10], [M.f32] * 3)])
    assert [c.parameter(i) for i in range(c.n_params)] == [(0, 1), (1, 1), (1, 2), (2, 0), (2, 1), (0, 2)]
    assert c.parameter_shapes() == [[4, 10, 3], [4, 6, 1], [4, 6, 1], [4, 6, 5], [4, 5, 10], [4, 6, 3]]


def test_chain_validation():
    mm = lambda shape, dts=(M.f32,) * 3, accum=False: M.Matmul(shape, list(dts), accum=accum)
    with pytest.raises(M.MorelloError):  # one component is not a Compose (spec.rs:3330)
        M.Compose([mm([1, 4, 4, 4])])
    with pytest.raises(M.MorelloError):  # shapes do not chain: [1,4,8] is not [1,4,4]
        M.Compose([mm([1, 4, 8, 4]), mm([1, 4, 4, 4])])
    with pytest.raises(M.MorelloError):  # dtypes do not chain: i32 output into an f32 input
        M.Compose([mm([1, 4, 4, 4]), mm([1, 4, 4, 4], (M.u8, M.i8, M.i32))])
    with pytest.raises(M.MorelloError):  # accumulating tail component (spec.rs:1760-1764, 3840-3847)
        M.Compose([mm([1, 4, 4, 4]), mm([1, 4, 4, 4], accum=True)])
    # An accumulating head is a Compose (spec.rs:3829-3838) with the same parameters.
    c = M.Compose([mm([1, 4, 4, 4], accum=True), mm([1, 4, 4, 4])])
    assert [c.parameter(i) for i in range(c.n_params)] == [(0, 1), (1, 0), (1, 1), (0, 2)]
    with pytest.raises(M.MorelloError):  # two written parameters: no unique output to chain on
        M.Compose([mm([1, 4, 4, 4]), M.SoftmaxDenominatorAndMax([1, 4, 4], 2)])
    with pytest.raises(M.MorelloError):  # DivideVec writes its first parameter
        M.Compose([M.DivideVec([1, 4, 4]), mm([1, 4, 4, 4])])


def _run(compose, arrays):
    bufs = [M.DeviceBuffer.from_numpy(a) for a in arrays]
    compose.run_device([b.ptr for b in bufs])
    out = bufs[-1].to_numpy(arrays[-1].dtype, arrays[-1].shape)
    for b in bufs:
        b.free()
    return out


@pytest.mark.gpu
def test_integer_matmul_chain_is_exact(gpu):
    """(A.B).C.D with wrapping integer intermediates, as the reference's interpreter chains
    `dot_inplace` (verification.rs:286-335), bit-exact against the oracle applied in order."""
    b, m = 2, 24
    a = synth.uniform_u8(901, 0, (b, m, 40))
    w2 = synth.uniform_i8(901, 1, (b, 40, 16))
    w1 = synth.uniform_i8(901, 2, (b, 16, 72)).astype(np.int32)
    w0 = synth.uniform_i8(901, 3, (b, 72, 8)).astype(np.int32)
    c = M.Compose([M.Matmul([b, m, 72, 8], [M.i32] * 3), M.Matmul([b, m, 16, 72], [M.i32] * 3),
                   M.Matmul([b, m, 40, 16], [M.u8, M.i8, M.i32])])
    got = _run(c, [w0, w1, a, w2, np.zeros((b, m, 8), np.int32)])
    t2 = orc.matmul([b, m, 40, 16], [orc.U8, orc.I8, orc.I32], a, w2, np.zeros((b, m, 16), np.int32))
    t1 = orc.matmul([b, m, 16, 72], [orc.I32] * 3, t2, w1, np.zeros((b, m, 72), np.int32))
    want = orc.matmul([b, m, 72, 8], [orc.I32] * 3, t1, w0, np.zeros((b, m, 8), np.int32))
    assert np.array_equal(got, want)


@pytest.mark.gpu
def test_accumulating_head(gpu):
    """components[0] = Matmul{accum: true} (spec.rs:3829-3838): the pipeline's result is added to
    what the output holds, wrapping for integers, and a second run adds it again."""
    b, m = 2, 24
    a = synth.uniform_u8(905, 0, (b, m, 40))
    w1 = synth.uniform_i8(905, 1, (b, 40, 16))
    w0 = synth.uniform_i8(905, 2, (b, 16, 72)).astype(np.int32)
    init = synth.uniform_i8(905, 3, (b, m, 72)).astype(np.int32) * 16777259
    c = M.Compose([M.Matmul([b, m, 16, 72], [M.i32] * 3, accum=True), M.Matmul([b, m, 40, 16], [M.u8, M.i8, M.i32])])
    t1 = orc.matmul([b, m, 40, 16], [orc.U8, orc.I8, orc.I32], a, w1, np.zeros((b, m, 16), np.int32))
    want = orc.matmul([b, m, 16, 72], [orc.I32] * 3, t1, w0, init.copy(), accum=True)
    got = _run(c, [w0, a, w1, init.copy()])
    assert np.array_equal(got, want)
    want2 = orc.matmul([b, m, 16, 72], [orc.I32] * 3, t1, w0, want.copy(), accum=True)
    assert np.array_equal(_run(c, [w0, a, w1, got.copy()]), want2)
    # The attention shape with an accumulating head: Matmul -> Softmax -> MatmulAccum.
    b, m, k, n2, n = 2, 128, 128, 256, 128
    q = synth.normal_bf16(906, 0, (b, m, k), 0.5)
    kmat = synth.normal_bf16(906, 1, (b, n2, k), 0.5)
    v = synth.normal_bf16(906, 2, (b, n2, n), 0.5)
    init = synth.normal_f32(906, 3, (b, m, n), 1.0)
    c = M.Compose([M.Matmul([b, m, n2, n], [M.f32, M.bf16, M.f32], accum=True), M.Softmax([b, m, n2], 2),
                   M.Matmul([b, m, k, n2], [M.bf16, M.bf16, M.f32])], layouts=[None, None, M.layout(0, 2, 1), None])
    got = _run(c, [v, q, kmat, init.copy()])
    kt = np.ascontiguousarray(kmat.transpose(0, 2, 1))
    want = init + orc.compose_msm(b, m, k, n2, n, [7, 7, 7, 6], v, q, kt, np.zeros((b, m, n), np.float32))
    assert np.abs(got - want).max() / np.abs(want).max() < 1e-2  # the Compose's tolerance: P is rounded to bf16
    assert np.abs(got - init).max() > 0.01


@pytest.mark.gpu
def test_general_compose_equals_the_attention_spec(gpu):
    b, m, k, n2, n = 2, 128, 128, 256, 128
    q = synth.normal_bf16(902, 0, (b, m, k), 0.5)
    kmat = synth.normal_bf16(902, 1, (b, n2, k), 0.5)
    v = synth.normal_bf16(902, 2, (b, n2, n), 0.5)
    kt_layout = M.layout(0, 2, 1)
    c = M.Compose([M.Matmul([b, m, n2, n], [M.f32, M.bf16, M.f32]), M.Softmax([b, m, n2], 2),
                   M.Matmul([b, m, k, n2], [M.bf16, M.bf16, M.f32])], layouts=[None, None, kt_layout, None])
    got = _run(c, [v, q, kmat, np.zeros((b, m, n), np.float32)])
    kt = np.ascontiguousarray(kmat.transpose(0, 2, 1))
    want = orc.compose_msm(b, m, k, n2, n, [7, 7, 7, 6], v, q, kt, np.zeros((b, m, n), np.float32))
    assert np.abs(got - want).max() / np.abs(want).max() < 1e-2
    # bufferize (scheduling/bufferize.rs): with the softmax input or output materialised the
    # pipeline runs component by component with f32 intermediates, as the reference's
    # interpreter does, and lands within 1e-5 of the oracle instead of the fused kernel's 1e-3.
    fused_err = np.abs(got - want).max() / np.abs(want).max()
    for idx in (0, 1):
        staged = _run(c.bufferize(idx), [v, q, kmat, np.zeros((b, m, n), np.float32)])
        assert np.abs(staged - want).max() / np.abs(want).max() < 1e-5 < fused_err
    with pytest.raises(M.MorelloError):
        c.bufferize(2)
    # A shape the fused kernel does not take (head dim 64) runs component by component.
    b, m, k, n2, n = 2, 48, 64, 80, 24
    q = synth.normal_f32(903, 0, (b, m, k), 0.5)
    kt = synth.normal_f32(903, 1, (b, k, n2), 0.5)
    v = synth.normal_f32(903, 2, (b, n2, n), 0.5)
    c = M.Compose([M.Matmul([b, m, n2, n], [M.f32] * 3), M.Softmax([b, m, n2], 2), M.Matmul([b, m, k, n2], [M.f32] * 3)])
    got = _run(c, [v, q, kt, np.zeros((b, m, n), np.float32)])
    want = orc.compose_msm(b, m, k, n2, n, [6, 6, 6, 6], v, q, kt, np.zeros((b, m, n), np.float32))
    np.testing.assert_allclose(got, want, rtol=1e-5, atol=1e-6)


@pytest.mark.gpu
def test_pipeline_of_softmax_primitives(gpu):
    """[DivideVecScalar is InOut and cannot chain; SoftmaxComplete can]:
    Matmul -> SoftmaxComplete(max, denom given) -> Max over the rows of the result."""
    b, m, k, n2 = 3, 10, 12, 33
    q = synth.normal_f32(904, 0, (b, m, k), 0.7)
    kt = synth.normal_f32(904, 1, (b, k, n2), 0.7)
    s = np.zeros((b, m, n2), np.float32)
    orc.matmul([b, m, k, n2], [orc.F32] * 3, q, kt, s)
    mx = s.max(axis=2, keepdims=True)
    dn = np.exp(s - mx).sum(axis=2, keepdims=True).astype(np.float32)
    c = M.Compose([M.Max([b, m, n2], 2), M.SoftmaxComplete([b, m, n2], 2), M.Matmul([b, m, k, n2], [M.f32] * 3)])
    assert [c.parameter(i) for i in range(c.n_params)] == [(1, 1), (1, 2), (2, 0), (2, 1), (0, 1)]
    got = _run(c, [mx, dn, q, kt, np.zeros((b, m, 1), np.float32)])
    p = orc.softmax_part(orc.PART_COMPLETE, (b, m, n2), 2, [s, mx, dn, np.zeros_like(s)])[3]
    want = orc.softmax_part(orc.PART_MAX, (b, m, n2), 2, [p, np.zeros((b, m, 1), np.float32)])[1]
    np.testing.assert_allclose(got, want, rtol=1e-5, atol=1e-7)
