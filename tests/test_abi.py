"""The C-ABI library loads and exports every symbol the header declares, and the host-side
Spec surface answers as the reference's does.  No compute, no GPU."""
import ctypes as C
import os
import re

import pytest

import morello_amd as M
from morello_amd import _binding as B

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_functions():
    text = open(os.path.join(ROOT, "include", "morello_amd.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(mrl_[a-z0-9_]+)\s*\(", text)))


def test_every_declared_symbol_is_exported_and_bound():
    lib = B.load()
    names = declared_functions()
    assert len(names) >= 30
    for n in names:
        assert hasattr(lib, n), f"{n} declared in the header but not exported"
        assert n in B.SIGNATURES, f"{n} has no ctypes signature"
    assert set(B.SIGNATURES) <= set(names)


def test_abi_version_of_library_header_and_binding_agree():
    text = open(os.path.join(ROOT, "include", "morello_amd.h")).read()
    declared = int(re.search(r"#define MRL_ABI_VERSION (\d+)u", text).group(1))
    assert B.load().mrl_abi_version() == declared == B.ABI_VERSION


def test_struct_sizes_match_the_header():
    # mrl_physdim {u8,u8,u32} = 8 bytes; mrl_layout = 4 + 10*8; mrl_spec as declared.
    assert C.sizeof(B.PhysDimC) == 8
    assert C.sizeof(B.LayoutC) == 84
    assert C.sizeof(B.SpecC) == 4 * 4 + 7 * 4 + 4 + 4 * 4 + 4 * 84
    # mrl_subspec = mrl_spec + 4 sources; mrl_rewrite = count, 4 of those, count, 4 sizes (8-byte aligned)
    assert C.sizeof(B.SubspecC) == C.sizeof(B.SpecC) + 16
    assert C.sizeof(B.RewriteC) == 4 + 4 * C.sizeof(B.SubspecC) + 4 + 4 * 8


def test_parameter_shapes_and_directions():
    # spec.rs:480-498, :523-526 and the Conv expectation of spec.rs:3788-3826
    mm = M.Matmul([32, 2, 3, 3], [M.u8, M.i8, M.u16], accum=True)  # spec.rs:3663-3698
    assert mm.parameter_shapes() == [[32, 2, 3], [32, 3, 3], [32, 2, 3]]
    assert mm.operand_directions() == [M.OperandDirection.In, M.OperandDirection.In, M.OperandDirection.InOut]
    assert M.Matmul([1, 2, 3, 4], [M.f32] * 3).operand_directions()[2] == M.OperandDirection.Out
    cv = M.Conv([1, 2, 3, 4, 5, 2, 2], [M.u8, M.i8, M.i32])
    assert cv.parameter_shapes() == [[1, 3, 5, 6], [2, 3, 2, 2], [1, 2, 4, 5]]
    sm = M.Softmax([4, 8, 16], 2)
    assert sm.parameter_shapes() == [[4, 8, 16]] * 2
    assert sm.operand_directions() == [M.OperandDirection.In, M.OperandDirection.Out]
    # Compose parameters: head's rhs, then the innermost Matmul's lhs and rhs, then the
    # output (spec.rs:3329-3365, test_compose_parameters spec.rs:3733-3785).
    cm = M.ComposeMSM(16, 2048, 128, 2048, 128)
    assert cm.parameter_shapes() == [[16, 2048, 128], [16, 2048, 128], [16, 128, 2048], [16, 2048, 128]]
    assert [int(d) for d in cm.operand_directions()] == [0, 0, 0, 1]
    assert cm.bytes_used(0) == 16 * 2048 * 128 * 2 and cm.bytes_used(3) == 16 * 2048 * 128 * 4


def test_primitive_spec_parameter_shapes_and_directions():
    # spec.rs:499-583 (shapes) and spec.rs:1204-1245 (directions); 0 In, 1 Out, 2 InOut.
    def dirs(spec):
        return [int(d) for d in spec.operand_directions()]

    full, red = [4, 6, 8], [4, 1, 8]
    mx = M.Max(full, 1)
    assert mx.parameter_shapes() == [full, red] and dirs(mx) == [0, 1]
    assert dirs(M.Max(full, 1, accum=True)) == [0, 2]
    sd = M.SoftmaxDenominator(full, 1)
    assert sd.parameter_shapes() == [full, red, red] and dirs(sd) == [0, 0, 1]
    assert dirs(M.SoftmaxDenominator(full, 1, accum=True)) == [0, 0, 2]
    sdm = M.SoftmaxDenominatorAndMax(full, 1)
    assert sdm.parameter_shapes() == [full, red, red] and dirs(sdm) == [0, 1, 1]
    assert dirs(M.SoftmaxDenominatorAndMax(full, 1, accum=True)) == [0, 2, 2]
    fp = M.SoftmaxDenominatorAndMaxFromParts(full, 1)
    assert fp.parameter_shapes() == [full, full, red, red] and dirs(fp) == [0, 0, 1, 1]
    assert dirs(M.SoftmaxDenominatorAndMaxFromParts(full, 1, accum=True)) == [0, 0, 2, 2]
    un = M.SoftmaxDenominatorAndUnscaled(full, 1)
    assert un.parameter_shapes() == [full, red, full] and dirs(un) == [0, 1, 1]
    ufm = M.SoftmaxDenominatorAndUnscaledFromMax(full, 1)
    assert ufm.parameter_shapes() == [full, red, red, full] and dirs(ufm) == [0, 0, 1, 1]
    assert dirs(M.SoftmaxDenominatorAndUnscaledFromMax(full, 1, accum=True)) == [0, 0, 2, 1]
    sc = M.SoftmaxComplete(full, 1)
    assert sc.parameter_shapes() == [full, red, red, full] and dirs(sc) == [0, 0, 0, 1]
    dv = M.DivideVec(full)
    assert dv.parameter_shapes() == [full, full] and dirs(dv) == [2, 0]
    dvs = M.DivideVecScalar(full, 1)
    assert dvs.parameter_shapes() == [full, red] and dirs(dvs) == [2, 0]
    bc = M.Broadcast(full, 1)
    assert bc.parameter_shapes() == [red, full] and dirs(bc) == [0, 1]
    op = M.OnePrefix([6, 8])
    assert op.parameter_shapes() == [[6, 8], [1, 6, 8]] and dirs(op) == [0, 1]
    fl = M.Fill(full, M.i32, M.FillValue.Min)
    assert fl.parameter_shapes() == [full] and dirs(fl) == [1]
    for s in (mx, sd, sdm, fp, un, ufm, sc, dv, dvs, bc, op, fl):
        assert s.check() == 0, s.kind
    # f32 only; scan_dim in range; no -inf among the integers; OnePrefix output rank <= 5.
    assert M.Spec(M.SpecKind.Max, full, [M.u8, M.u8], scan_dim=1).check() == 1
    with pytest.raises(M.MorelloError):
        M.Max(full, 3)  # no parameter shape exists for a dim outside the tensor
    assert M.Fill(full, M.i32, M.FillValue.NegInf).check() == 3
    with pytest.raises(M.MorelloError):
        M.OnePrefix([2, 2, 2, 2, 2])
    assert M.Spec(M.SpecKind.SoftmaxDenominatorAndUnscaled, full, [M.f32] * 3, accum=True, scan_dim=1).check() == 1


def test_flops_convention():
    # spec.rs:273-305: Matmul 2*b*m*k*n, Softmax 5*volume
    assert M.Matmul([1, 4096, 4096, 4096], [M.u8, M.i8, M.i32]).flops() == 137438953472
    assert M.Matmul([1, 8192, 8192, 8192], [M.bf16, M.bf16, M.f32]).flops() == 1099511627776
    assert M.Conv([32, 64, 64, 54, 54, 3, 3], [M.u8, M.i8, M.i32]).flops() == 6879707136
    assert M.Softmax([16, 2048, 2048], 2).flops() == 335544320
    assert M.ComposeMSM(16, 2048, 128, 2048, 128).flops() == 34359738368 + 335544320


def test_spec_check_status_codes():
    assert M.Matmul([1, 64, 64, 64], [M.f32] * 3).check() == 0
    assert M.Matmul([1, 64, 0, 64], [M.f32] * 3).check() == 3          # zero dim
    assert M.Spec(M.SpecKind.Matmul, [1, 2, 3], [M.f32] * 3, layouts=[M.Layout([])] * 3).check() == 3  # rank
    assert M.Matmul([1, 4, 4, 4], [M.f32, M.f32, M.bf16]).check() == 0  # bf16 output: a legal triple (spec.rs:3663-3698)
    assert M.Softmax([4, 4], 2).check() == 3                              # scan_dim out of range
    bad = M.layout((0, M.Packed(4)), 1)                                   # layout.rs:1520-1527
    assert M.Matmul([1, 8, 64, 64], [M.f32] * 3,
                    layouts=[M.Layout([(1, M.Packed(4)), (2, M.Dynamic)]), None, None]).check() == 2
    assert bad.applies_to_shape([1, 64]) and not bad.applies_to_shape([8, 64])
    assert M.Spec(M.SpecKind.Softmax, [4, 4], [M.u8, M.u8], scan_dim=1).check() == 1
    assert M.Matmul([1, 65536, 65536, 2], [M.u8, M.i8, M.i32]).check() == 7  # > i32 index range


def test_workspace_only_for_non_strided_layouts():
    assert M.Matmul([1, 64, 64, 64], [M.f32] * 3).workspace_bytes() == 0
    assert M.Conv([1, 8, 8, 4, 4, 3, 3], [M.u8, M.i8, M.i32]).workspace_bytes() == 0
    packed = M.layout(0, 2, 1, (2, M.Packed(16)))  # examples/matmul_x86.rs:34-53 style relayout
    s = M.Matmul([1, 64, 64, 64], [M.f32] * 3, layouts=[None, packed, None])
    assert s.workspace_bytes() == 64 * 64 * 4
    # Packed dims that leave the row-major order as it is are read in place.
    same_order = M.layout(0, 1, 2, (2, M.Packed(16)))
    assert M.Matmul([1, 64, 64, 64], [M.f32] * 3, layouts=[None, same_order, None]).workspace_bytes() == 0


def test_null_and_status_strings():
    lib = B.load()
    assert lib.mrl_run(None, None) in (5, 6)  # no device here, or NULL spec
    assert lib.mrl_status_string(0) == b"ok"
    assert lib.mrl_status_string(2).startswith(b"layout")
    assert lib.mrl_version().count(b".") == 2


@pytest.mark.gpu
def test_sustained_matrix_core_rate_is_sane(gpu):
    """All-zero operands run near the datasheet rate; benchmark-like operands lower, never
    higher, and both within physical bounds."""
    for kind, nominal in (("int8", 5033e12), ("bf16", 2516e12)):
        zero = M.measure_mfma_rate(kind, False, 4000)
        rand = M.measure_mfma_rate(kind, True, 4000)
        assert 0.2 * nominal < rand <= zero * 1.02 < 1.1 * nominal, (kind, zero, rand)
    lib = B.load()
    out = C.c_double()
    assert lib.mrl_measure_mfma_rate(2, 0, 10, C.byref(out)) == 3   # unknown kind
    assert lib.mrl_measure_mfma_rate(0, 0, 10, None) == 6           # NULL result pointer
