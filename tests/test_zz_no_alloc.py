"""mrl_run_noalloc: the entry point for callers that cannot allocate device memory, against
mrl_run on the same Specs.  Scratch-using paths only (operands padded to whole 16-byte chunks,
K shared out over workgroups with a summing pass, a Compose with materialised intermediates):
results must be the same bits, on calls that follow each other through the one shared array,
the later ones with smaller inputs."""
import numpy as np
import pytest

import morello_amd as M
from gpu_util import run_spec
from morello_amd import synth

pytestmark = pytest.mark.gpu


def both_ways(spec, arrays):
    """-> (output of mrl_run, output of mrl_run_noalloc) on fresh copies of `arrays`."""
    want = run_spec(spec, arrays)
    bufs = [M.DeviceBuffer.from_numpy(a) for a in arrays]
    M.synchronize()
    free_before = M.device_free_bytes()
    spec.run_noalloc([b.ptr for b in bufs])
    M.synchronize()
    assert M.device_free_bytes() == free_before      # the call took no device memory
    got = bufs[-1].to_numpy(arrays[-1].dtype, arrays[-1].shape)
    for b in bufs:
        b.free()
    return want, got


def test_noalloc_matches_run_on_two_calls_in_a_row(gpu):
    # K shared out over slices (partial results in scratch, then the sum): the larger first
    for seed, (m, k, n) in enumerate([(512, 8192, 512), (128, 4096, 192)]):
        spec = M.MatmulAccum([1, m, k, n], (M.u8, M.i8, M.i32))
        assert spec.plan().scratch_bytes > 0 and "k_sum_splits" in spec.plan().kernels
        arrays = [synth.uniform_u8(900 + seed, 0, (1, m, k)), synth.uniform_i8(900 + seed, 1, (1, k, n)),
                  (synth.uniform_u8(900 + seed, 2, (1, m, n)).astype(np.int32) - 77)]
        want, got = both_ways(spec, arrays)
        assert np.array_equal(got, want)
    # rows that are not whole 16-byte chunks (zero-padded copies of A and B in scratch): larger, then smaller
    for seed, (m, k, n) in enumerate([(1000, 1000, 1000), (520, 300, 410)]):
        spec = M.Matmul([1, m, k, n], (M.u8, M.i8, M.i32))
        assert spec.plan().scratch_bytes > 0
        arrays = [synth.uniform_u8(910 + seed, 0, (1, m, k)), synth.uniform_i8(910 + seed, 1, (1, k, n)),
                  np.full((1, m, n), -1, np.int32)]
        want, got = both_ways(spec, arrays)
        assert np.array_equal(got, want)


def test_noalloc_between_calls_that_use_the_arena(gpu):
    """mrl_run_async (scratch from the stream's arena) between two mrl_run_noalloc calls (scratch
    from the fixed array): neither disturbs the other."""
    m, k, n = 384, 4096, 256
    spec = M.MatmulAccum([1, m, k, n], (M.u8, M.i8, M.i32))
    assert spec.plan().scratch_bytes > 0
    a, b = synth.uniform_u8(930, 0, (1, m, k)), synth.uniform_i8(930, 1, (1, k, n))
    once = run_spec(spec, [a, b, np.zeros((1, m, n), np.int32)])
    bufs = [M.DeviceBuffer.from_numpy(x) for x in (a, b, np.zeros((1, m, n), np.int32))]
    ptrs = [x.ptr for x in bufs]
    spec.run_noalloc(ptrs)
    spec.run_device(ptrs)       # mrl_run: accumulates a second time
    spec.run_noalloc(ptrs)
    M.synchronize()
    got = bufs[2].to_numpy(np.int32, (1, m, n))
    for x in bufs:
        x.free()
    assert np.array_equal(got, once * 3)


def test_noalloc_wants_aligned_parameters(gpu):
    spec = M.MatmulAccum([1, 256, 256, 256], (M.u8, M.i8, M.i32))
    bufs = [M.DeviceBuffer(spec.bytes_used(i) + 256) for i in range(3)]
    with pytest.raises(M.MorelloError) as err:
        spec.run_noalloc([bufs[0].ptr + 16, bufs[1].ptr, bufs[2].ptr])
    assert err.value.status == 1 and "aligned" in str(err.value)
    for x in bufs:
        x.free()


def test_noalloc_turns_down_what_does_not_fit(gpu):
    # staged Compose with 16 x 2048 x 2048 f32 scores: 268 MB of intermediates
    spec = M.ComposeMSM(16, 2048, 256, 2048, 256, layouts=[None, None, M.layout(0, 2, 1), None])
    assert spec.plan().scratch_bytes > M.NOALLOC_SCRATCH_BYTES
    bufs = [M.DeviceBuffer(spec.bytes_used(i)) for i in range(4)]
    with pytest.raises(M.MorelloError) as err:
        spec.run_noalloc([b.ptr for b in bufs])
    assert "scratch" in str(err.value)
    for b in bufs:
        b.free()
    # and a Spec that needs no scratch at all runs
    spec = M.MatmulAccum([1, 256, 256, 256], (M.u8, M.i8, M.i32))
    arrays = [synth.uniform_u8(920, 0, (1, 256, 256)), synth.uniform_i8(920, 1, (1, 256, 256)), np.zeros((1, 256, 256), np.int32)]
    want, got = both_ways(spec, arrays)
    assert np.array_equal(got, want)
