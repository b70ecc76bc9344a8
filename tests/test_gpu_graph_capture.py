"""mrl_run_noalloc under HIP stream capture: the launches of several Specs recorded into one graph,
the graph replayed with the program's own eager work (fresh inputs uploaded, eager runs of the
same Specs) between the replays, every replay held against the eager result bit for bit.  The
HIP graph calls are made through ctypes on the runtime the library itself is linked to."""
import ctypes as C

import numpy as np
import pytest

import morello_amd as M
from gpu_util import run_spec
from morello_amd import synth

pytestmark = pytest.mark.gpu

NHWC = M.layout(0, 2, 3, 1)


def hip_runtime():
    for name in ("libamdhip64.so", "/opt/rocm/lib/libamdhip64.so"):
        try:
            hip = C.CDLL(name)
            hip.hipStreamBeginCapture.argtypes = [C.c_void_p, C.c_int]
            hip.hipStreamEndCapture.argtypes = [C.c_void_p, C.POINTER(C.c_void_p)]
            hip.hipGraphInstantiate.argtypes = [C.POINTER(C.c_void_p), C.c_void_p, C.c_void_p, C.c_char_p, C.c_size_t]
            hip.hipGraphLaunch.argtypes = [C.c_void_p, C.c_void_p]
            hip.hipGraphExecDestroy.argtypes = [C.c_void_p]
            hip.hipGraphDestroy.argtypes = [C.c_void_p]
            return hip
        except OSError:
            continue
    raise RuntimeError("the HIP runtime library was not found")


def inputs(seed):
    """Parameter buffers of the four Specs, outputs included (filled with a sentinel)."""
    return [
        [synth.uniform_u8(seed, 0, (4, 22, 22, 64)), synth.uniform_i8(seed, 1, (64, 3, 3, 64)), np.full((4, 20, 20, 64), -3, np.int32)],
        [synth.uniform_u8(seed, 2, (1, 512, 8192)), synth.uniform_i8(seed, 3, (1, 8192, 512)), np.full((1, 512, 512), -3, np.int32)],
        [(synth.normal_f32(seed, 4, (64, 2048)) * 3).astype(np.float32), np.full((64, 2048), -3, np.float32)],
        [synth.normal_bf16(seed, 5, (2, 256, 128), 0.5), synth.normal_bf16(seed, 6, (2, 256, 128), 0.5),
         synth.normal_bf16(seed, 7, (2, 256, 128), 0.5), np.full((2, 256, 128), -3, np.float32)],
    ]


def test_noalloc_launches_replay_from_a_graph(gpu):
    hip = hip_runtime()
    specs = [
        M.Conv([4, 64, 64, 20, 20, 3, 3], (M.u8, M.i8, M.i32)),                                # the fused Conv kernel
        M.Matmul([1, 512, 8192, 512], (M.u8, M.i8, M.i32)),                                    # K in slices: partial results in the fixed scratch array, then the sum
        M.Softmax([64, 2048], 1),
        M.ComposeMSM(2, 256, 128, 256, 128, layouts=[None, None, M.layout(0, 2, 1), None]),    # the fused attention kernel
    ]
    assert "k_sum_splits" in specs[1].plan().kernels and specs[3].plan().kernels == ["k_attn"]
    first = inputs(700)
    bufs = [[M.DeviceBuffer.from_numpy(a) for a in arrays] for arrays in first]
    stream = M.Stream()
    graph, graph_exec = C.c_void_p(), C.c_void_p()
    try:
        assert hip.hipStreamBeginCapture(stream.handle, 0) == 0          # hipStreamCaptureModeGlobal
        try:
            for spec, b in zip(specs, bufs):
                spec.run_noalloc([x.ptr for x in b], stream)
        finally:
            assert hip.hipStreamEndCapture(stream.handle, C.byref(graph)) == 0
        assert hip.hipGraphInstantiate(C.byref(graph_exec), graph, None, None, 0) == 0
        # nothing has run yet: the outputs still hold the sentinel
        assert np.all(bufs[0][2].to_numpy(np.int32, (4, 20, 20, 64)) == -3)
        for replay, seed in enumerate((700, 701, 702, 700)):
            arrays = inputs(seed)
            want = [run_spec(spec, a) for spec, a in zip(specs, arrays)]        # eager runs between the replays
            for b, a in zip(bufs, arrays):                                        # fresh inputs, outputs back to the sentinel
                for x, host in zip(b, a):
                    M._check(M.B.load().mrl_memcpy_h2d(x.ptr, np.ascontiguousarray(host).ctypes.data, host.nbytes), "mrl_memcpy_h2d")
            assert hip.hipGraphLaunch(graph_exec, stream.handle) == 0
            stream.synchronize()
            for spec, b, a, w in zip(specs, bufs, arrays, want):
                got = b[-1].to_numpy(a[-1].dtype, a[-1].shape)
                assert np.array_equal(got, w), (replay, spec.kind)
    finally:
        if graph_exec:
            hip.hipGraphExecDestroy(graph_exec)
        if graph:
            hip.hipGraphDestroy(graph)
        stream.destroy()
        for b in bufs:
            for x in b:
                x.free()
