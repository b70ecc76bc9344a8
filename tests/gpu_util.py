"""Helpers for the GPU parity tests: every call goes through the C ABI (mrl_run)."""
import numpy as np

import morello_amd as M


def run_spec(spec, arrays, out_index=-1):
    """Uploads `arrays` (raw parameter buffers in Spec order), runs the Spec on the device,
    returns the output parameter as a numpy array of the same dtype/shape as given."""
    bufs = [M.DeviceBuffer.from_numpy(a) for a in arrays]
    spec.run_device([b.ptr for b in bufs])
    out = arrays[out_index]
    res = bufs[out_index].to_numpy(out.dtype, out.shape)
    for b in bufs:
        b.free()
    return res


def rel_err(got, want):
    """Norm-wise relative error max|x - r| / max|r|."""
    return float(np.abs(got.astype(np.float64) - want.astype(np.float64)).max() /
                 max(float(np.abs(want).max()), 1e-30))


def elem_err(got, want, floor_frac=1e-2):
    """Element-wise relative error max(|x - r| / max(|r|, floor)) with the absolute floor
    floor_frac * rms(r): an output that is wrong where the result is small shows here and not in
    the norm-wise figure; the floor keeps elements that cancel to nearly zero from dividing by it."""
    g, w = got.astype(np.float64), want.astype(np.float64)
    floor = max(floor_frac * float(np.sqrt(np.mean(w * w))), 1e-30)
    return float((np.abs(g - w) / np.maximum(np.abs(w), floor)).max())
