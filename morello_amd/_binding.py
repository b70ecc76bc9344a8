"""ctypes binding of libmorello_amd.so (the C ABI in include/morello_amd.h).

Loading fails loudly: there is no CPU implementation behind this package, so a missing
library is an ImportError-grade problem, not something to paper over.
"""
from __future__ import annotations

import ctypes as C
import os

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libmorello_amd.so")

MAX_PHYS, MAX_RANK, MAX_SPEC_RANK, MAX_PARAMS = 10, 5, 7, 4
ABI_VERSION = 4   # MRL_ABI_VERSION of include/morello_amd.h


class PhysDimC(C.Structure):
    _fields_ = [("logical_dim", C.c_uint8), ("kind", C.c_uint8), ("size", C.c_uint32)]


class LayoutC(C.Structure):
    _fields_ = [("ndims", C.c_uint32), ("dims", PhysDimC * MAX_PHYS)]


class MatmulScheduleC(C.Structure):
    _fields_ = [("tile_m", C.c_uint32), ("tile_n", C.c_uint32), ("split_k", C.c_uint32), ("staging", C.c_uint32)]


class ActionC(C.Structure):
    _fields_ = [("kind", C.c_int32), ("tile_m", C.c_uint32), ("tile_n", C.c_uint32), ("split_k", C.c_uint32),
                ("parts", C.c_uint32), ("staging", C.c_uint32), ("n_steps", C.c_uint32), ("scratch_bytes", C.c_uint64), ("cost_ns", C.c_double)]


class SpecC(C.Structure):
    _fields_ = [
        ("kind", C.c_int32),
        ("accum", C.c_int32),
        ("scan_dim", C.c_uint32),
        ("rank", C.c_uint32),
        ("spec_shape", C.c_uint32 * MAX_SPEC_RANK),
        ("n_params", C.c_uint32),
        ("dtypes", C.c_int32 * MAX_PARAMS),
        ("layouts", LayoutC * MAX_PARAMS),
    ]


MAX_SUBSPECS = 4


class SubspecC(C.Structure):
    _fields_ = [("spec", SpecC), ("source", C.c_int32 * MAX_PARAMS)]


class RewriteC(C.Structure):
    _fields_ = [("n_subspecs", C.c_uint32), ("subspecs", SubspecC * MAX_SUBSPECS), ("n_intermediates", C.c_uint32),
                ("intermediate_bytes", C.c_uint64 * MAX_SUBSPECS)]


MAX_COMPONENTS = 8
MAX_COMPOSE_PARAMS = 12


class ComponentC(C.Structure):
    _fields_ = [
        ("kind", C.c_int32),
        ("accum", C.c_int32),
        ("scan_dim", C.c_uint32),
        ("rank", C.c_uint32),
        ("spec_shape", C.c_uint32 * MAX_SPEC_RANK),
        ("n_params", C.c_uint32),
        ("dtypes", C.c_int32 * MAX_PARAMS),
    ]


class ComposeC(C.Structure):
    _fields_ = [
        ("n_components", C.c_uint32),
        ("components", ComponentC * MAX_COMPONENTS),
        ("n_params", C.c_uint32),
        ("layouts", LayoutC * MAX_COMPOSE_PARAMS),
        ("bufferize_mask", C.c_uint32),
    ]


_U32P = C.POINTER(C.c_uint32)
_VPP = C.POINTER(C.c_void_p)

class TargetMemoryC(C.Structure):
    _fields_ = [("name", C.c_char * 8), ("is_addressed", C.c_uint8), ("can_parallel_tile", C.c_uint8),
                ("counts_registers", C.c_uint8), ("has_layout", C.c_uint8), ("vector_bytes", C.c_uint32 * 4),
                ("limit", C.c_uint64), ("cache_hit_cost", C.c_uint32)]


class PlanStepC(C.Structure):
    _fields_ = [("kernel", C.c_char * 160), ("grid", C.c_uint32 * 3), ("block", C.c_uint32 * 3),
                ("lds_bytes", C.c_uint32), ("unit", C.c_int32), ("ops", C.c_double), ("bytes", C.c_double),
                ("cost_ns", C.c_double)]


class PlanC(C.Structure):
    _fields_ = [("n_steps", C.c_uint32), ("scratch_bytes", C.c_uint64), ("cost_ns", C.c_double)]


# name -> (restype, argtypes); every symbol include/morello_amd.h declares.
SIGNATURES = {
    "mrl_init": (C.c_int, [C.c_int]),
    "mrl_status_string": (C.c_char_p, [C.c_int]),
    "mrl_last_error": (C.c_char_p, []),
    "mrl_version": (C.c_char_p, []),
    "mrl_dtype_size": (C.c_size_t, [C.c_int]),
    "mrl_dtype_name": (C.c_char_p, [C.c_int]),
    "mrl_layout_row_major": (C.c_int, [_U32P, C.c_uint32, C.POINTER(LayoutC)]),
    "mrl_layout_col_major": (C.c_int, [_U32P, C.c_uint32, C.POINTER(LayoutC)]),
    "mrl_layout_batched_col_major": (C.c_int, [_U32P, C.c_uint32, C.POINTER(LayoutC)]),
    "mrl_layout_nhwc": (C.c_int, [_U32P, C.c_uint32, C.POINTER(LayoutC)]),
    "mrl_layout_physical_shape": (C.c_int, [C.POINTER(LayoutC), _U32P, C.c_uint32, _U32P]),
    "mrl_layout_buffer_index": (C.c_int64, [C.POINTER(LayoutC), _U32P, C.c_uint32, _U32P]),
    "mrl_spec_parameter_shape": (C.c_int, [C.POINTER(SpecC), C.c_uint32, _U32P, _U32P]),
    "mrl_spec_parameter_direction": (C.c_int, [C.POINTER(SpecC), C.c_uint32]),
    "mrl_spec_parameter_bytes": (C.c_size_t, [C.POINTER(SpecC), C.c_uint32]),
    "mrl_spec_ops": (C.c_uint64, [C.POINTER(SpecC)]),
    "mrl_spec_check": (C.c_int, [C.POINTER(SpecC)]),
    "mrl_spec_workspace_bytes": (C.c_size_t, [C.POINTER(SpecC)]),
    "mrl_run": (C.c_int, [C.POINTER(SpecC), _VPP]),
    "mrl_run_async": (C.c_int, [C.POINTER(SpecC), _VPP, C.c_void_p]),
    "mrl_run_noalloc": (C.c_int, [C.POINTER(SpecC), _VPP, C.c_void_p]),
    "mrl_run_host": (C.c_int, [C.POINTER(SpecC), _VPP]),
    "mrl_matmul": (C.c_int, [C.c_uint32] * 4 + [C.c_int] * 4 + [C.c_void_p] * 4),
    "mrl_conv": (C.c_int, [C.c_uint32] * 7 + [C.c_int] * 4 + [C.c_void_p] * 4),
    "mrl_softmax": (C.c_int, [_U32P, C.c_uint32, C.c_uint32, C.c_void_p, C.c_void_p, C.c_void_p]),
    "mrl_move": (C.c_int, [_U32P, C.c_uint32, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p]),
    "mrl_compose_msm": (C.c_int, [C.c_uint32] * 5 + [C.c_int] * 4 + [C.c_void_p] * 5),
    "mrl_matmul_schedules": (C.c_uint32, [C.POINTER(SpecC), C.POINTER(MatmulScheduleC), C.c_uint32]),
    "mrl_run_matmul_scheduled": (C.c_int, [C.POINTER(SpecC), _VPP, C.POINTER(MatmulScheduleC), C.c_void_p]),
    "mrl_bench": (C.c_int, [C.POINTER(SpecC), _VPP, C.c_uint32, C.c_uint32,
                            C.POINTER(C.c_double), C.POINTER(C.c_double)]),
    "mrl_run_timed": (C.c_int, [C.POINTER(SpecC), _VPP, C.c_uint32, C.POINTER(C.c_double)]),
    "mrl_compose_init": (C.c_int, [C.POINTER(ComposeC)]),
    "mrl_compose_parameter": (C.c_int, [C.POINTER(ComposeC), C.c_uint32, _U32P, _U32P]),
    "mrl_compose_parameter_shape": (C.c_int, [C.POINTER(ComposeC), C.c_uint32, _U32P, _U32P]),
    "mrl_compose_parameter_dtype": (C.c_int, [C.POINTER(ComposeC), C.c_uint32]),
    "mrl_run_compose": (C.c_int, [C.POINTER(ComposeC), _VPP, C.c_void_p]),
    "mrl_measure_mfma_rate": (C.c_int, [C.c_int, C.c_int, C.c_uint32, C.POINTER(C.c_double)]),
    "mrl_device_malloc": (C.c_int, [_VPP, C.c_size_t]),
    "mrl_device_free": (C.c_int, [C.c_void_p]),
    "mrl_memcpy_h2d": (C.c_int, [C.c_void_p, C.c_void_p, C.c_size_t]),
    "mrl_memcpy_d2h": (C.c_int, [C.c_void_p, C.c_void_p, C.c_size_t]),
    "mrl_memset": (C.c_int, [C.c_void_p, C.c_int, C.c_size_t]),
    "mrl_device_synchronize": (C.c_int, []),
    "mrl_stream_create": (C.c_int, [_VPP]),
    "mrl_stream_synchronize": (C.c_int, [C.c_void_p]),
    "mrl_stream_release": (C.c_int, [C.c_void_p]),
    "mrl_device_mem_free": (C.c_int, [C.POINTER(C.c_size_t)]),
    "mrl_abi_version": (C.c_uint32, []),
    "mrl_action_apply": (C.c_int, [C.POINTER(SpecC), C.POINTER(ActionC), C.POINTER(RewriteC)]),
    "mrl_run_action_timed": (C.c_int, [C.POINTER(SpecC), _VPP, C.POINTER(ActionC), C.c_uint32, C.POINTER(C.c_double)]),
    "mrl_stream_destroy": (C.c_int, [C.c_void_p]),
    "mrl_target_id": (C.c_char_p, []),
    "mrl_target_line_size": (C.c_uint32, []),
    "mrl_target_processors": (C.c_uint32, []),
    "mrl_target_memories": (C.c_uint32, [C.POINTER(TargetMemoryC), C.c_uint32]),
    "mrl_target_default_memory": (C.c_uint32, []),
    "mrl_target_destination_memories": (C.c_uint32, [C.c_uint32, C.POINTER(C.c_uint32), C.c_uint32]),
    "mrl_target_layouts_for_shape": (C.c_uint32, [C.POINTER(C.c_uint32), C.c_uint32, C.c_int, C.POINTER(LayoutC),
                                                  C.c_uint32]),
    "mrl_target_kernels": (C.c_uint32, [C.POINTER(C.c_char_p), C.c_uint32]),
    "mrl_spec_plan": (C.c_int, [C.POINTER(SpecC), C.POINTER(PlanC), C.POINTER(PlanStepC), C.c_uint32]),
    "mrl_matmul_scheduled_plan": (C.c_int, [C.POINTER(SpecC), C.POINTER(MatmulScheduleC), C.POINTER(PlanC),
                                            C.POINTER(PlanStepC), C.c_uint32]),
    "mrl_matmul_search_schedule": (C.c_int, [C.POINTER(SpecC), C.POINTER(MatmulScheduleC), C.POINTER(C.c_double)]),
    "mrl_target_actions": (C.c_uint32, [C.POINTER(SpecC), C.POINTER(ActionC), C.c_uint32]),
    "mrl_action_plan": (C.c_int, [C.POINTER(SpecC), C.POINTER(ActionC), C.POINTER(PlanC), C.POINTER(PlanStepC), C.c_uint32]),
    "mrl_run_action": (C.c_int, [C.POINTER(SpecC), _VPP, C.POINTER(ActionC), C.c_void_p]),
    "mrl_launch_count": (C.c_uint64, []),
    "mrl_compose_plan": (C.c_int, [C.POINTER(ComposeC), C.POINTER(PlanC), C.POINTER(PlanStepC), C.c_uint32]),
    "mrl_device_info": (C.c_int, [C.c_char_p, C.c_size_t, C.POINTER(C.c_int), C.POINTER(C.c_int),
                                  C.POINTER(C.c_size_t)]),
}

_lib = None


def load() -> C.CDLL:
    """Loads the library (building nothing: run `python -m morello_amd.build` first)."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            f"{LIB_PATH} is missing: build it with `python -m morello_amd.build` "
            "(there is no CPU fallback)")
    lib = C.CDLL(LIB_PATH)
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)  # AttributeError if the ABI lost a symbol
        fn.restype = res
        fn.argtypes = args
    if lib.mrl_abi_version() != ABI_VERSION:
        raise ImportError(f"{LIB_PATH} has struct layout version {lib.mrl_abi_version()}, this binding is written "
                          f"for {ABI_VERSION}: rebuild with `python -m morello_amd.build`")
    _lib = lib
    return lib
