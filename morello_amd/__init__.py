"""morello_amd: MI355X execution backend for Morello Specs -- Python view of the C ABI.

The classes mirror the names of Morello's Spec surface so that a test written against the
reference reads the same here: `Dtype` (morello/src/common.rs:15-65), `PhysDim`/`Layout`
and the constructors `row_major`, `col_major`, `batched_col_major`, `nhwc`, `layout`
(morello/src/layout.rs:67-81, 1234-1302), and the Spec constructors `Matmul`, `Conv`,
`Softmax`, `ComposeMSM` (morello/src/spec.rs:57-162, 467-583).  All arithmetic happens in
libmorello_amd.so; this module only packs descriptors and moves bytes.
"""
from __future__ import annotations

import ctypes as C
import enum
from dataclasses import dataclass
from typing import Optional, Sequence, Tuple

import numpy as np

from . import _binding as B


class MorelloError(RuntimeError):
    def __init__(self, status: int, where: str):
        lib = B.load()
        msg = lib.mrl_status_string(status).decode()
        detail = lib.mrl_last_error().decode()
        with_detail = status == 4 or where == "mrl_run_noalloc"   # the calls that set the detail they fail with
        super().__init__(f"{where}: {msg}" + (f" ({detail})" if detail and with_detail else ""))
        self.status = status


def _check(status: int, where: str):
    if status != 0:
        raise MorelloError(status, where)


class Dtype(enum.IntEnum):
    """morello/src/common.rs:15-24."""
    Uint8 = 0
    Sint8 = 1
    Uint16 = 2
    Sint16 = 3
    Uint32 = 4
    Sint32 = 5
    Float32 = 6
    Bfloat16 = 7

    @property
    def size(self) -> int:
        return int(B.load().mrl_dtype_size(int(self)))

    def __str__(self) -> str:
        return B.load().mrl_dtype_name(int(self)).decode()

    @property
    def numpy(self):
        """Storage dtype; bf16 travels as its 16-bit pattern."""
        return {0: np.uint8, 1: np.int8, 2: np.uint16, 3: np.int16, 4: np.uint32, 5: np.int32,
                6: np.float32, 7: np.uint16}[int(self)]


u8, i8, u16, i16, u32, i32, f32, bf16 = (Dtype(i) for i in range(8))


@dataclass(frozen=True)
class PhysDim:
    """morello/src/layout.rs:74-81.  kind: 0 Dynamic, 1 Packed(size), 2 OddEven(size)."""
    kind: int = 0
    size: int = 0


Dynamic = PhysDim(0, 0)


def Packed(n: int) -> PhysDim:
    return PhysDim(1, n)


def OddEven(n: int) -> PhysDim:
    return PhysDim(2, n)


class Layout:
    """Physical dims, slowest to fastest, as (logical_dim, PhysDim) pairs."""

    def __init__(self, dims: Sequence[Tuple[int, PhysDim]]):
        self.dims = [(int(d), pd) for d, pd in dims]
        if len(self.dims) > B.MAX_PHYS:
            raise ValueError("too many physical dims")

    def to_c(self) -> B.LayoutC:
        out = B.LayoutC()
        out.ndims = len(self.dims)
        for i, (d, pd) in enumerate(self.dims):
            out.dims[i].logical_dim = d
            out.dims[i].kind = pd.kind
            out.dims[i].size = pd.size
        return out

    @staticmethod
    def from_c(c: B.LayoutC) -> "Layout":
        return Layout([(c.dims[i].logical_dim, PhysDim(c.dims[i].kind, c.dims[i].size if c.dims[i].kind else 0))
                       for i in range(c.ndims)])

    def physical_shape(self, shape: Sequence[int]):
        """expand_physical_shape (layout.rs:769-810); raises on shapes it does not apply to."""
        arr = (C.c_uint32 * len(shape))(*shape)
        out = (C.c_uint32 * B.MAX_PHYS)()
        lc = self.to_c()
        _check(B.load().mrl_layout_physical_shape(C.byref(lc), arr, len(shape), out), "physical_shape")
        return [int(out[i]) for i in range(len(self.dims))]

    def applies_to_shape(self, shape: Sequence[int]) -> bool:
        try:
            self.physical_shape(shape)
            return True
        except MorelloError:
            return False

    def buffer_index(self, shape: Sequence[int], point: Sequence[int]) -> int:
        """buffer_indexing_expr (layout.rs:221-272) evaluated at a logical point."""
        arr = (C.c_uint32 * len(shape))(*shape)
        pt = (C.c_uint32 * len(point))(*point)
        lc = self.to_c()
        idx = int(B.load().mrl_layout_buffer_index(C.byref(lc), arr, len(shape), pt))
        if idx < 0:
            raise MorelloError(2, "buffer_index")
        return idx

    def __eq__(self, other):
        return isinstance(other, Layout) and self.dims == other.dims

    def __repr__(self):
        def one(d, pd):
            return f"{d}" if pd.kind == 0 else f"{d} {'p' if pd.kind == 1 else 'oe'}({pd.size})"
        return "layout![" + ", ".join(one(d, pd) for d, pd in self.dims) + "]"


def layout(*dims) -> Layout:
    """The `layout!` macro (layout.rs:1283-1302): ints are Dynamic dims, `(d, Packed(n))` or
    `(d, OddEven(n))` tuples are packed dims."""
    out = []
    for d in dims:
        out.append((d, Dynamic) if isinstance(d, int) else (d[0], d[1]))
    return Layout(out)


def _ctor(name: str, shape: Sequence[int]) -> Layout:
    arr = (C.c_uint32 * len(shape))(*shape)
    out = B.LayoutC()
    _check(getattr(B.load(), name)(arr, len(shape), C.byref(out)), name)
    return Layout.from_c(out)


def row_major(shape):
    return _ctor("mrl_layout_row_major", shape)


def col_major(shape):
    return _ctor("mrl_layout_col_major", shape)


def batched_col_major(shape):
    return _ctor("mrl_layout_batched_col_major", shape)


def nhwc(shape):
    return _ctor("mrl_layout_nhwc", shape)


class SpecKind(enum.IntEnum):
    Matmul = 0
    Conv = 1
    Softmax = 2
    ComposeMSM = 3
    Move = 4
    Fill = 5
    Max = 6
    SoftmaxDenominator = 7
    SoftmaxDenominatorAndMax = 8
    SoftmaxDenominatorAndMaxFromParts = 9
    SoftmaxDenominatorAndUnscaled = 10
    SoftmaxDenominatorAndUnscaledFromMax = 11
    SoftmaxComplete = 12
    DivideVec = 13
    DivideVecScalar = 14
    Broadcast = 15
    OnePrefix = 16


class FillValue(enum.IntEnum):
    """morello/src/spec.rs:165-170."""
    Zero = 0
    NegInf = 1
    Min = 2


class OperandDirection(enum.IntEnum):
    """morello/src/spec.rs:1091-1095."""
    In = 0
    Out = 1
    InOut = 2


class Spec:
    """A logical Spec plus one (dtype, layout) per parameter (spec.rs:33-56, tensorspec.rs:19-32).

    `layouts=None` means row-major for every parameter, except Conv where it means NHWC
    image/output and KRSC filters.
    """

    def __init__(self, kind: SpecKind, spec_shape, dtypes, layouts=None, accum=False, scan_dim=0):
        self.kind = SpecKind(kind)
        self.spec_shape = [int(x) for x in spec_shape]
        self.dtypes = [Dtype(d) for d in dtypes]
        self.accum = bool(accum)
        self.scan_dim = int(scan_dim)
        self._c = B.SpecC()
        self._c.kind = int(self.kind)
        self._c.accum = int(self.accum)
        self._c.scan_dim = self.scan_dim
        if len(self.spec_shape) > B.MAX_SPEC_RANK or len(self.dtypes) > B.MAX_PARAMS:
            raise ValueError("spec_shape or dtypes too long")
        self._c.rank = len(self.spec_shape)
        for i, v in enumerate(self.spec_shape):
            self._c.spec_shape[i] = v
        self._c.n_params = len(self.dtypes)
        for i, d in enumerate(self.dtypes):
            self._c.dtypes[i] = int(d)
        if layouts is None:
            layouts = [None] * len(self.dtypes)
        self.layouts = []
        for i, l in enumerate(layouts):
            if l is None:
                shp = self.parameter_shape(i)
                l = nhwc(shp) if self.kind == SpecKind.Conv else row_major(shp)
            self.layouts.append(l)
            self._c.layouts[i] = l.to_c()

    # -- reference-named accessors ---------------------------------------------------
    def parameter_shape(self, idx: int):
        out = (C.c_uint32 * B.MAX_RANK)()
        rank = C.c_uint32()
        _check(B.load().mrl_spec_parameter_shape(C.byref(self._c), idx, out, C.byref(rank)),
               "parameter_shape")
        return [int(out[i]) for i in range(rank.value)]

    def parameter_shapes(self):
        return [self.parameter_shape(i) for i in range(len(self.dtypes))]

    def operand_directions(self):
        lib = B.load()
        return [OperandDirection(lib.mrl_spec_parameter_direction(C.byref(self._c), i))
                for i in range(len(self.dtypes))]

    def bytes_used(self, idx: int) -> int:
        return int(B.load().mrl_spec_parameter_bytes(C.byref(self._c), idx))

    def flops(self) -> int:
        return int(B.load().mrl_spec_ops(C.byref(self._c)))

    def check(self) -> int:
        return int(B.load().mrl_spec_check(C.byref(self._c)))

    def workspace_bytes(self) -> int:
        return int(B.load().mrl_spec_workspace_bytes(C.byref(self._c)))

    def plan(self) -> "Plan":
        """The kernels a run would launch and the cost model's prediction (no GPU needed)."""
        return _plan_of(B.load().mrl_spec_plan, self._c, "mrl_spec_plan")

    # -- execution -------------------------------------------------------------------
    def run_device(self, ptrs: Sequence[int]):
        """`ptrs`: device pointers in Spec parameter order.  Synchronous."""
        arr = (C.c_void_p * len(ptrs))(*ptrs)
        _check(B.load().mrl_run(C.byref(self._c), arr), "mrl_run")

    def run_async(self, ptrs: Sequence[int], stream: "Stream"):
        """Enqueues the Spec on `stream` and returns; `stream.synchronize()` waits for it."""
        arr = (C.c_void_p * len(ptrs))(*ptrs)
        _check(B.load().mrl_run_async(C.byref(self._c), arr, stream.handle), "mrl_run_async")

    def run_noalloc(self, ptrs: Sequence[int], stream: "Stream | None" = None):
        """As run_async without any device allocation: scratch comes from the library's fixed
        per-GPU array (NOALLOC_SCRATCH_BYTES); MorelloError (tensor too large) if the Spec needs more."""
        arr = (C.c_void_p * len(ptrs))(*ptrs)
        _check(B.load().mrl_run_noalloc(C.byref(self._c), arr, stream.handle if stream else None), "mrl_run_noalloc")

    def run_host(self, *arrays: np.ndarray):
        """`arrays`: numpy buffers in Spec parameter order, each already laid out by its
        parameter's layout; the output array is written in place."""
        if len(arrays) != len(self.dtypes):
            raise ValueError("one array per parameter")
        for i, a in enumerate(arrays):
            if not a.flags["C_CONTIGUOUS"] or a.nbytes != self.bytes_used(i):
                raise ValueError(f"parameter {i}: need a contiguous buffer of {self.bytes_used(i)} bytes")
        arr = (C.c_void_p * len(arrays))(*[a.ctypes.data for a in arrays])
        _check(B.load().mrl_run_host(C.byref(self._c), arr), "mrl_run_host")

    def run_timed(self, ptrs: Sequence[int], steps: int) -> float:
        """`steps` back-to-back launches between two HIP events; total device milliseconds."""
        arr = (C.c_void_p * len(ptrs))(*ptrs)
        ms = C.c_double()
        _check(B.load().mrl_run_timed(C.byref(self._c), arr, steps, C.byref(ms)), "mrl_run_timed")
        return ms.value

    # -- scheduling sugar (scheduling_sugar.rs:37-132), the subset with a knob in the kernels
    def available_schedules(self, with_staging: bool = False):
        """[(tile_m, tile_n, split_k)] the matrix-core Matmul kernel is built for; with_staging:
        [(tile_m, tile_n, split_k, Staging)], the explicitly staged variants included."""
        buf = (B.MatmulScheduleC * 16)()
        n = min(B.load().mrl_matmul_schedules(C.byref(self._c), buf, 16), 16)
        if with_staging:
            return [(buf[i].tile_m, buf[i].tile_n, buf[i].split_k, Staging(buf[i].staging)) for i in range(n)]
        return [(buf[i].tile_m, buf[i].tile_n, buf[i].split_k) for i in range(n) if buf[i].staging == 0]

    def search_schedule(self) -> "ScheduledMatmul":
        """The manual schedule the cost model predicts cheapest (host only)."""
        sched, cost = B.MatmulScheduleC(), C.c_double()
        _check(B.load().mrl_matmul_search_schedule(C.byref(self._c), C.byref(sched), C.byref(cost)),
               "mrl_matmul_search_schedule")
        return ScheduledMatmul(self, sched.tile_m, sched.tile_n, sched.split_k, Staging(sched.staging))

    def actions(self) -> "list[Action]":
        """Target::actions for this Spec (target/mod.rs:69): the lowerings the backend can run,
        each priced by the cost model (host only)."""
        buf = (B.ActionC * 32)()
        n = B.load().mrl_target_actions(C.byref(self._c), buf, 32)
        return [Action(self, buf[i]) for i in range(min(n, 32))]

    def tile_out(self, tile_shape: Sequence[int]) -> "ScheduledMatmul":
        """`spec.tile_out([1, m, n])`: one workgroup per m x n tile of the output."""
        if self.kind != SpecKind.Matmul or len(tile_shape) != 3 or tile_shape[0] != 1:
            raise MorelloError(1, "tile_out")
        return ScheduledMatmul(self, int(tile_shape[1]), int(tile_shape[2]), None)

    def bench(self, ptrs: Sequence[int], iters: int, repeats: int = 10):
        """CodeGen::bench protocol (codegen/mod.rs:133-169): (best, mean) ns per launch."""
        arr = (C.c_void_p * len(ptrs))(*ptrs)
        best, mean = C.c_double(), C.c_double()
        _check(B.load().mrl_bench(C.byref(self._c), arr, iters, repeats, C.byref(best), C.byref(mean)),
               "mrl_bench")
        return best.value, mean.value


class Staging(enum.IntEnum):
    """How the k loop brings operand tiles to the matrix cores: the GPU counterpart of a CPU
    schedule's move_param steps (mrl_staging)."""
    Default = 0
    Registers = 1      # A, B: HBM -> VGPR -> LDS, two LDS stages, eight waves
    DirectB = 2        # B: HBM -> LDS directly, three slots; eight waves of 128 x 64
    DirectBWide = 3    # the same on four waves of 128 x 128, one per SIMD


class ScheduledMatmul:
    """A Matmul Spec under a manual schedule: `spec.tile_out([1, m, n]).split(k)`, optionally
    `.staged(Staging.X)` for the move_param steps."""

    def __init__(self, spec: Spec, tile_m: int, tile_n: int, split_k: Optional[int], staging: "Staging" = Staging.Default):
        self.spec, self.tile_m, self.tile_n, self.split_k, self.staging = spec, tile_m, tile_n, split_k, Staging(staging)

    def split(self, k: int) -> "ScheduledMatmul":
        return ScheduledMatmul(self.spec, self.tile_m, self.tile_n, int(k), self.staging)

    def staged(self, staging: "Staging") -> "ScheduledMatmul":
        return ScheduledMatmul(self.spec, self.tile_m, self.tile_n, self.split_k, staging)

    def plan(self) -> "Plan":
        if self.split_k is None:
            raise MorelloError(1, "schedule needs .split(k)")
        sched = B.MatmulScheduleC(self.tile_m, self.tile_n, self.split_k, int(self.staging))
        fn = lambda spec, head, steps, cap: B.load().mrl_matmul_scheduled_plan(spec, C.byref(sched), head, steps, cap)
        return _plan_of(fn, self.spec._c, "mrl_matmul_scheduled_plan")

    def run_timed(self, ptrs: Sequence[int], steps: int) -> float:
        """Host-clock milliseconds for `steps` launches of this schedule, queue drained."""
        import time
        if self.split_k is None:
            raise MorelloError(1, "schedule needs .split(k)")
        sched = B.MatmulScheduleC(self.tile_m, self.tile_n, self.split_k, int(self.staging))
        arr = (C.c_void_p * len(ptrs))(*ptrs)
        lib = B.load()
        synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            _check(lib.mrl_run_matmul_scheduled(C.byref(self.spec._c), arr, C.byref(sched), None),
                   "mrl_run_matmul_scheduled")
        synchronize()
        return (time.perf_counter() - t0) * 1e3

    def run_device(self, ptrs: Sequence[int]):
        if self.split_k is None:
            raise MorelloError(1, "schedule needs .split(k)")
        sched = B.MatmulScheduleC(self.tile_m, self.tile_n, self.split_k, int(self.staging))
        arr = (C.c_void_p * len(ptrs))(*ptrs)
        _check(B.load().mrl_run_matmul_scheduled(C.byref(self.spec._c), arr, C.byref(sched), None),
               "mrl_run_matmul_scheduled")
        synchronize()


def Matmul(spec_shape, dtypes, layouts=None, accum=False) -> Spec:
    """Matmul{accum} with spec_shape [b, m, k, n] (spec.rs:480-485)."""
    return Spec(SpecKind.Matmul, spec_shape, dtypes, layouts, accum)


def MatmulAccum(spec_shape, dtypes, layouts=None) -> Spec:
    return Matmul(spec_shape, dtypes, layouts, accum=True)


def Conv(spec_shape, dtypes, layouts=None, accum=False) -> Spec:
    """Conv{accum} with spec_shape [b, f, c, oh, ow, fh, fw] (spec.rs:486-498)."""
    return Spec(SpecKind.Conv, spec_shape, dtypes, layouts, accum)


def Softmax(shape, scan_dim, layouts=None) -> Spec:
    """Softmax{scan_dim} on an f32 tensor (spec.rs:86-90, 523-526)."""
    return Spec(SpecKind.Softmax, shape, [f32, f32], layouts, scan_dim=scan_dim)


def ComposeMSM(b, m, k, n2, n, dtypes=(bf16, bf16, bf16, f32), layouts=None) -> Spec:
    """Compose [Matmul, Softmax{2}, Matmul] with external parameters [V, Q, KT, out]
    (spec.rs:3329-3365; examples/matmul_chain.rs:26-57)."""
    return Spec(SpecKind.ComposeMSM, [b, m, k, n2, n], dtypes, layouts)


def Move(shape, dtypes, layouts=None) -> Spec:
    """Move Spec: copy `in` to `out`, which may differ in layout and dtype (Rust `as`
    conversion; oracle: assign_cast in morello/src/verification.rs)."""
    return Spec(SpecKind.Move, shape, dtypes, layouts)


def Fill(shape, dtype, value: FillValue, layout=None) -> Spec:
    """Fill{value} (spec.rs:143-147): one Out parameter set to zero, -inf or the dtype's minimum."""
    return Spec(SpecKind.Fill, shape, [dtype], [layout], scan_dim=int(FillValue(value)))


def Max(shape, dim, layouts=None, accum=False) -> Spec:
    """Max{dim, accum} (spec.rs:142): params [in, out (size one on dim)], f32."""
    return Spec(SpecKind.Max, shape, [f32] * 2, layouts, accum, dim)


def SoftmaxDenominator(shape, scan_dim, layouts=None, accum=False) -> Spec:
    """params [in, max, denom]: denom (+)= sum exp(in - max) (spec.rs:91-95)."""
    return Spec(SpecKind.SoftmaxDenominator, shape, [f32] * 3, layouts, accum, scan_dim)


def SoftmaxDenominatorAndMax(shape, scan_dim, layouts=None, accum=False) -> Spec:
    """params [in, max, denom]: the online (max, denominator) pair (spec.rs:96-101)."""
    return Spec(SpecKind.SoftmaxDenominatorAndMax, shape, [f32] * 3, layouts, accum, scan_dim)


def SoftmaxDenominatorAndMaxFromParts(shape, scan_dim, layouts=None, accum=False) -> Spec:
    """params [tile_max, tile_denom, out_max, out_denom]: merges per-tile (max, denominator)
    pairs listed along scan_dim (spec.rs:102-132)."""
    return Spec(SpecKind.SoftmaxDenominatorAndMaxFromParts, shape, [f32] * 4, layouts, accum, scan_dim)


def SoftmaxDenominatorAndUnscaled(shape, scan_dim, layouts=None) -> Spec:
    """params [in, denom, unscaled] (spec.rs:133-136)."""
    return Spec(SpecKind.SoftmaxDenominatorAndUnscaled, shape, [f32] * 3, layouts, False, scan_dim)


def SoftmaxDenominatorAndUnscaledFromMax(shape, scan_dim, layouts=None, accum=False) -> Spec:
    """params [in, max, denom, unscaled] (spec.rs:137-141)."""
    return Spec(SpecKind.SoftmaxDenominatorAndUnscaledFromMax, shape, [f32] * 4, layouts, accum, scan_dim)


def SoftmaxComplete(shape, scan_dim, layouts=None) -> Spec:
    """params [in, max, denom, out]: out = exp(in - max) / denom (spec.rs:86-90)."""
    return Spec(SpecKind.SoftmaxComplete, shape, [f32] * 4, layouts, False, scan_dim)


def DivideVec(shape, layouts=None) -> Spec:
    """params [numer (InOut), denom], same shape (spec.rs:76)."""
    return Spec(SpecKind.DivideVec, shape, [f32] * 2, layouts)


def DivideVecScalar(shape, scan_dim, layouts=None) -> Spec:
    """params [numer (InOut), denom (size one on scan_dim)] (spec.rs:77-85)."""
    return Spec(SpecKind.DivideVecScalar, shape, [f32] * 2, layouts, False, scan_dim)


def Broadcast(shape, dim, dtype=f32, layouts=None) -> Spec:
    """Broadcast{dim} (spec.rs:70-75): params [in (size one on dim), out]."""
    return Spec(SpecKind.Broadcast, shape, [dtype] * 2, layouts, False, dim)


def OnePrefix(shape, dtype=f32, layouts=None) -> Spec:
    """OnePrefix (spec.rs:59, 469-479): params [in[shape], out[1, *shape]]."""
    return Spec(SpecKind.OnePrefix, shape, [dtype] * 2, layouts)


class Compose:
    """LogicalSpec::Compose (spec.rs:39-45, 1519-1590): `components` are Specs listed
    last-executed first, each consuming the output of the one listed after it as its first
    input.  External parameters follow compose_parameter_visit (spec.rs:3329-3365).
    `layouts`: one per external parameter, None = row-major."""

    def __init__(self, components: Sequence[Spec], layouts=None):
        self.components = list(components)
        self._c = B.ComposeC()
        if len(self.components) > B.MAX_COMPONENTS:
            raise ValueError("too many components")
        self._c.n_components = len(self.components)
        for i, comp in enumerate(self.components):
            cc = self._c.components[i]
            cc.kind, cc.accum, cc.scan_dim = int(comp.kind), int(comp.accum), comp.scan_dim
            cc.rank, cc.n_params = len(comp.spec_shape), len(comp.dtypes)
            for d, v in enumerate(comp.spec_shape):
                cc.spec_shape[d] = v
            for p, dt in enumerate(comp.dtypes):
                cc.dtypes[p] = int(dt)
        _check(B.load().mrl_compose_init(C.byref(self._c)), "mrl_compose_init")
        self.n_params = int(self._c.n_params)
        if layouts is not None:
            if len(layouts) != self.n_params:
                raise ValueError("one layout per external parameter")
            for i, l in enumerate(layouts):
                if l is not None:
                    self._c.layouts[i] = l.to_c()

    def bufferize(self, index: int) -> "Compose":
        """`spec.bufferize(index, GL, row_major)` (scheduling/bufferize.rs:24-116): the tensor
        feeding component `index` is materialised in device memory instead of staying inside a
        fused kernel.  Returns a new Compose; the knob accumulates."""
        if not 0 <= index < len(self.components) - 1:
            raise MorelloError(3, "bufferize")
        import copy
        other = copy.copy(self)
        other._c = B.ComposeC.from_buffer_copy(self._c)
        other._c.bufferize_mask |= 1 << index
        return other

    def parameter(self, idx: int):
        """(component index, component parameter index) of external parameter `idx`."""
        comp, par = C.c_uint32(), C.c_uint32()
        _check(B.load().mrl_compose_parameter(C.byref(self._c), idx, C.byref(comp), C.byref(par)),
               "mrl_compose_parameter")
        return comp.value, par.value

    def parameter_shape(self, idx: int):
        out = (C.c_uint32 * B.MAX_RANK)()
        rank = C.c_uint32()
        _check(B.load().mrl_compose_parameter_shape(C.byref(self._c), idx, out, C.byref(rank)),
               "mrl_compose_parameter_shape")
        return [int(out[i]) for i in range(rank.value)]

    def parameter_shapes(self):
        return [self.parameter_shape(i) for i in range(self.n_params)]

    def parameter_dtypes(self):
        lib = B.load()
        return [Dtype(lib.mrl_compose_parameter_dtype(C.byref(self._c), i)) for i in range(self.n_params)]

    def plan(self) -> "Plan":
        return _plan_of(B.load().mrl_compose_plan, self._c, "mrl_compose_plan")

    def run_device(self, ptrs: Sequence[int]):
        arr = (C.c_void_p * len(ptrs))(*ptrs)
        _check(B.load().mrl_run_compose(C.byref(self._c), arr, None), "mrl_run_compose")
        synchronize()


class PlanStep:
    """One planned launch: `kernel` (with its template arguments in brackets), `family` (the name before them),
    grid, block, LDS bytes, the bounding unit, declared ops / bytes and the predicted ns."""
    UNITS = ("hbm", "mfma_i8", "mfma_bf16", "mfma_f32", "valu")

    def __init__(self, c: B.PlanStepC):
        self.kernel = c.kernel.decode()
        self.family = self.kernel.split(" [")[0]
        self.grid, self.block = tuple(c.grid), tuple(c.block)
        self.lds_bytes, self.unit = int(c.lds_bytes), self.UNITS[c.unit]
        self.ops, self.bytes, self.cost_ns = c.ops, c.bytes, c.cost_ns

    def __repr__(self):
        return f"{self.kernel} grid={self.grid} block={self.block} {self.unit} {self.cost_ns:.0f} ns"


class Plan:
    """Kernel::applies_to_logical_spec / main_cost / memory_allocated (target/mod.rs:103-109) of
    the backend for one Spec: `steps`, `cost_ns` (their sum) and `scratch_bytes`."""

    def __init__(self, steps, cost_ns: float, scratch_bytes: int):
        self.steps, self.cost_ns, self.scratch_bytes = steps, cost_ns, scratch_bytes

    @property
    def kernels(self):
        return [s.family for s in self.steps]

    def __repr__(self):
        return f"Plan({self.cost_ns:.0f} ns, scratch {self.scratch_bytes} B, {self.steps})"


class ActionKind(enum.IntEnum):
    Select = 0
    TileOutSplit = 1
    Fused = 2
    SpatialSplit = 3
    Unfold = 4
    Bufferize = 5
    Generic = 6
    ToSoftmaxParts = 7
    ToSoftmaxPartsRecompute = 8
    ParallelSoftmax = 9
    ToAccum = 10
    MoveRelayout = 11
    Cast = 12
    ToMaxAndDenominator = 13
    ToMaxAndUnscaled = 14
    BroadcastFirst = 15


class Action:
    """One lowering of a Spec (mrl_action): what it is, what the cost model says of it, and a way
    to run the Spec under it."""

    def __init__(self, spec: "Spec", c: B.ActionC):
        self.spec = spec
        self._c = B.ActionC(c.kind, c.tile_m, c.tile_n, c.split_k, c.parts, c.staging, c.n_steps, c.scratch_bytes, c.cost_ns)
        self.kind = ActionKind(c.kind)
        self.tile_m, self.tile_n, self.split_k, self.parts = c.tile_m, c.tile_n, c.split_k, c.parts
        self.staging = Staging(c.staging)
        self.n_steps, self.scratch_bytes, self.cost_ns = c.n_steps, int(c.scratch_bytes), c.cost_ns

    def __repr__(self):
        knobs = {ActionKind.TileOutSplit: f" tile {self.tile_m}x{self.tile_n} split {self.split_k}" + (f" {self.staging.name}" if self.staging else ""),
                 ActionKind.SpatialSplit: f" tile {self.tile_m}x{self.tile_n}",
                 ActionKind.Fused: (f" rows {self.tile_m}" if self.tile_m else "") + (f" parts {self.parts}" if self.parts else ""),
                 ActionKind.ParallelSoftmax: f" parts {self.parts}",
                 ActionKind.MoveRelayout: f" parameter {self.tile_m}",
                 ActionKind.Cast: f" parameter {self.tile_m} to {Dtype(self.tile_n) if self.kind == ActionKind.Cast else ''}",
                 }.get(self.kind, "")
        return f"Action({self.kind.name}{knobs}: {self.cost_ns:.0f} ns, {self.n_steps} launches, scratch {self.scratch_bytes} B)"

    def plan(self) -> "Plan":
        head, cap = B.PlanC(), 64
        steps = (B.PlanStepC * cap)()
        _check(B.load().mrl_action_plan(C.byref(self.spec._c), C.byref(self._c), C.byref(head), steps, cap), "mrl_action_plan")
        return Plan([PlanStep(steps[i]) for i in range(min(cap, head.n_steps))], head.cost_ns, int(head.scratch_bytes))

    def run_device(self, ptrs: Sequence[int]):
        arr = (C.c_void_p * len(ptrs))(*ptrs)
        _check(B.load().mrl_run_action(C.byref(self.spec._c), arr, C.byref(self._c), None), "mrl_run_action")
        synchronize()

    def run_timed(self, ptrs: Sequence[int], steps: int) -> float:
        """`steps` back-to-back launches of this action between two HIP events; total device milliseconds."""
        arr = (C.c_void_p * len(ptrs))(*ptrs)
        ms = C.c_double()
        _check(B.load().mrl_run_action_timed(C.byref(self.spec._c), arr, C.byref(self._c), steps, C.byref(ms)),
               "mrl_run_action_timed")
        return ms.value

    def apply(self) -> "Rewrite":
        """The action's children (ActionT::apply, scheduling/mod.rs:40-63): for a rewrite, the
        sub-Specs it turns the Spec into, in execution order, with each parameter's source, and
        the sizes of the buffers between them; for a leaf, none."""
        c = B.RewriteC()
        _check(B.load().mrl_action_apply(C.byref(self.spec._c), C.byref(self._c), C.byref(c)), "mrl_action_apply")
        subs = []
        for i in range(c.n_subspecs):
            sc = c.subspecs[i].spec
            sub = Spec(SpecKind(sc.kind), list(sc.spec_shape[:sc.rank]), [Dtype(sc.dtypes[j]) for j in range(sc.n_params)],
                       layouts=[Layout.from_c(sc.layouts[j]) for j in range(sc.n_params)], accum=bool(sc.accum), scan_dim=sc.scan_dim)
            subs.append((sub, [int(c.subspecs[i].source[j]) for j in range(sc.n_params)]))
        return Rewrite(subs, [int(c.intermediate_bytes[j]) for j in range(c.n_intermediates)])

    def flops(self) -> float:
        return self.spec.flops()

    def bytes_used(self, i: int) -> int:
        return self.spec.bytes_used(i)


class Rewrite:
    """What Action.apply returns: `subspecs` = [(Spec, sources)], a source i >= 0 naming parameter i
    of the Spec the action was applied to and -1 - j the j-th of `intermediate_bytes`."""

    def __init__(self, subspecs, intermediate_bytes):
        self.subspecs, self.intermediate_bytes = subspecs, intermediate_bytes

    def is_leaf(self) -> bool:
        return not self.subspecs

    def run_device(self, ptrs: Sequence[int]):
        """Runs the sub-Specs one after the other with mrl_run, each on the buffers its sources name."""
        between = [DeviceBuffer(n) for n in self.intermediate_bytes]
        try:
            for sub, sources in self.subspecs:
                sub.run_device([ptrs[i] if i >= 0 else between[-1 - i].ptr for i in sources])
        finally:
            for b in between:
                b.free()


def _plan_of(fn, c_spec, where: str) -> Plan:
    head, cap = B.PlanC(), 64
    steps = (B.PlanStepC * cap)()
    _check(fn(C.byref(c_spec), C.byref(head), steps, cap), where)
    return Plan([PlanStep(steps[i]) for i in range(min(cap, head.n_steps))], head.cost_ns, int(head.scratch_bytes))


class TargetMemory:
    def __init__(self, c: B.TargetMemoryC):
        self.name = c.name.decode()
        self.is_addressed, self.can_parallel_tile = bool(c.is_addressed), bool(c.can_parallel_tile)
        self.counts_registers, self.has_layout = bool(c.counts_registers), bool(c.has_layout)
        self.vector_bytes = [v for v in c.vector_bytes if v]
        self.limit, self.cache_hit_cost = int(c.limit), int(c.cache_hit_cost)


class Target:
    """The backend as morello's `Target` trait sees it (target/mod.rs:37-78)."""

    @staticmethod
    def target_id() -> str:
        return B.load().mrl_target_id().decode()

    @staticmethod
    def line_size() -> int:
        return int(B.load().mrl_target_line_size())

    @staticmethod
    def processors() -> int:
        return int(B.load().mrl_target_processors())

    @staticmethod
    def memories():
        buf = (B.TargetMemoryC * 4)()
        n = B.load().mrl_target_memories(buf, 4)
        return [TargetMemory(buf[i]) for i in range(n)]

    @staticmethod
    def default_memory() -> "TargetMemory":
        return Target.memories()[B.load().mrl_target_default_memory()]

    @staticmethod
    def possible_destination_memories(slower: str):
        names = [m.name for m in Target.memories()]
        buf = (C.c_uint32 * 4)()
        n = B.load().mrl_target_destination_memories(names.index(slower), buf, 4)
        return [names[buf[i]] for i in range(n)]

    @staticmethod
    def all_layouts_for_shape(shape: Sequence[int], dtype: "Dtype"):
        arr = (C.c_uint32 * len(shape))(*shape)
        n = B.load().mrl_target_layouts_for_shape(arr, len(shape), int(dtype), None, 0)
        buf = (B.LayoutC * n)()
        B.load().mrl_target_layouts_for_shape(arr, len(shape), int(dtype), buf, n)
        return [Layout.from_c(buf[i]) for i in range(n)]

    move_destination_layouts = all_layouts_for_shape

    @staticmethod
    def kernels():
        buf = (C.c_char_p * 64)()
        n = B.load().mrl_target_kernels(buf, 64)
        return [buf[i].decode() for i in range(n)]


class Stream:
    """A HIP stream owned by Python; plumbing for asynchronous launches."""

    def __init__(self):
        h = C.c_void_p()
        _check(B.load().mrl_stream_create(C.byref(h)), "mrl_stream_create")
        self.handle = h

    def synchronize(self):
        _check(B.load().mrl_stream_synchronize(self.handle), "mrl_stream_synchronize")

    def destroy(self):
        if self.handle:
            B.load().mrl_stream_destroy(self.handle)
            self.handle = None


def device_free_bytes() -> int:
    """Device memory that is not allocated at the moment."""
    n = C.c_size_t()
    _check(B.load().mrl_device_mem_free(C.byref(n)), "mrl_device_mem_free")
    return n.value


def release_stream(stream=None) -> None:
    """Waits for a caller-owned HIP stream (an integer or ctypes handle; None = the default
    stream) and frees the scratch arena the library kept for it."""
    handle = stream.handle if isinstance(stream, Stream) else C.c_void_p(stream or 0)
    _check(B.load().mrl_stream_release(handle), "mrl_stream_release")


class DeviceBuffer:
    """A device allocation owned by Python; plumbing for tests and the benchmark."""

    def __init__(self, nbytes: int):
        self.nbytes = int(nbytes)
        p = C.c_void_p()
        _check(B.load().mrl_device_malloc(C.byref(p), self.nbytes), "mrl_device_malloc")
        self.ptr = p.value

    @staticmethod
    def from_numpy(a: np.ndarray) -> "DeviceBuffer":
        a = np.ascontiguousarray(a)
        buf = DeviceBuffer(a.nbytes)
        _check(B.load().mrl_memcpy_h2d(buf.ptr, a.ctypes.data, a.nbytes), "mrl_memcpy_h2d")
        return buf

    def to_numpy(self, dtype, shape) -> np.ndarray:
        out = np.empty(shape, dtype=dtype)
        assert out.nbytes <= self.nbytes
        _check(B.load().mrl_memcpy_d2h(out.ctypes.data, self.ptr, out.nbytes), "mrl_memcpy_d2h")
        return out

    def zero(self):
        _check(B.load().mrl_memset(self.ptr, 0, self.nbytes), "mrl_memset")

    def free(self):
        if self.ptr:
            B.load().mrl_device_free(self.ptr)
            self.ptr = None

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


def init(device: int = 0):
    _check(B.load().mrl_init(device), "mrl_init")


def measure_mfma_rate(kind: str, random_operands: bool, iters: int = 20000) -> float:
    """Operations per second the matrix cores sustain on register operands: `kind` "int8" or
    "bf16"; all-zero operands (near the datasheet rate) or benchmark-like random ones (the
    rate at the board's power limit)."""
    out = C.c_double()
    _check(B.load().mrl_measure_mfma_rate({"int8": 0, "bf16": 1}[kind], int(random_operands), iters,
                                          C.byref(out)), "mrl_measure_mfma_rate")
    return out.value


def launch_count() -> int:
    """Kernels this thread has launched through the library so far."""
    return int(B.load().mrl_launch_count())


def synchronize():
    _check(B.load().mrl_device_synchronize(), "mrl_device_synchronize")


NOALLOC_SCRATCH_BYTES = 32 << 20   # MRL_NOALLOC_SCRATCH_BYTES


def device_info():
    name = C.create_string_buffer(256)
    cus, khz, mem = C.c_int(), C.c_int(), C.c_size_t()
    _check(B.load().mrl_device_info(name, 256, C.byref(cus), C.byref(khz), C.byref(mem)), "mrl_device_info")
    return {"name": name.value.decode(), "compute_units": cus.value, "clock_khz": khz.value,
            "total_mem_bytes": mem.value}
