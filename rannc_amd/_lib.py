"""ctypes binding of libranncgrad.so (the C ABI declared in ``include/ranncgrad.h``).

The library is the only compute path: there is no CPU or PyTorch fallback.  If the
shared object is missing every import of this module raises.
"""
from __future__ import annotations

import ctypes as C
import os
from typing import List, Optional, Sequence

HERE = os.path.dirname(os.path.abspath(__file__))
# RANNC_AMD_LIB points at an alternative build of the same library (tuning experiments).
LIB_PATH = os.environ.get("RANNC_AMD_LIB") or os.path.join(HERE, "libranncgrad.so")

RG_OK, RG_EINVAL, RG_EALIGN, RG_EHIP, RG_ENOMEM = 0, 1, 2, 3, 4
RG_F32, RG_F16, RG_BF16 = 0, 1, 2
RG_STEP_DEFAULT, RG_STEP_WRITE_ON_OVERFLOW, RG_STEP_IGNORE_OVERFLOW, RG_STEP_EXPECT_NO_CLIP = 0, 1, 2, 4

DTYPE_CODES = {"f32": RG_F32, "f16": RG_F16, "bf16": RG_BF16}


class StepResult(C.Structure):
    _fields_ = [("norm", C.c_double), ("coef", C.c_float), ("overflow", C.c_int32),
                ("clipped", C.c_int32), ("skipped", C.c_int32)]


class AdamArgs(C.Structure):
    _fields_ = [("lr", C.c_double), ("beta1", C.c_double), ("beta2", C.c_double), ("eps", C.c_double),
                ("weight_decay", C.c_double), ("step", C.c_int64), ("decoupled_weight_decay", C.c_int32),
                ("maximize", C.c_int32), ("grad_scale", C.c_float), ("gate", C.c_void_p)]


class SgdArgs(C.Structure):
    _fields_ = [("lr", C.c_double), ("momentum", C.c_double), ("dampening", C.c_double), ("weight_decay", C.c_double),
                ("nesterov", C.c_int32), ("maximize", C.c_int32), ("first_step", C.c_int32),
                ("grad_scale", C.c_float), ("gate", C.c_void_p)]


# name -> (restype, argtypes); the complete export list of include/ranncgrad.h
_vp, _i, _i64, _f = C.c_void_p, C.c_int, C.c_int64, C.c_float
_pi64, _pi, _pvp = C.POINTER(C.c_int64), C.POINTER(C.c_int), C.POINTER(C.c_void_p)
SIGNATURES = {
    "rg_last_error": (C.c_char_p, []),
    "rg_version": (_i, []),
    "rg_elem_size": (_i, [_i]),
    "rg_aligned_numel": (_i64, [_i64, _i, _i]),
    "rg_segment_layout": (_i, [_i64, _i, _i, _pi64, _pi64, _pi64, _pi64]),
    "rg_bucket_layout": (_i, [_i, _pi64, _pi, _pi64, _pi64]),
    "rg_plan_create": (_i, [C.POINTER(_vp), _i, _i, _pvp, _pvp, _pi64, _pi, _pi, _i64]),
    "rg_plan_update_pointers": (_i, [_vp, _pvp, _pvp, _vp]),
    "rg_plan_destroy": (_i, [_vp]),
    "rg_plan_num_tensors": (_i, [_vp]),
    "rg_plan_num_chunks": (_i64, [_vp]),
    "rg_plan_chunk_elems": (_i64, [_vp]),
    "rg_plan_total_numel": (_i64, [_vp]),
    "rg_plan_set_streaming": (_i, [_vp, _i]),
    "rg_plan_tune": (_i, [_vp, _vp]),
    "rg_plan_write_order": (_i, [_vp]),
    "rg_plan_set_write_order": (_i, [_vp, _i]),
    "rg_fused_step": (_i, [_vp, _f, _f, _i, _vp]),
    "rg_step_begin": (_i, [_vp, _f, _vp]),
    "rg_step_begin_scaled": (_i, [_vp, _vp, _vp]),
    "rg_scaler_init": (_i, [_vp, _vp, _i, _vp]),
    "rg_scaler_update": (_i, [_vp, _vp, _i, _i, _vp]),
    "rg_optim_set_grad_scale_source": (_i, [_vp, _vp]),
    "rg_step_finish": (_i, [_vp, _f, _i, _vp]),
    "rg_step_decide": (_i, [_vp, _f, _i, _vp]),
    "rg_unscale_pack": (_i, [_vp, _f, _vp]),
    "rg_step_apply_clip": (_i, [_vp, _f, _i, _vp]),
    "rg_accumulate": (_i, [_vp, _f, _vp]),
    "rg_unscale_accumulate": (_i, [_vp, _f, _vp]),
    "rg_grad_norm": (_i, [_vp, _vp]),
    "rg_scale_cast": (_i, [_vp, _f, _vp]),
    "rg_scale_cast_single": (_i, [_vp, _vp, _i64, _i, _i, _f, _i, _vp]),
    "rg_fused_step_static": (_i, [_vp, _vp, _i64, _i, _i, _f, _f, _i, _vp, _i, _vp]),
    "rg_zero": (_i, [_vp, _vp]),
    "rg_fill_zero": (_i, [_vp, _i64, _i, _vp]),
    "rg_result_device_ptr": (_i, [_vp, C.POINTER(_vp)]),
    "rg_tensor_norms_device_ptr": (_i, [_vp, C.POINTER(_vp)]),
    "rg_read_result": (_i, [_vp, C.POINTER(StepResult), _vp]),
    "rg_read_tensor_norms": (_i, [_vp, C.POINTER(C.c_float), _vp]),
    "rg_optim_create": (_i, [C.POINTER(_vp), _i, _i, _pvp, _pvp, _pvp, _pvp, _pvp, _pi64, _pi, _pi]),
    "rg_optim_update_pointers": (_i, [_vp, _pvp, _pvp, _pvp, _pvp, _pvp, _vp]),
    "rg_optim_destroy": (_i, [_vp]),
    "rg_adam_step": (_i, [_vp, C.POINTER(AdamArgs), _vp]),
    "rg_adam_step_clocked": (_i, [_vp, C.POINTER(AdamArgs), _vp, _vp]),
    "rg_adam_clock_advance": (_i, [_vp, C.c_double, C.c_double, C.c_double, _vp, _i, _vp]),
    "rg_sgd_step": (_i, [_vp, C.POINTER(SgdArgs), _vp]),
    "rg_plan_enable_timing": (_i, [_vp, _i]),
    "rg_plan_timing_stride": (_i, [_vp, _i]),
    "rg_plan_read_timing": (_i, [_vp, _i, C.POINTER(C.c_float)]),
    "rg_ceiling_kernel": (_i, [_i, _pvp, _i, _i64, _i, _vp]),
}


class RanncGradError(RuntimeError):
    pass


def _load() -> C.CDLL:
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            f"{LIB_PATH} is missing: build it with `python rannc_amd/build.py` "
            "(there is no fallback path)")
    lib = C.CDLL(LIB_PATH)
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    return lib


lib = _load()


def check(rc: int) -> None:
    """Status -> exception, mirroring the reference's pybind translation
    (std::invalid_argument -> ValueError, std::runtime_error -> RuntimeError)."""
    if rc == RG_OK:
        return
    msg = (lib.rg_last_error() or b"").decode("utf-8", "replace")
    if rc in (RG_EINVAL, RG_EALIGN):
        raise ValueError(msg)
    if rc == RG_ENOMEM:
        raise MemoryError(msg)
    raise RanncGradError(msg)


# ------------------------------------------------------------------------- layout

def aligned_numel(numel: int, elem_size: int, split_num: int) -> int:
    r = lib.rg_aligned_numel(numel, elem_size, split_num)
    if r < 0:
        check(RG_EINVAL)
    return int(r)


def segment_layout(numel: int, elem_size: int, nranks: int):
    """-> (aligned_size, segment_size, offsets, src_sizes)."""
    if nranks < 1:
        raise ValueError("nranks must be >= 1")
    aligned, seg = C.c_int64(), C.c_int64()
    offs, srcs = (C.c_int64 * nranks)(), (C.c_int64 * nranks)()
    check(lib.rg_segment_layout(numel, elem_size, nranks, C.byref(aligned), C.byref(seg), offs, srcs))
    return int(aligned.value), int(seg.value), list(offs), list(srcs)


def bucket_layout(numels: Sequence[int], dtype_codes: Sequence[int]):
    """-> (offsets, [len_f32, len_f16, len_bf16])."""
    n = len(numels)
    a_n = (C.c_int64 * max(n, 1))(*numels)
    a_d = (C.c_int * max(n, 1))(*dtype_codes)
    offs = (C.c_int64 * max(n, 1))()
    lens = (C.c_int64 * 3)()
    check(lib.rg_bucket_layout(n, a_n, a_d, offs, lens))
    return list(offs)[:n], list(lens)


# ------------------------------------------------------------------------- plans

class Plan:
    """Owner of one ``rg_plan``.  Pointers are plain integers (``tensor.data_ptr()``)."""

    def __init__(self, device: int, src_ptrs: Sequence[Optional[int]], dst_ptrs: Sequence[Optional[int]],
                 numels: Sequence[int], src_dtypes: Sequence[int], dst_dtypes: Sequence[int],
                 chunk_elems: int = 0):
        n = len(numels)
        if not (len(src_ptrs) == len(dst_ptrs) == len(src_dtypes) == len(dst_dtypes) == n):
            raise ValueError("plan arrays differ in length")
        self._handle = _vp()
        self.n = n
        self.device = device
        m = max(n, 1)
        check(lib.rg_plan_create(
            C.byref(self._handle), device, n,
            (_vp * m)(*[p or None for p in src_ptrs]), (_vp * m)(*[p or None for p in dst_ptrs]),
            (C.c_int64 * m)(*numels), (C.c_int * m)(*src_dtypes), (C.c_int * m)(*dst_dtypes),
            chunk_elems))

    # -- bookkeeping
    def close(self) -> None:
        if getattr(self, "_handle", None) is not None and self._handle.value:
            lib.rg_plan_destroy(self._handle)
            self._handle = _vp()

    def is_open(self) -> bool:
        return bool(getattr(self, "_handle", None) is not None and self._handle.value)

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    @property
    def num_chunks(self) -> int:
        return int(lib.rg_plan_num_chunks(self._handle))

    @property
    def chunk_elems(self) -> int:
        return int(lib.rg_plan_chunk_elems(self._handle))

    @property
    def total_numel(self) -> int:
        return int(lib.rg_plan_total_numel(self._handle))

    def set_streaming(self, mode: int) -> None:
        """1 = nontemporal accesses, 0 = plain, -1 = decide from the plan's size."""
        check(lib.rg_plan_set_streaming(self._handle, mode))

    def tune(self, stream: int = 0) -> int:
        """Measure the block -> XCD orders on the plan's own tensors and keep the fastest (overwrites the
        destinations, waits for the stream).  Returns the order chosen."""
        check(lib.rg_plan_tune(self._handle, _vp(stream)))
        return int(lib.rg_plan_write_order(self._handle))

    @property
    def write_order(self) -> int:
        """Order in which the writing passes hand tiles to the XCDs (0 round robin, n runs of n, -1 eighths)."""
        return int(lib.rg_plan_write_order(self._handle))

    def set_write_order(self, order: int) -> None:
        check(lib.rg_plan_set_write_order(self._handle, order))

    def update_pointers(self, src_ptrs: Optional[Sequence[Optional[int]]],
                        dst_ptrs: Optional[Sequence[Optional[int]]], stream: int = 0) -> None:
        m = max(self.n, 1)
        a_s = (_vp * m)(*[p or None for p in src_ptrs]) if src_ptrs is not None else None
        a_d = (_vp * m)(*[p or None for p in dst_ptrs]) if dst_ptrs is not None else None
        check(lib.rg_plan_update_pointers(self._handle, a_s, a_d, _vp(stream)))

    # -- operations (all stream ordered)
    def fused_step(self, inv_scale: float, max_norm: float, flags: int = RG_STEP_DEFAULT, stream: int = 0) -> None:
        check(lib.rg_fused_step(self._handle, inv_scale, max_norm, flags, _vp(stream)))

    def step_begin(self, inv_scale: float, stream: int = 0) -> None:
        check(lib.rg_step_begin(self._handle, inv_scale, _vp(stream)))

    def step_begin_scaled(self, inv_scale_ptr: int, stream: int = 0) -> None:
        """``step_begin`` with ``inv_scale`` read by the kernels from device memory (a scaler state's ``inv_scale``)."""
        check(lib.rg_step_begin_scaled(self._handle, _vp(inv_scale_ptr), _vp(stream)))

    def step_finish(self, max_norm: float, flags: int = RG_STEP_DEFAULT, stream: int = 0) -> None:
        check(lib.rg_step_finish(self._handle, max_norm, flags, _vp(stream)))

    def step_decide(self, max_norm: float, flags: int = RG_STEP_DEFAULT, stream: int = 0) -> None:
        check(lib.rg_step_decide(self._handle, max_norm, flags, _vp(stream)))

    def unscale_pack(self, inv_scale: float, stream: int = 0) -> None:
        check(lib.rg_unscale_pack(self._handle, inv_scale, _vp(stream)))

    def step_apply_clip(self, max_norm: float, flags: int = RG_STEP_DEFAULT, stream: int = 0) -> None:
        check(lib.rg_step_apply_clip(self._handle, max_norm, flags, _vp(stream)))

    def accumulate(self, scale: float = 1.0, stream: int = 0) -> None:
        check(lib.rg_accumulate(self._handle, scale, _vp(stream)))

    def unscale_accumulate(self, inv_scale: float, stream: int = 0) -> None:
        check(lib.rg_unscale_accumulate(self._handle, inv_scale, _vp(stream)))

    def grad_norm(self, stream: int = 0) -> None:
        check(lib.rg_grad_norm(self._handle, _vp(stream)))

    def scale_cast(self, scale: float = 1.0, stream: int = 0) -> None:
        check(lib.rg_scale_cast(self._handle, scale, _vp(stream)))

    def zero(self, stream: int = 0) -> None:
        check(lib.rg_zero(self._handle, _vp(stream)))

    # -- results (these wait for the stream)
    def read_result(self, stream: int = 0) -> StepResult:
        out = StepResult()
        check(lib.rg_read_result(self._handle, C.byref(out), _vp(stream)))
        return out

    def read_tensor_norms(self, stream: int = 0) -> List[float]:
        buf = (C.c_float * max(self.n, 1))()
        check(lib.rg_read_tensor_norms(self._handle, buf, _vp(stream)))
        return list(buf)[: self.n]

    def enable_timing(self, slots: int) -> None:
        """slots > 0: bracket all stages of each fused step; < 0: only the write pass; 0: off."""
        check(lib.rg_plan_enable_timing(self._handle, slots))

    def timing_stride(self, stride: int) -> None:
        check(lib.rg_plan_timing_stride(self._handle, stride))

    def read_timing(self, slot: int) -> List[float]:
        """[reduce pass, reduce + decide, write pass, whole step] in milliseconds."""
        ms = (C.c_float * 4)()
        check(lib.rg_plan_read_timing(self._handle, slot, ms))
        return list(ms)

    def result_device_ptr(self) -> int:
        out = _vp()
        check(lib.rg_result_device_ptr(self._handle, C.byref(out)))
        return int(out.value)


def scale_cast_single(src_ptr: Optional[int], dst_ptr: int, numel: int, src_dtype: int, dst_dtype: int,
                      scale: float, device: int, stream: int = 0) -> None:
    check(lib.rg_scale_cast_single(_vp(src_ptr or None), _vp(dst_ptr or None), numel, src_dtype, dst_dtype,
                                   scale, device, _vp(stream)))


RG_STATIC_MAX_NUMEL = 1 << 32


def fused_step_static(src_ptr: int, dst_ptr: int, numel: int, src_dtype: int, dst_dtype: int, inv_scale: float,
                      max_norm: float, flags: int, result_ptr: Optional[int], device: int, stream: int = 0) -> None:
    """The fused step over one tensor pair with no plan and no allocation (``rg_fused_step_static``)."""
    check(lib.rg_fused_step_static(_vp(src_ptr or None), _vp(dst_ptr or None), numel, src_dtype, dst_dtype, inv_scale,
                                   max_norm, flags, _vp(result_ptr or None), device, _vp(stream)))


CEILING_KINDS = {"read": 0, "fill": 1, "copy_f32": 2, "widen_bf16_f32": 3, "adam_streams": 4, "copy_f32_nt": 5}


def ceiling_kernel(kind: int, array_ptrs: Sequence[int], nbytes: int, device: int, stream: int = 0) -> None:
    """One launch of a yardstick kernel (``rg_ceiling_kernel``) over caller-owned device arrays."""
    n = len(array_ptrs)
    check(lib.rg_ceiling_kernel(kind, (_vp * max(n, 1))(*array_ptrs), n, nbytes, device, _vp(stream)))


def fill_zero(ptr: int, nbytes: int, device: int, stream: int = 0) -> None:
    check(lib.rg_fill_zero(_vp(ptr), nbytes, device, _vp(stream)))


# ------------------------------------------------------------------------- optimizer tables

def _ptr_array(ptrs: Optional[Sequence[Optional[int]]], n: int):
    if ptrs is None:
        return None
    if len(ptrs) != n:
        raise ValueError("pointer arrays differ in length")
    return (C.c_void_p * max(n, 1))(*[p if p else None for p in ptrs])


class ScalerState(C.Structure):
    """``rg_scaler_state``: the loss scale and its schedule as they sit in 32 bytes of device memory."""
    _fields_ = [("loss_scale", C.c_float), ("inv_scale", C.c_float), ("unskipped", C.c_int32), ("skipped_steps", C.c_int32),
                ("min_loss_scale", C.c_float), ("max_loss_scale", C.c_float), ("scale_window", C.c_int32),
                ("scale_factor", C.c_float)]


SCALER_STATE_BYTES = C.sizeof(ScalerState)
SCALER_INV_SCALE_OFFSET = ScalerState.inv_scale.offset
RG_SCALER_DYNAMIC, RG_SCALER_TRUNCATE = 1, 2


def scaler_init(state_ptr: int, loss_scale: float, min_loss_scale: float, max_loss_scale: float, scale_window: int,
                scale_factor: float, device: int, stream: int = 0) -> None:
    init = ScalerState(loss_scale, 0.0, 0, 0, min_loss_scale or 0.0, max_loss_scale, scale_window, scale_factor)
    check(lib.rg_scaler_init(_vp(state_ptr), C.byref(init), device, _vp(stream)))


def scaler_update(state_ptr: int, result_ptr: int, flags: int, device: int, stream: int = 0) -> None:
    """One thread applies the loss-scale schedule to the overflow flag of a plan's result block."""
    check(lib.rg_scaler_update(_vp(state_ptr), _vp(result_ptr), flags, device, _vp(stream)))


ADAM_CLOCK_BYTES = 32     # sizeof(rg_adam_clock): int64 step, float neg_step_size, float bias2_sqrt, float step_f32, pad


def adam_clock_advance(clock_ptr: int, lr: float, beta1: float, beta2: float, gate: int, device: int, stream: int = 0) -> None:
    """One thread on the device: the clock's step count + 1 and the factors that depend on it - unless ``gate``
    (a result block's device address, or 0) says the step was skipped."""
    check(lib.rg_adam_clock_advance(_vp(clock_ptr), lr, beta1, beta2, _vp(gate or None), device, _vp(stream)))


class OptimTable:
    """Owner of one ``rg_optim``: parameter / gradient / state / model-copy pointers of the
    tensors one optimizer launch updates."""

    def __init__(self, device: int, params: Sequence[int], grads: Sequence[int], state1: Optional[Sequence[int]],
                 state2: Optional[Sequence[int]], copies: Optional[Sequence[Optional[int]]], numels: Sequence[int],
                 grad_dtypes: Sequence[int], copy_dtypes: Optional[Sequence[int]] = None):
        n = len(numels)
        self._handle = _vp()
        self.n = n
        self.device = device
        a_cd = (C.c_int * max(n, 1))(*(copy_dtypes if copy_dtypes is not None else [RG_F32] * n))
        check(lib.rg_optim_create(C.byref(self._handle), device, n, _ptr_array(params, n), _ptr_array(grads, n),
                                  _ptr_array(state1, n), _ptr_array(state2, n), _ptr_array(copies, n),
                                  (C.c_int64 * max(n, 1))(*numels), (C.c_int * max(n, 1))(*grad_dtypes), a_cd))

    def set_grad_scale_source(self, grad_scale_ptr: int) -> None:
        """Later steps multiply the gradients by the float at this device address instead of ``grad_scale`` (0: off)."""
        check(lib.rg_optim_set_grad_scale_source(self._handle, _vp(grad_scale_ptr or None)))

    @property
    def handle(self) -> int:
        """The ``rg_optim*`` as an integer, for another binding of the same library."""
        return self._handle.value

    def update_pointers(self, params=None, grads=None, state1=None, state2=None, copies=None, stream: int = 0) -> None:
        n = self.n
        check(lib.rg_optim_update_pointers(self._handle, _ptr_array(params, n), _ptr_array(grads, n),
                                           _ptr_array(state1, n), _ptr_array(state2, n), _ptr_array(copies, n),
                                           _vp(stream)))

    def adam_step(self, lr: float, beta1: float, beta2: float, eps: float, weight_decay: float, step: int,
                  decoupled: bool = False, maximize: bool = False, grad_scale: float = 1.0, gate: int = 0,
                  stream: int = 0) -> None:
        a = AdamArgs(lr, beta1, beta2, eps, weight_decay, step, int(decoupled), int(maximize), grad_scale, gate or None)
        check(lib.rg_adam_step(self._handle, C.byref(a), _vp(stream)))

    def adam_step_clocked(self, clock_ptr: int, lr: float, beta1: float, beta2: float, eps: float, weight_decay: float,
                          decoupled: bool = False, maximize: bool = False, grad_scale: float = 1.0, gate: int = 0,
                          stream: int = 0) -> None:
        """``adam_step`` with the step count and the factors that depend on it read from an ``rg_adam_clock`` on
        the device (``adam_clock_advance`` updates it), so that the launch can be replayed from a HIP graph."""
        a = AdamArgs(lr, beta1, beta2, eps, weight_decay, 0, int(decoupled), int(maximize), grad_scale, gate or None)
        check(lib.rg_adam_step_clocked(self._handle, C.byref(a), _vp(clock_ptr), _vp(stream)))

    def sgd_step(self, lr: float, momentum: float = 0.0, dampening: float = 0.0, weight_decay: float = 0.0,
                 nesterov: bool = False, maximize: bool = False, first_step: bool = False, grad_scale: float = 1.0,
                 gate: int = 0, stream: int = 0) -> None:
        a = SgdArgs(lr, momentum, dampening, weight_decay, int(nesterov), int(maximize), int(first_step), grad_scale,
                    gate or None)
        check(lib.rg_sgd_step(self._handle, C.byref(a), _vp(stream)))

    def close(self) -> None:
        if self._handle:
            lib.rg_optim_destroy(self._handle)
            self._handle = _vp()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass
