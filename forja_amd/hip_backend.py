"""ctypes binding of libforja_hip.so: the methods of `forja_core::Backend`
(crates/forja-core/src/backend.rs:650-984) over the C ABI in include/forja_hip.h.

There is no CPU fallback: loading fails loudly when the library is missing, and `HipBackend()`
raises when no gfx950 device is visible.
"""
from __future__ import annotations

import ctypes as C
import os
from typing import List, Optional, Sequence

import numpy as np

from .core import (BackendError, CommandList, DType, Dispatch, Layout, Program, Slice, Status,
                   Tensor)

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libforja_hip.so")

FH_MAX_RANK = 8
FH_MAX_INPUTS = 12
FH_MAX_OUTPUTS = 4


class FhTensor(C.Structure):
    _fields_ = [("buffer", C.c_uint64), ("dtype", C.c_uint32), ("rank", C.c_uint32),
                ("shape", C.c_uint32 * FH_MAX_RANK), ("stride", C.c_uint64 * FH_MAX_RANK),
                ("offset", C.c_uint64)]


class FhInst(C.Structure):
    _fields_ = [("kind", C.c_uint32), ("op", C.c_uint32), ("a", C.c_uint32), ("b", C.c_uint32),
                ("c", C.c_uint32)]


class FhDispatch(C.Structure):
    _fields_ = [("op", C.c_uint32), ("scale", C.c_float), ("eps", C.c_float), ("theta", C.c_float),
                ("bits", C.c_uint32), ("group_size", C.c_uint32), ("k", C.c_uint32),
                ("normalize", C.c_uint32), ("causal", C.c_uint32), ("q_start", C.c_uint32),
                ("key_length", C.c_uint32), ("page_tokens", C.c_uint32), ("direction", C.c_uint32),
                ("start", C.c_uint32), ("n_inputs", C.c_uint32), ("n_outputs", C.c_uint32),
                ("program", C.c_uint64), ("epilogue", C.c_uint64),
                ("accumulator_count", C.c_uint32), ("n_extras", C.c_uint32),
                ("inputs", FhTensor * FH_MAX_INPUTS), ("outputs", FhTensor * FH_MAX_OUTPUTS)]


class FhError(C.Structure):
    _fields_ = [("code", C.c_uint32), ("dispatch", C.c_uint32), ("submission", C.c_uint64),
                ("operation", C.c_uint32), ("flag", C.c_uint32), ("value", C.c_uint32),
                ("reserved", C.c_uint32)]


class FhDispatchTiming(C.Structure):
    _fields_ = [("dispatch", C.c_uint32), ("dispatches", C.c_uint32), ("op", C.c_uint32),
                ("reserved", C.c_uint32), ("start_ns", C.c_uint64), ("end_ns", C.c_uint64)]


class FhDeviceInfo(C.Structure):
    _fields_ = [("family", C.c_char * 64), ("total_memory", C.c_uint64), ("lds_bytes", C.c_uint64),
                ("compute_units", C.c_uint32), ("wavefront", C.c_uint32)]


EXPORTS = [
    "fh_create", "fh_destroy", "fh_alloc", "fh_release", "fh_import", "fh_write", "fh_read",
    "fh_read_tensor", "fh_prepare_program", "fh_release_program", "fh_submit", "fh_submit_static", "fh_wait",
    "fh_gpu_time_ns", "fh_submission_free", "fh_device_info_get", "fh_memory_usage", "fh_set_memory_limit",
    "fh_submit_profiled", "fh_submission_profile",
    "fh_synchronize", "fh_profile_enable", "fh_profile_select", "fh_profile_sample", "fh_profile_reset", "fh_profile_read",
    "fh_fusion_enable", "fh_fusion_stats", "fh_version",
]

_lib = None


def load_library():
    """Loads the in-tree shared library; raises if it was not built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(f"{LIB_PATH} is missing: run `python -m forja_amd.build` (there is no "
                           "CPU fallback)")
    lib = C.CDLL(LIB_PATH)
    vp, u64, u32 = C.c_void_p, C.c_uint64, C.c_uint32
    lib.fh_create.argtypes = [C.c_int, C.POINTER(vp)]
    lib.fh_destroy.argtypes = [vp]
    lib.fh_destroy.restype = None
    lib.fh_alloc.argtypes = [vp, u64, C.POINTER(u64)]
    lib.fh_release.argtypes = [vp, u64]
    lib.fh_import.argtypes = [vp, vp, u64, C.POINTER(u64)]
    lib.fh_write.argtypes = [vp, u64, u64, vp, u64]
    lib.fh_read.argtypes = [vp, u64, u64, vp, u64]
    lib.fh_read_tensor.argtypes = [vp, C.POINTER(FhTensor), vp, u64]
    lib.fh_prepare_program.argtypes = [vp, u32, C.POINTER(FhInst), u32, C.POINTER(u32), u32,
                                       C.POINTER(u64)]
    lib.fh_release_program.argtypes = [vp, u64]
    lib.fh_submit.argtypes = [vp, C.POINTER(FhDispatch), u32, C.POINTER(vp)]
    lib.fh_submit_static.argtypes = [vp, C.POINTER(FhDispatch), u32, C.POINTER(FhError)]
    lib.fh_wait.argtypes = [vp, u64, C.POINTER(FhError)]
    lib.fh_gpu_time_ns.argtypes = [vp]
    lib.fh_gpu_time_ns.restype = u64
    lib.fh_submission_free.argtypes = [vp]
    lib.fh_submission_free.restype = None
    lib.fh_device_info_get.argtypes = [vp, C.POINTER(FhDeviceInfo)]
    lib.fh_memory_usage.argtypes = [vp, C.POINTER(u64)]
    lib.fh_set_memory_limit.argtypes = [vp, u64]
    lib.fh_submission_profile.argtypes = [vp, C.POINTER(FhDispatchTiming), u32, C.POINTER(u32)]
    lib.fh_synchronize.argtypes = [vp]
    lib.fh_profile_enable.argtypes = [vp, C.c_int]
    lib.fh_profile_reset.argtypes = [vp]
    lib.fh_profile_select.argtypes = [vp, u32]
    lib.fh_profile_sample.argtypes = [vp, u32]
    lib.fh_profile_read.argtypes = [vp, u32, C.POINTER(u64), C.POINTER(u64)]
    lib.fh_fusion_enable.argtypes = [vp, C.c_int]
    lib.fh_fusion_stats.argtypes = [vp, C.POINTER(u64), C.POINTER(u64)]
    lib.fh_version.restype = C.c_char_p
    _lib = lib
    return lib


def _check(status: int):
    if status != 0:
        raise BackendError(Status(status))


def to_fh_tensor(tensor: Tensor, out: Optional[FhTensor] = None) -> FhTensor:
    t = out if out is not None else FhTensor()
    layout = tensor.layout
    t.buffer = tensor.buffer
    t.dtype = int(layout.dtype)
    t.rank = len(layout.shape)
    for axis in range(FH_MAX_RANK):
        t.shape[axis] = layout.shape[axis] if axis < t.rank else 0
        t.stride[axis] = layout.strides[axis] if axis < t.rank else 0
    t.offset = layout.offset
    return t


class PreparedProgram:
    def __init__(self, backend: "HipBackend", handle: int, program: Program):
        self.backend, self.handle, self.program = backend, handle, program


class HipSubmission:
    """`Submission` (backend.rs:609-647)."""

    def __init__(self, backend: "HipBackend", handle):
        self._backend, self._handle = backend, handle
        self._lib = backend._lib

    def wait(self, timeout_ns: int = 0):
        error = FhError()
        status = self._lib.fh_wait(self._handle, timeout_ns, C.byref(error))
        if status != 0:
            raise BackendError(Status(status), index=error.value, dispatch=error.dispatch,
                               operation=error.operation, flag=error.flag)

    def gpu_time_ns(self) -> int:
        return int(self._lib.fh_gpu_time_ns(self._handle))

    def profile(self) -> list:
        """`Submission::profile`: per-dispatch device timeline of a submission made by
        `submit_profiled`, as (first dispatch, dispatches covered, op, start_ns, end_ns)."""
        count = C.c_uint32()
        _check(self._lib.fh_submission_profile(self._handle, None, 0, C.byref(count)))
        entries = (FhDispatchTiming * max(count.value, 1))()
        _check(self._lib.fh_submission_profile(self._handle, entries, count.value, C.byref(count)))
        return [(e.dispatch, e.dispatches, e.op, e.start_ns, e.end_ns) for e in entries[:count.value]]

    def free(self):
        if self._handle is not None:
            self._lib.fh_submission_free(self._handle)
            self._handle = None

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


class EncodedCommands:
    """A command list already lowered to the C ABI's dispatch array, reusable across submits."""

    def __init__(self, array, count):
        self.array, self.count = array, count


class HipBackend:
    """`impl Backend for HipBackend` over the C ABI."""

    def __init__(self, device: int = 0):
        self._lib = load_library()
        handle = C.c_void_p()
        status = self._lib.fh_create(device, C.byref(handle))
        if status != 0:
            raise BackendError(Status(status))
        self._handle = handle

    def close(self):
        if self._handle is not None:
            self._lib.fh_destroy(self._handle)
            self._handle = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    # ---- storage
    def alloc(self, dtype: DType, shape: Sequence[int]) -> Tensor:
        count = 1
        for extent in shape:
            count *= extent
        byte_len = count * DType(dtype).byte_size
        buffer = C.c_uint64()
        _check(self._lib.fh_alloc(self._handle, byte_len, C.byref(buffer)))
        return Tensor(buffer.value, Layout.contiguous(DType(dtype), 0, tuple(shape), byte_len), True)

    def import_readonly(self, data: bytes, dtype: DType, shape: Sequence[int]) -> Tensor:
        buffer = C.c_uint64()
        _check(self._lib.fh_import(self._handle, data, len(data), C.byref(buffer)))
        return Tensor(buffer.value, Layout.contiguous(DType(dtype), 0, tuple(shape), len(data)), False)

    def view(self, tensor: Tensor, op) -> Tensor:
        kind, arg = op
        layout = getattr(tensor.layout, kind)(arg)
        return tensor.with_layout(layout)

    def write(self, tensor: Tensor, data) -> None:
        data = bytes(data) if not isinstance(data, (bytes, bytearray, memoryview)) else data
        layout = tensor.layout
        if (not tensor.writable or not layout.is_contiguous()
                or len(data) != layout.element_count * layout.dtype.byte_size):
            raise BackendError(Status.INVALID_INPUT)
        start, _ = layout.byte_span()
        buf = (C.c_char * len(data)).from_buffer_copy(data)
        _check(self._lib.fh_write(self._handle, tensor.buffer, start, buf, len(data)))

    def write_array(self, tensor: Tensor, array) -> None:
        """numpy convenience: writes a C-contiguous array's bytes."""
        import numpy as np
        array = np.ascontiguousarray(array)
        layout = tensor.layout
        if (not tensor.writable or not layout.is_contiguous()
                or array.nbytes != layout.element_count * layout.dtype.byte_size):
            raise BackendError(Status.INVALID_INPUT)
        start, _ = layout.byte_span()
        _check(self._lib.fh_write(self._handle, tensor.buffer, start,
                                  array.ctypes.data_as(C.c_void_p), array.nbytes))

    def read(self, tensor: Tensor) -> bytes:
        layout = tensor.layout
        length = layout.element_count * layout.dtype.byte_size
        out = (C.c_char * max(length, 1))()
        fh = to_fh_tensor(tensor)
        _check(self._lib.fh_read_tensor(self._handle, C.byref(fh), out, length))
        return bytes(out[:length])

    def read_buffer_range(self, buffer: int, start: int, end: int) -> bytes:
        out = (C.c_char * max(end - start, 1))()
        _check(self._lib.fh_read(self._handle, buffer, start, out, end - start))
        return bytes(out[:end - start])

    def release(self, tensor: Tensor) -> None:
        _check(self._lib.fh_release(self._handle, tensor.buffer))

    # ---- programs
    def prepare_program(self, program: Program) -> PreparedProgram:
        insts = (FhInst * len(program.insts))()
        for i, inst in enumerate(program.insts):
            insts[i].kind, insts[i].op = inst.kind, inst.op
            insts[i].a, insts[i].b, insts[i].c = inst.a, inst.b, inst.c
        pairs = (C.c_uint32 * (2 * len(program.outputs)))()
        for i, (slot, value) in enumerate(program.outputs):
            pairs[2 * i], pairs[2 * i + 1] = slot, value
        handle = C.c_uint64()
        _check(self._lib.fh_prepare_program(self._handle, int(program.kind), insts,
                                            len(program.insts), pairs, len(program.outputs),
                                            C.byref(handle)))
        return PreparedProgram(self, handle.value, program)

    prepare_epilogue = prepare_program

    # ---- execution
    def encode(self, commands: CommandList) -> EncodedCommands:
        count = len(commands.dispatches)
        array = (FhDispatch * max(count, 1))()
        for i, d in enumerate(commands.dispatches):
            self._encode_dispatch(d, array[i])
        return EncodedCommands(array, count)

    @staticmethod
    def _encode_dispatch(d: Dispatch, out: FhDispatch):
        op = d.op
        out.op = int(op.kind)
        out.scale, out.eps, out.theta = op.scale, op.eps, op.theta
        out.bits, out.group_size = op.bits, op.group_size
        out.k, out.normalize = op.k, int(op.normalize)
        out.causal, out.q_start = int(op.causal), op.q_start
        out.key_length, out.page_tokens = op.key_length, op.page_tokens
        out.direction, out.start = op.direction, op.start
        if len(d.inputs) > FH_MAX_INPUTS or len(d.outputs) > FH_MAX_OUTPUTS:
            raise BackendError(Status.INVALID_INPUT)
        out.n_inputs, out.n_outputs = len(d.inputs), len(d.outputs)
        out.program = d.program.handle if d.program is not None else 0
        out.epilogue = d.epilogue.handle if d.epilogue is not None else 0
        out.accumulator_count, out.n_extras = d.accumulator_count, d.n_extras
        for i, t in enumerate(d.inputs):
            to_fh_tensor(t, out.inputs[i])
        for i, t in enumerate(d.outputs):
            to_fh_tensor(t, out.outputs[i])

    @staticmethod
    def patch_query_starts(encoded: EncodedCommands, dispatch_indices, starts):
        """Rewrites the q_start attribute of the named dispatches of an encoded list in place."""
        raw = np.frombuffer(encoded.array, dtype=np.uint8).reshape(-1, C.sizeof(FhDispatch))
        at = FhDispatch.q_start.offset
        field = raw[:, at:at + 4].view(np.uint32)
        field[np.asarray(dispatch_indices), 0] = np.asarray(starts, dtype=np.uint32)

    def submit(self, commands) -> HipSubmission:
        encoded = commands if isinstance(commands, EncodedCommands) else self.encode(commands)
        handle = C.c_void_p()
        _check(self._lib.fh_submit(self._handle, encoded.array, encoded.count, C.byref(handle)))
        return HipSubmission(self, handle)

    def submit_profiled(self, commands) -> HipSubmission:
        """`Backend::submit_profiled_retained`: a device timer around every dispatch."""
        encoded = commands if isinstance(commands, EncodedCommands) else self.encode(commands)
        handle = C.c_void_p()
        _check(self._lib.fh_submit_profiled(self._handle, encoded.array, encoded.count, C.byref(handle)))
        return HipSubmission(self, handle)

    def submit_static(self, commands, wait: bool = True) -> None:
        """fh_submit_static: the same dispatches executed without any allocation, all device
        scratch taken from the library's fixed array.  `wait` false only enqueues."""
        encoded = commands if isinstance(commands, EncodedCommands) else self.encode(commands)
        error = FhError()
        status = self._lib.fh_submit_static(self._handle, encoded.array, encoded.count,
                                            C.byref(error) if wait else None)
        if status != 0:
            raise BackendError(Status(status), index=error.value, dispatch=error.dispatch,
                               operation=error.operation, flag=error.flag)

    def synchronize(self):
        _check(self._lib.fh_synchronize(self._handle))

    def device_info(self) -> dict:
        info = FhDeviceInfo()
        _check(self._lib.fh_device_info_get(self._handle, C.byref(info)))
        return {"family": info.family.decode(), "total_memory": info.total_memory,
                "lds_bytes": info.lds_bytes, "compute_units": info.compute_units,
                "wavefront": info.wavefront}

    def memory_usage(self) -> int:
        """MemoryUsage::charged_bytes: every device byte the backend holds."""
        value = C.c_uint64()
        _check(self._lib.fh_memory_usage(self._handle, C.byref(value)))
        return value.value

    def set_memory_limit(self, limit: int):
        """Backend::set_memory_limit: quota over allocations plus kept operands; 0 lifts it."""
        _check(self._lib.fh_set_memory_limit(self._handle, int(limit)))

    # ---- profiling aid
    def profile_enable(self, level: int):
        """0 off, 1 single-kernel timers, 2 also one timer per dispatch."""
        _check(self._lib.fh_profile_enable(self._handle, int(level)))

    def profile_select(self, class_mask: int):
        """Kernel classes (bit i = class i) the kernel-level timers cover; all by default."""
        _check(self._lib.fh_profile_select(self._handle, int(class_mask) & 0xffffffff))

    def profile_sample(self, every: int):
        """The kernel-level timers take one launch in `every` of each selected class."""
        _check(self._lib.fh_profile_sample(self._handle, int(every)))

    def fusion_enable(self, enabled: bool):
        """Whether runs of per-lane attention dispatches are executed as one ragged launch."""
        _check(self._lib.fh_fusion_enable(self._handle, 1 if enabled else 0))

    def fusion_stats(self):
        """(runs fused, dispatches they replaced) since the backend was created."""
        runs, dispatches = C.c_uint64(), C.c_uint64()
        _check(self._lib.fh_fusion_stats(self._handle, C.byref(runs), C.byref(dispatches)))
        return runs.value, dispatches.value

    def profile_reset(self):
        _check(self._lib.fh_profile_reset(self._handle))

    def profile_read(self, kernel_class: int):
        ns, launches = C.c_uint64(), C.c_uint64()
        _check(self._lib.fh_profile_read(self._handle, kernel_class, C.byref(ns), C.byref(launches)))
        return ns.value, launches.value
