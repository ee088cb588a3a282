"""Python face of the CPU oracle: a `CpuBackend` with the same method names as the reference's
(crates/forja-cpu/src/lib.rs) that executes command lists through liboracle.so.

TEST INFRASTRUCTURE ONLY.  Nothing under forja_amd/ imports this module; only tests/,
__graft_entry__.smoke() and bench.py's cpu_baseline leg do.

Every op follows `CpuBackend::submit` (lib.rs:1419-1516): gather each operand into logical
row-major order (`read`), decode to f32 / u32, run the sequential f32 routine, round to the output
dtype (`encode`) and scatter into the output layout.  The first failing dispatch stops the list.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess
from typing import List, Sequence

import numpy as np

from forja_amd.core import (BackendError, CommandList, DType, Dispatch, Layout, OpKind, Program,
                            Status, Tensor, INTO_PAGES)

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "liboracle.so")


def build():
    subprocess.run(["make", "-s", "-C", _HERE, "-B"], check=True)
    return LIB_PATH


class OrcInst(C.Structure):
    _fields_ = [("kind", C.c_uint32), ("op", C.c_uint32), ("a", C.c_uint32), ("b", C.c_uint32),
                ("c", C.c_uint32)]


class OrcInput(C.Structure):
    _fields_ = [("data", C.c_void_p), ("is_u32", C.c_int)]


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            build()
        l = C.CDLL(LIB_PATH)
        l.orc_affine_quant_dot.restype = C.c_float
        l.orc_route_pack.restype = C.c_long
        l.orc_splitmix64.restype = C.c_uint64
        l.orc_splitmix64.argtypes = [C.c_uint64]
        l.orc_stream_u64.restype = C.c_uint64
        l.orc_stream_u64.argtypes = [C.c_uint64] * 3
        l.orc_f32_to_bf16.restype = C.c_uint16
        l.orc_f32_to_bf16.argtypes = [C.c_float]
        l.orc_f32_to_f16.restype = C.c_uint16
        l.orc_f32_to_f16.argtypes = [C.c_float]
        l.orc_bf16_to_f32.restype = C.c_float
        l.orc_bf16_to_f32.argtypes = [C.c_uint16]
        l.orc_f16_to_f32.restype = C.c_float
        l.orc_f16_to_f32.argtypes = [C.c_uint16]
        _lib = l
    return _lib


def _p(array):
    return array.ctypes.data_as(C.c_void_p)


def _sz(value):
    return C.c_size_t(int(value))


def _ok(status, err=Status.EXECUTION_FAILED):
    if status != 0:
        raise BackendError(Status(status) if status in Status._value2member_map_ else err)


_NP = {DType.F32: np.float32, DType.F16: np.uint16, DType.BF16: np.uint16, DType.I32: np.int32,
       DType.U32: np.uint32}


def sampling_words(temperature: float, top_k: int, top_p: float, seed: int) -> np.ndarray:
    """The five parameter words of Op::Sample (SamplingParameters::from_words, lib.rs:1553-1575)."""
    bits = np.array([temperature, top_p], dtype=np.float32).view(np.uint32)
    return np.array([bits[0], top_k, bits[1], seed & 0xffffffff, (seed >> 32) & 0xffffffff],
                    dtype=np.uint32)


def sample_rows(values: np.ndarray, params: np.ndarray, position: int, allow=None) -> np.ndarray:
    """sample_row / sample_row_masked (lib.rs:1577-1597) over the rows of a 2-D f32 array."""
    values = np.ascontiguousarray(values, dtype=np.float32)
    rows, width = values.shape
    out = np.empty(rows, dtype=np.uint32)
    params = np.ascontiguousarray(params, dtype=np.uint32)
    if allow is not None:
        allow = np.ascontiguousarray(allow, dtype=np.uint32)
    _ok(lib().orc_sample(_p(values), _sz(rows), _sz(width), _p(params), C.c_uint32(position),
                         _p(allow) if allow is not None else None, _p(out)))
    return out


def top_p_keep(row: np.ndarray, temperature: float, top_p: float) -> int:
    """Candidates truncate_top_p (lib.rs:1654-1679) keeps out of a whole row."""
    row = np.ascontiguousarray(row, dtype=np.float32)
    keep = C.c_size_t()
    _ok(lib().orc_top_p_keep(_p(row), _sz(row.size), C.c_float(temperature), C.c_float(top_p),
                             C.byref(keep)))
    return keep.value


def validate_allow_mask(allow, width: int) -> bool:
    """validate_allow_mask (lib.rs:1639-1652): True when accepted."""
    allow = np.ascontiguousarray(allow, dtype=np.uint32)
    return lib().orc_validate_allow_mask(_p(allow), _sz(allow.size), _sz(width)) == 0


def decode(raw: np.ndarray, dtype: DType) -> np.ndarray:
    """lib.rs:1790-1809"""
    count = raw.size // dtype.byte_size
    out = np.empty(count, dtype=np.float32)
    _ok(lib().orc_decode(_p(raw), int(dtype), _sz(count), _p(out)))
    return out


def encode(values: np.ndarray, dtype: DType) -> np.ndarray:
    """lib.rs:1836-1847"""
    values = np.ascontiguousarray(values, dtype=np.float32)
    out = np.empty(values.size * dtype.byte_size, dtype=np.uint8)
    _ok(lib().orc_encode(_p(values), int(dtype), _sz(values.size), _p(out)))
    return out


# ---- seeded synthetic data (identical arithmetic to FH_OP_FILL_SEEDED) ----

def fill_words(seed, stream, count, first=0):
    out = np.empty(count, dtype=np.uint32)
    lib().orc_fill_words(C.c_uint64(seed), C.c_uint64(stream), C.c_uint64(first), _sz(count), _p(out))
    return out


def fill_uniform_bf16(seed, stream, count, lo, hi, first=0):
    out = np.empty(count, dtype=np.uint16)
    lib().orc_fill_uniform_bf16(C.c_uint64(seed), C.c_uint64(stream), C.c_uint64(first), _sz(count),
                                C.c_float(lo), C.c_float(hi), _p(out))
    return out


def fill_normal_bf16(seed, stream, count, first=0):
    out = np.empty(count, dtype=np.uint16)
    lib().orc_fill_normal_bf16(C.c_uint64(seed), C.c_uint64(stream), C.c_uint64(first), _sz(count),
                               _p(out))
    return out


def fill_normal_f32(seed, stream, count, first=0):
    out = np.empty(count, dtype=np.float32)
    lib().orc_fill_normal_f32(C.c_uint64(seed), C.c_uint64(stream), C.c_uint64(first), _sz(count),
                              _p(out))
    return out


def bf16_to_f32(bits: np.ndarray) -> np.ndarray:
    return (bits.astype(np.uint32) << 16).view(np.float32)


def f32_to_bf16(values: np.ndarray) -> np.ndarray:
    return encode(np.asarray(values, dtype=np.float32).ravel(), DType.BF16).view(np.uint16)


def route_pack(indices: np.ndarray, experts: int, tile_rows: int):
    """Closed-form packing; returns counts, offsets, sorted_routes (valid prefix), blocks, invalid."""
    indices = np.ascontiguousarray(indices, dtype=np.uint32)
    rows, k = indices.shape
    counts = np.zeros(experts, np.uint32)
    offsets = np.zeros(experts + 1, np.uint32)
    sorted_routes = np.zeros(rows * k, np.uint32)
    max_blocks = experts + (rows * k) // tile_rows + 1
    blocks = np.zeros((max_blocks, 3), np.uint32)
    invalid = np.zeros(2, np.uint32)
    n = lib().orc_route_pack(_p(indices), _sz(rows), _sz(k), _sz(experts), _sz(tile_rows),
                             _p(counts), _p(offsets), _p(sorted_routes), _p(blocks),
                             _sz(max_blocks), _p(invalid))
    if n < 0:
        raise BackendError(Status.INVALID_INPUT)
    return counts, offsets, sorted_routes[:offsets[-1]], blocks[:n], invalid


class CpuSubmission:
    def __init__(self, error):
        self._error = error

    def wait(self, timeout_ns: int = 0):
        if self._error is not None:
            raise self._error


class CpuBackend:
    """Reference-semantics backend over plain host memory."""

    def __init__(self, threads: int = 0):
        self._buffers = {}
        self._next = 1
        lib().orc_set_threads(int(threads))

    # ---- storage (lib.rs:67-161)
    def alloc(self, dtype: DType, shape: Sequence[int]) -> Tensor:
        count = int(np.prod(shape, dtype=np.int64)) if len(shape) else 1
        byte_len = count * DType(dtype).byte_size
        buffer = self._next
        self._next += 1
        self._buffers[buffer] = np.zeros(byte_len, dtype=np.uint8)
        return Tensor(buffer, Layout.contiguous(DType(dtype), 0, tuple(shape), byte_len), True)

    def import_readonly(self, data: bytes, dtype: DType, shape) -> Tensor:
        buffer = self._next
        self._next += 1
        self._buffers[buffer] = np.frombuffer(bytes(data), dtype=np.uint8).copy()
        return Tensor(buffer, Layout.contiguous(DType(dtype), 0, tuple(shape), len(data)), False)

    def view(self, tensor: Tensor, op) -> Tensor:
        kind, arg = op
        return tensor.with_layout(getattr(tensor.layout, kind)(arg))

    def write(self, tensor: Tensor, data) -> None:
        layout = tensor.layout
        raw = np.frombuffer(bytes(data), dtype=np.uint8)
        if (not tensor.writable or not layout.is_contiguous()
                or raw.size != layout.element_count * layout.dtype.byte_size):
            raise BackendError(Status.INVALID_INPUT)
        start, end = layout.byte_span()
        self._storage(tensor)[start:end] = raw

    def write_array(self, tensor: Tensor, array) -> None:
        self.write(tensor, np.ascontiguousarray(array).tobytes())

    def read(self, tensor: Tensor) -> bytes:
        return self._gather(tensor).tobytes()

    def release(self, tensor: Tensor) -> None:
        if self._buffers.pop(tensor.buffer, None) is None:
            raise BackendError(Status.INVALID_INPUT)

    def prepare_program(self, program: Program):
        """The structural limits of validate_structure (crates/forja-core/src/program.rs:25-31,
        1052-1094): at most 256 instructions, 8 input slots, 4 outputs and 4 reductions, operands
        defined earlier, no reduction in a map program.  Typing is checked when the program runs."""
        if len(program.insts) > 256 or not program.outputs:
            raise BackendError(Status.INVALID_INPUT)
        reductions = 0
        for index, inst in enumerate(program.insts):
            if inst.kind == 0 and inst.a >= 8:
                raise BackendError(Status.INVALID_INPUT)
            if inst.kind == 8:
                reductions += 1
                if int(program.kind) == 0 or reductions > 4:
                    raise BackendError(Status.INVALID_INPUT)
            operands = {4: (inst.a,), 5: (inst.a, inst.b), 6: (inst.a, inst.b, inst.c), 7: (inst.a,),
                        8: (inst.a,)}.get(inst.kind, ())
            if any(operand >= index for operand in operands):
                raise BackendError(Status.INVALID_INPUT)
        if any(slot >= 4 for slot, _ in program.outputs):
            raise BackendError(Status.INVALID_INPUT)
        return program

    prepare_epilogue = prepare_program

    def synchronize(self):
        pass

    # ---- helpers
    def _storage(self, tensor: Tensor) -> np.ndarray:
        try:
            return self._buffers[tensor.buffer]
        except KeyError:
            raise BackendError(Status.INVALID_INPUT)

    def _gather(self, tensor: Tensor) -> np.ndarray:
        """gather (lib.rs:1747-1765) through the C restatement."""
        layout = tensor.layout
        storage = self._storage(tensor)
        size = layout.dtype.byte_size
        out = np.empty(layout.element_count * size, dtype=np.uint8)
        if layout.element_count == 0:
            return out
        shape = (C.c_uint32 * max(layout.rank, 1))(*layout.shape)
        strides = (C.c_uint64 * max(layout.rank, 1))(*layout.strides)
        _ok(lib().orc_gather(_p(storage), _sz(storage.size), size, layout.rank, shape, strides,
                             C.c_uint64(layout.offset), _p(out)), Status.INVALID_INPUT)
        return out

    def _scatter(self, tensor: Tensor, raw: np.ndarray) -> None:
        layout = tensor.layout
        if not tensor.writable:
            raise BackendError(Status.INVALID_INPUT)
        storage = self._storage(tensor)
        if layout.element_count == 0:
            return
        raw = np.ascontiguousarray(raw).view(np.uint8).ravel()
        shape = (C.c_uint32 * max(layout.rank, 1))(*layout.shape)
        strides = (C.c_uint64 * max(layout.rank, 1))(*layout.strides)
        _ok(lib().orc_scatter(_p(storage), _sz(storage.size), layout.dtype.byte_size, layout.rank,
                              shape, strides, C.c_uint64(layout.offset), _p(raw)),
            Status.INVALID_INPUT)

    def _floats(self, tensor: Tensor) -> np.ndarray:
        return decode(self._gather(tensor), tensor.dtype)

    def _u32(self, tensor: Tensor) -> np.ndarray:
        return self._gather(tensor).view(np.uint32).copy()

    def _write_output(self, tensor: Tensor, values: np.ndarray) -> None:
        """write_output (lib.rs:484-493)"""
        self._scatter(tensor, encode(values, tensor.dtype))

    # ---- submit (lib.rs:1419-1516)
    def submit(self, commands: CommandList) -> CpuSubmission:
        for d in commands.dispatches:
            for t in list(d.inputs) + list(d.outputs):
                self._storage(t)
        error = None
        for index, d in enumerate(commands.dispatches):
            try:
                self._execute(d)
            except BackendError as e:
                e.dispatch = index
                error = e
                break
        return CpuSubmission(error)

    def _execute(self, d: Dispatch) -> None:
        kind = d.op.kind
        handler = {
            OpKind.PROGRAM: self._program, OpKind.COPY: self._copy,
            OpKind.PAGED_COPY: self._paged_copy_op, OpKind.RMS_NORM: self._rms_norm,
            OpKind.ARGMAX: self._argmax, OpKind.TOP_K: self._top_k, OpKind.ROPE: self._rope,
            OpKind.SAMPLE: self._sample, OpKind.SAMPLE_MASKED: self._sample,
            OpKind.QUANT_EMBED: self._quant_embed, OpKind.MATMUL: self._matmul,
            OpKind.QUANT_MATMUL: self._quant_matmul,
            OpKind.GATHER_QUANT_MATMUL: self._gather_quant,
            OpKind.PAGED_SDPA_APPEND: self._paged_append, OpKind.PAGED_SDPA: self._paged_sdpa_op,
            OpKind.PAGED_ATTENTION_RAGGED: self._ragged, OpKind.ROUTE_PACK: self._route_pack,
            OpKind.FILL_SEEDED: self._fill,
        }.get(kind)
        if handler is None:
            raise BackendError(Status.UNSUPPORTED_OPERATION)
        handler(d)

    # ---- scalar programs (lib.rs:395-482)
    def _interpret(self, program: Program, shape, inputs: List[np.ndarray]) -> List[np.ndarray]:
        insts = (OrcInst * len(program.insts))()
        for i, inst in enumerate(program.insts):
            insts[i].kind, insts[i].op = inst.kind, inst.op
            insts[i].a, insts[i].b, insts[i].c = inst.a, inst.b, inst.c
        pairs = (C.c_uint32 * (2 * len(program.outputs)))()
        for i, (slot, value) in enumerate(program.outputs):
            pairs[2 * i], pairs[2 * i + 1] = slot, value
        elements = int(np.prod(shape, dtype=np.int64))
        ins = (OrcInput * max(len(inputs), 1))()
        keep = []
        for i, array in enumerate(inputs):
            array = np.ascontiguousarray(array)
            if array.size != elements:
                raise BackendError(Status.EXECUTION_FAILED)
            keep.append(array)
            ins[i].data = array.ctypes.data
            ins[i].is_u32 = int(array.dtype == np.uint32)
        outs = [np.zeros(elements, dtype=np.float32) for _ in range(program.output_count)]
        out_ptrs = (C.c_void_p * len(outs))(*[o.ctypes.data for o in outs])
        cshape = (C.c_uint32 * len(shape))(*shape)
        _ok(lib().orc_interpret(int(program.kind), insts, _sz(len(program.insts)), pairs,
                                _sz(len(program.outputs)), _sz(program.output_count), len(shape),
                                cshape, ins, _sz(len(inputs)), out_ptrs))
        return outs

    def _decode_inputs(self, tensors):
        out = []
        for t in tensors:
            if t.dtype.is_float:
                out.append(self._floats(t))
            elif t.dtype == DType.U32:
                out.append(self._u32(t))
            else:
                raise BackendError(Status.EXECUTION_FAILED)
        return out

    def _program(self, d: Dispatch):
        outs = self._interpret(d.program, d.outputs[0].shape, self._decode_inputs(d.inputs))
        for tensor, values in zip(d.outputs, outs):
            self._write_output(tensor, values)

    def _apply_epilogue(self, d: Dispatch, primitive: int, accumulators: List[np.ndarray]):
        if d.epilogue is None:
            if len(accumulators) != 1:
                raise BackendError(Status.EXECUTION_FAILED)
            return accumulators[0]
        extras = self._decode_inputs(d.inputs[primitive:])
        outs = self._interpret(d.epilogue, d.outputs[0].shape, list(accumulators) + extras)
        return outs[-1]

    # ---- ops
    def _copy(self, d):
        src = d.inputs[0]
        if src.dtype in (DType.I32, DType.U32):
            self._scatter(d.outputs[0], self._gather(src))
        else:
            self._write_output(d.outputs[0], self._floats(src))

    def _quant_matmul(self, d):
        x, packed, scales, biases = d.inputs[:4]
        rows, inner = x.shape
        columns = packed.shape[0]
        out = np.empty(rows * columns, dtype=np.float32)
        xs, ps, ss, bs = self._floats(x), self._u32(packed), self._floats(scales), self._floats(biases)
        _ok(lib().orc_quant_matmul(_p(xs), _p(ps), _p(ss), _p(bs), _sz(rows), _sz(inner),
                                   _sz(columns), d.op.bits, _sz(d.op.group_size), _p(out)))
        self._write_output(d.outputs[0], self._apply_epilogue(d, 4, [out]))

    def _projection(self, d, positions):
        x, packed, scales, biases, indices = (d.inputs[p] for p in positions)
        rows, inner = x.shape
        experts, columns, _ = packed.shape
        k = indices.shape[1]
        out = np.empty(rows * k * columns, dtype=np.float32)
        invalid = np.zeros(2, dtype=np.uint32)
        xs, ps, ss, bs, ix = (self._floats(x), self._u32(packed), self._floats(scales),
                              self._floats(biases), self._u32(indices))
        _ok(lib().orc_gather_quant_projection(_p(xs), _p(ps), _p(ss), _p(bs), _p(ix), _sz(rows),
                                              _sz(inner), _sz(experts), _sz(columns), _sz(k),
                                              d.op.bits, _sz(d.op.group_size), _p(out), _p(invalid)))
        return out, invalid

    def _gather_quant(self, d):
        primitive = len(d.inputs) - d.n_extras
        if primitive == 6:
            return self._weighted_sum(d)
        first, invalid = self._projection(d, [0, 1, 2, 3, primitive - 1])
        accumulators = [first]
        if primitive == 8:
            second, _ = self._projection(d, [0, 4, 5, 6, 7])
            accumulators.append(second)
        self._write_output(d.outputs[0], self._apply_epilogue(d, primitive, accumulators))
        if invalid[0]:
            raise BackendError(Status.INDEX_OUT_OF_RANGE, index=int(invalid[1]))

    def _weighted_sum(self, d):
        x, packed, scales, biases, indices, weights = d.inputs[:6]
        rows, routes, inner = x.shape
        experts, columns, _ = packed.shape
        out = np.empty(rows * columns, dtype=np.float32)
        invalid = np.zeros(2, dtype=np.uint32)
        xs, ps, ss, bs, ix, ws = (self._floats(x), self._u32(packed), self._floats(scales),
                                  self._floats(biases), self._u32(indices), self._floats(weights))
        _ok(lib().orc_gather_quant_weighted_sum(_p(xs), _p(ps), _p(ss), _p(bs), _p(ix), _p(ws), None,
                                                _sz(rows), _sz(routes), _sz(inner), _sz(experts),
                                                _sz(columns), d.op.bits, _sz(d.op.group_size),
                                                _p(out), _p(invalid)))
        self._write_output(d.outputs[0], self._apply_epilogue(d, 6, [out]))
        if invalid[0]:
            raise BackendError(Status.INDEX_OUT_OF_RANGE, index=int(invalid[1]))

    def _top_k(self, d):
        src = d.inputs[0]
        width = src.shape[-1]
        rows = src.layout.element_count // width
        k = d.op.k
        values = np.empty(rows * k, dtype=np.float32)
        indices = np.empty(rows * k, dtype=np.uint32)
        xs = self._floats(src)
        _ok(lib().orc_top_k(_p(xs), _sz(rows), _sz(width), _sz(k), int(d.op.normalize), _p(values),
                            _p(indices)))
        self._write_output(d.outputs[0], values)
        self._scatter(d.outputs[1], indices)

    def _argmax(self, d):
        src = d.inputs[0]
        width = src.shape[-1]
        rows = src.layout.element_count // width
        out = np.empty(rows, dtype=np.uint32)
        xs = self._floats(src)
        _ok(lib().orc_argmax(_p(xs), _sz(rows), _sz(width), _p(out)))
        self._scatter(d.outputs[0], out)

    def _sample(self, d):
        """execute_sample / execute_sample_masked (crates/forja-cpu/src/lib.rs:610-678)."""
        src = d.inputs[0]
        width = src.shape[-1]
        rows = src.layout.element_count // width
        xs = self._floats(src)
        params = np.ascontiguousarray(self._gather(d.inputs[1]).view(np.uint32))
        allow = None
        if d.op.kind == OpKind.SAMPLE_MASKED:
            allow = np.ascontiguousarray(self._gather(d.inputs[2]).view(np.uint32))
        out = np.empty(rows, dtype=np.uint32)
        _ok(lib().orc_sample(_p(xs), _sz(rows), _sz(width), _p(params), C.c_uint32(d.op.start),
                             _p(allow) if allow is not None else None, _p(out)))
        self._scatter(d.outputs[0], out)

    def _rms_norm(self, d):
        x, w = d.inputs
        width = w.shape[0]
        rows = x.layout.element_count // width
        out = np.empty(rows * width, dtype=np.float32)
        xs, ws = self._floats(x), self._floats(w)
        _ok(lib().orc_rms_norm(_p(xs), _p(ws), _sz(rows), _sz(width), C.c_float(d.op.eps), _p(out)))
        self._write_output(d.outputs[0], out)

    def _rope(self, d):
        x, pos = d.inputs
        rows, heads, width = x.shape
        values = self._floats(x).copy()
        ps = self._u32(pos)
        _ok(lib().orc_rope(_p(values), _p(ps), _sz(rows), _sz(heads), _sz(width),
                           C.c_float(d.op.theta)))
        self._write_output(d.outputs[0], values)

    def _quant_embed(self, d):
        packed, scales, biases, ids = d.inputs
        vocab, packed_width = packed.shape
        width = packed_width * (32 // d.op.bits)
        id_values = self._u32(ids)
        out = np.empty(id_values.size * width, dtype=np.float32)
        invalid = np.zeros(2, dtype=np.uint32)
        ps, ss, bs = self._u32(packed), self._floats(scales), self._floats(biases)
        _ok(lib().orc_quant_embed(_p(ps), _p(ss), _p(bs), _p(id_values), _sz(id_values.size),
                                  _sz(vocab), _sz(packed_width), d.op.bits, _sz(d.op.group_size),
                                  _p(out), _p(invalid)))
        self._write_output(d.outputs[0], out)
        if invalid[0]:
            raise BackendError(Status.INDEX_OUT_OF_RANGE, index=int(invalid[1]))

    def _matmul(self, d):
        l, r = d.inputs[:2]
        rank = len(l.shape)
        batches = l.shape[0] if rank == 3 else 1
        rows, inner, columns = l.shape[-2], l.shape[-1], r.shape[-1]
        out = np.empty(batches * rows * columns, dtype=np.float32)
        ls, rs = self._floats(l), self._floats(r)
        _ok(lib().orc_matmul(_p(ls), _p(rs), _sz(batches), _sz(rows), _sz(inner), _sz(columns),
                             _p(out)))
        self._write_output(d.outputs[0], self._apply_epilogue(d, 2, [out]))

    # ---- paged storage (lib.rs:189-393)
    def _lane_active(self, activity):
        if activity is None:
            return True
        return int(self._gather(activity).view(np.uint32)[0]) != 0

    def _page_table(self, table: Tensor, generations: Tensor):
        """cpu_page_table (lib.rs:1519-1535)"""
        entries = self._u32(table)
        gens = self._u32(generations)
        if entries.size % 2:
            raise BackendError(Status.INVALID_INPUT)
        if lib().orc_page_table_from_padded(_p(entries), _sz(entries.size // 2), _p(gens),
                                            _sz(gens.size)):
            raise BackendError(Status.EXECUTION_FAILED)
        return entries, gens

    def _paged_copy(self, ordinary: Tensor, pool: Tensor, table, generations, activity, direction,
                    start, page_tokens, held=None):
        """`held`: the pool's bytes, already gathered by a caller that runs many copies and
        writes the pool back itself (the ragged op); the copy then lands there."""
        if not self._lane_active(activity):
            return
        entries, gens = self._page_table(table, generations)
        physical_pages, _, elements = pool.shape
        row_bytes = elements * pool.dtype.byte_size
        pool_raw = self._gather(pool) if held is None else held
        tokens = ordinary.shape[0]
        if direction == INTO_PAGES:
            rows = encode(self._floats(ordinary), pool.dtype)
            status = lib().orc_paged_copy_in(_p(pool_raw), _sz(physical_pages), _sz(page_tokens),
                                             _sz(row_bytes), _p(entries), _sz(entries.size // 2),
                                             _p(gens), C.c_uint64(start), C.c_uint64(tokens),
                                             _p(rows))
            _ok(status, Status.INVALID_INPUT)
            if held is None:
                self.write(pool, pool_raw.tobytes())
        else:
            rows = np.empty(tokens * row_bytes, dtype=np.uint8)
            status = lib().orc_paged_copy_out(_p(pool_raw), _sz(physical_pages), _sz(page_tokens),
                                              _sz(row_bytes), _p(entries), _sz(entries.size // 2),
                                              _p(gens), C.c_uint64(start), C.c_uint64(tokens),
                                              _p(rows))
            _ok(status, Status.INVALID_INPUT)
            self.write(ordinary, encode(decode(rows, pool.dtype), ordinary.dtype).tobytes())

    def _paged_copy_op(self, d):
        direction = d.op.direction
        activity = d.inputs[3] if len(d.inputs) == 4 else None
        ordinary, pool = (d.inputs[0], d.outputs[0]) if direction == INTO_PAGES else (d.outputs[0], d.inputs[0])
        self._paged_copy(ordinary, pool, d.inputs[1], d.inputs[2], activity, direction, d.op.start,
                         d.op.page_tokens)

    def _paged_sdpa(self, q, key_pool, value_pool, table, generations, activity, output, scale,
                    causal, q_start, key_length, page_tokens, held=None):
        """`held`: the bytes of both pools, already gathered (see _paged_copy)."""
        if not self._lane_active(activity):
            self._write_output(output, np.zeros(output.layout.element_count, dtype=np.float32))
            return
        kp, vp = (self._gather(key_pool), self._gather(value_pool)) if held is None else held
        entries, gens = self._page_table(table, generations)
        query = self._floats(q)
        hq, sq, width = q.shape
        physical_pages, _, kv_heads, _ = key_pool.shape
        value_width = value_pool.shape[3]
        out = np.empty(hq * sq * value_width, dtype=np.float32)
        status = lib().orc_paged_sdpa(_p(query), _p(kp), _p(vp), int(key_pool.dtype),
                                      int(value_pool.dtype), _sz(physical_pages), _sz(page_tokens),
                                      _p(entries), _sz(entries.size // 2), _p(gens), hq, sq,
                                      kv_heads, width, value_width, key_length, q_start,
                                      C.c_float(scale), int(causal), _p(out))
        _ok(status, Status.INVALID_INPUT)
        self._write_output(output, out)

    def _paged_sdpa_op(self, d):
        activity = d.inputs[5] if len(d.inputs) == 6 else None
        self._paged_sdpa(d.inputs[0], d.inputs[1], d.inputs[2], d.inputs[3], d.inputs[4], activity,
                         d.outputs[0], d.op.scale, d.op.causal, d.op.q_start, d.op.key_length,
                         d.op.page_tokens)

    def _paged_append(self, d):
        """execute_paged_append (lib.rs:262-306)"""
        activity = d.inputs[5] if len(d.inputs) == 6 else None
        for index in (1, 2):
            pool = d.outputs[index]
            p, t, h, w = pool.shape
            plane = pool.reshape([p, t, h * w])
            self._paged_copy(d.inputs[index], plane, d.inputs[3], d.inputs[4], activity,
                             INTO_PAGES, d.op.q_start, d.op.page_tokens)
        self._paged_sdpa(d.inputs[0], d.outputs[1], d.outputs[2], d.inputs[3], d.inputs[4],
                         activity, d.outputs[0], d.op.scale, True, d.op.q_start, d.op.q_start + 1,
                         d.op.page_tokens)

    def _ragged(self, d):
        """The fused ragged op, executed lane by lane as the per-lane sequence it replaces:
        two PagedCopy{IntoPages} then one causal PagedSdpa (engines/qwen3-coder/src/lib.rs:917-935,
        crates/forja-sdk/src/paged.rs:420-478)."""
        q, k_new, v_new, tables, generations, cu, starts = d.inputs[:7]
        activity = d.inputs[7] if len(d.inputs) == 8 else None
        out, key_pool, value_pool = d.outputs
        cu_values, start_values = self._u32(cu), self._u32(starts)
        lanes = tables.shape[0]
        # cu_seqlens is data: token ranges must be non-decreasing and end inside the packed batch,
        # else the dispatch is refused whole (zero rows, pools untouched, lowest offending lane).
        ends = cu_values.astype(np.int64)
        malformed = (ends[1:] < ends[:-1]) | (ends[1:] > q.shape[0])
        if malformed.any():
            self._write_output(out, np.zeros(out.layout.element_count, dtype=np.float32))
            raise BackendError(Status.DEVICE_ERROR_FLAG, index=int(np.argmax(malformed)))
        if d.op.k == 1:     # the recorder promised at most one query row per lane
            counts = np.diff(cu_values.astype(np.int64))
            if (counts > 1).any():
                lane = int(np.argmax(counts > 1))
                raise BackendError(Status.DEVICE_ERROR_FLAG, index=int(cu_values[lane]))
        p, pt, hkv, width = key_pool.shape
        value_width = value_pool.shape[3]
        # The same sequence of calls per lane, on one copy of each pool's bytes that is written
        # back when the lanes are through (or a lane has failed): gathering and rewriting both
        # pools for every lane costs more than the attention itself.
        whole = (key_pool.layout.is_contiguous() and value_pool.layout.is_contiguous()
                 and key_pool.writable and value_pool.writable)
        held = (self._gather(key_pool), self._gather(value_pool)) if whole else None
        try:
            for lane in range(lanes):
                first, last = int(cu_values[lane]), int(cu_values[lane + 1])
                count = last - first
                if count <= 0:
                    continue
                act = activity.narrow(0, lane, 1) if activity is not None else None
                table = tables.narrow(0, lane, 1).reshape([tables.shape[1], 2])
                q_start = int(start_values[lane])
                key_plane = key_pool.reshape([p, pt, hkv * width])
                value_plane = value_pool.reshape([p, pt, hkv * value_width])
                self._paged_copy(k_new.narrow(0, first, count), key_plane, table, generations, act,
                                 INTO_PAGES, q_start, d.op.page_tokens, held=held and held[0])
                self._paged_copy(v_new.narrow(0, first, count), value_plane, table, generations, act,
                                 INTO_PAGES, q_start, d.op.page_tokens, held=held and held[1])
                lane_q = q.narrow(0, first, count).permute([1, 0, 2])
                lane_out = out.narrow(0, first, count).permute([1, 0, 2])
                self._paged_sdpa(lane_q, key_pool, value_pool, table, generations, act, lane_out,
                                 d.op.scale, True, q_start, q_start + count, d.op.page_tokens, held=held)
        finally:
            if held is not None:
                self.write(key_pool, held[0].tobytes())
                self.write(value_pool, held[1].tobytes())

    def _route_pack(self, d):
        indices = self._u32(d.inputs[0]).reshape(d.inputs[0].shape)
        experts = d.outputs[0].shape[0]
        counts, offsets, sorted_routes, blocks, invalid = route_pack(indices, experts, d.op.k)
        full_sorted = np.zeros(d.outputs[2].shape[0], np.uint32)
        full_sorted[:sorted_routes.size] = sorted_routes
        full_blocks = np.zeros(d.outputs[3].shape, np.uint32)
        full_blocks[:, 0] = 0xffffffff
        full_blocks[:blocks.shape[0]] = blocks
        self._scatter(d.outputs[0], counts)
        self._scatter(d.outputs[1], offsets)
        self._scatter(d.outputs[2], full_sorted)
        self._scatter(d.outputs[3], full_blocks)
        if invalid[0]:
            raise BackendError(Status.INDEX_OUT_OF_RANGE, index=int(invalid[1]))

    def _fill(self, d):
        out = d.outputs[0]
        seed = d.op.q_start | (d.op.key_length << 32)
        count = out.layout.element_count
        if d.op.k == 0:
            self._scatter(out, fill_words(seed, d.op.start, count, d.op.direction))
            return
        if d.op.k == 1:
            # uniform in f32, then the output dtype's rounding
            unit = np.empty(count, dtype=np.uint16)
            values = bf16_to_f32(fill_uniform_bf16(seed, d.op.start, count, d.op.scale, d.op.eps,
                                                   d.op.direction)) if out.dtype == DType.BF16 else None
            if values is None:
                raise BackendError(Status.UNSUPPORTED_OPERATION)
            self._write_output(out, values)
            return
        self._write_output(out, fill_normal_f32(seed, d.op.start, count, d.op.direction))
