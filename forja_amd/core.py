"""Host-side contract types shared by every backend binding.

These restate the parts of `forja-core` a backend's callers use on the ragged forward step:
`DType`, `Layout` (crates/forja-core/src/layout.rs), `Tensor` and `Op`
(crates/forja-core/src/ops.rs:62-302), the scalar Program IR (wit/compute.wit:75-141) and
`BackendError` (crates/forja-core/src/backend.rs:363-426).  They are metadata only; no compute.
"""
from __future__ import annotations

import enum
import struct
from dataclasses import dataclass, field
from typing import List, Optional, Sequence, Tuple

MAX_RANK = 8


class DType(enum.IntEnum):
    F32 = 0
    F16 = 1
    BF16 = 2
    I32 = 3
    U32 = 4

    @property
    def byte_size(self) -> int:
        return 2 if self in (DType.F16, DType.BF16) else 4

    @property
    def is_float(self) -> bool:
        return self in (DType.F32, DType.F16, DType.BF16)


class Status(enum.IntEnum):
    OK = 0
    QUOTA_EXCEEDED = 1
    ALLOCATION_FAILED = 2
    INVALID_DEVICE_WORKING_SET = 3
    EXECUTION_FAILED = 4
    DEVICE_EXECUTION_FAILED = 5
    DEVICE_ERROR_FLAG = 6
    GPU_PREDICTION_EXCEEDED = 7
    IMPOSSIBLE_RATE = 8
    TIMEOUT = 9
    INVALID_INPUT = 10
    UNSUPPORTED_OPERATION = 11
    INDEX_OUT_OF_RANGE = 12


class BackendError(Exception):
    """`forja_core::BackendError` with its payload."""

    def __init__(self, status: Status, index: Optional[int] = None, dispatch: Optional[int] = None,
                 operation: Optional[int] = None, flag: Optional[int] = None):
        self.status = Status(status)
        self.index = index
        self.dispatch = dispatch
        self.operation = operation
        self.flag = flag
        super().__init__(f"{self.status.name}(index={index}, dispatch={dispatch})")


class LayoutError(ValueError):
    pass


@dataclass(frozen=True)
class Slice:
    start: int
    len: int
    step: int = 1


@dataclass(frozen=True)
class Layout:
    """Element-unit offset/strides over a buffer of `buffer_len` bytes (layout.rs)."""
    dtype: DType
    offset: int
    shape: Tuple[int, ...]
    strides: Tuple[int, ...]
    buffer_len: int

    def __post_init__(self):
        if len(self.shape) != len(self.strides) or len(self.shape) > MAX_RANK:
            raise LayoutError("rank")
        if self.element_count:
            last = self.offset + sum((e - 1) * s for e, s in zip(self.shape, self.strides))
            if (last + 1) * self.dtype.byte_size > self.buffer_len:
                raise LayoutError("span exceeds buffer")

    @staticmethod
    def contiguous(dtype: DType, offset: int, shape: Sequence[int], buffer_len: int) -> "Layout":
        strides, stride = [], 1
        for extent in reversed(shape):
            strides.append(stride)
            stride *= extent
        return Layout(dtype, offset, tuple(shape), tuple(reversed(strides)), buffer_len)

    @property
    def element_count(self) -> int:
        count = 1
        for extent in self.shape:
            count *= extent
        return count

    @property
    def rank(self) -> int:
        return len(self.shape)

    def is_contiguous(self) -> bool:
        expected = 1
        for extent, stride in zip(reversed(self.shape), reversed(self.strides)):
            if extent == 1:
                continue
            if stride != expected:
                return False
            expected *= extent
        return True

    def byte_span(self) -> Tuple[int, int]:
        if not self.element_count:
            return (self.offset * self.dtype.byte_size,) * 2
        last = self.offset + sum((e - 1) * s for e, s in zip(self.shape, self.strides))
        return self.offset * self.dtype.byte_size, (last + 1) * self.dtype.byte_size

    def slice(self, specs: Sequence[Slice]) -> "Layout":
        if len(specs) != self.rank:
            raise LayoutError("slice rank")
        offset, shape, strides = self.offset, [], []
        for spec, extent, stride in zip(specs, self.shape, self.strides):
            if spec.step == 0 or spec.len == 0:
                raise LayoutError("empty slice")
            if spec.start + (spec.len - 1) * spec.step >= extent:
                raise LayoutError("slice out of range")
            offset += spec.start * stride
            shape.append(spec.len)
            strides.append(stride * spec.step)
        return Layout(self.dtype, offset, tuple(shape), tuple(strides), self.buffer_len)

    def permute(self, axes: Sequence[int]) -> "Layout":
        if sorted(axes) != list(range(self.rank)):
            raise LayoutError("permutation")
        return Layout(self.dtype, self.offset, tuple(self.shape[a] for a in axes),
                      tuple(self.strides[a] for a in axes), self.buffer_len)

    def broadcast(self, shape: Sequence[int]) -> "Layout":
        if len(shape) < self.rank:
            raise LayoutError("broadcast rank")
        pad = len(shape) - self.rank
        strides = []
        for axis, extent in enumerate(shape):
            if axis < pad:
                strides.append(0)
                continue
            own, stride = self.shape[axis - pad], self.strides[axis - pad]
            if own == extent:
                strides.append(stride)
            elif own == 1:
                strides.append(0)
            else:
                raise LayoutError("broadcast extent")
        return Layout(self.dtype, self.offset, tuple(shape), tuple(strides), self.buffer_len)

    def reshape(self, shape: Sequence[int]) -> "Layout":
        if not self.is_contiguous():
            raise LayoutError("reshape of a non-contiguous view")
        count = 1
        for extent in shape:
            count *= extent
        if count != self.element_count:
            raise LayoutError("reshape element count")
        return Layout.contiguous(self.dtype, self.offset, shape, self.buffer_len)


@dataclass(frozen=True)
class Tensor:
    """`Tensor` = (BufferId, Layout, writable)."""
    buffer: int
    layout: Layout
    writable: bool = True

    @property
    def shape(self):
        return self.layout.shape

    @property
    def dtype(self):
        return self.layout.dtype

    def with_layout(self, layout: Layout) -> "Tensor":
        return Tensor(self.buffer, layout, self.writable)

    # view helpers in the style of the SDK's tensor methods
    def slice(self, specs):
        return self.with_layout(self.layout.slice(specs))

    def narrow(self, axis: int, start: int, length: int) -> "Tensor":
        specs = [Slice(0, e) for e in self.shape]
        specs[axis] = Slice(start, length)
        return self.slice(specs)

    def permute(self, axes):
        return self.with_layout(self.layout.permute(axes))

    def broadcast(self, shape):
        return self.with_layout(self.layout.broadcast(shape))

    def reshape(self, shape):
        return self.with_layout(self.layout.reshape(shape))


# ---------------------------------------------------------------- scalar programs

class UnOp(enum.IntEnum):
    NEG = 0; ABS = 1; EXP = 2; LOG = 3; SQRT = 4; RSQRT = 5; SIN = 6; COS = 7; TANH = 8
    SIGMOID = 9; RECIP = 10; FLOOR = 11; LOG1P = 12; EXP_ROUNDED = 13


class BinOp(enum.IntEnum):
    ADD = 0; SUB = 1; MUL = 2; DIV = 3; MIN = 4; MAX = 5; POW = 6
    LT = 7; LE = 8; EQ = 9; NE = 10; GE = 11; GT = 12


class RedOp(enum.IntEnum):
    SUM = 0; MAX = 1; MIN = 2


class ValueType(enum.IntEnum):
    F32 = 0; U32 = 1; BOOL = 2


class ProgramKind(enum.IntEnum):
    MAP = 0; ROW = 1


@dataclass(frozen=True)
class Inst:
    kind: int
    op: int = 0
    a: int = 0
    b: int = 0
    c: int = 0

    @staticmethod
    def input(slot): return Inst(0, 0, slot)

    @staticmethod
    def const(value: float): return Inst(1, 0, struct.unpack("<I", struct.pack("<f", value))[0])

    @staticmethod
    def index(axis): return Inst(2, axis)

    @staticmethod
    def extent(axis): return Inst(3, axis)

    @staticmethod
    def unary(op, value): return Inst(4, int(op), value)

    @staticmethod
    def binary(op, left, right): return Inst(5, int(op), left, right)

    @staticmethod
    def select(cond, accepted, rejected): return Inst(6, 0, cond, accepted, rejected)

    @staticmethod
    def cast(to, value): return Inst(7, int(to), value)

    @staticmethod
    def reduce(op, value): return Inst(8, int(op), value)


@dataclass
class Program:
    kind: ProgramKind
    insts: List[Inst]
    outputs: List[Tuple[int, int]]  # (slot, value)

    @property
    def input_count(self) -> int:
        slots = [i.a for i in self.insts if i.kind == 0]
        return max(slots) + 1 if slots else 0

    @property
    def output_count(self) -> int:
        return max(slot for slot, _ in self.outputs) + 1


class ProgramBuilder:
    """Small SSA builder used by tests and drivers to write guest-style programs."""

    def __init__(self, kind: ProgramKind, rank_hint: int = 0):
        self.kind = kind
        self.insts: List[Inst] = []
        self.outputs: List[Tuple[int, int]] = []

    def _push(self, inst):
        self.insts.append(inst)
        return len(self.insts) - 1

    def input(self, slot): return self._push(Inst.input(slot))
    def const(self, value): return self._push(Inst.const(value))
    def index(self, axis): return self._push(Inst.index(axis))
    def extent(self, axis): return self._push(Inst.extent(axis))
    def unary(self, op, v): return self._push(Inst.unary(op, v))
    def binary(self, op, l, r): return self._push(Inst.binary(op, l, r))
    def add(self, l, r): return self.binary(BinOp.ADD, l, r)
    def sub(self, l, r): return self.binary(BinOp.SUB, l, r)
    def mul(self, l, r): return self.binary(BinOp.MUL, l, r)
    def div(self, l, r): return self.binary(BinOp.DIV, l, r)
    def select(self, c, a, r): return self._push(Inst.select(c, a, r))
    def cast(self, to, v): return self._push(Inst.cast(to, v))
    def reduce(self, op, v): return self._push(Inst.reduce(op, v))
    def output(self, slot, v): self.outputs.append((slot, v))
    def finish(self): return Program(self.kind, list(self.insts), list(self.outputs))


# ---------------------------------------------------------------- ops

class OpKind(enum.IntEnum):
    PROGRAM = 1
    COPY = 2
    PAGED_COPY = 3
    RMS_NORM = 4
    ARGMAX = 5
    TOP_K = 6
    ROPE = 7
    QUANT_EMBED = 8
    MATMUL = 9
    QUANT_MATMUL = 10
    GATHER_QUANT_MATMUL = 11
    PAGED_SDPA_APPEND = 12
    PAGED_SDPA = 13
    SAMPLE = 14
    SAMPLE_MASKED = 15
    PAGED_ATTENTION_RAGGED = 32
    ROUTE_PACK = 33
    FILL_SEEDED = 34


INTO_PAGES = 0
OUT_OF_PAGES = 1


@dataclass(frozen=True)
class Op:
    kind: OpKind
    scale: float = 0.0
    eps: float = 0.0
    theta: float = 0.0
    bits: int = 0
    group_size: int = 0
    k: int = 0
    normalize: bool = False
    causal: bool = False
    q_start: int = 0
    key_length: int = 0
    page_tokens: int = 0
    direction: int = 0
    start: int = 0

    @staticmethod
    def copy(): return Op(OpKind.COPY)

    @staticmethod
    def paged_copy(direction, start, page_tokens):
        return Op(OpKind.PAGED_COPY, direction=direction, start=start, page_tokens=page_tokens)

    @staticmethod
    def rms_norm(eps): return Op(OpKind.RMS_NORM, eps=eps)

    @staticmethod
    def argmax(): return Op(OpKind.ARGMAX)

    @staticmethod
    def top_k(k, normalize): return Op(OpKind.TOP_K, k=k, normalize=normalize)

    @staticmethod
    def sample(position): return Op(OpKind.SAMPLE, start=position)

    @staticmethod
    def sample_masked(position): return Op(OpKind.SAMPLE_MASKED, start=position)

    @staticmethod
    def rope(theta): return Op(OpKind.ROPE, theta=theta)

    @staticmethod
    def quant_embed(bits, group_size): return Op(OpKind.QUANT_EMBED, bits=bits, group_size=group_size)

    @staticmethod
    def matmul(): return Op(OpKind.MATMUL)

    @staticmethod
    def quant_matmul(bits, group_size): return Op(OpKind.QUANT_MATMUL, bits=bits, group_size=group_size)

    @staticmethod
    def gather_quant_matmul(bits, group_size):
        return Op(OpKind.GATHER_QUANT_MATMUL, bits=bits, group_size=group_size)

    @staticmethod
    def paged_sdpa_append(scale, q_start, page_tokens):
        return Op(OpKind.PAGED_SDPA_APPEND, scale=scale, q_start=q_start, page_tokens=page_tokens)

    @staticmethod
    def paged_sdpa(scale, causal, q_start, key_length, page_tokens):
        return Op(OpKind.PAGED_SDPA, scale=scale, causal=causal, q_start=q_start,
                  key_length=key_length, page_tokens=page_tokens)

    @staticmethod
    def paged_attention_ragged(scale, page_tokens, one_row_per_lane=False):
        """`one_row_per_lane`: the recorder's promise that no lane brings more than one query row
        (a decode batch); checked when the dispatch runs."""
        return Op(OpKind.PAGED_ATTENTION_RAGGED, scale=scale, page_tokens=page_tokens,
                  k=1 if one_row_per_lane else 0)

    @staticmethod
    def route_pack(tile_rows): return Op(OpKind.ROUTE_PACK, k=tile_rows)

    @staticmethod
    def fill_seeded(kind, seed, stream, first=0, lo=0.0, hi=0.0):
        return Op(OpKind.FILL_SEEDED, k=kind, q_start=seed & 0xffffffff, key_length=seed >> 32,
                  start=stream, direction=first, scale=lo, eps=hi)


@dataclass
class Dispatch:
    op: Op
    inputs: List[Tensor]
    outputs: List[Tensor]
    program: object = None     # prepared program handle (Op PROGRAM)
    epilogue: object = None    # prepared epilogue handle
    accumulator_count: int = 0
    n_extras: int = 0


class CommandList:
    """`CommandList` (crates/forja-core/src/ops.rs:1001-1053): an ordered list of dispatches."""

    def __init__(self):
        self.dispatches: List[Dispatch] = []

    def dispatch(self, op: Op, inputs: Sequence[Tensor], output: Tensor):
        self.dispatches.append(Dispatch(op, list(inputs), [output]))

    def dispatch_many(self, op: Op, inputs: Sequence[Tensor], outputs: Sequence[Tensor]):
        self.dispatches.append(Dispatch(op, list(inputs), list(outputs)))

    def dispatch_kernel(self, kernel, inputs: Sequence[Tensor], outputs: Sequence[Tensor]):
        self.dispatches.append(Dispatch(Op(OpKind.PROGRAM), list(inputs), list(outputs), program=kernel))

    def dispatch_epilogue(self, op: Op, inputs: Sequence[Tensor], output: Tensor, epilogue,
                          extras: Sequence[Tensor], accumulator_count: Optional[int] = None):
        if accumulator_count is None:
            accumulator_count = 2 if (op.kind == OpKind.GATHER_QUANT_MATMUL and len(inputs) == 8) else 1
        self.dispatches.append(Dispatch(op, list(inputs) + list(extras), [output], epilogue=epilogue,
                                        accumulator_count=accumulator_count, n_extras=len(extras)))

    def __len__(self):
        return len(self.dispatches)
