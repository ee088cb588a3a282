"""Weight import: a safetensors file becomes one read-only device buffer and its tensors become
views into it, the way the reference host does it (crates/forja-host/src/weights.rs:175-226 for
the validation, :76-87 for the layouts, `import_readonly(MappedRegion)` for the single buffer).

MLX 4-bit checkpoints name a quantised matrix `<prefix>.weight` (u32 [N, K/8], eight nibbles per
word, low nibble first), `<prefix>.scales` and `<prefix>.biases` (bf16 [N, K/group]); expert
matrices are stacked `[E, N, K/8]` under `switch_mlp.{gate,up,down}_proj`
(engines/qwen3-coder/src/lib.rs:430-437).  Nothing is re-tiled: `read` of an imported tensor
returns the file's bytes.
"""
from __future__ import annotations

import json
import mmap
import os
import struct
from dataclasses import dataclass
from typing import Dict, List, Tuple

from .core import DType, Layout, Tensor

# Prevents the length prefix from forcing an arbitrary allocation (weights.rs:17-20).
MAX_HEADER_BYTES = 100 * 1024 * 1024
_DTYPES = {"F32": DType.F32, "F16": DType.F16, "BF16": DType.BF16, "U32": DType.U32}


class WeightError(ValueError):
    """WeightError of the reference host (weights.rs:330-392); `kind` names the variant."""

    def __init__(self, kind: str, detail: str = ""):
        self.kind = kind
        super().__init__(f"{kind}: {detail}" if detail else kind)


@dataclass(frozen=True)
class WeightTensor:
    name: str
    dtype: DType
    shape: Tuple[int, ...]
    byte_offset: int   # in the data region
    byte_len: int

    @property
    def is_dtype_aligned(self) -> bool:
        return self.byte_offset % self.dtype.byte_size == 0


def _no_duplicates(pairs):
    seen = {}
    for name, value in pairs:
        if name in seen:
            raise WeightError("InvalidHeader", f"duplicate safetensors entry {name!r}")
        seen[name] = value
    return seen


def _parse_tensor(name: str, entry, data_len: int) -> WeightTensor:
    def bad(message):
        return WeightError("InvalidHeader", f"tensor {name!r}: {message}")
    if not isinstance(entry, dict):
        raise bad("entry is not an object")
    dtype_name = entry.get("dtype")
    if not isinstance(dtype_name, str):
        raise bad("dtype is missing")
    if dtype_name not in _DTYPES:
        raise WeightError("UnsupportedDtype", dtype_name)
    dtype = _DTYPES[dtype_name]
    shape = entry.get("shape")
    if not isinstance(shape, list):
        raise bad("shape is missing")
    for extent in shape:
        if not isinstance(extent, int) or isinstance(extent, bool) or not 0 <= extent < 2 ** 32:
            raise bad("shape extent is not a u32")
    offsets = entry.get("data_offsets")
    if not isinstance(offsets, list) or len(offsets) != 2:
        raise bad("data_offsets must contain two values")
    for offset in offsets:
        if not isinstance(offset, int) or isinstance(offset, bool) or not 0 <= offset < 2 ** 64:
            raise bad("data offset is not a u64")
    start, end = offsets
    if end < start:
        raise WeightError("InvalidRange")
    elements = 1
    for extent in shape:
        elements *= extent
    if elements * dtype.byte_size >= 2 ** 64 or end - start != elements * dtype.byte_size:
        raise WeightError("InvalidRange")
    if end > data_len:
        raise WeightError("Truncated")
    return WeightTensor(name, dtype, tuple(shape), start, end - start)


class SafetensorsFile:
    """A validated safetensors file (SafetensorsFile::open, weights.rs:175-226)."""

    def __init__(self, path: str):
        if os.path.islink(path) or not os.path.isfile(path):
            raise WeightError("NotRegularFile", path)
        self.path = path
        self.file_len = os.path.getsize(path)
        with open(path, "rb") as handle:
            prefix = handle.read(8)
            if len(prefix) != 8:
                raise WeightError("Truncated")
            header_len = struct.unpack("<Q", prefix)[0]
            if header_len > MAX_HEADER_BYTES:
                raise WeightError("HeaderTooLarge", str(header_len))
            header = handle.read(header_len)
            if len(header) != header_len:
                raise WeightError("Truncated")
        self.data_start = 8 + header_len
        data_len = self.file_len - self.data_start
        try:
            entries = json.loads(header, object_pairs_hook=_no_duplicates)
        except WeightError:
            raise
        except (ValueError, RecursionError) as error:
            raise WeightError("InvalidHeader", str(error)) from None
        if not isinstance(entries, dict):
            raise WeightError("InvalidHeader", "a safetensors metadata object is expected")
        tensors = [_parse_tensor(name, value, data_len) for name, value in entries.items()
                   if name != "__metadata__"]
        tensors.sort(key=lambda tensor: tensor.byte_offset)
        for left, right in zip(tensors, tensors[1:]):
            if left.byte_offset + left.byte_len > right.byte_offset:
                raise WeightError("OverlappingRanges")
        self.tensors: List[WeightTensor] = tensors
        self.data_len = data_len


class ImportedWeights:
    """The data region of one file as a single read-only allocation; tensors are views of it."""

    def __init__(self, backend, file: SafetensorsFile):
        self.file = file
        self._by_name: Dict[str, WeightTensor] = {tensor.name: tensor for tensor in file.tensors}
        with open(file.path, "rb") as handle:
            with mmap.mmap(handle.fileno(), 0, access=mmap.ACCESS_READ) as mapped:
                data = mapped[file.data_start:]
        data += bytes(-len(data) % 4)      # the whole-buffer tensor below is counted in u32 words
        self._whole = backend.import_readonly(data, DType.U32, (len(data) // 4,))
        self.buffer = self._whole.buffer
        self.byte_len = len(data)

    def names(self):
        return list(self._by_name)

    def tensor(self, name: str, shape=None) -> Tensor:
        """The named tensor as a view of the imported buffer; `shape`, when given, must be what
        the file declares (Weights::tensor of the SDK refuses a mismatch)."""
        if name not in self._by_name:
            raise KeyError(name)
        entry = self._by_name[name]
        if shape is not None and tuple(shape) != entry.shape:
            raise WeightError("Shape", f"{name}: file has {entry.shape}, caller expects {tuple(shape)}")
        if not entry.is_dtype_aligned:
            raise WeightError("Misaligned", name)
        layout = Layout.contiguous(entry.dtype, entry.byte_offset // entry.dtype.byte_size, entry.shape,
                                   self.byte_len)
        return Tensor(self.buffer, layout, False)

    def quantised(self, prefix: str):
        """(packed u32, scales, biases) of the matrix, or stack of expert matrices, at `prefix`."""
        packed = self.tensor(prefix + ".weight")
        scales = self.tensor(prefix + ".scales")
        biases = self.tensor(prefix + ".biases")
        if packed.dtype != DType.U32 or scales.dtype != biases.dtype or scales.shape != biases.shape:
            raise WeightError("Shape", f"{prefix}: not an MLX affine-quantised triple")
        if packed.shape[:-1] != scales.shape[:-1]:
            raise WeightError("Shape", f"{prefix}: scales do not match the packed rows")
        return packed, scales, biases


def import_safetensors(backend, path: str) -> ImportedWeights:
    return ImportedWeights(backend, SafetensorsFile(path))
