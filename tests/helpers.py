"""Shared helpers for the parity tests: seeded operands, quantised weight builders and the
comparison rules (support/forja-testing/src/lib.rs:22-29, :481-565 plus the elementwise
rel 1e-2 / abs 1e-2 rule for bf16 outputs)."""
import numpy as np

from forja_amd.core import DType
from oracle import cpu_backend as orc

NP_OF = {DType.F32: np.float32, DType.F16: np.float16, DType.BF16: np.uint16, DType.U32: np.uint32,
         DType.I32: np.int32}


def to_f32(raw: bytes, dtype: DType) -> np.ndarray:
    if dtype == DType.F32:
        return np.frombuffer(raw, dtype=np.float32).copy()
    if dtype == DType.F16:
        return np.frombuffer(raw, dtype=np.float16).astype(np.float32)
    if dtype == DType.BF16:
        return orc.bf16_to_f32(np.frombuffer(raw, dtype=np.uint16))
    raise ValueError(dtype)


def from_f32(values: np.ndarray, dtype: DType) -> bytes:
    return orc.encode(np.asarray(values, dtype=np.float32).ravel(), dtype).tobytes()


def upload(backend, values, dtype: DType, shape=None):
    """Allocates a tensor and writes `values` (float array, or integer array for U32)."""
    values = np.asarray(values)
    shape = tuple(values.shape if shape is None else shape)
    tensor = backend.alloc(dtype, shape)
    if dtype in (DType.U32, DType.I32):
        backend.write(tensor, np.ascontiguousarray(values, dtype=NP_OF[dtype]).tobytes())
    else:
        backend.write(tensor, from_f32(values, dtype))
    return tensor


def upload_raw(backend, raw: np.ndarray, dtype: DType, shape):
    tensor = backend.alloc(dtype, tuple(shape))
    backend.write(tensor, np.ascontiguousarray(raw).tobytes())
    return tensor


def both(backends, fn):
    return [fn(b) for b in backends]


class Quantised:
    """Random MLX-affine weights: packed words uniform over u32, bf16 scale~U(0.001,0.02),
    bf16 bias~U(-0.1,0.1)."""

    def __init__(self, seed, stream, shape_nk, bits=4, group=64, experts=None):
        n, k = shape_nk
        lead = () if experts is None else (experts,)
        total_rows = n * (experts or 1)
        self.bits, self.group = bits, group
        self.packed = orc.fill_words(seed, stream, total_rows * k * bits // 32).reshape(lead + (n, k * bits // 32))
        self.scales = orc.fill_uniform_bf16(seed, stream + 1, total_rows * (k // group), 0.001, 0.02).reshape(lead + (n, k // group))
        self.biases = orc.fill_uniform_bf16(seed, stream + 2, total_rows * (k // group), -0.1, 0.1).reshape(lead + (n, k // group))

    def upload(self, backend, scale_dtype=DType.BF16):
        packed = upload_raw(backend, self.packed, DType.U32, self.packed.shape)
        if scale_dtype == DType.BF16:
            scales = upload_raw(backend, self.scales, DType.BF16, self.scales.shape)
            biases = upload_raw(backend, self.biases, DType.BF16, self.biases.shape)
        else:
            scales = upload(backend, orc.bf16_to_f32(self.scales), scale_dtype, self.scales.shape)
            biases = upload(backend, orc.bf16_to_f32(self.biases), scale_dtype, self.biases.shape)
        return packed, scales, biases

    def dequantised(self) -> np.ndarray:
        """float64 dense weights [.., N, K] (independent of the oracle's C code)."""
        vpw = 32 // self.bits
        shifts = (np.arange(vpw, dtype=np.uint32) * self.bits)
        q = (self.packed[..., None] >> shifts) & ((1 << self.bits) - 1)
        q = q.reshape(self.packed.shape[:-1] + (-1,)).astype(np.float64)
        s = np.repeat(orc.bf16_to_f32(self.scales).astype(np.float64), self.group, axis=-1)
        b = np.repeat(orc.bf16_to_f32(self.biases).astype(np.float64), self.group, axis=-1)
        return s * q + b


def normal_bf16(seed, stream, shape):
    count = int(np.prod(shape))
    return orc.bf16_to_f32(orc.fill_normal_bf16(seed, stream, count)).reshape(shape)


def assert_close(candidate, reference, dtype: DType, rel=1e-2, abs_=1e-2, norm_tol=None):
    """Elementwise |c-r| <= abs + rel*|r| (the stated bf16 bar) and the reference's normwise
    relative error bound for the dtype."""
    candidate = np.asarray(candidate, dtype=np.float64).ravel()
    reference = np.asarray(reference, dtype=np.float64).ravel()
    assert candidate.shape == reference.shape
    assert np.array_equal(np.isnan(candidate), np.isnan(reference))
    finite = np.isfinite(reference)
    assert np.array_equal(candidate[~finite & ~np.isnan(reference)], reference[~finite & ~np.isnan(reference)])
    c, r = candidate[finite], reference[finite]
    if dtype == DType.F32:
        # f32 sums differ by their order of summation: eps times the size of the terms, which for
        # outputs that cancel is set by the typical output, not by the element itself
        scale = float(np.sqrt(np.mean(r * r))) if r.size else 0.0
        rel, abs_ = 1e-4, 1e-5 * max(1.0, scale)
    error = np.abs(c - r)
    bound = abs_ + rel * np.abs(r)
    worst = int(np.argmax(error - bound)) if error.size else 0
    assert np.all(error <= bound), f"elementwise: |{c[worst]} - {r[worst]}| = {error[worst]} > {bound[worst]}"
    if norm_tol is None:
        norm_tol = {DType.F32: 1e-5, DType.F16: 2e-3, DType.BF16: 1e-2}[dtype]
    denom = np.linalg.norm(r)
    if denom > 0:
        assert np.linalg.norm(c - r) / denom <= norm_tol, f"normwise {np.linalg.norm(c - r) / denom}"
