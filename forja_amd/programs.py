"""The guest scalar programs the qwen3 / qwen3-coder engines dispatch on the forward step,
written in the Program IR exactly as the SDK's `#[kernel]` functions lower them
(crates/forja-sdk/src/nn/blocks.rs:380-443, engines/qwen3-coder/src/lib.rs:26-40).
Scalars (epsilon, head_dim, theta) are baked in as constants, as the SDK does.
"""
from .core import BinOp, ProgramBuilder, ProgramKind, RedOp, UnOp, ValueType


def _row_mean(b: ProgramBuilder, value: int, axis: int) -> int:
    # RowCtx::row_mean = row_sum / extent(-1) as f32 (crates/forja-sdk/src/program.rs:445-447)
    total = b.reduce(RedOp.SUM, value)
    return b.div(total, b.cast(ValueType.F32, b.extent(axis)))


def rms_norm_rows(epsilon: float, rank: int = 2):
    """blocks.rs:392-400: inputs (input, weight) -> input * rsqrt(mean(input^2)+eps) * weight"""
    b = ProgramBuilder(ProgramKind.ROW)
    x, w = b.input(0), b.input(1)
    mean = _row_mean(b, b.mul(x, x), rank - 1)
    inverse = b.unary(UnOp.RSQRT, b.add(mean, b.const(epsilon)))
    b.output(0, b.mul(b.mul(x, inverse), w))
    return b.finish()


def residual_norm_rows(epsilon: float, rank: int = 2):
    """blocks.rs:380-390: inputs (residual, update, weight) -> (value, value*rsqrt(..)*weight)"""
    b = ProgramBuilder(ProgramKind.ROW)
    residual, update, w = b.input(0), b.input(1), b.input(2)
    value = b.add(residual, update)
    mean = _row_mean(b, b.mul(value, value), rank - 1)
    inverse = b.unary(UnOp.RSQRT, b.add(mean, b.const(epsilon)))
    b.output(0, value)
    b.output(1, b.mul(b.mul(value, inverse), w))
    return b.finish()


def qk_norm_rope_rows(head_dim: float, epsilon: float, theta: float, rank: int = 3):
    """blocks.rs:421-443: inputs (lo, hi, weight_lo, weight_hi, positions) over [rows, heads, D/2]."""
    b = ProgramBuilder(ProgramKind.ROW)
    lo, hi, w_lo, w_hi, positions = (b.input(i) for i in range(5))
    square_sum = b.reduce(RedOp.SUM, b.add(b.mul(lo, lo), b.mul(hi, hi)))
    inverse = b.unary(UnOp.RSQRT, b.add(b.div(square_sum, b.const(head_dim)), b.const(epsilon)))
    n_lo = b.mul(b.mul(lo, inverse), w_lo)
    n_hi = b.mul(b.mul(hi, inverse), w_hi)
    exponent = b.mul(b.cast(ValueType.F32, b.index(rank - 1)), b.const(-2.0 / head_dim))
    angle = b.mul(positions, b.binary(BinOp.POW, b.const(theta), exponent))
    cosine, sine = b.unary(UnOp.COS, angle), b.unary(UnOp.SIN, angle)
    b.output(0, b.sub(b.mul(n_lo, cosine), b.mul(n_hi, sine)))
    b.output(1, b.add(b.mul(n_hi, cosine), b.mul(n_lo, sine)))
    return b.finish()


def silu_mul_elements():
    """blocks.rs:413-416 / moe_gate_up (engines/qwen3-coder/src/lib.rs:26-32): gate*sigmoid(gate)*up"""
    b = ProgramBuilder(ProgramKind.MAP)
    gate, up = b.input(0), b.input(1)
    b.output(0, b.mul(b.mul(gate, b.unary(UnOp.SIGMOID, gate)), up))
    return b.finish()


def add_elements():
    """blocks.rs:408-411 / moe_add_residual (engines/qwen3-coder/src/lib.rs:34-40)"""
    b = ProgramBuilder(ProgramKind.MAP)
    b.output(0, b.add(b.input(0), b.input(1)))
    return b.finish()


def centered_bias_elements(bits: int = 4):
    """bias = noise - ((2^bits - 1) / 2) * scale: the affine bias that centres the quantised values
    0..2^bits-1 on zero (the zero-mean weight law of the model-level tests; not a reference
    program)."""
    b = ProgramBuilder(ProgramKind.MAP)
    scale, noise = b.input(0), b.input(1)
    b.output(0, b.add(b.mul(scale, b.const(-((1 << bits) - 1) / 2.0)), noise))
    return b.finish()
