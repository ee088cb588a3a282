"""Differential tests: the HIP library (through the C ABI) against the CPU oracle on identical
seeded bytes, in the manner of crates/forja-metal/tests/*.rs (CpuBackend = reference,
candidate = device backend).  Integer results are bit-exact; float results meet the elementwise
rel 1e-2 / abs 1e-2 bar and the reference's normwise bound for the dtype."""
import math

import numpy as np
import pytest

from forja_amd import programs
from forja_amd.core import (BackendError, BinOp, CommandList, DType, Inst, Layout, Op, Program,
                            ProgramBuilder, ProgramKind, RedOp, Slice, Status, UnOp, ValueType,
                            INTO_PAGES, OUT_OF_PAGES)
from oracle import cpu_backend as orc
from tests.helpers import (Quantised, assert_close, from_f32, normal_bf16, to_f32, upload,
                           upload_raw)
from tests.test_oracle_golden import paged_case, top_k_case

pytestmark = pytest.mark.gpu


def run(backend, commands):
    backend.submit(commands).wait()


def coarser(*dtypes):
    """The dtype whose tolerance judges an attention output: the reference holds f32 outputs
    computed from f16 or bf16 pools to the pools' tolerance (crates/forja-metal/tests/paged.rs:982-988)."""
    return max(dtypes, key=[DType.F32, DType.F16, DType.BF16].index)


def compare(cpu, hip, cpu_tensor, hip_tensor, bar=None, **kw):
    """`bar`: the dtype whose tolerance applies to float outputs (their own when not given)."""
    dtype = cpu_tensor.dtype
    a, b = cpu.read(cpu_tensor), hip.read(hip_tensor)
    if dtype in (DType.U32, DType.I32):
        assert a == b
    else:
        assert_close(to_f32(b, dtype), to_f32(a, dtype), coarser(dtype, bar or dtype), **kw)


def differential(cpu, hip, build, expect_error=None, **kw):
    """build(backend) -> (commands, [outputs]); runs on both and compares every output."""
    results = []
    for backend in (cpu, hip):
        commands, outputs = build(backend)
        error = None
        try:
            run(backend, commands)
        except BackendError as e:
            error = e
        results.append((outputs, error))
    (cpu_out, cpu_err), (hip_out, hip_err) = results
    if expect_error is None:
        assert cpu_err is None and hip_err is None, (cpu_err, hip_err)
    else:
        assert cpu_err is not None and hip_err is not None
        assert hip_err.status in expect_error
    for a, b in zip(cpu_out, hip_out):
        compare(cpu, hip, a, b, **kw)
    return results


# ------------------------------------------------------------------ device info / storage

def test_device_is_gfx950_and_storage_round_trips(hip):
    info = hip.device_info()
    assert info["family"].startswith("gfx950"), info
    assert info["wavefront"] == 64
    t = hip.alloc(DType.U32, (5, 7))
    assert hip.read(t) == bytes(5 * 7 * 4)                      # zero-initialised
    data = np.arange(35, dtype=np.uint32)
    hip.write(t, data.tobytes())
    assert np.frombuffer(hip.read(t), np.uint32).tolist() == data.tolist()
    view = t.slice([Slice(1, 2, 2), Slice(0, 3, 3)]).permute([1, 0])
    assert np.frombuffer(hip.read(view), np.uint32).tolist() == data.reshape(5, 7)[1::2, 0::3][:2, :3].T.ravel().tolist()
    with pytest.raises(BackendError):
        hip.write(view, bytes(24))                              # non-contiguous write refused
    hip.release(t)
    with pytest.raises(BackendError):
        hip.read(t)                                             # released allocation


def test_submit_refuses_foreign_tensors_and_bad_shapes(hip):
    x = hip.alloc(DType.BF16, (4, 64))
    out = hip.alloc(DType.BF16, (4, 8))
    packed = hip.alloc(DType.U32, (8, 8))
    scales, biases = hip.alloc(DType.BF16, (8, 1)), hip.alloc(DType.BF16, (8, 1))
    wrong = hip.alloc(DType.BF16, (4, 9))
    commands = CommandList()
    commands.dispatch(Op.quant_matmul(4, 64), [x, packed, scales, biases], wrong)
    with pytest.raises(BackendError) as info:
        hip.submit(commands)
    assert info.value.status == Status.INVALID_INPUT
    hip.release(scales)
    commands = CommandList()
    commands.dispatch(Op.quant_matmul(4, 64), [x, packed, scales, biases], out)
    with pytest.raises(BackendError):
        hip.submit(commands)


def test_seeded_fill_matches_the_host_generator_bit_for_bit(cpu, hip):
    def build(backend):
        words = backend.alloc(DType.U32, (3, 1000))
        uniform = backend.alloc(DType.BF16, (777,))
        normal = backend.alloc(DType.BF16, (5, 999))
        normal32 = backend.alloc(DType.F32, (4096,))
        commands = CommandList()
        commands.dispatch(Op.fill_seeded(0, 0x1234_5678_9abc, 3, first=17), [], words)
        commands.dispatch(Op.fill_seeded(1, 99, 4, lo=0.001, hi=0.02), [], uniform)
        commands.dispatch(Op.fill_seeded(2, 99, 5, first=1 << 20), [], normal)
        commands.dispatch(Op.fill_seeded(2, 7, 6), [], normal32)
        return commands, [words, uniform, normal, normal32]
    (cpu_out, _), (hip_out, _) = differential(cpu, hip, build)
    for a, b in zip(cpu_out, hip_out):
        assert cpu.read(a) == hip.read(b)


def test_kernel_timers_follow_the_selected_classes(hip):
    """fh_profile_select: only the selected kernel classes are timed (class 6 = the kernels of a
    dense quantised product)."""
    weights = Quantised(20, 1, (64, 256))
    x = upload(hip, normal_bf16(20, 2, (8, 256)), DType.BF16)
    out = hip.alloc(DType.BF16, (8, 64))
    commands = CommandList()
    commands.dispatch(Op.quant_matmul(4, 64), [x, *weights.upload(hip)], out)
    try:
        hip.profile_enable(1)
        for mask, expected in ((1 << 4, 0), (1 << 6, 1), (0xffffffff, 1)):
            hip.profile_select(mask)
            hip.profile_reset()
            run(hip, commands)
            nanoseconds, launches = hip.profile_read(6)
            assert launches == expected and (nanoseconds > 0) == (expected > 0)
        # fh_profile_sample: one launch in three is timed
        hip.profile_sample(3)
        hip.profile_reset()
        for _ in range(7):
            run(hip, commands)
        assert hip.profile_read(6)[1] == 3
    finally:
        hip.profile_sample(1)
        hip.profile_select(0xffffffff)
        hip.profile_enable(0)


# ------------------------------------------------------------------ quantised matmul

QMM_CASES = [
    # rows, N, K, bits, group, activation dtype
    (1, 64, 64, 4, 64, DType.F32),
    (7, 48, 128, 4, 64, DType.BF16),
    (33, 40, 256, 4, 64, DType.BF16),
    (4, 4096, 1024, 4, 64, DType.BF16),     # C0 stacked qkv
    (4, 1024, 3072, 4, 64, DType.BF16),     # C0 down
    (128, 160, 2048, 4, 64, DType.BF16),    # C3 row count, narrow N
    (128, 128, 2048, 8, 64, DType.BF16),    # router (q8 in the reference engine)
    (5, 24, 256, 4, 32, DType.F16),
    (3, 24, 256, 8, 128, DType.F32),
    (40, 72, 192, 4, 64, DType.BF16),
    (1, 2048, 2048, 4, 64, DType.BF16),
    (64, 100, 512, 4, 64, DType.BF16),      # column tail inside a wave
    (130, 96, 768, 4, 64, DType.BF16),      # row tail across row blocks
    (8, 512, 4096, 4, 64, DType.BF16),
    (128, 5120, 2048, 4, 64, DType.BF16),   # C3 stacked qkv: packed-activation path, 2 splits
    (128, 2048, 4096, 4, 64, DType.BF16),   # C3 o_proj: 4 splits
    (100, 130, 2048, 4, 64, DType.BF16),    # row and column tails, 8 splits
    (64, 96, 256, 4, 64, DType.BF16),       # a single group per wave, no split
    (65, 32, 3072, 4, 64, DType.BF16),      # 12 splits
    (192, 4096, 2048, 4, 64, DType.BF16),   # more rows than the decode path takes: tiled GEMM
    (257, 300, 512, 4, 64, DType.BF16),     # GEMM with row and column tails
    (1000, 96, 256, 4, 64, DType.BF16),     # GEMM, a single column tile, four row tiles
    (512, 1024, 2048, 4, 64, DType.BF16),   # GEMM, whole tiles
    # f32 / f16 activations and 8-bit weights: the f32 vector-ALU kernel
    (8, 5120, 2048, 4, 64, DType.F32),      # the qwen3-coder engine's decode batch: stacked qkv
    (8, 128, 2048, 8, 64, DType.F32),       # its 8-bit router
    (128, 2048, 4096, 4, 64, DType.F32),    # o_proj on a full decode batch
    (19, 130, 1056, 4, 32, DType.F16),      # row, column and wave tails; 33 pieces over 8 waves
    (70, 200, 384, 8, 128, DType.F16),
    (3, 70, 32, 4, 32, DType.F32),          # a single piece: one wave
    (300, 96, 256, 8, 32, DType.BF16),      # prefill rows with 8-bit weights
]


@pytest.mark.parametrize("rows,n,k,bits,group,dtype", QMM_CASES)
def test_quant_matmul(cpu, hip, rows, n, k, bits, group, dtype):
    weights = Quantised(21, 100 + n + k, (n, k), bits=bits, group=group)
    x_values = normal_bf16(21, 7, (rows, k))

    def build(backend):
        x = upload(backend, x_values, dtype)
        packed, scales, biases = weights.upload(backend)
        out = backend.alloc(dtype, (rows, n))
        commands = CommandList()
        commands.dispatch(Op.quant_matmul(bits, group), [x, packed, scales, biases], out)
        return commands, [out]
    differential(cpu, hip, build)


@pytest.mark.parametrize("rows,n,k,residual", [(8, 5120, 2048, False), (1, 2048, 768, False), (16, 768, 2048, True),
                                               (20, 2048, 1024, True), (31, 96, 512, False),
                                               (8, 2048, 4096, True), (24, 512, 4096, False)])   # o_proj: two K ranges
def test_quant_matmul_on_f32_activations_that_use_their_whole_mantissa(cpu, hip, rows, n, k, residual):
    """The engines' activations are f32 (engines/qwen3-coder/src/lib.rs:296-437) and carry 24
    significant bits, unlike the bf16-valued inputs of the cases above: a kernel that rounded them
    to bf16, or to two bf16 pieces, on its way to the matrix cores would miss the f32 bar."""
    weights = Quantised(25, n + k, (n, k))
    x_values = orc.fill_normal_f32(25, 1, rows * k).reshape(rows, k)
    extra_values = orc.fill_normal_f32(25, 2, rows * n).reshape(rows, n)

    def build(backend):
        x = upload(backend, x_values, DType.F32)
        out = backend.alloc(DType.F32, (rows, n))
        commands = CommandList()
        if residual:
            extra = upload(backend, extra_values, DType.F32)
            add = backend.prepare_epilogue(programs.add_elements())
            commands.dispatch_epilogue(Op.quant_matmul(4, 64), [x, *weights.upload(backend)], out, add, [extra])
        else:
            commands.dispatch(Op.quant_matmul(4, 64), [x, *weights.upload(backend)], out)
        return commands, [out]
    differential(cpu, hip, build)


@pytest.mark.parametrize("rows,k,experts,n,inner", [(8, 8, 128, 768, 2048), (3, 4, 16, 512, 1024), (40, 2, 64, 256, 512)])
def test_routed_products_on_f32_activations_that_use_their_whole_mantissa(cpu, hip, rows, k, experts, n, inner):
    """The MoE block of a small decode batch in the engine's dtypes: gate/up pair with SwiGLU, the
    down projection as a weighted sum with the residual, all f32."""
    gate = Quantised(26, 1, (n, inner), experts=experts)
    up = Quantised(26, 11, (n, inner), experts=experts)
    down = Quantised(26, 21, (inner, n), experts=experts)
    indices = routed_case(26, rows, k, experts, n, inner)
    x_values = orc.fill_normal_f32(26, 40, rows * inner).reshape(rows, inner)
    logits = orc.fill_normal_f32(26, 41, rows * k).reshape(rows, k)
    w_values = np.exp(logits) / np.exp(logits).sum(axis=1, keepdims=True)
    residual_values = orc.fill_normal_f32(26, 42, rows * inner).reshape(rows, inner)

    def build(backend):
        x = upload(backend, x_values, DType.F32)
        idx = upload(backend, indices, DType.U32)
        g, u, d = gate.upload(backend), up.upload(backend), down.upload(backend)
        plain = backend.alloc(DType.F32, (rows, k, n))
        activated = backend.alloc(DType.F32, (rows, k, n))
        combined = backend.alloc(DType.F32, (rows, inner))
        weights = upload(backend, w_values, DType.F32)
        residual = upload(backend, residual_values, DType.F32)
        swiglu = backend.prepare_epilogue(programs.silu_mul_elements())
        add = backend.prepare_epilogue(programs.add_elements())
        commands = CommandList()
        commands.dispatch(Op.gather_quant_matmul(4, 64), [x, *g, idx], plain)
        commands.dispatch_epilogue(Op.gather_quant_matmul(4, 64), [x, *g, *u, idx], activated, swiglu, [])
        commands.dispatch_epilogue(Op.gather_quant_matmul(4, 64), [activated, *d, idx, weights], combined,
                                   add, [residual])
        return commands, [plain, activated, combined]
    differential(cpu, hip, build)


@pytest.mark.parametrize("dtype,bits,group", [(DType.F32, 4, 64), (DType.F16, 8, 32), (DType.BF16, 4, 128)])
def test_quant_matmul_with_f16_scales_and_a_residual_in_other_dtypes(cpu, hip, dtype, bits, group):
    """f16 affine parameters (the reference allows f16 or bf16, quantized.rs:78-121) and the
    residual-add epilogue on activations that are not bf16, plus an unrecognised epilogue."""
    rows, n, k = 40, 200, 768
    weights = Quantised(24, n + k, (n, k), bits=bits, group=group)
    x_values = normal_bf16(24, 1, (rows, k))
    extra_values = normal_bf16(24, 2, (rows, n))

    def build(backend):
        x = upload(backend, x_values, dtype)
        extra = upload(backend, extra_values, dtype)
        plain, added, scaled = (backend.alloc(dtype, (rows, n)) for _ in range(3))
        triple = weights.upload(backend, scale_dtype=DType.F16)
        b = ProgramBuilder(ProgramKind.MAP)
        b.output(0, b.mul(b.input(0), b.input(1)))
        commands = CommandList()
        commands.dispatch(Op.quant_matmul(bits, group), [x, *triple], plain)
        commands.dispatch_epilogue(Op.quant_matmul(bits, group), [x, *triple], added,
                                   backend.prepare_epilogue(programs.add_elements()), [extra])
        commands.dispatch_epilogue(Op.quant_matmul(bits, group), [x, *triple], scaled,
                                   backend.prepare_epilogue(b.finish()), [extra])
        return commands, [plain, added, scaled]
    differential(cpu, hip, build)


def test_quant_gemm_with_scales_outside_the_fp16_range_and_huge_activations(cpu, hip):
    """Prefill-sized product whose affine parameters are not fp16 normal numbers (tiny scales, a
    zero bias, a large scale) and whose activations exceed the fp16 range in some rows: the
    f32 dequantisation path and the per-row power-of-two scaling."""
    rows, n, k = 300, 200, 512
    weights = Quantised(61, 3, (n, k))
    scales = orc.bf16_to_f32(weights.scales).copy()
    biases = orc.bf16_to_f32(weights.biases).copy()
    scales[::3, 0] = 3.0e-6
    scales[1::7, 1] = 7000.0
    biases[::5, 2] = 0.0
    biases[2::5, 3] = 1.0e-7
    weights.scales = orc.f32_to_bf16(scales.ravel()).reshape(scales.shape)
    weights.biases = orc.f32_to_bf16(biases.ravel()).reshape(biases.shape)
    x_values = orc.bf16_to_f32(normal_bf16(61, 9, (rows, k))).copy()
    x_values[5] *= 3.0e6
    x_values[17, 3] = 1.0e9
    x_values[40] *= 1.0e-6

    def build(backend):
        x = upload(backend, x_values, DType.BF16)
        packed, sc, bi = weights.upload(backend)
        out = backend.alloc(DType.BF16, (rows, n))
        commands = CommandList()
        commands.dispatch(Op.quant_matmul(4, 64), [x, packed, sc, bi], out)
        return commands, [out]
    differential(cpu, hip, build)


def test_quant_matmul_on_strided_views_with_bias_epilogue(cpu, hip):
    """Every operand sliced with step 2 (crates/forja-metal/tests/quant_matmul/shared.rs:95-107)
    plus a fused epilogue that adds a broadcast bias."""
    rows, n, k = 6, 32, 128
    weights = Quantised(22, 5, (2 * n, 2 * k), bits=4, group=64)
    x_values = normal_bf16(22, 8, (2 * rows, 2 * k))
    bias_values = normal_bf16(22, 9, (n,))

    def build(backend):
        x = upload(backend, x_values, DType.BF16).slice([Slice(0, rows, 2), Slice(0, k)])
        packed, scales, biases = weights.upload(backend)
        packed = packed.slice([Slice(1, n, 2), Slice(0, k // 8)])
        scales = scales.slice([Slice(1, n, 2), Slice(0, k // 64)])
        biases = biases.slice([Slice(1, n, 2), Slice(0, k // 64)])
        big = backend.alloc(DType.BF16, (rows, 2 * n))
        out = big.slice([Slice(0, rows), Slice(1, n, 2)])
        bias = upload(backend, bias_values, DType.BF16).broadcast((rows, n))
        epilogue = backend.prepare_epilogue(programs.add_elements())
        commands = CommandList()
        commands.dispatch_epilogue(Op.quant_matmul(4, 64), [x, packed, scales, biases], out, epilogue, [bias])
        return commands, [big]
    differential(cpu, hip, build)


def test_prefill_products_follow_weights_that_are_rewritten(cpu, hip):
    """Products of more than 128 rows keep a prepared copy of their weights from one product to the
    next.  The copy must go when any of the three tensors is written: by the host, by a dispatch,
    or when the allocation is released and its memory taken by other weights."""
    rows, n, k = 200, 320, 512
    first, second, third = (Quantised(27, seed, (n, k)) for seed in (1, 2, 3))
    x_values = normal_bf16(27, 9, (rows, k))

    def build(backend):
        x = upload(backend, x_values, DType.BF16)
        packed, scales, biases = first.upload(backend)
        outs = [backend.alloc(DType.BF16, (rows, n)) for _ in range(5)]
        op = Op.quant_matmul(4, 64)

        def product(out, triple):
            commands = CommandList()
            commands.dispatch(op, [x, *triple], out)
            run(backend, commands)
        product(outs[0], (packed, scales, biases))
        product(outs[1], (packed, scales, biases))                      # the kept copy serves
        backend.write(scales, np.ascontiguousarray(second.scales).tobytes())   # written by the host
        product(outs[2], (packed, scales, biases))
        commands = CommandList()                                        # written by a dispatch
        commands.dispatch(Op.copy(), [upload_raw(backend, third.packed, DType.U32, third.packed.shape)], packed)
        commands.dispatch(op, [x, packed, scales, biases], outs[3])
        run(backend, commands)
        for tensor in (packed, scales, biases):                         # released: the memory may come back
            backend.release(tensor)
        product(outs[4], second.upload(backend))
        return CommandList(), outs
    differential(cpu, hip, build)


def test_prefill_products_without_kept_weights(cpu, monkeypatch):
    """FORJA_HIP_PREPARED_MB=0: nothing is kept, every product prepares its weights into the
    workspace and stands by with the conditioned second kernel, as it does when the memory set
    aside for kept weights is used up."""
    from forja_amd.hip_backend import HipBackend
    monkeypatch.setenv("FORJA_HIP_PREPARED_MB", "0")
    frugal = HipBackend(0)
    try:
        rows, n, k = 300, 520, 512
        weights = Quantised(28, 1, (n, k))
        x_values = normal_bf16(28, 2, (rows, k))

        def build(backend):
            x = upload(backend, x_values, DType.BF16)
            triple = weights.upload(backend)
            outs = [backend.alloc(DType.BF16, (rows, n)) for _ in range(2)]
            commands = CommandList()
            for out in outs:
                commands.dispatch(Op.quant_matmul(4, 64), [x, *triple], out)
            return commands, outs
        differential(cpu, frugal, build)
    finally:
        frugal.close()


def test_memory_limit_counts_and_evicts_what_the_library_keeps(cpu):
    """`Backend::set_memory_limit` (crates/forja-core/src/backend.rs:683-686) covers the caller's
    allocations and the operands the library keeps for prefill products; `memory_usage` counts
    both.  An allocation that would pass the limit drops the kept operands first and succeeds;
    one that cannot fit is refused with QuotaExceeded; results do not depend on any of it."""
    from forja_amd.hip_backend import HipBackend
    own = HipBackend(0)     # its own backend: the shared one holds other tests' allocations
    try:
        rows, n, k = 200, 2048, 512
        weights = Quantised(29, 1, (n, k))
        x_values = normal_bf16(29, 2, (rows, k))
        kept = n * 64 * 2 + 256     # fp16 bias columns (3 per group of 64, padded to 64 a row) + flag
        names = ("kept", "served by the kept operand", "prepared into workspace", "kept again")
        x = upload(own, x_values, DType.BF16)
        triple = weights.upload(own)
        outs = {name: own.alloc(DType.BF16, (rows, n)) for name in names}
        allocated = sum(t.layout.buffer_len for t in (x, *triple, *outs.values()))

        def product(backend, x, triple, out):
            commands = CommandList()
            commands.dispatch(Op.quant_matmul(4, 64), [x, *triple], out)
            run(backend, commands)
        before = own.memory_usage()
        assert before >= allocated
        product(own, x, triple, outs["kept"])
        held = own.memory_usage()
        assert held >= before + kept                       # the kept operand is counted (and the workspace)
        product(own, x, triple, outs["served by the kept operand"])
        assert own.memory_usage() == held
        # room for half the kept operand more: an allocation of its size fits only once it is dropped
        own.set_memory_limit(allocated + kept + kept // 2)
        extra = own.alloc(DType.U32, ((kept - 256) // 4,))
        assert own.memory_usage() == held - kept + (kept - 256)
        product(own, x, triple, outs["prepared into workspace"])     # no room to keep anything
        assert own.memory_usage() <= held + (kept - 256)
        with pytest.raises(BackendError) as refused:
            own.alloc(DType.U32, (kept,))
        assert refused.value.status == Status.QUOTA_EXCEEDED
        own.set_memory_limit(0)
        own.release(extra)
        product(own, x, triple, outs["kept again"])
        assert own.memory_usage() >= held
        expected = cpu.alloc(DType.BF16, (rows, n))
        product(cpu, upload(cpu, x_values, DType.BF16), weights.upload(cpu), expected)
        for name in names:
            compare(cpu, own, expected, outs[name])
    finally:
        own.close()


def test_profiled_submission_reports_an_ordered_timeline(hip):
    """`submit_profiled_retained` / `Submission::profile` (crates/forja-core/src/backend.rs:455-579):
    one entry per executed dispatch, in order, intervals that do not overlap, inside the
    submission's device time."""
    weights = Quantised(30, 1, (512, 1024))
    x = upload(hip, normal_bf16(30, 2, (8, 1024)), DType.BF16)
    triple = weights.upload(hip)
    outs = [hip.alloc(DType.BF16, (8, 512)) for _ in range(3)]
    total = hip.alloc(DType.BF16, (8, 512))
    commands = CommandList()
    for out in outs:
        commands.dispatch(Op.quant_matmul(4, 64), [x, *triple], out)
    commands.dispatch(Op.copy(), [outs[0]], total)
    plain = hip.submit(commands)
    plain.wait()
    assert plain.profile() == []                       # not asked for: nothing recorded
    submission = hip.submit_profiled(commands)
    with pytest.raises(BackendError):
        submission.profile()                           # the timeline exists after the wait
    submission.wait()
    timeline = submission.profile()
    assert [entry[0] for entry in timeline] == [0, 1, 2, 3]
    assert [entry[1] for entry in timeline] == [1, 1, 1, 1]
    assert [entry[2] for entry in timeline] == [int(d.op.kind) for d in commands.dispatches]
    previous_end = 0
    for _, _, _, start, end in timeline:
        assert previous_end <= start <= end
        previous_end = end
    assert sum(end - start for _, _, _, start, end in timeline) <= submission.gpu_time_ns() * 1.05 + 2000
    assert previous_end <= submission.gpu_time_ns() * 1.05 + 2000


@pytest.mark.parametrize("rows,n,k,kind", [
    (128, 256, 1024, "add"),    # decode rows: the add joins the slab sum
    (8, 64, 256, "add"),        # a single K slab: accumulators + epilogue program
    (300, 520, 512, "add"),     # prefill rows: the add joins the tiled GEMM's store
    (300, 130, 512, "add"),     # residual rows not 8-byte aligned: accumulators + epilogue program
    (700, 768, 1024, "mul"),    # unrecognised epilogue over a GEMM of several tiles
    (96, 512, 2048, "mul"),     # unrecognised epilogue over the slab kernels
])
def test_quant_matmul_with_elementwise_epilogue(cpu, hip, rows, n, k, kind):
    """out = epilogue(f32 accumulator, extra) with a full [rows, N] extra operand: the residual add
    after the dense down projection (crates/forja-sdk/src/nn/blocks.rs:408-411) and a product."""
    weights = Quantised(23, n + k, (n, k))
    x_values = normal_bf16(23, 1, (rows, k))
    extra_values = normal_bf16(23, 2, (rows, n))

    def build(backend):
        x = upload(backend, x_values, DType.BF16)
        extra = upload(backend, extra_values, DType.BF16)
        out = backend.alloc(DType.BF16, (rows, n))
        if kind == "add":
            program = programs.add_elements()
        else:
            b = ProgramBuilder(ProgramKind.MAP)
            b.output(0, b.mul(b.input(0), b.input(1)))
            program = b.finish()
        epilogue = backend.prepare_epilogue(program)
        commands = CommandList()
        commands.dispatch_epilogue(Op.quant_matmul(4, 64), [x, *weights.upload(backend)], out, epilogue,
                                   [extra])
        return commands, [out]
    differential(cpu, hip, build)


# ------------------------------------------------------------------ routed projections

def routed_case(seed, rows, k, experts, n, inner, bad=()):
    rng = np.random.default_rng(seed)
    indices = np.stack([rng.permutation(experts)[:k] for _ in range(rows)]).astype(np.uint32)
    for (r, s, value) in bad:
        indices[r, s] = value
    return indices


@pytest.mark.parametrize("rows,k,experts,n,inner", [(24, 4, 16, 128, 128), (256, 8, 128, 64, 128),
                                                   (5, 2, 3, 64, 64), (40, 8, 8, 192, 256),
                                                   (64, 8, 16, 256, 256), (33, 4, 7, 512, 256),
                                                   (256, 8, 128, 768, 2048)])   # last: BASELINE config 2
def test_gather_projection_pair_and_weighted_sum(cpu, hip, rows, k, experts, n, inner):
    gate = Quantised(31, 1, (n, inner), experts=experts)
    up = Quantised(31, 11, (n, inner), experts=experts)
    down = Quantised(31, 21, (inner, n), experts=experts)
    indices = routed_case(31, rows, k, experts, n, inner)
    x_values = normal_bf16(31, 40, (rows, inner))
    logits = orc.fill_normal_f32(31, 41, rows * k).reshape(rows, k)
    w_values = np.exp(logits) / np.exp(logits).sum(axis=1, keepdims=True)
    residual_values = normal_bf16(31, 42, (rows, inner))

    def build(backend):
        x = upload(backend, x_values, DType.BF16)
        idx = upload(backend, indices, DType.U32)
        g, u, d = gate.upload(backend), up.upload(backend), down.upload(backend)
        plain = backend.alloc(DType.BF16, (rows, k, n))
        activated = backend.alloc(DType.BF16, (rows, k, n))
        combined = backend.alloc(DType.BF16, (rows, inner))
        summed = backend.alloc(DType.BF16, (rows, inner))
        weights = upload(backend, w_values, DType.BF16)
        residual = upload(backend, residual_values, DType.BF16)
        swiglu = backend.prepare_epilogue(programs.silu_mul_elements())
        add = backend.prepare_epilogue(programs.add_elements())
        commands = CommandList()
        commands.dispatch(Op.gather_quant_matmul(4, 64), [x, *g, idx], plain)
        commands.dispatch_epilogue(Op.gather_quant_matmul(4, 64), [x, *g, *u, idx], activated, swiglu, [])
        commands.dispatch_epilogue(Op.gather_quant_matmul(4, 64), [activated, *d, idx, weights], combined,
                                   add, [residual])
        commands.dispatch(Op.gather_quant_matmul(4, 64), [activated, *d, idx, weights], summed)
        return commands, [plain, activated, combined, summed]
    differential(cpu, hip, build)


@pytest.mark.parametrize("form", ["plain", "residual", "norm_into_residual", "norm_of_a_slice",
                                  "weights_in_the_sum"])
@pytest.mark.parametrize("rows,k,experts,n,inner", [(128, 8, 128, 768, 2048), (19, 4, 7, 256, 256)])
def test_weighted_sum_followed_by_the_normalisation_of_its_rows(cpu, hip, rows, k, experts, n, inner, form):
    """A decoder layer ends with the routed weighted sum and the next begins by normalising those
    rows (engines/qwen3-coder/src/lib.rs): the backend may run the two as one kernel.  The result
    must be that of the two dispatches, also where the second is not what the first can absorb: a
    normalisation that overwrites the sum's residual, one that reads only part of the rows, one
    whose weights are the rows themselves."""
    down = Quantised(33, 21, (inner, n), experts=experts)
    indices = routed_case(33, rows, k, experts, n, inner)
    activated_values = normal_bf16(33, 40, (rows, k, n))
    logits = orc.fill_normal_f32(33, 41, rows * k).reshape(rows, k)
    w_values = np.exp(logits) / np.exp(logits).sum(axis=1, keepdims=True)
    residual_values = normal_bf16(33, 42, (rows, inner))
    norm_values = normal_bf16(33, 43, (inner,))

    def build(backend):
        activated = upload(backend, activated_values, DType.BF16)
        idx = upload(backend, indices, DType.U32)
        d = down.upload(backend)
        weights = upload(backend, w_values, DType.BF16)
        residual = upload(backend, residual_values, DType.BF16)
        norm_weight = upload(backend, norm_values, DType.BF16).broadcast((rows, inner))
        summed = backend.alloc(DType.BF16, (rows, inner))
        normed = backend.alloc(DType.BF16, (rows, inner))
        add = backend.prepare_epilogue(programs.add_elements())
        norm = backend.prepare_program(programs.rms_norm_rows(1e-6))
        commands = CommandList()
        outputs = [summed, normed]
        if form == "plain":
            commands.dispatch(Op.gather_quant_matmul(4, 64), [activated, *d, idx, weights], summed)
        else:
            commands.dispatch_epilogue(Op.gather_quant_matmul(4, 64), [activated, *d, idx, weights], summed,
                                       add, [residual])
        if form == "norm_into_residual":
            commands.dispatch_kernel(norm, [summed, norm_weight], [residual])
            outputs = [summed, residual]
        elif form == "norm_of_a_slice":
            half = rows // 2
            commands.dispatch_kernel(norm, [summed.narrow(0, 0, half), norm_weight.narrow(0, 0, half)],
                                     [normed.narrow(0, 0, half)])
            commands.dispatch(Op.copy(), [summed.narrow(0, half, rows - half)], normed.narrow(0, half, rows - half))
        elif form == "weights_in_the_sum":
            commands.dispatch_kernel(norm, [summed, summed], [normed])
        else:
            commands.dispatch_kernel(norm, [summed, norm_weight], [normed])
        return commands, outputs
    # rows normalised by themselves square the one-ulp differences the sums may have: twice the bar
    differential(cpu, hip, build, **({"rel": 3e-2} if form == "weights_in_the_sum" else {}))


@pytest.mark.parametrize("with_residual", [False, True])
def test_f32_weighted_sum_followed_by_the_normalisation_of_its_rows(cpu, hip, with_residual):
    """The same pair in the engine's dtypes: an 8-row decode batch, everything f32."""
    rows, k, experts, n, inner = 8, 8, 128, 768, 2048
    down = Quantised(34, 21, (inner, n), experts=experts)
    indices = routed_case(34, rows, k, experts, n, inner)
    activated_values = orc.fill_normal_f32(34, 40, rows * k * n).reshape(rows, k, n)
    logits = orc.fill_normal_f32(34, 41, rows * k).reshape(rows, k)
    w_values = np.exp(logits) / np.exp(logits).sum(axis=1, keepdims=True)
    residual_values = orc.fill_normal_f32(34, 42, rows * inner).reshape(rows, inner)
    norm_values = orc.fill_normal_f32(34, 43, inner)

    def build(backend):
        activated = upload(backend, activated_values, DType.F32)
        idx = upload(backend, indices, DType.U32)
        weights = upload(backend, w_values, DType.F32)
        residual = upload(backend, residual_values, DType.F32)
        norm_weight = upload(backend, norm_values, DType.F32).broadcast((rows, inner))
        summed = backend.alloc(DType.F32, (rows, inner))
        normed = backend.alloc(DType.F32, (rows, inner))
        commands = CommandList()
        if with_residual:
            add = backend.prepare_epilogue(programs.add_elements())
            commands.dispatch_epilogue(Op.gather_quant_matmul(4, 64), [activated, *down.upload(backend), idx, weights],
                                       summed, add, [residual])
        else:
            commands.dispatch(Op.gather_quant_matmul(4, 64), [activated, *down.upload(backend), idx, weights], summed)
        commands.dispatch_kernel(backend.prepare_program(programs.rms_norm_rows(1e-6)), [summed, norm_weight], [normed])
        return commands, [summed, normed]
    differential(cpu, hip, build)


@pytest.mark.parametrize("dtype,bits,group,scale_dtype", [
    (DType.F32, 4, 64, DType.BF16),      # the qwen3-coder engine: f32 activations
    (DType.F16, 8, 32, DType.F16),
    (DType.BF16, 4, 128, DType.BF16),    # a group size the matrix-core kernels do not take
])
@pytest.mark.parametrize("rows,k,experts,n,inner", [(8, 8, 128, 768, 2048), (37, 3, 5, 96, 256),
                                                   (70, 8, 16, 192, 512)])   # ≈35 routes per expert: two tiles
def test_gather_in_other_dtypes_bits_and_groups(cpu, hip, rows, k, experts, n, inner, dtype, bits, group,
                                                scale_dtype):
    """The routed forms through the f32 vector-ALU kernels (route by route for the first case, grouped
    by expert for the others), with two bad routes: the valid routes
    agree with the oracle, the lowest bad expert is reported, bad projection rows read zero and bad
    routes are left out of the weighted sum."""
    gate = Quantised(35, 1, (n, inner), bits=bits, group=group, experts=experts)
    up = Quantised(35, 11, (n, inner), bits=bits, group=group, experts=experts)
    down = Quantised(35, 21, (inner, n), bits=bits, group=group if n % group == 0 else 32, experts=experts)
    down_group = down.group
    indices = routed_case(35, rows, k, experts, n, inner, bad=[(1, 2, experts + 9), (rows - 1, 0, experts)])
    x_values = normal_bf16(35, 40, (rows, inner))
    logits = orc.fill_normal_f32(35, 41, rows * k).reshape(rows, k)
    w_values = np.exp(logits) / np.exp(logits).sum(axis=1, keepdims=True)
    residual_values = normal_bf16(35, 42, (rows, inner))

    def build(backend, good_only):
        x = upload(backend, x_values, dtype)
        idx = upload(backend, indices if not good_only else indices % experts, DType.U32)
        g, u, d = (w.upload(backend, scale_dtype=scale_dtype) for w in (gate, up, down))
        plain, activated = (backend.alloc(dtype, (rows, k, n)) for _ in range(2))
        combined, summed = (backend.alloc(dtype, (rows, inner)) for _ in range(2))
        weights = upload(backend, w_values, dtype)
        residual = upload(backend, residual_values, dtype)
        swiglu = backend.prepare_epilogue(programs.silu_mul_elements())
        add = backend.prepare_epilogue(programs.add_elements())
        first, second = CommandList(), CommandList()
        first.dispatch(Op.gather_quant_matmul(bits, group), [x, *g, idx], plain)
        second.dispatch_epilogue(Op.gather_quant_matmul(bits, group), [x, *g, *u, idx], activated, swiglu, [])
        second.dispatch_epilogue(Op.gather_quant_matmul(bits, down_group), [activated, *d, idx, weights],
                                 combined, add, [residual])
        second.dispatch(Op.gather_quant_matmul(bits, down_group), [activated, *d, idx, weights], summed)
        return (first, second), [plain, activated, combined, summed]

    # without bad routes: every output against the oracle
    outputs = []
    for backend in (cpu, hip):
        lists, tensors = build(backend, True)
        for commands in lists:
            run(backend, commands)
        outputs.append(tensors)
    for a, b in zip(*outputs):
        compare(cpu, hip, a, b)
    # with them: the lowest bad expert is reported by both, the projection's bad rows are zero
    for backend in (cpu, hip):
        lists, tensors = build(backend, False)
        with pytest.raises(BackendError) as info:
            run(backend, lists[0])
        assert info.value.index == experts
        if backend is hip:
            values = to_f32(hip.read(tensors[0]), dtype).reshape(rows, k, n)
            assert not values[1, 2].any() and not values[rows - 1, 0].any() and values[0, 0].any()
            with pytest.raises(BackendError) as info:
                run(backend, lists[1])
            assert info.value.index == experts


def test_gather_reports_lowest_bad_expert_and_zeroes_its_rows(cpu, hip):
    """lib.rs:2929-2950, crates/forja-metal/tests/gather_quant_matmul.rs:644-764"""
    rows, k, experts, n, inner = 6, 3, 4, 32, 64
    gate = Quantised(32, 1, (n, inner), experts=experts)
    indices = routed_case(32, rows, k, experts, n, inner, bad=[(1, 2, 99), (4, 0, 7)])
    x_values = normal_bf16(32, 40, (rows, inner))

    def build(backend):
        x = upload(backend, x_values, DType.BF16)
        idx = upload(backend, indices, DType.U32)
        out = upload(backend, np.full((rows, k, n), 3.0), DType.BF16)
        commands = CommandList()
        commands.dispatch(Op.gather_quant_matmul(4, 64), [x, *gate.upload(backend), idx], out)
        return commands, [out]
    results = differential(cpu, hip, build, expect_error={Status.INDEX_OUT_OF_RANGE, Status.DEVICE_ERROR_FLAG})
    (cpu_out, cpu_err), (hip_out, hip_err) = results
    assert cpu_err.index == 7 and hip_err.index == 7
    values = to_f32(hip.read(hip_out[0]), DType.BF16).reshape(rows, k, n)
    assert not values[1, 2].any() and not values[4, 0].any() and values[0, 0].any()


def test_gather_with_an_unrecognised_epilogue_uses_the_interpreter(cpu, hip):
    rows, k, experts, n, inner = 8, 2, 4, 32, 64
    gate, up = Quantised(33, 1, (n, inner), experts=experts), Quantised(33, 2, (n, inner), experts=experts)
    indices = routed_case(33, rows, k, experts, n, inner)
    x_values = normal_bf16(33, 3, (rows, inner))
    program = Program(ProgramKind.MAP, [
        Inst.input(0), Inst.input(1), Inst.unary(UnOp.TANH, 0), Inst.binary(BinOp.MAX, 1, 2),
        Inst.const(0.5), Inst.binary(BinOp.MUL, 3, 4)], [(0, 5)])

    def build(backend):
        x = upload(backend, x_values, DType.F32)
        idx = upload(backend, indices, DType.U32)
        out = backend.alloc(DType.F32, (rows, k, n))
        commands = CommandList()
        commands.dispatch_epilogue(Op.gather_quant_matmul(4, 64),
                                   [x, *gate.upload(backend), *up.upload(backend), idx], out,
                                   backend.prepare_epilogue(program), [])
        return commands, [out]
    differential(cpu, hip, build, rel=1e-4, abs_=1e-4, norm_tol=1e-4)


@pytest.mark.parametrize("rows,k,experts,tile", [(256, 8, 128, 16), (128, 8, 128, 32), (7, 3, 5, 2),
                                                (1, 1, 1, 1), (300, 8, 128, 32), (64, 2, 200, 8),
                                                (100, 8, 512, 32), (333, 8, 3, 32)])
def test_route_pack_is_bit_exact(cpu, hip, rows, k, experts, tile):
    rng = np.random.default_rng(rows * 31 + k)
    indices = rng.integers(0, experts, (rows, k)).astype(np.uint32)
    if experts == 3:
        indices[:] = 1      # every route names the same expert: one long run across rounds
        indices[5, 2] = 0

    def build(backend):
        idx = upload(backend, indices, DType.U32)
        max_blocks = experts + rows * k // tile + 1
        outs = [backend.alloc(DType.U32, (experts,)), backend.alloc(DType.U32, (experts + 1,)),
                backend.alloc(DType.U32, (rows * k,)), backend.alloc(DType.U32, (max_blocks, 3))]
        commands = CommandList()
        commands.dispatch_many(Op.route_pack(tile), [idx], outs)
        return commands, outs
    (cpu_out, _), (hip_out, _) = differential(cpu, hip, build)
    flat = indices.ravel().astype(np.int64)
    order = np.argsort(flat, kind="stable")
    assert np.frombuffer(hip.read(hip_out[2]), np.uint32).tolist() == order.tolist()


def test_route_pack_skips_bad_routes_and_reports_the_lowest(cpu, hip):
    indices = np.array([[0, 9, 2], [7, 1, 1], [2, 2, 50]], dtype=np.uint32)

    def build(backend):
        idx = upload(backend, indices, DType.U32)
        outs = [backend.alloc(DType.U32, (3,)), backend.alloc(DType.U32, (4,)),
                backend.alloc(DType.U32, (9,)), backend.alloc(DType.U32, (8, 3))]
        commands = CommandList()
        commands.dispatch_many(Op.route_pack(2), [idx], outs)
        return commands, outs[:2]
    results = differential(cpu, hip, build, expect_error={Status.INDEX_OUT_OF_RANGE})
    assert results[1][1].index == 7


# ------------------------------------------------------------------ selection

@pytest.mark.parametrize("width,k", [(1, 1), (64, 8), (100, 8), (128, 8), (300, 16), (512, 64),
                                     (2050, 64)])
def test_top_k_edge_widths_ties_and_nans(cpu, hip, width, k):
    values = top_k_case(width)

    def build(backend):
        x = upload_raw(backend, values, DType.F32, (1, width))
        outs = [backend.alloc(DType.F32, (1, k)), backend.alloc(DType.U32, (1, k))]
        commands = CommandList()
        commands.dispatch_many(Op.top_k(k, False), [x], outs)
        return commands, outs
    (cpu_out, _), (hip_out, _) = differential(cpu, hip, build)
    assert cpu.read(cpu_out[0]) == hip.read(hip_out[0])       # values copied bit for bit


@pytest.mark.parametrize("dtype", [DType.BF16, DType.F32])
def test_router_top_k_is_bit_exact_in_order_and_close_in_weight(cpu, hip, dtype):
    logits = orc.fill_normal_f32(41, 1, 256 * 128).reshape(256, 128)

    def build(backend):
        x = upload(backend, logits, dtype)
        outs = [backend.alloc(dtype, (256, 8)), backend.alloc(DType.U32, (256, 8))]
        commands = CommandList()
        commands.dispatch_many(Op.top_k(8, True), [x], outs)
        return commands, outs
    differential(cpu, hip, build)


@pytest.mark.parametrize("case", ["chain", "indices_rewritten", "fewer_logits_than_experts", "one_allocation"])
@pytest.mark.parametrize("rows,dtype", [(1, DType.BF16), (8, DType.BF16), (16, DType.F32), (17, DType.BF16)])
def test_top_k_of_a_small_batch_feeds_the_routed_products(cpu, hip, rows, dtype, case):
    """A small decode batch: router logits -> top-k -> routed gate/up + SwiGLU -> routed down with
    the weighted sum, the two products sharing the route plan packed from the selected indices.
    The result is the oracle's, also where the indices are overwritten before the products read
    them, the products know more experts than there were logits, or values and indices live in
    one allocation."""
    k, experts, n, inner = 8, 128, 128, 256
    width = 64 if case == "fewer_logits_than_experts" else experts
    gate = Quantised(47, 1, (n, inner), experts=experts)
    up = Quantised(47, 11, (n, inner), experts=experts)
    down = Quantised(47, 21, (inner, n), experts=experts)
    logits = orc.fill_normal_f32(47, 31, rows * width).reshape(rows, width)
    other = routed_case(47, rows, k, experts, n, inner)
    x_values = normal_bf16(47, 40, (rows, inner))

    def build(backend):
        x = upload(backend, x_values, DType.BF16)
        g, u, d = gate.upload(backend), up.upload(backend), down.upload(backend)
        router = upload(backend, logits, dtype)
        if case == "one_allocation":      # u32 indices behind the weights in the same allocation
            both = backend.alloc(DType.U32, (2 * rows, k))
            span = both.layout.buffer_len
            weights = both.with_layout(Layout.contiguous(dtype, 0, (rows, k), span))
            idx = both.with_layout(Layout.contiguous(DType.U32, rows * k, (rows, k), span))
        else:
            weights, idx = backend.alloc(dtype, (rows, k)), backend.alloc(DType.U32, (rows, k))
        activated = backend.alloc(DType.BF16, (rows, k, n))
        summed = backend.alloc(DType.BF16, (rows, inner))
        bf16_weights = backend.alloc(DType.BF16, (rows, k))
        swiglu = backend.prepare_epilogue(programs.silu_mul_elements())
        commands = CommandList()
        commands.dispatch_many(Op.top_k(k, True), [router], [weights, idx])
        if case == "indices_rewritten":
            commands.dispatch(Op.copy(), [upload(backend, other, DType.U32)], idx)
        commands.dispatch(Op.copy(), [weights], bf16_weights)
        commands.dispatch_epilogue(Op.gather_quant_matmul(4, 64), [x, *g, *u, idx], activated, swiglu, [])
        commands.dispatch(Op.gather_quant_matmul(4, 64), [activated, *d, idx, bf16_weights], summed)
        return commands, [weights, idx, activated, summed]
    differential(cpu, hip, build)


def test_argmax_ties_and_vocabulary_width(cpu, hip):
    rng = np.random.default_rng(3)
    logits = rng.standard_normal((4, 151936)).astype(np.float32)
    logits[1, 77] = logits[1, 150000] = 99.0            # tie: highest index wins
    logits[2, 5] = np.inf
    logits[3, 100] = np.nan                             # +NaN is the maximum under total order
    small = np.array([[1.0, 9.0, 2.0, 9.0, 3.0]], dtype=np.float32)

    def build(backend):
        a, b = upload(backend, logits, DType.BF16), upload(backend, small, DType.F32)
        c = upload(backend, logits, DType.F32)             # the engine's f32 logits
        outs = [backend.alloc(DType.U32, (4,)), backend.alloc(DType.U32, (1,)), backend.alloc(DType.U32, (4,))]
        commands = CommandList()
        commands.dispatch(Op.argmax(), [a], outs[0])
        commands.dispatch(Op.argmax(), [b], outs[1])
        commands.dispatch(Op.argmax(), [c], outs[2])
        return commands, outs
    (_, _), (hip_out, _) = differential(cpu, hip, build)
    assert np.frombuffer(hip.read(hip_out[1]), np.uint32).tolist() == [3]
    assert np.frombuffer(hip.read(hip_out[0]), np.uint32).tolist()[1:] == [150000, 5, 100]


# ------------------------------------------------------------------ paged storage

def test_paged_copy_round_trip_with_conversion(cpu, hip):
    values = np.arange(21, dtype=np.float32) / 8.0

    def build(backend):
        source = upload(backend, values.reshape(7, 3), DType.F32)
        pool = backend.alloc(DType.F16, (3, 4, 3))
        table = upload(backend, np.array([[2, 5], [0, 7]]), DType.U32)
        generations = upload(backend, np.array([7, 0, 5]), DType.U32)
        output = backend.alloc(DType.F32, (7, 3))
        commands = CommandList()
        commands.dispatch(Op.paged_copy(INTO_PAGES, 1, 4), [source, table, generations], pool)
        commands.dispatch(Op.paged_copy(OUT_OF_PAGES, 1, 4), [pool, table, generations], output)
        return commands, [pool, output]
    (cpu_out, _), (hip_out, _) = differential(cpu, hip, build)
    assert cpu.read(cpu_out[0]) == hip.read(hip_out[0]) and cpu.read(cpu_out[1]) == hip.read(hip_out[1])


def test_paged_copy_refuses_stale_entries_without_writing(hip):
    """crates/forja-metal/tests/paged.rs:239-277: rejected rows are not written, others are."""
    source = upload(hip, np.arange(16, dtype=np.float32).reshape(8, 2) + 1.0, DType.F32)
    pool = hip.alloc(DType.F32, (3, 4, 2))
    generations = upload(hip, np.array([7, 8, 9]), DType.U32)
    table = upload(hip, np.array([[1, 8], [2, 1]]), DType.U32)     # second entry is stale
    commands = CommandList()
    commands.dispatch(Op.paged_copy(INTO_PAGES, 0, 4), [source, table, generations], pool)
    with pytest.raises(BackendError) as info:
        run(hip, commands)
    assert info.value.status == Status.DEVICE_ERROR_FLAG and info.value.index == 1
    values = to_f32(hip.read(pool), DType.F32).reshape(3, 4, 2)
    assert values[1].ravel().tolist() == list(np.arange(8) + 1.0) and not values[2].any()


PAGED_CASES = [
    # hq, hkv, sq, key_length, q_start, causal, pool dtype, page_tokens
    (16, 8, 1, 18, 17, True, DType.BF16, 16),
    (16, 8, 1, 65, 64, True, DType.BF16, 16),
    (16, 8, 1, 131, 130, True, DType.BF16, 16),
    (16, 8, 1, 512, 511, True, DType.BF16, 16),
    (32, 4, 1, 1000, 999, True, DType.BF16, 16),
    (32, 4, 1, 300, 299, True, DType.BF16, 64),
    (4, 2, 5, 37, 32, True, DType.BF16, 16),
    (4, 4, 3, 33, 0, False, DType.F16, 16),
    (2, 1, 4, 20, 16, True, DType.F32, 4),
    (40, 8, 77, 177, 100, True, DType.BF16, 16),     # prefill chunk through the single-lane op
    (16, 8, 50, 90, 0, False, DType.BF16, 16),       # non-causal: every row attends key_length
    (32, 4, 130, 130, 0, True, DType.BF16, 16),
]


@pytest.mark.parametrize("hq,hkv,sq,key_length,q_start,causal,dtype,pt", PAGED_CASES)
def test_paged_sdpa(cpu, hip, hq, hkv, sq, key_length, q_start, causal, dtype, pt):
    scale = 1.0 / math.sqrt(128)

    def build(backend):
        t, _ = paged_case(backend, hq, hkv, sq, key_length, pt, q_start, pool_dtype=dtype)
        commands = CommandList()
        commands.dispatch(Op.paged_sdpa(scale, causal, q_start, key_length, pt),
                          [t["q"], t["keys"], t["values"], t["table"], t["generations"]], t["out"])
        return commands, [t["out"]]
    differential(cpu, hip, build)


@pytest.mark.parametrize("sq,key_length,q_start", [(1, 300, 299), (77, 177, 100)])
@pytest.mark.parametrize("q_dtype", [DType.F32, DType.F16])
def test_paged_sdpa_and_append_with_f16_pools(cpu, hip, q_dtype, sq, key_length, q_start):
    """The qwen3-coder engine's dtypes: f32 activations against an f16 KV cache
    (engines/qwen3-coder/src/lib.rs: the pools are allocated as F16, the rows arrive as F32)."""
    hq, hkv, pt = 32, 4, 64
    scale = 1.0 / math.sqrt(128)
    k_new = normal_bf16(52, 1, (sq, hkv, 128)) * 1.001      # not representable in f16 as they stand
    v_new = normal_bf16(52, 2, (sq, hkv, 128)) * 1.001

    def build(backend):
        t, _ = paged_case(backend, hq, hkv, sq, key_length, pt, q_start, pool_dtype=DType.F16, q_dtype=q_dtype)
        appended = backend.alloc(q_dtype, (hq, sq, 128))
        commands = CommandList()
        commands.dispatch(Op.paged_sdpa(scale, True, q_start, key_length, pt),
                          [t["q"], t["keys"], t["values"], t["table"], t["generations"]], t["out"])
        if sq == 1:       # the appending form takes a single query row (check_paged_append, ops.rs:2266)
            commands.dispatch_many(Op.paged_sdpa_append(scale, q_start, pt),
                                   [t["q"], upload(backend, k_new, q_dtype), upload(backend, v_new, q_dtype),
                                    t["table"], t["generations"]], [appended, t["keys"], t["values"]])
        return commands, [t["out"], appended, t["keys"], t["values"]]
    (cpu_out, _), (hip_out, _) = differential(cpu, hip, build, bar=DType.F16)
    assert cpu.read(cpu_out[2]) == hip.read(hip_out[2]) and cpu.read(cpu_out[3]) == hip.read(hip_out[3])


def test_paged_sdpa_through_a_permuted_query_view(cpu, hip):
    """Engines pass q as a permuted [Hq,Sq,D] view of [Sq,Hq,D] storage and read the output the
    same way (crates/forja-host/src/lib.rs:6223-6333)."""
    hq, hkv, sq, key_length, q_start = 8, 2, 3, 40, 37
    scale = 0.1

    def build(backend):
        t, host = paged_case(backend, hq, hkv, sq, key_length, 16, q_start)
        stored_q = upload(backend, np.transpose(host["q"], (1, 0, 2)), DType.BF16)
        stored_out = backend.alloc(DType.BF16, (sq, hq, 128))
        commands = CommandList()
        commands.dispatch(Op.paged_sdpa(scale, True, q_start, key_length, 16),
                          [stored_q.permute([1, 0, 2]), t["keys"], t["values"], t["table"], t["generations"]],
                          stored_out.permute([1, 0, 2]))
        return commands, [stored_out]
    differential(cpu, hip, build)


def test_paged_append_then_attend(cpu, hip):
    hq, hkv, q_start = 16, 8, 130
    scale = 1.0 / math.sqrt(128)
    k_new = normal_bf16(51, 1, (1, hkv, 128))
    v_new = normal_bf16(51, 2, (1, hkv, 128))

    def build(backend):
        t, _ = paged_case(backend, hq, hkv, 1, q_start + 1, 16, q_start)
        kn, vn = upload(backend, k_new, DType.BF16), upload(backend, v_new, DType.BF16)
        commands = CommandList()
        commands.dispatch_many(Op.paged_sdpa_append(scale, q_start, 16),
                               [t["q"], kn, vn, t["table"], t["generations"]],
                               [t["out"], t["keys"], t["values"]])
        return commands, [t["out"]]
    (cpu_out, _), (hip_out, _) = differential(cpu, hip, build)


def test_inactive_lane_is_zero_and_touches_nothing(hip):
    query = upload(hip, np.ones((2, 1, 4)), DType.F32)
    key = upload(hip, np.ones((1, 1, 4)), DType.F32)
    value = upload(hip, np.ones((1, 1, 4)), DType.F32)
    table = upload(hip, np.array([[0, 0xffffffff]]), DType.U32)
    generations = upload(hip, np.array([1]), DType.U32)
    activity = upload(hip, np.array([0]), DType.U32)
    key_pages, value_pages = hip.alloc(DType.F32, (1, 4, 1, 4)), hip.alloc(DType.F32, (1, 4, 1, 4))
    output = upload(hip, np.full((2, 1, 4), 5.0), DType.F32)
    commands = CommandList()
    commands.dispatch_many(Op.paged_sdpa_append(1.0, 0, 4), [query, key, value, table, generations, activity],
                           [output, key_pages, value_pages])
    run(hip, commands)
    assert not any(hip.read(output)) and not any(hip.read(key_pages)) and not any(hip.read(value_pages))


def test_stale_generation_is_reported_and_never_dereferenced(hip):
    t, _ = paged_case(hip, 4, 2, 1, 40, 16, 39)
    generations = np.frombuffer(hip.read(t["generations"]), np.uint32).copy()
    table = np.frombuffer(hip.read(t["table"]), np.uint32).reshape(-1, 2)
    generations[table[1, 0]] += 1                       # logical page 1 is now stale
    hip.write(t["generations"], generations.tobytes())
    commands = CommandList()
    commands.dispatch(Op.paged_sdpa(0.1, True, 39, 40, 16),
                      [t["q"], t["keys"], t["values"], t["table"], t["generations"]], t["out"])
    with pytest.raises(BackendError) as info:
        run(hip, commands)
    assert info.value.status == Status.DEVICE_ERROR_FLAG and info.value.index == 1
    assert not any(hip.read(t["out"]))


# ------------------------------------------------------------------ ragged batch

def ragged_case(backend, contexts, counts, hq, hkv, pt, seed, activity=None, dtype=DType.BF16,
                corrupt=None, pool_dtype=None, out_dtype=None):
    """Lanes with `contexts[l]` tokens already cached and `counts[l]` new queries each.  Shuffled
    physical pages shared by all lanes, generations 11+page, poisoned table tails.  `dtype` is
    that of the query and of the new rows; pools and output follow it unless named."""
    width = 128
    pool_dtype = dtype if pool_dtype is None else pool_dtype
    out_dtype = dtype if out_dtype is None else out_dtype
    lanes = len(contexts)
    pages_needed = [(c + n + pt - 1) // pt for c, n in zip(contexts, counts)]
    table_pages = max(pages_needed) + 2
    physical = sum(pages_needed) + 5
    rng = np.random.default_rng(seed)
    free = list(rng.permutation(physical))
    tables = np.zeros((lanes, table_pages, 2), np.uint32)
    tables[:, :, 1] = 0xffffffff
    for lane, need in enumerate(pages_needed):
        for logical in range(need):
            page = free.pop()
            tables[lane, logical] = (page, 11 + page)
    if corrupt is not None:
        lane, logical = corrupt
        tables[lane, logical, 1] += 1
    pool_k = orc.bf16_to_f32(orc.fill_normal_bf16(seed, 1, physical * pt * hkv * width))
    pool_v = orc.bf16_to_f32(orc.fill_normal_bf16(seed, 2, physical * pt * hkv * width))
    total = sum(counts)
    cu = np.concatenate([[0], np.cumsum(counts)]).astype(np.uint32)
    tensors = dict(
        q=upload(backend, normal_bf16(seed, 3, (total, hq, width)), dtype),
        k_new=upload(backend, normal_bf16(seed, 4, (total, hkv, width)), dtype),
        v_new=upload(backend, normal_bf16(seed, 5, (total, hkv, width)), dtype),
        tables=upload(backend, tables, DType.U32),
        generations=upload(backend, 11 + np.arange(physical), DType.U32),
        cu=upload(backend, cu, DType.U32),
        starts=upload(backend, np.array(contexts), DType.U32),
        out=backend.alloc(out_dtype, (total, hq, width)),
        keys=upload(backend, pool_k.reshape(physical, pt, hkv, width), pool_dtype),
        values=upload(backend, pool_v.reshape(physical, pt, hkv, width), pool_dtype))
    inputs = [tensors[n] for n in ("q", "k_new", "v_new", "tables", "generations", "cu", "starts")]
    if activity is not None:
        inputs.append(upload(backend, np.array(activity), DType.U32))
    return tensors, inputs


RAGGED_CASES = [
    # contexts, new tokens per lane, hq, hkv, page_tokens
    ([17, 64, 130, 511], [1, 1, 1, 1], 16, 8, 16),                 # BASELINE config 0
    ([300, 1, 2047, 700, 15, 16, 0], [1, 1, 1, 1, 1, 1, 1], 32, 4, 16),
    ([40, 0, 100], [1, 5, 3], 8, 2, 16),                           # decode + prefill chunks
    ([100, 257], [1, 1], 32, 4, 64),                               # engine page size
    ([0, 130, 33, 900], [70, 1, 45, 1], 40, 8, 16),                # prefill chunks of a 5-head group + decode rows
    ([0, 64], [200, 37], 16, 8, 16),                               # 16 tokens per query group, ragged tails
    ([500], [96], 32, 4, 16),                                      # a chunk continuing a long context
    ([0, 5], [33, 31], 4, 4, 16),                                  # one head per kv head: 32 tokens per group
    # decode lanes of very different lengths: the split length is the shortest that gives every
    # work item a place on the device at once
    ([5000, 100, 2500, 3100, 33, 4000, 777, 1500, 6000, 9000, 7000, 8990], [1] * 12, 8, 8, 16),
    # more decode lanes than the device holds workgroups, two of them long: split at the even
    # share of a place, up to the split limit of so many tokens
    ([3000 if i == 5 else 2000 if i == 200 else (37 * i) % 60 for i in range(300)], [1] * 300, 8, 8, 16),
]


@pytest.mark.parametrize("contexts,counts,hq,hkv,pt", RAGGED_CASES)
def test_ragged_attention_equals_the_per_lane_sequence(cpu, hip, contexts, counts, hq, hkv, pt):
    scale = 1.0 / math.sqrt(128)

    def build(backend):
        t, inputs = ragged_case(backend, contexts, counts, hq, hkv, pt, seed=61)
        commands = CommandList()
        commands.dispatch_many(Op.paged_attention_ragged(scale, pt), inputs, [t["out"], t["keys"], t["values"]])
        return commands, [t["out"], t["keys"], t["values"]]
    (cpu_out, _), (hip_out, _) = differential(cpu, hip, build)
    # block-table gather and append placement are pure addressing: pools must match bit for bit
    assert cpu.read(cpu_out[1]) == hip.read(hip_out[1]) and cpu.read(cpu_out[2]) == hip.read(hip_out[2])


DTYPE_MIXES = [
    # query and new rows, pools, output
    (DType.F32, DType.F16, DType.F32),      # the qwen3-coder engine
    (DType.F16, DType.F16, DType.F16),
    (DType.F16, DType.F16, DType.BF16),
    (DType.BF16, DType.BF16, DType.F32),
    (DType.F32, DType.BF16, DType.F32),     # f32 activations against a bf16 cache
    (DType.F32, DType.BF16, DType.BF16),
]


@pytest.mark.parametrize("dtype,pool_dtype,out_dtype", DTYPE_MIXES)
@pytest.mark.parametrize("contexts,counts,hq,hkv,pt,promise", [
    ([300, 1, 2047, 700, 15, 16, 0], [1] * 7, 32, 4, 16, True),
    ([300, 1, 2047, 700, 15, 16, 0], [1] * 7, 32, 4, 64, False),
    ([0, 130, 33, 900], [70, 1, 45, 1], 40, 8, 16, False),
    (list(range(0, 520, 13)), [1] * 40, 16, 8, 16, True)])
def test_ragged_attention_across_activation_and_pool_dtypes(cpu, hip, dtype, pool_dtype, out_dtype, contexts,
                                                            counts, hq, hkv, pt, promise):
    """f16 or bf16 pools fed by rows of their own dtype or by f32 rows, any float output: the
    stored rows are rounded once, exactly as the oracle rounds them, so the pools match bit for
    bit; a second layer reuses the work plan on other pools."""
    scale = 1.0 / math.sqrt(128)

    def build(backend):
        t, inputs = ragged_case(backend, contexts, counts, hq, hkv, pt, seed=69, dtype=dtype,
                                pool_dtype=pool_dtype, out_dtype=out_dtype)
        # new rows with more significand bits than the pools hold
        rows = sum(counts)
        inputs[1] = upload(backend, normal_bf16(69, 6, (rows, hkv, 128)) * 1.001, dtype)
        inputs[2] = upload(backend, normal_bf16(69, 7, (rows, hkv, 128)) * 1.001, dtype)
        physical = t["keys"].shape[0]
        other_k = upload(backend, normal_bf16(69, 8, (physical, pt, hkv, 128)), pool_dtype)
        other_v = upload(backend, normal_bf16(69, 9, (physical, pt, hkv, 128)), pool_dtype)
        out2 = backend.alloc(out_dtype, t["out"].shape)
        op = Op.paged_attention_ragged(scale, pt, one_row_per_lane=promise)
        commands = CommandList()
        commands.dispatch_many(op, inputs, [t["out"], t["keys"], t["values"]])
        commands.dispatch_many(op, inputs, [out2, other_k, other_v])
        return commands, [t["out"], out2, t["keys"], t["values"], other_k, other_v]
    (cpu_out, _), (hip_out, _) = differential(cpu, hip, build, bar=pool_dtype)
    for index in (2, 3, 4, 5):
        assert cpu.read(cpu_out[index]) == hip.read(hip_out[index])


def test_f32_queries_beyond_the_f16_range_stay_finite(cpu, hip):
    """An f32 query element no f16 holds: the oracle's scores are huge but finite, and so are the
    device's (the element is held at the largest finite f16); the winner of such a softmax is
    one key on both sides."""
    def build(backend):
        t, inputs = ragged_case(backend, [40, 7], [1, 1], 8, 2, 16, seed=70, dtype=DType.F32,
                                pool_dtype=DType.F16)
        values = normal_bf16(70, 3, (2, 8, 128)).astype(np.float32)
        values[0, 3, 5] = 3.0e6
        values[1, 0, 100] = -1.0e9
        inputs[0] = upload(backend, values, DType.F32)
        commands = CommandList()
        commands.dispatch_many(Op.paged_attention_ragged(0.09, 16), inputs, [t["out"], t["keys"], t["values"]])
        return commands, [t["out"]]
    (cpu_out, _), (hip_out, _) = differential(cpu, hip, build, bar=DType.F16)
    assert np.isfinite(to_f32(hip.read(hip_out[0]), DType.F32)).all()


@pytest.mark.parametrize("contexts,counts,hq,hkv", [([300, 40, 2047, 700], [1, 1, 1, 1], 32, 4),
                                                    ([0, 130, 33], [70, 1, 45], 16, 8)])
def test_ragged_attention_layers_share_metadata_until_it_is_rewritten(cpu, hip, contexts, counts, hq, hkv):
    """One command list the way a model step records it: two layers (their own pools) attend with
    the same tables, starts and cu_seqlens, then the starts are overwritten on the device and a third
    dispatch must follow the new values."""
    scale, pt = 1.0 / math.sqrt(128), 16
    moved = [max(0, c - 5) for c in contexts]

    def build(backend):
        t, inputs = ragged_case(backend, contexts, counts, hq, hkv, pt, seed=64)
        physical = t["keys"].shape[0]
        other_k = upload(backend, normal_bf16(64, 8, (physical, pt, hkv, 128)), DType.BF16)
        other_v = upload(backend, normal_bf16(64, 9, (physical, pt, hkv, 128)), DType.BF16)
        out2, out3 = (backend.alloc(DType.BF16, t["out"].shape) for _ in range(2))
        new_starts = upload(backend, np.array(moved), DType.U32)
        op = Op.paged_attention_ragged(scale, pt)
        commands = CommandList()
        commands.dispatch_many(op, inputs, [t["out"], t["keys"], t["values"]])
        commands.dispatch_many(op, inputs, [out2, other_k, other_v])
        commands.dispatch(Op.copy(), [new_starts], t["starts"])
        commands.dispatch_many(op, inputs, [out3, t["keys"], t["values"]])
        return commands, [t["out"], out2, out3, t["keys"], other_k]
    (cpu_out, _), (hip_out, _) = differential(cpu, hip, build)
    assert cpu.read(cpu_out[3]) == hip.read(hip_out[3]) and cpu.read(cpu_out[4]) == hip.read(hip_out[4])


@pytest.mark.parametrize("contexts,hq,hkv,pt", [
    ([17, 64, 130, 511], 16, 8, 16), ([300, 1, 2047, 700, 15, 16, 0], 32, 4, 16), ([100, 257], 32, 4, 64),
    ([0], 8, 2, 16), (list(range(0, 520, 13)), 32, 4, 16)])
def test_decode_batch_with_the_one_row_promise_stores_the_new_rows_itself(cpu, hip, contexts, hq, hkv, pt):
    """With the recorder's promise of one query row per lane the attention kernel stores the new
    key/value rows itself: pools still match the oracle bit for bit (lanes at context 0 attend
    nothing but the row just stored), and so does a second layer that reuses the work plan."""
    scale = 1.0 / math.sqrt(128)

    def build(backend):
        t, inputs = ragged_case(backend, contexts, [1] * len(contexts), hq, hkv, pt, seed=66)
        physical = t["keys"].shape[0]
        other_k = upload(backend, normal_bf16(66, 8, (physical, pt, hkv, 128)), DType.BF16)
        other_v = upload(backend, normal_bf16(66, 9, (physical, pt, hkv, 128)), DType.BF16)
        out2 = backend.alloc(DType.BF16, t["out"].shape)
        op = Op.paged_attention_ragged(scale, pt, one_row_per_lane=True)
        commands = CommandList()
        commands.dispatch_many(op, inputs, [t["out"], t["keys"], t["values"]])
        commands.dispatch_many(op, inputs, [out2, other_k, other_v])
        return commands, [t["out"], out2, t["keys"], t["values"], other_k, other_v]
    (cpu_out, _), (hip_out, _) = differential(cpu, hip, build)
    for index in (2, 3, 4, 5):
        assert cpu.read(cpu_out[index]) == hip.read(hip_out[index])


def test_a_broken_one_row_promise_is_reported(cpu, hip):
    def build(backend):
        t, inputs = ragged_case(backend, [40, 0, 100], [1, 2, 1], 8, 2, 16, seed=67)
        commands = CommandList()
        commands.dispatch_many(Op.paged_attention_ragged(0.09, 16, one_row_per_lane=True), inputs,
                               [t["out"], t["keys"], t["values"]])
        return commands, []
    for backend in (cpu, hip):
        commands, _ = build(backend)
        with pytest.raises(BackendError) as info:
            run(backend, commands)
        assert info.value.status == Status.DEVICE_ERROR_FLAG and info.value.index == 1


def test_the_one_row_promise_keeps_inactive_lanes_and_stale_pages_unwritten(cpu, hip):
    def build(backend, corrupt):
        t, inputs = ragged_case(backend, [33, 70, 5], [1, 1, 1], 8, 4, 16, seed=68,
                                activity=[1, 0, 1], corrupt=corrupt)
        commands = CommandList()
        commands.dispatch_many(Op.paged_attention_ragged(0.09, 16, one_row_per_lane=True), inputs,
                               [t["out"], t["keys"], t["values"]])
        return commands, [t["out"], t["keys"], t["values"]]
    (cpu_out, _), (hip_out, _) = differential(cpu, hip, lambda backend: build(backend, None))
    assert cpu.read(cpu_out[1]) == hip.read(hip_out[1]) and cpu.read(cpu_out[2]) == hip.read(hip_out[2])
    # lane 0 appends at position 33 = logical page 2: stale there, nothing of lane 0 is written
    commands, tensors = build(hip, (0, 2))
    before = hip.read(tensors[1])
    with pytest.raises(BackendError) as info:
        run(hip, commands)
    assert info.value.status == Status.DEVICE_ERROR_FLAG and info.value.index == 2
    # exactly one token row of the key pool changed: lane 2's (lane 1 is inactive, lane 0 refused)
    token_row = 4 * 128 * 2
    changed = np.frombuffer(hip.read(tensors[1]), np.uint8).reshape(-1, token_row) != \
        np.frombuffer(before, np.uint8).reshape(-1, token_row)
    assert changed.any(axis=1).sum() == 1
    assert not to_f32(hip.read(tensors[0]), DType.BF16).reshape(3, -1)[0].any()


@pytest.mark.parametrize("hq,hkv,pt,counts,cu", [
    (8, 4, 16, [1, 1, 1, 1], [0, 100, 4, 4, 4]),      # decode batch: lane 0 claims 100 rows of 4
    (8, 4, 16, [20, 30, 14], [0, 20, 10, 64]),        # prefill groups: lane 1 runs backwards
    (8, 4, 16, [20, 30, 14], [0, 20, 50, 4000]),      # the last lane runs past the packed batch
    (6, 2, 8, [3, 2, 1], [0, 3, 70, 6])])             # a page size only the generic kernels take
def test_ragged_attention_refuses_malformed_cu_seqlens(cpu, hip, hq, hkv, pt, counts, cu):
    """cu_seqlens is read on the device: ranges that run backwards or beyond the packed batch fail
    the dispatch (lowest offending lane reported), every output row reads zero, and neither the
    pools nor the allocations around q and out are touched.  Every kernel exits normally."""
    contexts = [40 + 3 * lane for lane in range(len(counts))]
    bad_lane = next(l for l in range(len(counts)) if cu[l + 1] < cu[l] or cu[l + 1] > sum(counts))
    for promise in (False, True) if max(counts) == 1 else (False,):
        for backend in (cpu, hip):
            guard_before = upload(backend, normal_bf16(72, 1, (4096,)), DType.BF16)
            t, inputs = ragged_case(backend, contexts, counts, hq, hkv, pt, seed=71)
            guard_after = upload(backend, normal_bf16(72, 2, (4096,)), DType.BF16)
            inputs[5] = upload(backend, np.array(cu), DType.U32)
            backend.write(t["out"], np.full(sum(counts) * hq * 128, 0x3f80, np.uint16).tobytes())
            pools = backend.read(t["keys"]), backend.read(t["values"])
            guards = backend.read(guard_before), backend.read(guard_after)
            commands = CommandList()
            commands.dispatch_many(Op.paged_attention_ragged(0.09, pt, one_row_per_lane=promise), inputs,
                                   [t["out"], t["keys"], t["values"]])
            with pytest.raises(BackendError) as info:
                run(backend, commands)
            assert info.value.status == Status.DEVICE_ERROR_FLAG and info.value.index == bad_lane
            assert not np.frombuffer(backend.read(t["out"]), np.uint16).any()
            assert (backend.read(t["keys"]), backend.read(t["values"])) == pools
            assert (backend.read(guard_before), backend.read(guard_after)) == guards
            # and the backend keeps working: the same batch with its real cu_seqlens succeeds
            inputs[5] = t["cu"]
            commands = CommandList()
            commands.dispatch_many(Op.paged_attention_ragged(0.09, pt), inputs, [t["out"], t["keys"], t["values"]])
            run(backend, commands)
            assert np.frombuffer(backend.read(t["out"]), np.uint16).any()


def test_ragged_attention_skips_inactive_lanes(cpu, hip):
    def build(backend):
        t, inputs = ragged_case(backend, [33, 70, 5], [1, 1, 1], 8, 4, 16, seed=62, activity=[1, 0, 1])
        commands = CommandList()
        commands.dispatch_many(Op.paged_attention_ragged(0.09, 16), inputs, [t["out"], t["keys"], t["values"]])
        return commands, [t["out"], t["keys"], t["values"]]
    (cpu_out, _), (hip_out, _) = differential(cpu, hip, build)
    assert cpu.read(cpu_out[1]) == hip.read(hip_out[1])
    assert not to_f32(hip.read(hip_out[0]), DType.BF16).reshape(3, -1)[1].any()


def test_ragged_attention_reports_a_stale_page(hip):
    t, inputs = ragged_case(hip, [33, 70, 5], [1, 1, 1], 8, 4, 16, seed=63, corrupt=(1, 2))
    commands = CommandList()
    commands.dispatch_many(Op.paged_attention_ragged(0.09, 16), inputs, [t["out"], t["keys"], t["values"]])
    with pytest.raises(BackendError) as info:
        run(hip, commands)
    assert info.value.status == Status.DEVICE_ERROR_FLAG and info.value.index == 2
    out = to_f32(hip.read(t["out"]), DType.BF16).reshape(3, -1)
    assert not out[1].any() and out[0].any() and out[2].any()


def test_empty_batches_are_accepted_and_change_nothing(cpu, hip):
    """Zero rows through the projections, the router and a program, and a ragged batch whose lanes
    bring no query tokens: both backends accept them, write nothing and report nothing."""
    weights = Quantised(81, 1, (64, 128))
    stacked = Quantised(81, 2, (64, 128), experts=4)

    def build(backend):
        x = backend.alloc(DType.BF16, (0, 128))
        out = backend.alloc(DType.BF16, (0, 64))
        logits = backend.alloc(DType.BF16, (0, 4))
        route_weights, route_ids = backend.alloc(DType.BF16, (0, 2)), backend.alloc(DType.U32, (0, 2))
        routed = backend.alloc(DType.BF16, (0, 2, 64))
        t, inputs = ragged_case(backend, [5, 9], [0, 0], 8, 4, 16, seed=82)
        commands = CommandList()
        commands.dispatch(Op.quant_matmul(4, 64), [x, *weights.upload(backend)], out)
        commands.dispatch_many(Op.top_k(2, True), [logits], [route_weights, route_ids])
        commands.dispatch(Op.gather_quant_matmul(4, 64), [x, *stacked.upload(backend), route_ids], routed)
        commands.dispatch_kernel(backend.prepare_program(programs.add_elements()), [out, out],
                                 [backend.alloc(DType.BF16, (0, 64))])
        commands.dispatch_many(Op.paged_attention_ragged(0.1, 16), inputs, [t["out"], t["keys"], t["values"]])
        return commands, [t["keys"], t["values"]]
    (cpu_out, _), (hip_out, _) = differential(cpu, hip, build)
    assert cpu.read(cpu_out[0]) == hip.read(hip_out[0]) and cpu.read(cpu_out[1]) == hip.read(hip_out[1])


# ------------------------------------------------------------------ programs and glue

@pytest.mark.parametrize("dtype", [DType.BF16, DType.F32])
def test_engine_row_programs(cpu, hip, dtype):
    """The fused row-program kernels on bf16 and on f32 rows.  f32 results are held to the f16 bar:
    the rotation angle at position 32767 carries the few-ulp difference between the device's and
    the host's powf, about 3e-3 rad."""
    rows, hidden, heads, half = 6, 1024, 24, 64
    x_values = normal_bf16(71, 1, (rows, hidden))
    u_values = normal_bf16(71, 2, (rows, hidden))
    w_values = 1.0 + 0.1 * normal_bf16(71, 3, (hidden,))
    qk_values = normal_bf16(71, 4, (rows, heads, 2 * half))
    norm_values = 1.0 + 0.1 * normal_bf16(71, 5, (heads, 2 * half))
    positions = np.array([0, 1, 17, 511, 4095, 32767], dtype=np.float32)

    def build(backend):
        x, u = upload(backend, x_values, dtype), upload(backend, u_values, dtype)
        w = upload(backend, w_values, dtype).broadcast((rows, hidden))
        normed = backend.alloc(dtype, (rows, hidden))
        hidden_out, normed2 = backend.alloc(dtype, (rows, hidden)), backend.alloc(dtype, (rows, hidden))
        qk = upload(backend, qk_values, dtype)
        norm = upload(backend, norm_values, dtype).broadcast((rows, heads, 2 * half))
        pos = upload(backend, positions, DType.F32).reshape((rows, 1, 1)).broadcast((rows, heads, half))
        rotated = backend.alloc(dtype, (rows, heads, 2 * half))
        commands = CommandList()
        commands.dispatch_kernel(backend.prepare_program(programs.rms_norm_rows(1e-6)), [x, w], [normed])
        commands.dispatch_kernel(backend.prepare_program(programs.residual_norm_rows(1e-6)), [x, u, w],
                                 [hidden_out, normed2])
        commands.dispatch_kernel(
            backend.prepare_program(programs.qk_norm_rope_rows(128.0, 1e-6, 1e6)),
            [qk.narrow(2, 0, half), qk.narrow(2, half, half), norm.narrow(2, 0, half),
             norm.narrow(2, half, half), pos],
            [rotated.narrow(2, 0, half), rotated.narrow(2, half, half)])
        return commands, [normed, hidden_out, normed2, rotated]
    differential(cpu, hip, build, abs_=2e-2, bar=DType.F16 if dtype == DType.F32 else None)


@pytest.mark.parametrize("rows,width", [(5, 64), (130, 1024), (3, 20)])
def test_engine_element_programs_on_the_halves_of_a_stacked_projection(cpu, hip, rows, width):
    """silu_mul_elements over the gate and up halves of one [rows, 2 * width] tensor and
    add_elements (crates/forja-sdk/src/nn/blocks.rs:408-416); the last width is not a multiple of
    eight."""
    stacked_values = 3.0 * normal_bf16(72, 1, (rows, 2 * width))
    residual_values = normal_bf16(72, 2, (rows, width))

    def build(backend):
        stacked = upload(backend, stacked_values, DType.BF16)
        residual = upload(backend, residual_values, DType.BF16)
        activated, summed = (backend.alloc(DType.BF16, (rows, width)) for _ in range(2))
        commands = CommandList()
        commands.dispatch_kernel(backend.prepare_program(programs.silu_mul_elements()),
                                 [stacked.narrow(1, 0, width), stacked.narrow(1, width, width)], [activated])
        commands.dispatch_kernel(backend.prepare_program(programs.add_elements()), [residual, activated],
                                 [summed])
        return commands, [activated, summed]
    differential(cpu, hip, build)


def test_map_programs_casts_index_select(cpu, hip):
    values = np.array([[-1.5, 3.7, np.nan, 5e9, 0.25, -0.0, 7.0, 1e-3]], dtype=np.float32).repeat(3, axis=0)
    b = ProgramBuilder(ProgramKind.MAP)
    v, w = b.input(0), b.input(1)
    as_u32 = b.cast(ValueType.U32, v)
    b.output(0, b.cast(ValueType.F32, as_u32))
    column = b.cast(ValueType.F32, b.index(1))
    big = b.binary(BinOp.GT, column, b.const(3.5))
    b.output(1, b.select(big, b.binary(BinOp.MAX, v, b.const(0.0)), b.unary(UnOp.ABS, v)))
    b.output(2, b.cast(ValueType.F32, b.binary(BinOp.ADD, w, b.extent(1))))
    program = b.finish()

    def build(backend):
        x = upload_raw(backend, values, DType.F32, values.shape)
        ids = upload(backend, np.arange(24).reshape(3, 8), DType.U32)
        outs = [backend.alloc(DType.F32, values.shape) for _ in range(3)]
        commands = CommandList()
        commands.dispatch_kernel(backend.prepare_program(program), [x, ids], outs)
        return commands, outs
    (cpu_out, _), (hip_out, _) = differential(cpu, hip, build)
    for a, b_ in zip(cpu_out, hip_out):
        assert cpu.read(a) == hip.read(b_)


def random_program(rng, kind, inputs, length, exact):
    """A typed random SSA program over `inputs` = [ValueType of input slot ...]: every operand is
    drawn from earlier values of the right type, the way the reference's proptest generator does
    (crates/forja-metal/tests/map_programs.rs).  `exact` keeps to operations IEEE fixes bit for bit
    (no division, roots or transcendentals, no sum reduction)."""
    b = ProgramBuilder(kind)
    of_type = {ValueType.F32: [], ValueType.U32: [], ValueType.BOOL: []}
    for slot, value_type in enumerate(inputs):
        of_type[value_type].append(b.input(slot))
    of_type[ValueType.F32].append(b.const(float(rng.choice([0.0, -1.5, 2.0, 0.3, 1e-3]))))
    of_type[ValueType.U32].append(b.index(1))
    of_type[ValueType.U32].append(b.extent(1))
    pick = lambda t: int(rng.choice(of_type[t]))
    reductions = 0
    exact_unary = [UnOp.NEG, UnOp.ABS, UnOp.FLOOR]
    loose_unary = [UnOp.NEG, UnOp.ABS, UnOp.TANH, UnOp.SIGMOID, UnOp.SIN, UnOp.COS]
    exact_binary = [BinOp.ADD, BinOp.SUB, BinOp.MUL, BinOp.MIN, BinOp.MAX]
    compare = [BinOp.LT, BinOp.LE, BinOp.EQ, BinOp.NE, BinOp.GE, BinOp.GT]
    for _ in range(length):
        # the loose set stays with continuous operations: a comparison, floor or integer cast of a
        # value that differs in its last bit may legitimately take the other branch
        choice = int(rng.integers(0, 9)) if exact else int(rng.choice([0, 1, 2, 7, 8]))
        if choice == 0:
            of_type[ValueType.F32].append(b.unary(rng.choice(exact_unary if exact else loose_unary),
                                                  pick(ValueType.F32)))
        elif choice in (1, 2):
            ops = exact_binary
            of_type[ValueType.F32].append(b.binary(rng.choice(ops), pick(ValueType.F32), pick(ValueType.F32)))
        elif choice == 3:
            of_type[ValueType.U32].append(b.binary(rng.choice(exact_binary), pick(ValueType.U32),
                                                   pick(ValueType.U32)))
        elif choice == 4:
            operand = ValueType.F32 if rng.integers(0, 2) else ValueType.U32
            of_type[ValueType.BOOL].append(b.binary(rng.choice(compare), pick(operand), pick(operand)))
        elif choice == 5 and of_type[ValueType.BOOL]:
            chosen = ValueType.F32 if rng.integers(0, 2) else ValueType.U32
            of_type[chosen].append(b.select(pick(ValueType.BOOL), pick(chosen), pick(chosen)))
        elif choice == 6:
            source = [t for t in of_type if of_type[t]][int(rng.integers(0, sum(1 for t in of_type if of_type[t])))]
            target = ValueType(int(rng.integers(0, 3)))
            of_type[target].append(b.cast(target, pick(source)))
        elif choice == 7 and kind == ProgramKind.ROW and reductions < 4:   # MAX_REDUCTIONS, program.rs:27
            reductions += 1
            ops = [RedOp.MAX, RedOp.MIN] if exact else [RedOp.MAX, RedOp.MIN, RedOp.SUM]
            of_type[ValueType.F32].append(b.reduce(rng.choice(ops), pick(ValueType.F32)))
        else:
            of_type[ValueType.F32].append(b.cast(ValueType.F32, pick(ValueType.U32)))
    for slot in range(2):
        b.output(slot, int(of_type[ValueType.F32][-1 - slot]))
    return b.finish()


@pytest.mark.parametrize("kind", [ProgramKind.MAP, ProgramKind.ROW])
@pytest.mark.parametrize("exact", [True, False])
def test_random_typed_programs_agree_with_the_interpreter(cpu, hip, kind, exact):
    """25 seeded random programs per case over a broadcast row, a strided view and an integer
    tensor: bit for bit where IEEE fixes the result, to 1e-5 where libm or the order of a sum does
    not."""
    rows, width = 5, 37
    rng = np.random.default_rng(1234 + 2 * int(kind) + int(exact))
    first = orc.fill_normal_f32(73, 1, rows * width).reshape(rows, width)
    second = orc.fill_normal_f32(73, 2, 2 * width).reshape(1, 2 * width)
    for case in range(25):
        program = random_program(rng, kind, [ValueType.F32, ValueType.F32, ValueType.U32],
                                 length=int(rng.integers(4, 24)), exact=exact)

        def build(backend):
            x = upload(backend, first, DType.F32)
            y = upload(backend, second, DType.F32).slice([Slice(0, 1), Slice(1, width, 2)]).broadcast(
                (rows, width))
            ids = upload(backend, (np.arange(rows * width) * 7919) % 1000, DType.U32).reshape((rows, width))
            outs = [backend.alloc(DType.F32, (rows, width)) for _ in range(2)]
            commands = CommandList()
            commands.dispatch_kernel(backend.prepare_program(program), [x, y, ids], outs)
            return commands, outs
        try:
            if exact:
                (cpu_out, _), (hip_out, _) = differential(cpu, hip, build, rel=0.0, abs_=0.0, norm_tol=0.0)
                for a, b_ in zip(cpu_out, hip_out):
                    assert cpu.read(a) == hip.read(b_), (case, program)
            else:
                differential(cpu, hip, build, rel=1e-5, abs_=1e-6, norm_tol=1e-5)
        except AssertionError as error:
            raise AssertionError(f"program {case}: {program}") from error


def test_program_limits_are_refused_when_prepared(cpu, hip):
    """Five reductions, a reduction in a map program, an operand that is not earlier
    (validate_structure, crates/forja-core/src/program.rs:1052-1094)."""
    five = ProgramBuilder(ProgramKind.ROW)
    value = five.input(0)
    for _ in range(5):
        value = five.reduce(RedOp.MAX, value)
    five.output(0, value)
    in_map = ProgramBuilder(ProgramKind.MAP)
    in_map.output(0, in_map.reduce(RedOp.SUM, in_map.input(0)))
    forward = Program(ProgramKind.MAP, [Inst.input(0), Inst.unary(UnOp.NEG, 2), Inst.const(1.0)], [(0, 1)])
    for backend in (cpu, hip):
        for program in (five.finish(), in_map.finish(), forward):
            with pytest.raises(BackendError) as info:
                backend.prepare_program(program)
            assert info.value.status == Status.INVALID_INPUT


def test_softmax_row_program_with_max_and_sum_reductions(cpu, hip):
    b = ProgramBuilder(ProgramKind.ROW)
    x = b.input(0)
    e = b.unary(UnOp.EXP, b.sub(x, b.reduce(RedOp.MAX, x)))
    b.output(0, b.div(e, b.reduce(RedOp.SUM, e)))
    program = b.finish()
    values = orc.fill_normal_f32(72, 1, 5 * 700).reshape(5, 700)

    def build(backend):
        x = upload(backend, values, DType.F32)
        out = backend.alloc(DType.F32, (5, 700))
        commands = CommandList()
        commands.dispatch_kernel(backend.prepare_program(program), [x], [out])
        return commands, [out]
    differential(cpu, hip, build, rel=1e-4, abs_=1e-6, norm_tol=1e-5)


def test_quant_embed_copy_matmul_rms_norm_rope(cpu, hip):
    table = Quantised(81, 1, (300, 128))
    ids_values = np.array([[5, 299, 0], [17, 100, 3]], dtype=np.uint32)
    experts_values = normal_bf16(81, 2, (6, 32, 4))
    weights_values = normal_bf16(81, 3, (6, 4, 1))
    x_values = normal_bf16(81, 4, (7, 16, 128))

    def build(backend):
        ids = upload(backend, ids_values, DType.U32)
        embedded = backend.alloc(DType.BF16, (2, 3, 128))
        experts = upload(backend, experts_values, DType.BF16)
        weights = upload(backend, weights_values, DType.BF16)
        combined = backend.alloc(DType.BF16, (6, 32, 1))
        x = upload(backend, x_values, DType.BF16)
        copied = backend.alloc(DType.F32, (16, 7, 128))
        normed = backend.alloc(DType.BF16, (7, 16, 128))
        w = upload(backend, np.linspace(0.5, 1.5, 128), DType.F32)
        roped = backend.alloc(DType.BF16, (7, 16, 128))
        pos = upload(backend, np.array([0, 1, 2, 100, 1000, 20000, 32767]), DType.U32)
        commands = CommandList()
        commands.dispatch(Op.quant_embed(4, 64), [*table.upload(backend), ids], embedded)
        commands.dispatch(Op.matmul(), [experts, weights], combined)     # MoE combine shape
        commands.dispatch(Op.copy(), [x.permute([1, 0, 2])], copied)
        commands.dispatch(Op.rms_norm(1e-6), [x, w], normed)
        commands.dispatch(Op.rope(1e6), [x, pos], roped)
        return commands, [embedded, combined, copied, normed, roped]
    differential(cpu, hip, build, abs_=2e-2)


def test_quant_embed_zeroes_bad_rows_and_reports_the_lowest_bad_id(cpu, hip):
    """lib.rs:3020-3037 for the quantised table"""
    table = Quantised(82, 1, (300, 128))
    ids_values = np.array([5, 1000, 0, 999], dtype=np.uint32)

    def build(backend):
        ids = upload(backend, ids_values, DType.U32)
        embedded = upload(backend, np.ones((4, 128)), DType.BF16)
        commands = CommandList()
        commands.dispatch(Op.quant_embed(4, 64), [*table.upload(backend), ids], embedded)
        return commands, [embedded]
    results = differential(cpu, hip, build, expect_error={Status.INDEX_OUT_OF_RANGE})
    assert results[0][1].index == 999 and results[1][1].index == 999
