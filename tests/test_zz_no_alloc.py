"""fh_submit_static (the entry point that allocates nothing: all device scratch comes from a fixed
array in the library's image) against fh_submit on the same dispatches and the same seeded
operands.  The two run the same kernels, so every output must match bit for bit; the second call
of each test is smaller than the first, so it meets whatever the first left in the array."""

import numpy as np
import pytest

from forja_amd.core import (BackendError, CommandList, DType, Op, ProgramBuilder, ProgramKind, RedOp,
                            Status, UnOp)
from forja_amd.model import Model, ModelConfig, PackedStep
from oracle import cpu_backend as orc
from tests.helpers import Quantised, normal_bf16, upload

pytestmark = pytest.mark.gpu

MOE = ModelConfig("no-alloc-moe", hidden=512, layers=2, q_heads=8, kv_heads=2, head_dim=128,
                  vocab=4096, experts=16, top_k=4, expert_intermediate=256, rope_theta=1e7)
DENSE = ModelConfig("no-alloc-dense", hidden=512, layers=2, q_heads=8, kv_heads=4, head_dim=128,
                    vocab=4096, intermediate=768)


def step_outputs(step):
    backend, b, cache = step.model.backend, step.buffers, step.cache
    tensors = [b.logits, b.next_tokens, b.attended, b.hidden[0], b.hidden[1], *cache.keys, *cache.values]
    return [backend.read(t) for t in tensors]


@pytest.mark.parametrize("config", [MOE, DENSE], ids=["moe", "dense"])
def test_packed_steps_match_fh_submit_bit_for_bit(hip, config):
    """A packed prefill + decode step of a whole (small) model: embed, norms, stacked QKV,
    qk-norm + rope, ragged paged attention with split-KV partials and in-pool append, routed MoE
    (route plan, weighted partial sums) or dense SwiGLU, lm_head, argmax."""
    model = Model(hip, config, seed=21)
    for contexts, counts in (([0, 700, 33, 1500, 5], [70, 1, 45, 1, 1]),    # first call
                             ([12, 300], [1, 1])):                          # then a smaller one
        ordinary = PackedStep(model, contexts, counts, seed=9)
        static = PackedStep(model, contexts, counts, seed=9)
        hip.submit(ordinary.encoded).wait()
        hip.submit_static(static.encoded)
        expected, got = step_outputs(ordinary), step_outputs(static)
        assert np.frombuffer(expected[0], np.uint16).any()
        for a, b in zip(expected, got):
            assert a == b


def other_scratch_users(backend, rows, seed):
    """Dispatches whose kernels use the kinds of scratch the model step does not: f32 accumulators
    under an unrecognised epilogue, a generic row program (typed instructions), sampling scratch,
    route packing on its own, and a long single-lane attention with split partials."""
    weights = Quantised(seed, 1, (192, 256))
    x = upload(backend, normal_bf16(seed, 2, (rows, 256)), DType.BF16)
    extra = upload(backend, normal_bf16(seed, 3, (rows, 192)), DType.BF16)
    product = backend.alloc(DType.BF16, (rows, 192))
    b = ProgramBuilder(ProgramKind.MAP)
    b.output(0, b.mul(b.unary(UnOp.TANH, b.input(0)), b.input(1)))
    epilogue = backend.prepare_epilogue(b.finish())
    r = ProgramBuilder(ProgramKind.ROW)
    value = r.input(0)
    r.output(0, r.sub(value, r.reduce(RedOp.MAX, value)))
    row_program = backend.prepare_program(r.finish())
    shifted = backend.alloc(DType.F32, (rows, 192))
    params = upload(backend, orc.sampling_words(0.8, 40, 0.9, 1234), DType.U32)
    sampled = backend.alloc(DType.U32, (rows,))
    indices = upload(backend, np.random.default_rng(seed).integers(0, 8, (rows, 2)), DType.U32)
    experts, tile = 8, 4
    blocks = experts + rows * 2 // tile + 1
    packed = [backend.alloc(DType.U32, shape) for shape in ((experts,), (experts + 1,), (rows * 2,), (blocks, 3))]
    commands = CommandList()
    commands.dispatch_epilogue(Op.quant_matmul(4, 64), [x, *weights.upload(backend)], product, epilogue, [extra])
    commands.dispatch_kernel(row_program, [product], [shifted])
    commands.dispatch_many(Op.sample(3), [shifted, params], [sampled])
    commands.dispatch_many(Op.route_pack(tile), [indices], packed)
    return commands, [product, shifted, sampled, *packed]


def test_accumulators_programs_sampling_and_packing_match(hip):
    for rows in (48, 5):
        results = []
        for static in (False, True):
            commands, outputs = other_scratch_users(hip, rows, seed=33)
            if static:
                hip.submit_static(commands)
            else:
                hip.submit(commands).wait()
            results.append([hip.read(t) for t in outputs])
        assert np.frombuffer(results[0][0], np.uint16).any()
        assert results[0] == results[1]


def test_enqueue_only_form_and_data_dependent_errors(hip):
    """`error` null: the call only enqueues; a later synchronisation sees the results.  `error`
    given: a stale page is reported as fh_wait reports it, with the same zero row."""
    from tests.test_parity_gpu import ragged_case
    results = []
    for static in (False, True):
        t, inputs = ragged_case(hip, [300, 40, 2047], [1, 1, 1], 32, 4, 16, seed=44)
        commands = CommandList()
        commands.dispatch_many(Op.paged_attention_ragged(0.09, 16, one_row_per_lane=True), inputs,
                               [t["out"], t["keys"], t["values"]])
        if static:
            hip.submit_static(commands, wait=False)
            hip.synchronize()
        else:
            hip.submit(commands).wait()
        results.append([hip.read(t[name]) for name in ("out", "keys", "values")])
    assert results[0] == results[1]
    results = []
    for static in (False, True):
        t, inputs = ragged_case(hip, [33, 70, 5], [1, 1, 1], 8, 4, 16, seed=45, corrupt=(1, 2))
        commands = CommandList()
        commands.dispatch_many(Op.paged_attention_ragged(0.09, 16), inputs, [t["out"], t["keys"], t["values"]])
        with pytest.raises(BackendError) as info:
            hip.submit_static(commands) if static else hip.submit(commands).wait()
        assert info.value.status == Status.DEVICE_ERROR_FLAG and info.value.index == 2 and info.value.dispatch == 0
        results.append(hip.read(t["out"]))
    assert results[0] == results[1]


def test_a_need_beyond_the_fixed_array_is_refused(hip):
    """8 MiB of f32 accumulators hold 2 Mi elements: a 2048 x 2048 product under an unrecognised
    epilogue needs twice that.  The call names the dispatch; the one before it has run; the same
    list goes through fh_submit; and the static entry point still works afterwards."""
    weights = Quantised(55, 1, (2048, 64))
    small = Quantised(55, 4, (64, 64))
    x = upload(hip, normal_bf16(55, 2, (2048, 64)), DType.BF16)
    extra = hip.alloc(DType.BF16, (2048, 2048))
    out, first = hip.alloc(DType.BF16, (2048, 2048)), hip.alloc(DType.BF16, (2048, 64))
    b = ProgramBuilder(ProgramKind.MAP)
    b.output(0, b.mul(b.input(0), b.input(1)))
    epilogue = hip.prepare_epilogue(b.finish())
    commands = CommandList()
    commands.dispatch(Op.quant_matmul(4, 64), [x, *small.upload(hip)], first)
    commands.dispatch_epilogue(Op.quant_matmul(4, 64), [x, *weights.upload(hip)], out, epilogue, [extra])
    with pytest.raises(BackendError) as info:
        hip.submit_static(commands)
    assert info.value.status == Status.QUOTA_EXCEEDED and info.value.dispatch == 1
    assert np.frombuffer(hip.read(first), np.uint16).any()
    hip.submit(commands).wait()
    many = CommandList()
    many.dispatch(Op.copy(), [first], hip.alloc(DType.BF16, (2048, 64)))
    many.dispatches.extend([many.dispatches[0]] * 8192)     # one more than the error records hold
    with pytest.raises(BackendError) as info:
        hip.submit_static(many)
    assert info.value.status == Status.QUOTA_EXCEEDED
    test_accumulators_programs_sampling_and_packing_match(hip)
