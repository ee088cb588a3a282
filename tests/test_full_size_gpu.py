"""The BASELINE configurations at their full sizes, where the CPU oracle is out of reach.

Each case runs the operation twice on the device with the same seeded data, through two
independent implementations that must agree to the stated bf16 bar, |a - b| <= 1e-2 + 1e-2 |b|:
once through the specialised bf16 matrix-core kernels and once with the activations given as f32,
which selects the f32 vector-ALU kernels for the quantised products (qmm_valu.hip) and the strided
f32 kernel for attention; both follow the oracle's arithmetic order and are checked against it at
small sizes in test_parity_gpu.py.  The cases named "strided" go further and hand over views with
padded rows, which only the any-stride kernels of generic_ops.hip accept.  Paging is checked
through its round-trip property: rows appended through block tables read back bit for bit."""
import math

import numpy as np
import pytest

from forja_amd import programs
from forja_amd.core import CommandList, DType, Op
from tests.helpers import assert_close, to_f32

pytestmark = pytest.mark.gpu


def seeded(hip, dtype, shape, seed, stream, kind=2, lo=0.0, hi=0.0):
    tensor = hip.alloc(dtype, shape)
    commands = CommandList()
    commands.dispatch(Op.fill_seeded(kind, seed, stream, lo=lo, hi=hi), [], tensor)
    hip.submit(commands).wait()
    return tensor


def as_f32(hip, tensor):
    wide = hip.alloc(DType.F32, tensor.shape)
    commands = CommandList()
    commands.dispatch(Op.copy(), [tensor], wide)
    hip.submit(commands).wait()
    return wide


def quantised(hip, n, k, seed, experts=None):
    lead = () if experts is None else (experts,)
    packed = seeded(hip, DType.U32, lead + (n, k // 8), seed, 1, kind=0)
    scales = seeded(hip, DType.BF16, lead + (n, k // 64), seed, 2, kind=1, lo=0.001, hi=0.02)
    biases = seeded(hip, DType.BF16, lead + (n, k // 64), seed, 3, kind=1, lo=-0.1, hi=0.1)
    return [packed, scales, biases]


def run(hip, commands):
    hip.submit(commands).wait()


def release(hip, *tensors):
    for tensor in tensors:
        hip.release(tensor)


@pytest.mark.parametrize("rows,n,k,note", [
    (128, 5120, 2048, "config 3 stacked qkv"),
    (128, 2048, 4096, "config 3 o_proj"),
    (128, 128, 2048, "config 3 router"),
    (128, 151936, 2048, "config 3 lm_head"),
    (2048, 4096, 1024, "config 1 stacked qkv over the packed 2048-token batch"),
    (8256, 512, 5120, "config 4 prefill rows, a 512-column slice of a projection"),
    (8256, 256, 17408, "config 4 down projection depth, a 256-column slice (128 x 128 tiles)"),
    (8256, 1536, 17408, "config 4 down projection depth in 256 x 256 tiles (33 x 6 of them)"),
])
def test_quantised_projection_fast_and_generic_paths_agree(hip, rows, n, k, note):
    weights = quantised(hip, n, k, seed=101)
    x = seeded(hip, DType.BF16, (rows, k), 101, 4)
    x_wide = as_f32(hip, x)
    fast = hip.alloc(DType.BF16, (rows, n))
    generic = hip.alloc(DType.F32, (rows, n))
    commands = CommandList()
    commands.dispatch(Op.quant_matmul(4, 64), [x, *weights], fast)
    commands.dispatch(Op.quant_matmul(4, 64), [x_wide, *weights], generic)
    run(hip, commands)
    assert_close(to_f32(hip.read(fast), DType.BF16), to_f32(hip.read(generic), DType.F32), DType.BF16)
    release(hip, x, x_wide, fast, generic, *weights)


def test_config3_qkv_projection_through_the_strided_kernel(hip):
    """Config 3 stacked qkv (128 x 5120 x 2048) against the any-stride kernel: its activations and
    output are views into rows padded by one element, which no specialised kernel accepts."""
    rows, n, k = 128, 5120, 2048
    weights = quantised(hip, n, k, seed=121)
    x = seeded(hip, DType.BF16, (rows, k), 121, 4)
    padded_x = hip.alloc(DType.BF16, (rows, k + 1))
    padded_out = hip.alloc(DType.BF16, (rows, n + 1))
    fast = hip.alloc(DType.BF16, (rows, n))
    commands = CommandList()
    commands.dispatch(Op.copy(), [x], padded_x.narrow(1, 0, k))
    commands.dispatch(Op.quant_matmul(4, 64), [x, *weights], fast)
    commands.dispatch(Op.quant_matmul(4, 64), [padded_x.narrow(1, 0, k), *weights], padded_out.narrow(1, 0, n))
    run(hip, commands)
    strided = to_f32(hip.read(padded_out), DType.BF16).reshape(rows, n + 1)[:, :n]
    assert_close(to_f32(hip.read(fast), DType.BF16).reshape(rows, n), strided, DType.BF16)
    release(hip, x, padded_x, padded_out, fast, *weights)


def test_config4_gate_up_projection_at_full_width(hip):
    """Config 4's stacked gate/up projection at its real shape, 8256 rows x 34816 columns x 5120:
    one product on the matrix cores over all rows, and the f32 kernels over three 64-row blocks of
    the same rows (first, middle, last), every column."""
    rows, n, k = 8256, 34816, 5120
    weights = quantised(hip, n, k, seed=131)
    x = seeded(hip, DType.BF16, (rows, k), 131, 4)
    fast = hip.alloc(DType.BF16, (rows, n))
    commands = CommandList()
    commands.dispatch(Op.quant_matmul(4, 64), [x, *weights], fast)
    run(hip, commands)
    for first in (0, 4096, rows - 64):
        block = as_f32(hip, x.narrow(0, first, 64))
        generic = hip.alloc(DType.F32, (64, n))
        commands = CommandList()
        commands.dispatch(Op.quant_matmul(4, 64), [block, *weights], generic)
        run(hip, commands)
        assert_close(to_f32(hip.read(fast.narrow(0, first, 64)), DType.BF16),
                     to_f32(hip.read(generic), DType.F32), DType.BF16)
        release(hip, block, generic)
    release(hip, x, fast, *weights)


def test_config4_down_projection_at_full_depth(hip):
    """Config 4's down projection at its real shape, 8256 rows x 5120 columns x 17408, the deepest
    contraction of the configurations (the case the centred weights and the scaled rows of the
    tiled GEMM exist for): one product on the matrix cores over all rows, and the f32 kernels over
    three 64-row blocks of the same rows (first, middle, last), every column."""
    rows, n, k = 8256, 5120, 17408
    weights = quantised(hip, n, k, seed=133)
    x = seeded(hip, DType.BF16, (rows, k), 133, 4)
    fast = hip.alloc(DType.BF16, (rows, n))
    commands = CommandList()
    commands.dispatch(Op.quant_matmul(4, 64), [x, *weights], fast)
    run(hip, commands)
    for first in (0, 4096, rows - 64):
        block = as_f32(hip, x.narrow(0, first, 64))
        generic = hip.alloc(DType.F32, (64, n))
        commands = CommandList()
        commands.dispatch(Op.quant_matmul(4, 64), [block, *weights], generic)
        run(hip, commands)
        assert_close(to_f32(hip.read(fast.narrow(0, first, 64)), DType.BF16),
                     to_f32(hip.read(generic), DType.F32), DType.BF16)
        release(hip, block, generic)
    release(hip, x, fast, *weights)


@pytest.mark.parametrize("rows,n,k,note", [
    (8256, 1024, 2048, "config 4 prefill rows: residual add joined to the tiled GEMM"),
    (128, 5120, 17408, "config 4 decode rows: residual add joined to the slab sum"),
])
def test_projection_with_residual_add_fast_and_generic_paths_agree(hip, rows, n, k, note):
    weights = quantised(hip, n, k, seed=111)
    x = seeded(hip, DType.BF16, (rows, k), 111, 4)
    residual = seeded(hip, DType.BF16, (rows, n), 111, 5)
    x_wide = as_f32(hip, x)
    add = hip.prepare_epilogue(programs.add_elements())
    fast = hip.alloc(DType.BF16, (rows, n))
    generic = hip.alloc(DType.F32, (rows, n))
    commands = CommandList()
    commands.dispatch_epilogue(Op.quant_matmul(4, 64), [x, *weights], fast, add, [residual])
    commands.dispatch_epilogue(Op.quant_matmul(4, 64), [x_wide, *weights], generic, add, [residual])
    run(hip, commands)
    assert_close(to_f32(hip.read(fast), DType.BF16), to_f32(hip.read(generic), DType.F32), DType.BF16)
    release(hip, x, x_wide, residual, fast, generic, *weights)


def test_config2_moe_block_fast_and_generic_paths_agree(hip):
    """256 decode tokens, 128 experts, top-8 of N(0,1) router logits, expert SwiGLU 2048 x 768."""
    tokens, hidden, experts, top_k, inner = 256, 2048, 128, 8, 768
    gate, up = quantised(hip, inner, hidden, 201, experts), quantised(hip, inner, hidden, 202, experts)
    down = quantised(hip, hidden, inner, 203, experts)
    x = seeded(hip, DType.BF16, (tokens, hidden), 204, 1)
    logits = seeded(hip, DType.BF16, (tokens, experts), 204, 2)
    weights = hip.alloc(DType.BF16, (tokens, top_k))
    indices = hip.alloc(DType.U32, (tokens, top_k))
    swiglu = hip.prepare_epilogue(programs.silu_mul_elements())
    activated = hip.alloc(DType.BF16, (tokens, top_k, inner))
    out = hip.alloc(DType.BF16, (tokens, hidden))
    gq = Op.gather_quant_matmul(4, 64)
    commands = CommandList()
    commands.dispatch_many(Op.top_k(top_k, True), [logits], [weights, indices])
    commands.dispatch_epilogue(gq, [x, *gate, *up, indices], activated, swiglu, [])
    commands.dispatch(gq, [activated, *down, indices, weights], out)
    run(hip, commands)
    chosen = np.frombuffer(hip.read(indices), np.uint32)
    counts = np.bincount(chosen, minlength=experts)
    assert counts.sum() == tokens * top_k and counts.max() <= 40 and len(np.unique(chosen)) > 120
    # the same block through the generic kernels: f32 activations and route weights
    x_wide, weights_wide, activated_from_fast = as_f32(hip, x), as_f32(hip, weights), as_f32(hip, activated)
    activated_wide = hip.alloc(DType.F32, (tokens, top_k, inner))
    out_wide = hip.alloc(DType.F32, (tokens, hidden))
    commands = CommandList()
    commands.dispatch_epilogue(gq, [x_wide, *gate, *up, indices], activated_wide, swiglu, [])
    commands.dispatch(gq, [activated_from_fast, *down, indices, weights_wide], out_wide)
    run(hip, commands)
    assert_close(to_f32(hip.read(activated), DType.BF16), to_f32(hip.read(activated_wide), DType.F32),
                 DType.BF16)
    assert_close(to_f32(hip.read(out), DType.BF16), to_f32(hip.read(out_wide), DType.F32), DType.BF16)


def ragged_batch(hip, contexts, counts, hq, hkv, pt, seed):
    """Device-seeded ragged batch with shuffled block tables; returns the tensors by name."""
    rng = np.random.default_rng(seed)
    lanes = len(contexts)
    pages_of = [(c + n + pt - 1) // pt for c, n in zip(contexts, counts)]
    table_pages, physical = max(pages_of) + 1, sum(pages_of) + 3
    order = rng.permutation(physical)
    tables = np.zeros((lanes, table_pages, 2), np.uint32)
    tables[:, :, 1] = 0xffffffff
    cursor = 0
    for lane, need in enumerate(pages_of):
        pages = order[cursor:cursor + need]
        cursor += need
        tables[lane, :need, 0] = pages
        tables[lane, :need, 1] = 11 + pages
    total = sum(counts)

    def up(array, shape):
        tensor = hip.alloc(DType.U32, shape)
        hip.write(tensor, np.ascontiguousarray(array, dtype=np.uint32).tobytes())
        return tensor
    return dict(
        tables=up(tables, tables.shape), generations=up(11 + np.arange(physical), (physical,)),
        cu=up(np.concatenate([[0], np.cumsum(counts)]), (lanes + 1,)), starts=up(contexts, (lanes,)),
        activity=up(np.ones(lanes), (lanes,)),
        q=seeded(hip, DType.BF16, (total, hq, 128), seed, 1),
        k_new=seeded(hip, DType.BF16, (total, hkv, 128), seed, 2),
        v_new=seeded(hip, DType.BF16, (total, hkv, 128), seed, 3),
        keys=seeded(hip, DType.BF16, (physical, pt, hkv, 128), seed, 4),
        values=seeded(hip, DType.BF16, (physical, pt, hkv, 128), seed, 5),
        table_array=tables, total=total)


def attention_both_ways(hip, contexts, counts, hq, hkv):
    pt, scale = 16, 1.0 / math.sqrt(128)
    t = ragged_batch(hip, contexts, counts, hq, hkv, pt, seed=301)
    tail = [t["tables"], t["generations"], t["cu"], t["starts"], t["activity"]]
    fast = hip.alloc(DType.BF16, (t["total"], hq, 128))
    commands = CommandList()
    commands.dispatch_many(Op.paged_attention_ragged(scale, pt), [t["q"], t["k_new"], t["v_new"], *tail],
                           [fast, t["keys"], t["values"]])
    run(hip, commands)
    keys_after = hip.read(t["keys"])
    wide = [as_f32(hip, t[name]) for name in ("q", "k_new", "v_new")]
    generic = hip.alloc(DType.F32, (t["total"], hq, 128))
    commands = CommandList()
    commands.dispatch_many(Op.paged_attention_ragged(scale, pt), [*wide, *tail],
                           [generic, t["keys"], t["values"]])
    run(hip, commands)
    assert hip.read(t["keys"]) == keys_after          # appending the same rows again changes nothing
    assert_close(to_f32(hip.read(fast), DType.BF16), to_f32(hip.read(generic), DType.F32), DType.BF16)
    # round trip of the appended rows of the longest lane through its block table
    lane = int(np.argmax(np.array(contexts) + np.array(counts)))
    first = int(np.cumsum([0] + list(counts))[lane])
    new_rows = np.frombuffer(hip.read(t["k_new"]), np.uint16).reshape(t["total"], hkv * 128)
    pool = np.frombuffer(keys_after, np.uint16).reshape(-1, pt, hkv * 128)
    for offset in range(counts[lane]):
        position = contexts[lane] + offset
        page = int(t["table_array"][lane, position // pt, 0])
        assert np.array_equal(pool[page, position % pt], new_rows[first + offset])


def test_config3_decode_attention_full_batch(hip):
    """128 decode lanes, contexts log-uniform over 256..32768, 32 query / 4 kv heads."""
    rng = np.random.default_rng(7)
    contexts = np.exp(rng.uniform(math.log(256), math.log(32768), 128)).astype(int).tolist()
    attention_both_ways(hip, contexts, [1] * 128, 32, 4)


def test_config3_decode_attention_with_the_engine_dtypes(hip):
    """The same batch with the qwen3-coder engine's dtypes: f32 rows against an f16 KV cache.  The
    specialised kernels against the strided ones, which an output view with unaligned rows selects;
    both round the new rows into the pools identically."""
    rng = np.random.default_rng(7)
    contexts = np.exp(rng.uniform(math.log(256), math.log(32768), 128)).astype(int).tolist()
    hq, hkv, pt, scale = 32, 4, 16, 1.0 / math.sqrt(128)
    t = ragged_batch(hip, contexts, [1] * 128, hq, hkv, pt, seed=302)
    rows = [seeded(hip, DType.F32, t[name].shape, 302, 6 + index) for index, name in enumerate(("q", "k_new", "v_new"))]
    pools = [seeded(hip, DType.F16, t["keys"].shape, 302, 9 + index) for index in range(2)]
    tail = [t["tables"], t["generations"], t["cu"], t["starts"], t["activity"]]
    fast = hip.alloc(DType.F32, (128, hq, 128))
    commands = CommandList()
    commands.dispatch_many(Op.paged_attention_ragged(scale, pt, one_row_per_lane=True), [*rows, *tail],
                           [fast, *pools])
    run(hip, commands)
    keys_after, values_after = hip.read(pools[0]), hip.read(pools[1])
    padded = hip.alloc(DType.F32, (128, hq, 129))
    commands = CommandList()
    commands.dispatch_many(Op.paged_attention_ragged(scale, pt), [*rows, *tail],
                           [padded.narrow(2, 0, 128), *pools])
    run(hip, commands)
    assert hip.read(pools[0]) == keys_after and hip.read(pools[1]) == values_after
    generic = to_f32(hip.read(padded), DType.F32).reshape(128, hq, 129)[:, :, :128]
    assert_close(to_f32(hip.read(fast), DType.F32), generic, DType.F16)
    # the stored rows are the f32 rows rounded to f16, at the positions the tables name
    new_rows = to_f32(hip.read(rows[1]), DType.F32).reshape(128, hkv * 128).astype(np.float16)
    pool = np.frombuffer(keys_after, np.float16).reshape(-1, pt, hkv * 128)
    for lane in (0, 17, 127):
        page = int(t["table_array"][lane, contexts[lane] // pt, 0])
        assert np.array_equal(pool[page, contexts[lane] % pt], new_rows[lane])


def test_config1_packed_batch_attention(hip):
    """48 decode lanes (contexts uniform 128..4096) and prefill chunks of 256, 384, 512 and 848
    tokens packed into 2048 tokens, 16 query / 8 kv heads."""
    rng = np.random.default_rng(8)
    contexts = rng.integers(128, 4097, 48).tolist() + [0, 0, 0, 0]
    attention_both_ways(hip, contexts, [1] * 48 + [256, 384, 512, 848], 16, 8)


def test_config4_prefill_attention_largest_prompt(hip):
    """The 3072-token prompt of the config 4 chunk plus decode rows, 40 query / 8 kv heads."""
    attention_both_ways(hip, [0, 1500, 4000], [3072, 1, 1], 40, 8)


def test_config4_prefill_chunk_full_batch(hip):
    """The whole config 4 batch: an 8192-token prefill chunk packed from six prompts of 512 to 3072
    tokens (two of them continuing an earlier chunk) plus 64 decode rows, 40 query / 8 kv heads."""
    rng = np.random.default_rng(10)
    prompts = [512, 768, 1024, 1280, 1536, 3072]
    assert sum(prompts) == 8192
    contexts = [0, 0, 2048, 0, 512, 0] + rng.integers(64, 8193, 64).tolist()
    attention_both_ways(hip, contexts, prompts + [1] * 64, 40, 8)


def test_config3_churn_lane_by_lane_equals_the_packed_recording(hip):
    """Config 3's continuous batch under churn: 128 lanes, contexts log-uniform over 256..32768,
    eight steps, and before every step eight sequences retire and eight are admitted into the freed
    pages.  The lane-by-lane recording (fused by the library) and the packed recording run on
    separate storage with the same seeds: tokens every step and the final logits must be equal bit
    for bit, and the last layer's newly appended key rows must read back from the pool through the
    block tables bit for bit."""
    from forja_amd.model import QWEN3_CODER_30B_A3B, DecodeSession, Model
    rng = np.random.default_rng(12)
    lanes, pt = 128, 16
    contexts = np.exp(rng.uniform(math.log(256), math.log(32768), lanes)).astype(int).tolist()
    pages = int(sum((c + 64 + pt) // pt for c in contexts) * 1.4)
    sessions = [DecodeSession(Model(hip, QWEN3_CODER_30B_A3B, seed=23, layers=2), contexts, seed=23,
                              physical_pages=pages, table_pages=(32768 + 4096) // pt)
                for _ in range(2)]
    packed, by_lane = sessions
    by_lane.record_lane_by_lane()
    before = hip.fusion_stats()
    retired = 0
    for step in range(8):
        for _ in range(8):
            lane = retired % lanes
            retired += 1
            context = int(math.exp(rng.uniform(math.log(256), math.log(8192))))
            for session in sessions:
                session.replace_lane(lane, context)
        expected = packed.step()
        actual = by_lane.step(lane_by_lane=True)
        assert expected.tolist() == actual.tolist(), step
    assert hip.read(packed.buffers.logits) == hip.read(by_lane.buffers.logits)
    runs, replaced = (after - start for after, start in zip(hip.fusion_stats(), before))
    assert (runs, replaced) == (8 * 2, 8 * 2 * 2 * lanes)
    # round trip: the key rows the last step appended in the last layer, through the tables
    c = QWEN3_CODER_30B_A3B
    for session in sessions:
        qk = np.frombuffer(hip.read(session.buffers.qk), np.uint16).reshape(lanes, c.q_heads + c.kv_heads, c.head_dim)
        pool = np.frombuffer(hip.read(session.cache.keys[-1]), np.uint16).reshape(-1, pt, c.kv_heads, c.head_dim)
        for lane in range(lanes):
            position = int(session.contexts[lane]) - 1          # the token this step appended
            page = int(session.cache.table_values[lane, position // pt, 0])
            assert np.array_equal(pool[page, position % pt], qk[lane, c.q_heads:]), lane


def test_config3_step_recorded_lane_by_lane_equals_the_packed_recording(hip):
    """Two layers of the config 3 model on 128 lanes with contexts log-uniform over 256..32768:
    the step recorded the way the engines record it (per lane one PagedSdpaAppend and one Copy per
    layer) goes through the library's run fusion and must give the packed recording's tokens and
    logits bit for bit over several steps, with every layer's run fused."""
    from forja_amd.model import QWEN3_CODER_30B_A3B, DecodeSession, Model
    rng = np.random.default_rng(9)
    contexts = np.exp(rng.uniform(math.log(256), math.log(32768), 128)).astype(int).tolist()
    packed, by_lane = (DecodeSession(Model(hip, QWEN3_CODER_30B_A3B, seed=21, layers=2), contexts, seed=21)
                       for _ in range(2))
    by_lane.record_lane_by_lane()
    before = hip.fusion_stats()
    for _ in range(3):
        expected = packed.step()
        actual = by_lane.step(lane_by_lane=True)
        assert expected.tolist() == actual.tolist()
    assert hip.read(packed.buffers.logits) == hip.read(by_lane.buffers.logits)
    runs, replaced = (after - start for after, start in zip(hip.fusion_stats(), before))
    assert (runs, replaced) == (3 * 2, 3 * 2 * 2 * 128)
