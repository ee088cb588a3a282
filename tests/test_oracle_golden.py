"""Pins the CPU oracle against the reference's own known-answer tests and against independent
mathematics (float64 numpy, closed forms).  No GPU.  Each test names the reference test it
restates (crates/forja-cpu/src/lib.rs unless noted)."""
import math
import os

import numpy as np
import pytest

from forja_amd.core import (BinOp, CommandList, DType, Inst, Op, Program, ProgramBuilder,
                            ProgramKind, RedOp, Slice, Status, BackendError, UnOp, ValueType,
                            INTO_PAGES, OUT_OF_PAGES)
from oracle import cpu_backend as orc
from tests.helpers import Quantised, assert_close, from_f32, normal_bf16, to_f32, upload, upload_raw

GOLDEN = os.path.join(os.path.dirname(__file__), "golden")


def run(backend, commands):
    backend.submit(commands).wait()


# ------------------------------------------------------------------ conversions

def test_bf16_round_to_nearest_even_and_round_trip():
    lib = orc.lib()
    # ties: 1 + 2^-8 is exactly half way between bf16(1.0) and the next value -> even (1.0)
    assert lib.orc_f32_to_bf16(np.float32(1.0 + 2.0 ** -8)) == 0x3f80
    assert lib.orc_f32_to_bf16(np.float32(1.0 + 3 * 2.0 ** -8)) == 0x3f82
    assert lib.orc_f32_to_bf16(np.float32(1.0 + 2.0 ** -8 + 2.0 ** -20)) == 0x3f81
    # every bf16 bit pattern survives f32 and back (NaNs become quiet)
    bits = np.arange(65536, dtype=np.uint16)
    back = orc.f32_to_bf16(orc.bf16_to_f32(bits))
    nan = (bits & 0x7fff) > 0x7f80
    assert np.array_equal(back[~nan], bits[~nan])
    assert np.array_equal(back[nan], bits[nan] | 0x40)


def test_f16_matches_numpy_half_including_subnormals():
    rng = np.random.default_rng(7)
    values = np.concatenate([
        rng.standard_normal(20000).astype(np.float32) * np.float32(10.0) ** rng.integers(-9, 6, 20000),
        np.array([0.0, -0.0, 65504.0, 65520.0, 70000.0, 5.96e-8, 2.98e-8, 2.99e-8, 6.1e-5, np.inf,
                  -np.inf], dtype=np.float32)])
    ours = orc.encode(values, DType.F16).view(np.uint16)
    with np.errstate(over="ignore"):
        theirs = values.astype(np.float16).view(np.uint16)
    assert np.array_equal(ours, theirs)
    bits = np.arange(65536, dtype=np.uint16)
    decoded = orc.decode(bits.view(np.uint8), DType.F16)
    expected = bits.view(np.float16).astype(np.float32)
    keep = ~np.isnan(expected)
    assert np.array_equal(decoded[keep], expected[keep])


# ------------------------------------------------------------------ quantised matmul

@pytest.mark.parametrize("bits,param_dtype", [(4, DType.BF16), (8, DType.F16)])
@pytest.mark.parametrize("rows", [1, 7, 33])
def test_quant_matmul_dequantizes_q4_and_q8_in_mlx_order(cpu, bits, param_dtype, rows):
    """lib.rs:2786-2845"""
    inner = 64
    activations = (np.arange(rows * inner) % 17).astype(np.float32) / 8.0 - 1.0
    x = upload(cpu, activations.reshape(rows, inner), DType.F32)
    vpw = 32 // bits
    repeats = inner // vpw
    pattern = 0x11111111 if bits == 4 else 0x01010101
    maximum = (1 << bits) - 1
    words = np.repeat(np.array([0, pattern, pattern * maximum], dtype=np.uint32), repeats)
    packed = upload_raw(cpu, words, DType.U32, (3, repeats))
    scale_values, bias_values = [0.5, -0.25, 0.125], [1.0, 2.0, -1.0]
    scales = upload(cpu, np.array(scale_values).reshape(3, 1), param_dtype)
    biases = upload(cpu, np.array(bias_values).reshape(3, 1), param_dtype)
    out = cpu.alloc(DType.F32, (rows, 3))
    commands = CommandList()
    commands.dispatch(Op.quant_matmul(bits, 64), [x, packed, scales, biases], out)
    run(cpu, commands)
    sums = activations.reshape(rows, inner).astype(np.float32).sum(axis=1, dtype=np.float32)
    expected = np.stack([sums * bias_values[0], sums * (scale_values[1] + bias_values[1]),
                         sums * (scale_values[2] * maximum + bias_values[2])], axis=1)
    actual = to_f32(cpu.read(out), DType.F32).reshape(rows, 3)
    np.testing.assert_allclose(actual, expected, rtol=1e-5, atol=1e-5)


def test_quant_matmul_matches_float64_dequantise_then_matmul(cpu):
    """Reduces to a library routine: dequantise in float64, numpy matmul."""
    for bits, group in [(4, 64), (4, 32), (8, 128)]:
        weights = Quantised(11, 10 * bits + group, (24, 256), bits=bits, group=group)
        x_values = normal_bf16(11, 3, (5, 256))
        x = upload(cpu, x_values, DType.BF16)
        packed, scales, biases = weights.upload(cpu)
        out = cpu.alloc(DType.BF16, (5, 24))
        commands = CommandList()
        commands.dispatch(Op.quant_matmul(bits, group), [x, packed, scales, biases], out)
        run(cpu, commands)
        expected = x_values.astype(np.float64) @ weights.dequantised().T
        assert_close(to_f32(cpu.read(out), DType.BF16), expected, DType.BF16)


def test_tiny_model_fixture_pins_nibble_order_and_dequantisation(cpu):
    """Derived from crates/forja-host/tests/fixtures/qwen38 (see golden/make_tiny_qwen_fixture.py)."""
    z = np.load(os.path.join(GOLDEN, "tiny_qwen_mlx4.npz"))
    packed = upload_raw(cpu, z["embed_packed"], DType.U32, z["embed_packed"].shape)
    scales = upload_raw(cpu, z["embed_scales_bf16"], DType.BF16, z["embed_scales_bf16"].shape)
    biases = upload_raw(cpu, z["embed_biases_bf16"], DType.BF16, z["embed_biases_bf16"].shape)
    ids = upload_raw(cpu, z["prompt_token_ids"], DType.U32, (3,))
    rows = cpu.alloc(DType.BF16, (3, 64))
    commands = CommandList()
    commands.dispatch(Op.quant_embed(4, 64), [packed, scales, biases, ids], rows)
    run(cpu, commands)
    assert np.array_equal(to_f32(cpu.read(rows), DType.BF16), z["hidden_state_0"].ravel())

    hidden = upload(cpu, z["final_hidden_last"].reshape(1, 64), DType.F32)
    lp = upload_raw(cpu, z["lm_head_packed"], DType.U32, z["lm_head_packed"].shape)
    ls = upload_raw(cpu, z["lm_head_scales_bf16"], DType.BF16, z["lm_head_scales_bf16"].shape)
    lb = upload_raw(cpu, z["lm_head_biases_bf16"], DType.BF16, z["lm_head_biases_bf16"].shape)
    logits = cpu.alloc(DType.F32, (1, 33))
    token = cpu.alloc(DType.U32, (1,))
    commands = CommandList()
    commands.dispatch(Op.quant_matmul(4, 64), [hidden, lp, ls, lb], logits)
    commands.dispatch(Op.argmax(), [logits], token)
    run(cpu, commands)
    actual = to_f32(cpu.read(logits), DType.F32)
    expected = z["prompt_last_logits"]
    assert np.linalg.norm(actual - expected) / np.linalg.norm(expected) < 5e-3  # bf16 model rounding
    assert np.frombuffer(cpu.read(token), np.uint32)[0] == z["first_greedy_token"][0]


def _small_experts(cpu, first_value):
    words = np.repeat(np.arange(first_value, first_value + 6, dtype=np.uint32) * np.uint32(0x11111111), 8)
    return upload_raw(cpu, words, DType.U32, (3, 2, 8))


def test_gathered_quantized_matmul_selects_duplicate_routes_and_reports_lowest_bad_index(cpu):
    """lib.rs:2848-2951"""
    x = upload(cpu, np.ones((1, 64)), DType.F32)
    packed = _small_experts(cpu, 0)
    scales = upload(cpu, np.ones((3, 2, 1)), DType.BF16)
    biases = upload(cpu, np.zeros((3, 2, 1)), DType.BF16)
    indices = upload(cpu, np.array([[2, 0, 2]]), DType.U32)
    out = cpu.alloc(DType.F32, (1, 3, 2))
    commands = CommandList()
    commands.dispatch(Op.gather_quant_matmul(4, 64), [x, packed, scales, biases, indices], out)
    run(cpu, commands)
    assert to_f32(cpu.read(out), DType.F32).tolist() == [256.0, 320.0, 0.0, 64.0, 256.0, 320.0]

    epilogue = Program(ProgramKind.MAP, [
        Inst.input(0), Inst.input(1), Inst.unary(UnOp.NEG, 0), Inst.unary(UnOp.EXP, 2),
        Inst.const(1.0), Inst.binary(BinOp.ADD, 4, 3), Inst.binary(BinOp.DIV, 0, 5),
        Inst.binary(BinOp.MUL, 6, 1)], [(0, 7)])
    fused = cpu.alloc(DType.F32, (1, 3, 2))
    commands = CommandList()
    commands.dispatch_epilogue(Op.gather_quant_matmul(4, 64),
                               [x, packed, scales, biases, packed, scales, biases, indices], fused,
                               cpu.prepare_epilogue(epilogue), [])
    run(cpu, commands)
    base = np.array([256.0, 320.0, 0.0, 64.0, 256.0, 320.0], dtype=np.float32)
    expected = base / (1.0 + np.exp(-base)) * base
    np.testing.assert_allclose(to_f32(cpu.read(fused), DType.F32), expected, rtol=1e-5)

    invalid = upload(cpu, np.array([[99, 7]]), DType.U32)
    out = cpu.alloc(DType.F32, (1, 2, 2))
    commands = CommandList()
    commands.dispatch(Op.gather_quant_matmul(4, 64), [x, packed, scales, biases, invalid], out)
    with pytest.raises(BackendError) as info:
        run(cpu, commands)
    assert info.value.status == Status.INDEX_OUT_OF_RANGE and info.value.index == 7
    assert cpu.read(out) == bytes(16)


def test_combined_quantized_matmul_keeps_valid_routes_and_reports_lowest_bad_index(cpu):
    """lib.rs:2954-3017"""
    activations = np.repeat(np.arange(1, 6, dtype=np.float32), 64).reshape(1, 5, 64)
    x = upload(cpu, activations, DType.F32)
    packed = _small_experts(cpu, 1)
    scales = upload(cpu, np.full((3, 2, 1), 0.5), DType.BF16)
    biases = upload(cpu, np.full((3, 2, 1), 0.25), DType.BF16)
    indices = upload(cpu, np.array([[2, 99, 0, 7, 1]]), DType.U32)
    weights = upload(cpu, np.array([[0.5, 1.0, -0.25, 2.0, 0.75]]), DType.F32)
    residual = upload(cpu, np.array([[1.5, -2.0]]), DType.F32)
    out = cpu.alloc(DType.F32, (1, 2))
    epilogue = Program(ProgramKind.MAP, [Inst.input(0), Inst.input(1), Inst.binary(BinOp.ADD, 0, 1)],
                       [(0, 2)])
    commands = CommandList()
    commands.dispatch_epilogue(Op.gather_quant_matmul(4, 64),
                               [x, packed, scales, biases, indices, weights], out,
                               cpu.prepare_epilogue(epilogue), [residual])
    with pytest.raises(BackendError) as info:
        run(cpu, commands)
    assert info.value.status == Status.INDEX_OUT_OF_RANGE and info.value.index == 7
    assert to_f32(cpu.read(out), DType.F32).tolist() == [473.5, 582.0]


# ------------------------------------------------------------------ selection

def _total_order_key(values):
    bits = values.view(np.int32).astype(np.int64)
    return np.where(bits < 0, bits ^ 0x7fffffff, bits)


def test_argmax_prefers_the_last_equal_value(cpu):
    """lib.rs:2386-2395"""
    x = upload(cpu, np.array([[1.0, 9.0, 2.0, 9.0, 3.0]]), DType.F32)
    out = cpu.alloc(DType.U32, (1,))
    commands = CommandList()
    commands.dispatch(Op.argmax(), [x], out)
    run(cpu, commands)
    assert np.frombuffer(cpu.read(out), np.uint32).tolist() == [3]


def top_k_case(width):
    values = (np.arange(width) % 11).astype(np.float32)
    if width >= 128:
        bits = values.view(np.uint32)
        bits[3], bits[9], bits[17] = 0x7fc00001, 0x7fc00002, 0xffc00001
    if width == 2050:
        values[2048], values[2049] = 1000.0, 999.0
    return values


@pytest.mark.parametrize("width,k", [(1, 1), (64, 8), (128, 8), (2050, 64)])
def test_top_k_orders_rows_for_edge_widths_ties_and_nans(cpu, width, k):
    """lib.rs:2398-2447; expectation = closed form: stable sort by (total order desc, index asc)."""
    values = top_k_case(width)
    keys = _total_order_key(values)
    expected = np.lexsort((np.arange(width), -keys))[:k]
    x = upload_raw(cpu, values, DType.F32, (1, width))
    out_values, out_indices = cpu.alloc(DType.F32, (1, k)), cpu.alloc(DType.U32, (1, k))
    commands = CommandList()
    commands.dispatch_many(Op.top_k(k, False), [x], [out_values, out_indices])
    run(cpu, commands)
    assert np.frombuffer(cpu.read(out_indices), np.uint32).tolist() == expected.tolist()
    assert np.array_equal(np.frombuffer(cpu.read(out_values), np.uint32), values.view(np.uint32)[expected])


def test_top_k_normalises_over_the_selected_set(cpu):
    x = upload(cpu, np.array([[1.0, 4.0, 2.0, 3.0]]), DType.F32)
    out_values, out_indices = cpu.alloc(DType.F32, (1, 2)), cpu.alloc(DType.U32, (1, 2))
    commands = CommandList()
    commands.dispatch_many(Op.top_k(2, True), [x], [out_values, out_indices])
    run(cpu, commands)
    denominator = 1.0 + math.exp(-1.0)
    np.testing.assert_allclose(to_f32(cpu.read(out_values), DType.F32),
                               [1.0 / denominator, math.exp(-1.0) / denominator], rtol=1e-6)
    assert np.frombuffer(cpu.read(out_indices), np.uint32).tolist() == [1, 3]


def test_route_pack_is_a_stable_counting_sort():
    rng = np.random.default_rng(5)
    for rows, k, experts, tile in [(256, 8, 128, 16), (7, 3, 5, 2), (128, 8, 128, 32), (1, 1, 1, 1)]:
        indices = rng.integers(0, experts, (rows, k)).astype(np.uint32)
        if rows > 4:
            indices[3, 0] = experts + 9   # one bad route
            indices[1, k - 1] = experts + 4
        counts, offsets, sorted_routes, blocks, invalid = orc.route_pack(indices, experts, tile)
        flat = indices.ravel().astype(np.int64)
        valid = np.nonzero(flat < experts)[0]
        order = valid[np.argsort(flat[valid], kind="stable")]
        assert np.array_equal(sorted_routes, order.astype(np.uint32))
        assert np.array_equal(counts, np.bincount(flat[valid], minlength=experts))
        assert np.array_equal(offsets, np.concatenate([[0], np.cumsum(counts)]))
        assert int(counts.sum()) == valid.size == sorted_routes.size
        expected_blocks = [(e, offsets[e] + s, min(tile, counts[e] - s))
                           for e in range(experts) for s in range(0, counts[e], tile)]
        assert blocks.tolist() == [list(map(int, b)) for b in expected_blocks]
        if rows > 4:
            assert invalid.tolist() == [1, experts + 4]


# ------------------------------------------------------------------ paged storage

def test_paged_copy_converts_directly_into_reduced_storage(cpu):
    """lib.rs:1883-1924"""
    values = np.arange(21, dtype=np.float32) / 8.0
    source = upload(cpu, values.reshape(7, 3), DType.F32)
    pool = cpu.alloc(DType.F16, (3, 4, 3))
    table = upload(cpu, np.array([[2, 5], [0, 7]]), DType.U32)
    generations = upload(cpu, np.array([7, 0, 5]), DType.U32)
    output = cpu.alloc(DType.F32, (7, 3))
    commands = CommandList()
    commands.dispatch(Op.paged_copy(INTO_PAGES, 1, 4), [source, table, generations], pool)
    commands.dispatch(Op.paged_copy(OUT_OF_PAGES, 1, 4), [pool, table, generations], output)
    run(cpu, commands)
    expected = values.astype(np.float16).astype(np.float32)
    assert np.array_equal(to_f32(cpu.read(output), DType.F32), expected)
    # placement: token t lands at table[(1+t)//4].page*4 + (1+t)%4
    pool_values = to_f32(cpu.read(pool), DType.F16).reshape(12, 3)
    for token in range(7):
        logical = 1 + token
        row = [2, 0][logical // 4] * 4 + logical % 4
        assert np.array_equal(pool_values[row], expected.reshape(7, 3)[token])


def test_paged_copy_crosses_nonconsecutive_pages(cpu):
    """crates/forja-cpu/src/paged.rs:408-419"""
    values = np.arange(12, dtype=np.float32).reshape(6, 2)
    source = upload(cpu, values, DType.F32)
    pool = cpu.alloc(DType.F32, (3, 4, 2))
    table = upload(cpu, np.array([[2, 1], [0, 1]]), DType.U32)
    generations = upload(cpu, np.array([1, 1, 1]), DType.U32)
    output = cpu.alloc(DType.F32, (6, 2))
    commands = CommandList()
    commands.dispatch(Op.paged_copy(INTO_PAGES, 2, 4), [source, table, generations], pool)
    commands.dispatch(Op.paged_copy(OUT_OF_PAGES, 2, 4), [pool, table, generations], output)
    run(cpu, commands)
    assert np.array_equal(to_f32(cpu.read(output), DType.F32), values.ravel())


def test_paged_append_stores_both_planes_before_attention(cpu):
    """lib.rs:1926-1970"""
    query = cpu.alloc(DType.F32, (16, 1, 128))
    key = cpu.alloc(DType.F32, (1, 8, 128))
    value = upload(cpu, np.ones((1, 8, 128)), DType.F32)
    table = upload(cpu, np.array([[0, 1]]), DType.U32)
    generations = upload(cpu, np.array([1]), DType.U32)
    key_pages = cpu.alloc(DType.F16, (1, 16, 8, 128))
    value_pages = cpu.alloc(DType.F16, (1, 16, 8, 128))
    output = cpu.alloc(DType.F32, (16, 1, 128))
    commands = CommandList()
    commands.dispatch_many(Op.paged_sdpa_append(0.125, 0, 16), [query, key, value, table, generations],
                           [output, key_pages, value_pages])
    run(cpu, commands)
    assert np.array_equal(to_f32(cpu.read(output), DType.F32), np.ones(16 * 128, np.float32))
    raw = cpu.read(value_pages)
    assert raw[:2048] == np.float16(1.0).tobytes() * 1024
    assert not any(raw[2048:])


def test_page_tables_are_authenticated_and_poison_is_never_dereferenced(cpu):
    """crates/forja-core/src/paged.rs:381-420 and cpu_page_table (lib.rs:1519-1535)."""
    source = upload(cpu, np.ones((4, 2)), DType.F32)
    pool = cpu.alloc(DType.F32, (3, 4, 2))
    generations = upload(cpu, np.array([7, 8, 9]), DType.U32)
    poison = [0, 0xffffffff]
    ok = upload(cpu, np.array([[1, 8], poison]), DType.U32)
    commands = CommandList()
    commands.dispatch(Op.paged_copy(INTO_PAGES, 0, 4), [source, ok, generations], pool)
    run(cpu, commands)  # padded tail is accepted while untouched
    for bad in ([[1, 7], poison], [[3, 8], poison]):   # stale generation; page out of range
        table = upload(cpu, np.array(bad), DType.U32)
        commands = CommandList()
        commands.dispatch(Op.paged_copy(INTO_PAGES, 0, 4), [source, table, generations], pool)
        with pytest.raises(BackendError) as info:
            run(cpu, commands)
        assert info.value.status == Status.EXECUTION_FAILED
    # dereferencing the poison entry is refused
    commands = CommandList()
    commands.dispatch(Op.paged_copy(INTO_PAGES, 2, 4), [source, ok, generations], pool)
    with pytest.raises(BackendError):
        run(cpu, commands)


def test_inactive_lane_writes_zeros_and_leaves_pools_untouched(cpu):
    """lib.rs:197-199, :319-328, :1972-1982"""
    query = upload(cpu, np.ones((2, 1, 4)), DType.F32)
    key = upload(cpu, np.ones((1, 1, 4)), DType.F32)
    value = upload(cpu, np.ones((1, 1, 4)), DType.F32)
    table = upload(cpu, np.array([[0, 0xffffffff]]), DType.U32)   # poison: must not be read
    generations = upload(cpu, np.array([1]), DType.U32)
    activity = upload(cpu, np.array([0]), DType.U32)
    key_pages, value_pages = cpu.alloc(DType.F32, (1, 4, 1, 4)), cpu.alloc(DType.F32, (1, 4, 1, 4))
    output = upload(cpu, np.full((2, 1, 4), 5.0), DType.F32)
    commands = CommandList()
    commands.dispatch_many(Op.paged_sdpa_append(1.0, 0, 4),
                           [query, key, value, table, generations, activity],
                           [output, key_pages, value_pages])
    run(cpu, commands)
    assert not any(cpu.read(output)) and not any(cpu.read(key_pages)) and not any(cpu.read(value_pages))


def test_paged_attention_matches_a_hand_checked_case(cpu):
    """crates/forja-cpu/src/paged.rs:457-476: e/(e+1)"""
    pool_values = np.zeros((2, 4, 1, 2), np.float32)
    pool_values[1, 0, 0] = [1.0, 0.0]
    pool_values[1, 1, 0] = [0.0, 1.0]
    keys = upload(cpu, pool_values, DType.F32)
    values = upload(cpu, pool_values, DType.F32)
    table = upload(cpu, np.array([[1, 4], [0, 3]]), DType.U32)
    generations = upload(cpu, np.array([3, 4]), DType.U32)
    query = upload(cpu, np.array([[[1.0, 0.0]]]), DType.F32)
    out = cpu.alloc(DType.F32, (1, 1, 2))
    commands = CommandList()
    commands.dispatch(Op.paged_sdpa(1.0, False, 0, 2, 4), [query, keys, values, table, generations], out)
    run(cpu, commands)
    expected = math.e / (math.e + 1.0)
    np.testing.assert_allclose(to_f32(cpu.read(out), DType.F32), [expected, 1 - expected], atol=1e-6)


def paged_case(backend, hq, hkv, sq, key_length, pt, q_start, pool_dtype=DType.BF16, seed=3, q_dtype=None):
    """Deterministic paged K/V in the style of crates/forja-metal/tests/paged.rs:645-659 with a
    shuffled table, generations 11+page, NaN in unused slots and a poisoned table tail."""
    width = 128
    logical = (key_length + pt - 1) // pt
    physical = logical + 3
    rng = np.random.default_rng(seed)
    pages = rng.permutation(physical)[:logical]
    keys = np.full((physical * pt, hkv * width), np.nan, np.float32)
    vals = np.full((physical * pt, hkv * width), np.nan, np.float32)
    token = np.arange(key_length)[:, None]
    element = np.arange(hkv * width)[None, :]
    rows = pages[token[:, 0] // pt] * pt + token[:, 0] % pt
    keys[rows] = ((token * 13 + element * 7) % 101) / 100.0 - 0.5
    vals[rows] = ((token * 5 + element * 11) % 97) / 96.0 - 0.5
    table = np.zeros((logical + 2, 2), np.uint32)
    table[:logical, 0] = pages
    table[:logical, 1] = 11 + pages
    table[logical:] = [0, 0xffffffff]
    index = np.arange(hq * sq * width)
    query = ((index * 17) % 89) / 88.0 - 0.5
    q_dtype = pool_dtype if q_dtype is None else q_dtype      # the dtype of the query and of the output
    tensors = dict(
        q=upload(backend, query.reshape(hq, sq, width), q_dtype),
        keys=upload(backend, keys.reshape(physical, pt, hkv, width), pool_dtype),
        values=upload(backend, vals.reshape(physical, pt, hkv, width), pool_dtype),
        table=upload(backend, table, DType.U32),
        generations=upload(backend, 11 + np.arange(physical), DType.U32),
        out=backend.alloc(q_dtype, (hq, sq, width)))
    host = dict(q=query.reshape(hq, sq, width), keys=keys, vals=vals, rows=rows, pt=pt)
    return tensors, host


def float64_attention(host, hq, hkv, sq, key_length, q_start, scale, causal, dtype):
    width = 128
    round_ = lambda a: to_f32(from_f32(a, dtype), dtype).reshape(np.shape(a)).astype(np.float64)
    q = round_(host["q"])
    k = round_(np.nan_to_num(host["keys"][host["rows"]])).reshape(key_length, hkv, width)
    v = round_(np.nan_to_num(host["vals"][host["rows"]])).reshape(key_length, hkv, width)
    out = np.zeros((hq, sq, width))
    for head in range(hq):
        kv = head // (hq // hkv)
        for row in range(sq):
            attended = min(key_length, q_start + row + 1) if causal else key_length
            s = (k[:attended, kv] @ q[head, row]) * scale
            p = np.exp(s - s.max())
            out[head, row] = (p / p.sum()) @ v[:attended, kv]
    return out


@pytest.mark.parametrize("hq,hkv,sq,key_length,q_start,causal", [
    (16, 8, 1, 18, 17, True), (4, 2, 5, 37, 32, True), (4, 4, 3, 33, 0, False)])
def test_paged_sdpa_matches_float64_softmax(cpu, hq, hkv, sq, key_length, q_start, causal):
    """GQA grouping (lib.rs:3109-3138), causal limit and softmax against numpy float64."""
    scale = 1.0 / math.sqrt(128)
    t, host = paged_case(cpu, hq, hkv, sq, key_length, 16, q_start)
    commands = CommandList()
    commands.dispatch(Op.paged_sdpa(scale, causal, q_start, key_length, 16),
                      [t["q"], t["keys"], t["values"], t["table"], t["generations"]], t["out"])
    run(cpu, commands)
    expected = float64_attention(host, hq, hkv, sq, key_length, q_start, scale, causal, DType.BF16)
    assert_close(to_f32(cpu.read(t["out"]), DType.BF16), expected, DType.BF16)


def test_decode_equals_the_last_prefill_row(cpu):
    """lib.rs:3140-3153 restated on pages"""
    scale = 0.5
    t, _ = paged_case(cpu, 2, 1, 4, 20, 16, 16, pool_dtype=DType.F32)
    commands = CommandList()
    commands.dispatch(Op.paged_sdpa(scale, True, 16, 20, 16),
                      [t["q"], t["keys"], t["values"], t["table"], t["generations"]], t["out"])
    last = t["q"].narrow(1, 3, 1)
    out_last = cpu.alloc(DType.F32, (2, 1, 128))
    commands.dispatch(Op.paged_sdpa(scale, True, 19, 20, 16),
                      [last, t["keys"], t["values"], t["table"], t["generations"]], out_last)
    run(cpu, commands)
    prefill = to_f32(cpu.read(t["out"]), DType.F32).reshape(2, 4, 128)
    assert np.array_equal(to_f32(cpu.read(out_last), DType.F32).reshape(2, 128), prefill[:, 3])


# ------------------------------------------------------------------ programs and glue

def test_row_reduction_folds_left_to_right(cpu):
    """interpreter.rs: [1e20, -1e20, 3] sums to 3 only in sequential order."""
    x = upload(cpu, np.array([[1e20, -1e20, 3.0]]), DType.F32)
    out = cpu.alloc(DType.F32, (1, 3))
    b = ProgramBuilder(ProgramKind.ROW)
    v = b.input(0)
    b.output(0, b.reduce(RedOp.SUM, v))
    commands = CommandList()
    commands.dispatch_kernel(cpu.prepare_program(b.finish()), [x], [out])
    run(cpu, commands)
    assert to_f32(cpu.read(out), DType.F32).tolist() == [3.0, 3.0, 3.0]


def test_program_semantics_casts_select_and_nan_propagation(cpu):
    x = upload(cpu, np.array([[-1.5, 3.7, np.nan, 5e9]]), DType.F32)
    out_cast, out_max = cpu.alloc(DType.F32, (1, 4)), cpu.alloc(DType.F32, (1, 4))
    b = ProgramBuilder(ProgramKind.MAP)
    v = b.input(0)
    u = b.cast(ValueType.U32, v)                       # saturating, NaN -> 0
    b.output(0, b.cast(ValueType.F32, u))
    zero = b.const(0.0)
    b.output(1, b.binary(BinOp.MAX, v, zero))          # NaN-propagating
    commands = CommandList()
    commands.dispatch_kernel(cpu.prepare_program(b.finish()), [x], [out_cast, out_max])
    run(cpu, commands)
    assert to_f32(cpu.read(out_cast), DType.F32).tolist() == [0.0, 3.0, 0.0, 4294967296.0]
    result = to_f32(cpu.read(out_max), DType.F32)
    assert result[0] == 0.0 and result[1] == np.float32(3.7) and np.isnan(result[2])


def test_normalizes_1024_wide_rows_with_epsilon(cpu):
    """lib.rs:2688-2711"""
    values = np.concatenate([np.full(1024, 2.0), np.full(1024, -4.0), np.tile([3.0, 4.0], 512)])
    x = upload(cpu, values.reshape(3, 1024), DType.F32)
    w = upload(cpu, np.full(1024, 0.5), DType.F32)
    out = cpu.alloc(DType.F32, (3, 1024))
    commands = CommandList()
    commands.dispatch(Op.rms_norm(0.25), [x, w], out)
    run(cpu, commands)
    expected = np.concatenate([np.full(1024, 1.0 / math.sqrt(4.25)), np.full(1024, -2.0 / math.sqrt(16.25)),
                               np.tile([1.5 / math.sqrt(12.75), 2.0 / math.sqrt(12.75)], 512)])
    np.testing.assert_allclose(to_f32(cpu.read(out), DType.F32), expected, rtol=1e-5)


def test_rope_matches_independent_16_head_computation(cpu):
    """lib.rs:2713-2757"""
    values = (np.arange(14336) % 33).astype(np.float32) / 16.0 - 1.0
    x = upload(cpu, values.reshape(7, 16, 128), DType.F32)
    positions = upload(cpu, np.arange(7), DType.U32)
    out = cpu.alloc(DType.F32, (7, 16, 128))
    commands = CommandList()
    commands.dispatch(Op.rope(1e6), [x, positions], out)
    run(cpu, commands)
    expected = values.astype(np.float64).reshape(7, 16, 128).copy()
    index = np.arange(64)
    for position in range(7):
        angle = position / 1e6 ** (2.0 * index / 128.0)
        first, second = expected[position, :, :64].copy(), expected[position, :, 64:].copy()
        expected[position, :, :64] = first * np.cos(angle) - second * np.sin(angle)
        expected[position, :, 64:] = second * np.cos(angle) + first * np.sin(angle)
    np.testing.assert_allclose(to_f32(cpu.read(out), DType.F32), expected.ravel(), rtol=1e-5, atol=1e-6)
    identity = cpu.alloc(DType.F32, (1, 1, 4))
    x0 = upload(cpu, np.array([[[1.0, -2.0, 3.0, -4.0]]]), DType.F32)
    commands = CommandList()
    commands.dispatch(Op.rope(10000.0), [x0, upload(cpu, np.array([0]), DType.U32)], identity)
    run(cpu, commands)
    assert to_f32(cpu.read(identity), DType.F32).tolist() == [1.0, -2.0, 3.0, -4.0]


def test_strided_views_gather_in_row_major_order(cpu):
    """gather/scatter (lib.rs:1736-1788) through slice(step 2) + permute views."""
    base = np.arange(4 * 6, dtype=np.float32).reshape(4, 6)
    t = upload(cpu, base, DType.F32)
    view = t.slice([Slice(1, 2, 2), Slice(0, 3, 2)]).permute([1, 0])
    assert to_f32(cpu.read(view), DType.F32).tolist() == base[1::2, 0:5:2].T.ravel().tolist()
    out = cpu.alloc(DType.F32, (3, 2))
    commands = CommandList()
    commands.dispatch(Op.copy(), [view], out)
    run(cpu, commands)
    assert to_f32(cpu.read(out), DType.F32).tolist() == base[1::2, 0:5:2].T.ravel().tolist()


def test_matmul_handles_unit_contraction_and_batches(cpu):
    """lib.rs:3079-3092"""
    l = upload(cpu, np.array([[2.0], [3.0]]), DType.F32)
    r = upload(cpu, np.array([[4.0, 5.0, 6.0]]), DType.F32)
    out = cpu.alloc(DType.F32, (2, 3))
    commands = CommandList()
    commands.dispatch(Op.matmul(), [l, r], out)
    l3 = upload(cpu, np.array([1.0, 2.0, 3.0, 4.0]).reshape(2, 1, 2), DType.F32)
    r3 = upload(cpu, np.array([5.0, 6.0, 7.0, 8.0]).reshape(2, 2, 1), DType.F32)
    out3 = cpu.alloc(DType.F32, (2, 1, 1))
    commands.dispatch(Op.matmul(), [l3, r3], out3)
    run(cpu, commands)
    assert to_f32(cpu.read(out), DType.F32).tolist() == [8.0, 10.0, 12.0, 12.0, 15.0, 18.0]
    assert to_f32(cpu.read(out3), DType.F32).tolist() == [17.0, 53.0]


def test_seeded_generators_have_the_stated_distributions():
    normal = orc.fill_normal_f32(1234, 5, 200000)
    assert abs(float(normal.mean())) < 0.01 and abs(float(normal.std()) - 1.0) < 0.01
    uniform = orc.bf16_to_f32(orc.fill_uniform_bf16(1234, 6, 100000, 0.001, 0.02))
    assert uniform.min() >= 0.001 - 1e-5 and uniform.max() <= 0.02 + 1e-4
    words = orc.fill_words(1234, 7, 100000)
    nibbles = (words[:, None] >> (np.arange(8, dtype=np.uint32) * 4)) & 15
    assert np.all(np.abs(np.bincount(nibbles.ravel(), minlength=16) / nibbles.size - 1 / 16) < 0.002)
    # counter-based: a window equals the same indices of the full stream
    assert np.array_equal(orc.fill_words(1234, 7, 100, first=500), words[500:600])


# ------------------------------------------------------------------ sampling
# The reference's own tests of Op::Sample (crates/forja-cpu/src/lib.rs:2520-2690, 3283-3306),
# restated on the oracle, plus the closed form Gumbel-max sampling has to reproduce.

def _sample(row, temperature, top_k, top_p, seed, position, allow=None):
    words = orc.sampling_words(temperature, top_k, top_p, seed)
    return int(orc.sample_rows(np.array([row], dtype=np.float32), words, position, allow)[0])


def _chi_squared(row, temperature, top_k, top_p, seed, expected, trials=20_000):
    counts = np.zeros(len(row))
    for position in range(trials):
        counts[_sample(row, temperature, top_k, top_p, seed, position)] += 1
    expected = np.asarray(expected, dtype=np.float64)
    live = expected > 0
    statistic = (((counts - expected * trials) ** 2)[live] / (expected * trials)[live]).sum()
    assert statistic < 16.3, statistic               # the reference's bound (lib.rs:3300)
    assert not counts[~live].any()


def test_sampled_tokens_are_counter_deterministic():
    row = [0.1, -0.3, 1.2, 0.7, 0.0, 0.9, -1.0]
    first = [_sample(row, 0.7, 0, 1.0, 0xfeedbeefdeadcafe, p) for p in range(128)]
    second = [_sample(row, 0.7, 0, 1.0, 0xfeedbeefdeadcafe, p) for p in range(128)]
    assert first == second and len(set(first)) > 1


def test_sampling_top_k_and_top_p_keep_only_the_exact_allowed_set():
    row = [10.0, 9.0, 8.0, 1.0, 0.0, -1.0, -2.0]
    for position in range(4096):
        assert _sample(row, 1.0, 3, 1.0, 11, position) <= 2
        assert _sample(row, 1.0, 0, 0.7, 11, position) <= 1
        assert _sample(row, 1.0, 2, 0.999, 11, position) <= 1


def test_masked_sampling_conditions_every_sampling_mode():
    row = [10.0, 9.0, 8.0, 7.0, 6.0, 5.0, 4.0]
    allow = [0b01010010]
    for temperature, top_k, top_p, seed in [(0.0, 0, 1.0, 11), (1.0, 2, 1.0, 12), (1.0, 0, 0.8, 13),
                                            (0.7, 0, 1.0, 14)]:
        for position in range(256):
            assert _sample(row, temperature, top_k, top_p, seed, position, allow) in (1, 4, 6)


def test_all_allowed_mask_preserves_unconstrained_sampling():
    row = [index / 7.0 for index in range(33)]
    for position in range(512):
        assert _sample(row, 0.7, 7, 0.9, 0xfeedbeef, position, [0xffffffff, 1]) == \
            _sample(row, 0.7, 7, 0.9, 0xfeedbeef, position)


def test_masked_sampling_refuses_empty_and_padding_bits():
    assert not orc.validate_allow_mask([0], 7)
    assert not orc.validate_allow_mask([1 << 7], 7)
    assert orc.validate_allow_mask([1 << 6], 7)


def test_top_p_uses_the_full_candidate_set_beyond_1024_values():
    assert orc.top_p_keep(np.zeros(1025), 1.0, 0.9995) == 1025


def test_sampling_distributions_match_known_probabilities():
    _chi_squared([0.0, 0.0, 0.0, 0.0], 1.0, 0, 1.0, 91, [0.25] * 4)
    _chi_squared([2.0, 1.0, 0.0], 1.0, 2, 1.0, 92, [0.7310586, 0.2689414, 0.0])
    _chi_squared([2.0, 1.0, 0.0], 1.0, 0, 0.8, 93, [0.7310586, 0.2689414, 0.0])
    _chi_squared([2.0, 1.0, 0.0, -1.0], 1.0, 3, 0.95, 94, [0.66524094, 0.24472848, 0.09003057, 0.0])


def test_gumbel_max_reproduces_the_softmax_at_other_temperatures():
    """Closed form the noise term has to give: P(i) = softmax(logits / T)_i."""
    row = np.array([0.3, -1.2, 2.0, 0.9, 0.0])
    for temperature, seed in ((0.5, 95), (2.5, 96)):
        expected = np.exp(row / temperature)
        _chi_squared(list(row), temperature, 0, 1.0, seed, expected / expected.sum())


def test_greedy_sampling_takes_the_largest_value_and_the_last_of_equals():
    row = [1.0, 5.0, -2.0, 5.0, 3.0, float("-inf")]
    assert _sample(row, 0.0, 0, 1.0, 7, 3) == 3           # temperature 0
    assert _sample(row, 1.3, 1, 0.5, 7, 3) == 3           # top_k 1
    assert _sample(row, 0.0, 0, 1.0, 7, 3, [0b010111]) == 1
    assert _sample([float("nan"), 2.0, float("inf")], 0.0, 0, 1.0, 1, 0) == 0   # total order: NaN above inf


def test_sample_refuses_invalid_live_parameters(cpu):
    logits = upload(cpu, np.zeros(7), DType.F32)
    output = cpu.alloc(DType.U32, ())
    for words in ([np.float32("nan").view(np.uint32), 0, np.float32(1.0).view(np.uint32), 0, 0],
                  list(orc.sampling_words(-1.0, 0, 1.0, 0)), list(orc.sampling_words(1.0, 0, 0.0, 0)),
                  list(orc.sampling_words(1.0, 0, 1.5, 0))):
        params = upload(cpu, np.array(words, dtype=np.uint32), DType.U32)
        commands = CommandList()
        commands.dispatch(Op.sample(0), [logits, params], output)
        with pytest.raises(orc.BackendError) as info:
            run(cpu, commands)
        assert info.value.status == orc.Status.INVALID_INPUT
