"""The logical-work accounting (forja_amd/cost.py) against the known answers the reference's own
tests hold: crates/forja-core/src/cost.rs:199-315, cost/attention.rs:131-231,
cost/routed.rs:93-154 and roofline.rs:180-293.  Tensors are built the way those tests build them
(contiguous, one allocation each); no backend is involved."""
import pytest

from forja_amd import cost as C
from forja_amd.core import CommandList, DType, Layout, Op, Tensor, INTO_PAGES, OUT_OF_PAGES


def tensor(identity, dtype, shape):
    size = dtype.byte_size
    for extent in shape:
        size *= extent
    return Tensor(identity, Layout.contiguous(dtype, 0, tuple(shape), size), True)


def last(commands):
    return C.of(commands.dispatches[-1])


def test_composite_work_preserves_subsets_and_refuses_overflow():
    """cost.rs:230-279"""
    cost = C.KernelCost(read_bytes=C.U64_MAX, scratch_read_bytes=64, state_read_bytes=32, write_bytes=96,
                        scratch_write_bytes=64, state_write_bytes=32, flops=128, scalar_ops=7, sfu_ops=3,
                        weight_bytes=48, minimum_weight_bytes=16, maximum_weight_bytes=48, kv_bytes=8,
                        metadata_read_bytes=24)
    assert cost.checked_add(C.KernelCost()) == cost
    assert cost.checked_add(C.KernelCost(read_bytes=1)) is None
    from dataclasses import replace
    half = replace(cost, read_bytes=96)
    total = half.checked_add(half)
    assert (total.metadata_read_bytes, total.scratch_read_bytes, total.state_read_bytes) == (48, 128, 64)
    assert (total.sfu_ops, total.flops, total.weight_bytes) == (6, 256, 96)
    assert (total.minimum_weight_bytes, total.maximum_weight_bytes, total.kv_bytes) == (32, 96, 16)


@pytest.mark.parametrize("rows", [1, 7, 33])
def test_dense_gemv_and_gemm_count_logical_work(rows):
    """cost.rs:281-294"""
    commands = CommandList()
    commands.dispatch(Op.matmul(), [tensor(1, DType.BF16, (rows, 1024)), tensor(2, DType.BF16, (1024, 4097))],
                      tensor(3, DType.BF16, (rows, 4097)))
    cost = last(commands)
    assert cost.flops == 2 * rows * 1024 * 4097
    assert cost.read_bytes == 2 * (rows * 1024 + 1024 * 4097)
    assert cost.write_bytes == 2 * rows * 4097


def test_quantized_weights_include_scales_and_biases():
    """cost.rs:296-314"""
    commands = CommandList()
    commands.dispatch(Op.quant_matmul(4, 64),
                      [tensor(1, DType.BF16, (7, 1024)), tensor(2, DType.U32, (33, 128)),
                       tensor(3, DType.BF16, (33, 16)), tensor(4, DType.BF16, (33, 16))],
                      tensor(5, DType.BF16, (7, 33)))
    cost = last(commands)
    assert cost.flops == 2 * 7 * 1024 * 33
    assert cost.weight_bytes == 33 * (128 * 4 + 16 * 4)
    assert cost.read_bytes == 7 * 1024 * 2 + cost.weight_bytes and cost.write_bytes == 7 * 33 * 2


def test_paged_append_counts_one_token_write_and_logical_pool_reads():
    """cost/attention.rs:136-163"""
    commands = CommandList()
    commands.dispatch_many(
        Op.paged_sdpa_append(1.0, 0, 16),
        [tensor(1, DType.F32, (16, 1, 128)), tensor(2, DType.F32, (1, 8, 128)), tensor(3, DType.F32, (1, 8, 128)),
         tensor(6, DType.U32, (1, 2)), tensor(7, DType.U32, (99,))],
        [tensor(8, DType.F32, (16, 1, 128)), tensor(4, DType.F16, (99, 16, 8, 128)),
         tensor(5, DType.F16, (99, 16, 8, 128))])
    cost = last(commands)
    assert cost.metadata_read_bytes == 12
    assert cost.flops == 8192
    assert cost.write_bytes == 12288
    assert cost.kv_bytes == 4096
    assert cost.read_bytes == 8192 + 8192 + 4096 + 12


def test_attention_counts_causal_pairs_and_kv_once():
    """cost/attention.rs:165-192, through the paged form: 7 query rows from position 26 over 33
    keys give 27 + ... + 33 pairs, and K/V bytes are counted once per kv head."""
    commands = CommandList()
    commands.dispatch(
        Op.paged_sdpa(1.0, True, 26, 33, 16),
        [tensor(1, DType.F32, (16, 7, 128)), tensor(2, DType.F16, (9, 16, 8, 128)),
         tensor(3, DType.F16, (9, 16, 8, 128)), tensor(4, DType.U32, (3, 2)), tensor(5, DType.U32, (9,))],
        tensor(6, DType.F32, (16, 7, 128)))
    cost = last(commands)
    pairs = 27 + 28 + 29 + 30 + 31 + 32 + 33
    assert cost.flops == 2 * 16 * pairs * 256
    assert cost.sfu_ops == 16 * (pairs + 7)
    assert cost.kv_bytes == 2 * 8 * 33 * 128 * 2


@pytest.mark.parametrize("capacity", [99, 4097])
def test_paged_attention_ignores_unused_pool_capacity(capacity):
    """cost/attention.rs:194-230"""
    commands = CommandList()
    commands.dispatch(
        Op.paged_sdpa(1.0, True, 32, 33, 16),
        [tensor(1, DType.F32, (16, 1, 128)), tensor(2, DType.F16, (capacity, 16, 8, 128)),
         tensor(3, DType.F16, (capacity, 16, 8, 128)), tensor(4, DType.U32, (3, 2)),
         tensor(5, DType.U32, (capacity,))],
        tensor(6, DType.F32, (16, 1, 128)))
    cost = last(commands)
    assert cost.flops == 4 * 16 * 33 * 128
    assert cost.metadata_read_bytes == 36
    assert cost.read_bytes == 16 * 128 * 4 + 2 * 8 * 33 * 128 * 2 + 36
    assert cost.kv_bytes == 2 * 8 * 33 * 128 * 2


def test_paged_copy_counts_rows_in_the_pool_dtype_and_touched_pages():
    """cost/attention.rs:87-129: 5 f32 rows of 64 elements from position 30 touch pages 1 and 2 of
    16-token pages; the pool side is counted in the pool's dtype; an activity word adds 4 bytes."""
    ordinary, pool = tensor(1, DType.F32, (5, 64)), tensor(2, DType.F16, (9, 16, 64))
    table, generations, activity = tensor(3, DType.U32, (4, 2)), tensor(4, DType.U32, (9,)), tensor(5, DType.U32, (1,))
    commands = CommandList()
    commands.dispatch(Op.paged_copy(INTO_PAGES, 30, 16), [ordinary, table, generations, activity], pool)
    into = last(commands)
    assert (into.read_bytes, into.write_bytes, into.metadata_read_bytes) == (5 * 64 * 4 + 28, 5 * 64 * 2, 28)
    commands.dispatch(Op.paged_copy(OUT_OF_PAGES, 30, 16), [pool, table, generations], ordinary)
    out = last(commands)
    assert (out.read_bytes, out.write_bytes, out.metadata_read_bytes) == (5 * 64 * 2 + 24, 5 * 64 * 4, 24)


def test_routed_index_slots_refuse_unknown_arities():
    """cost/routed.rs:98-106"""
    assert [C.quantized_route_index(n) for n in (5, 6, 8, 7)] == [4, 4, 7, None]
    assert C.per_expert_bytes(7, 2) is None and C.per_expert_bytes(8, 0) is None


@pytest.mark.parametrize("rows", [1, 7, 33])
def test_routed_quantized_cost_counts_assignments_and_reuse_bounds(rows):
    """cost/routed.rs:108-141"""
    operands = [tensor(1, DType.F32, (rows, 1024)), tensor(2, DType.U32, (16, 33, 128)),
                tensor(3, DType.BF16, (16, 33, 16)), tensor(4, DType.BF16, (16, 33, 16)),
                tensor(5, DType.U32, (rows, 8))]
    commands = CommandList()
    commands.dispatch(Op.gather_quant_matmul(4, 64), operands, tensor(6, DType.F32, (rows, 8, 33)))
    cost = last(commands)
    expert_bytes = 33 * (128 * 4 + 16 * 4)
    assert cost.flops == 2 * rows * 8 * 1024 * 33
    assert cost.weight_bytes == expert_bytes * rows * 8
    assert cost.minimum_weight_bytes == expert_bytes * 8
    assert cost.maximum_weight_bytes == expert_bytes * min(rows * 8, 16)
    if rows == 1:
        assert cost.minimum_weight_bytes == cost.maximum_weight_bytes
    # the pair doubles the arithmetic and counts both projections' weights per assignment
    pair = operands[:4] + [tensor(7, DType.U32, (16, 33, 128)), tensor(8, DType.BF16, (16, 33, 16)),
                           tensor(9, DType.BF16, (16, 33, 16)), operands[4]]
    commands.dispatch_epilogue(Op.gather_quant_matmul(4, 64), pair, tensor(6, DType.F32, (rows, 8, 33)), None, [])
    both = last(commands)
    assert both.flops == 2 * cost.flops and both.weight_bytes == 2 * cost.weight_bytes
    # the measured point inside the interval: weights of the experts actually touched
    touched = min(rows * 8, 16)
    assert C.distinct_expert_traffic(commands.dispatches[0], touched) == C.traffic(cost, False)
    assert C.distinct_expert_traffic(commands.dispatches[0], 17) is None


def test_weighted_sum_counts_every_route_once():
    """gather_quant_matmul_weighted_flops (crates/forja-core/src/ops.rs:2167-2181): x [R, k, K]."""
    commands = CommandList()
    commands.dispatch(Op.gather_quant_matmul(4, 64),
                      [tensor(1, DType.BF16, (5, 8, 768)), tensor(2, DType.U32, (128, 2048, 96)),
                       tensor(3, DType.BF16, (128, 2048, 12)), tensor(4, DType.BF16, (128, 2048, 12)),
                       tensor(5, DType.U32, (5, 8)), tensor(6, DType.BF16, (5, 8))],
                      tensor(7, DType.BF16, (5, 2048)))
    cost = last(commands)
    assert cost.flops == 2 * 5 * 8 * 768 * 2048
    assert cost.maximum_weight_bytes == 40 * 2048 * (96 * 4 + 12 * 4)


def test_quantised_embedding_reads_only_selected_rows():
    """cost/routed.rs:49-57 (the quantised counterpart of embeddings_read_only_selected_rows)."""
    commands = CommandList()
    commands.dispatch(Op.quant_embed(4, 64),
                      [tensor(1, DType.U32, (4097, 128)), tensor(2, DType.BF16, (4097, 16)),
                       tensor(3, DType.BF16, (4097, 16)), tensor(4, DType.U32, (7,))],
                      tensor(5, DType.BF16, (7, 1024)))
    assert last(commands).read_bytes == 7 * (128 * 4 + 16 * 2 + 16 * 2 + 4)


def test_resource_bounds_compete_instead_of_being_added():
    """roofline.rs:222-248"""
    ceilings = C.Ceilings.new(100.0, 200.0, 1000.0, 0.01)
    limit = C.limits(C.KernelCost(read_bytes=100, write_bytes=100, flops=500), 1, ceilings)
    assert limit.bound() == "memory" and abs(limit.seconds() - 1.0) < 1e-15
    assert abs(limit.target_seconds(0.8) - 1.25) < 1e-15
    assert C.limits(C.KernelCost(flops=2000), 1, ceilings).bound() == "compute"
    floor = C.limits(C.KernelCost(), 7, ceilings)
    assert floor.bound() == "dispatch-floor" and abs(floor.seconds() - 0.07) < 1e-15


def test_expert_reuse_uncertainty_remains_explicit():
    """roofline.rs:250-279"""
    cost = C.KernelCost(read_bytes=1000, weight_bytes=900, minimum_weight_bytes=10, maximum_weight_bytes=100)
    assert C.traffic(cost, True) == 110 and C.traffic(cost, False) == 200
    assert C.traffic(C.KernelCost(read_bytes=C.U64_MAX, write_bytes=1), True) is None
    assert C.traffic(C.KernelCost(read_bytes=0, weight_bytes=1), True) is None


def test_ceilings_refuse_nonfinite_or_nonpositive_values():
    """roofline.rs:280-292"""
    assert C.Ceilings.new(0.0, 1.0, 1.0, 1.0) is None
    assert C.Ceilings.new(1.0, float("inf"), 1.0, 1.0) is None
    assert C.limits(C.KernelCost(), 1, C.Ceilings.new(100.0, 200.0, 1000.0, 0.01)).target_seconds(0.0) is None


def test_the_packed_ragged_batch_costs_what_its_lanes_cost():
    """One decode lane at position 40 of 16-token pages, 32 query / 4 kv heads of 128, bf16: the
    K/V bytes of 41 keys, q and o rows, the appended rows read and written, 12 bytes for each of
    the 3 pages the attention walks and for the page each copy touches, 3 activity words."""
    cost = C.ragged_attention_cost(32, 4, 128, 128, [1, 0], [40, 7], 16, 2, 2)
    kv = 4 * 41 * 256 * 2
    assert cost.kv_bytes == kv
    assert cost.metadata_read_bytes == 3 * 12 + 2 * 12 + 3 * 4
    assert cost.read_bytes == kv + 32 * 128 * 2 + 2 * 4 * 128 * 2 + cost.metadata_read_bytes
    assert cost.write_bytes == 32 * 128 * 2 + 2 * 4 * 128 * 2
    assert cost.flops == 2 * 32 * 41 * 256
    # a 3-row chunk from position 5: 6 + 7 + 8 pairs
    chunk = C.ragged_attention_cost(8, 2, 128, 128, [3], [5], 16, 2, 2, activity=False)
    assert chunk.flops == 2 * 8 * (6 + 7 + 8) * 256 and chunk.kv_bytes == 2 * 8 * 256 * 2
