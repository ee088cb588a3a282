"""Logical work of a recorded dispatch, as the reference counts it: `KernelCost::of`
(crates/forja-core/src/cost.rs:111-153) with the attention rules of cost/attention.rs:5-129 and the
routed rules of cost/routed.rs:19-91, and the roofline arithmetic of roofline.rs:144-178.

The counts are logical: operand bytes once, whatever a kernel re-reads; weights with their scales
and biases; K/V rows once per kv head; 12 bytes of table entry and generation per page touched;
for routed products the weight bytes of every assignment, bracketed by the smallest and the
largest set of distinct experts the shape allows.  Scalar-program instruction counts
(cost/scalar.rs) are not restated: nothing on the measured path is priced by them.

`ragged_attention_cost` prices the one dispatch that has no counterpart in the reference, the
packed ragged batch, as the per-lane dispatches it stands for.
"""
from __future__ import annotations

import math
from dataclasses import dataclass, fields, replace
from typing import Optional, Sequence

from .core import INTO_PAGES, Dispatch, DType, OpKind, Tensor

U64_MAX = (1 << 64) - 1


@dataclass(frozen=True)
class KernelCost:
    """`KernelCost` (cost.rs:27-58); every field is a u64 and sums refuse overflow."""
    read_bytes: int = 0
    write_bytes: int = 0
    flops: int = 0
    scalar_ops: int = 0
    sfu_ops: int = 0
    metadata_read_bytes: int = 0
    state_read_bytes: int = 0
    state_write_bytes: int = 0
    scratch_read_bytes: int = 0
    scratch_write_bytes: int = 0
    weight_bytes: int = 0
    minimum_weight_bytes: int = 0
    maximum_weight_bytes: int = 0
    kv_bytes: int = 0

    def checked_add(self, other: "KernelCost") -> Optional["KernelCost"]:
        """cost.rs:62-88: field by field, None when any sum leaves u64."""
        values = {}
        for field in fields(self):
            total = getattr(self, field.name) + getattr(other, field.name)
            if total > U64_MAX:
                return None
            values[field.name] = total
        return KernelCost(**values)


def tensor_bytes(tensor: Tensor) -> int:
    """cost.rs:162-174: logical elements times the element size (strides do not matter)."""
    count = 1
    for extent in tensor.shape:
        count *= extent
    return count * tensor.dtype.byte_size


def _bytes(tensors: Sequence[Tensor]) -> int:
    return sum(tensor_bytes(t) for t in tensors)


def _elements(tensor: Tensor) -> int:
    return tensor_bytes(tensor) // tensor.dtype.byte_size


def _metadata(start: int, tokens: int, page_tokens: int, activity_bytes: int) -> KernelCost:
    """attention.rs:112-129: 8 bytes of entry and 4 of generation per page touched."""
    last = (start + tokens - 1) // page_tokens
    pages = last - start // page_tokens + 1
    total = pages * 12 + activity_bytes
    return KernelCost(read_bytes=total, metadata_read_bytes=total,
                      scalar_ops=pages * 3 + (1 if activity_bytes else 0))


def _paged_copy(d: Dispatch, cost: KernelCost) -> KernelCost:
    """attention.rs:87-110."""
    into = d.op.direction == INTO_PAGES
    ordinary, pool = (d.inputs[0], d.outputs[0]) if into else (d.outputs[0], d.inputs[0])
    pool_bytes = _elements(ordinary) * pool.dtype.byte_size
    read, write = (tensor_bytes(ordinary), pool_bytes) if into else (pool_bytes, tensor_bytes(ordinary))
    cost = replace(cost, read_bytes=read, write_bytes=write)
    return cost.checked_add(_metadata(d.op.start, ordinary.shape[0], d.op.page_tokens,
                                      _bytes(d.inputs[3:])))


def _attention(d: Dispatch, cost: KernelCost) -> KernelCost:
    """attention.rs:5-85 for the paged forms."""
    kind = d.op.kind
    if kind == OpKind.PAGED_COPY:
        return _paged_copy(d, cost)
    if kind == OpKind.PAGED_SDPA_APPEND:
        causal, q_start, key_length = True, d.op.q_start, d.op.q_start + 1
        key, value = d.outputs[1], d.outputs[2]
    elif kind == OpKind.PAGED_SDPA:
        causal, q_start, key_length = d.op.causal, d.op.q_start, d.op.key_length
        key, value = d.inputs[1], d.inputs[2]
    else:
        return cost
    inputs = d.inputs[:len(d.inputs) - d.n_extras]
    heads, queries, width = inputs[0].shape
    value_width, kv_heads = value.shape[-1], key.shape[2]
    pairs = queries * (q_start + 1) + queries * (queries - 1) // 2 if causal else queries * key_length
    kv_bytes = kv_heads * key_length * (width + value_width) * key.dtype.byte_size
    cost = replace(cost, flops=2 * heads * pairs * (width + value_width),
                   sfu_ops=heads * (pairs + queries),
                   scalar_ops=heads * pairs * 5 + heads * queries, kv_bytes=kv_bytes,
                   read_bytes=tensor_bytes(inputs[0]) + kv_bytes)
    cost = cost.checked_add(_metadata(0, key_length, d.op.page_tokens, _bytes(inputs[5:])))
    if kind == OpKind.PAGED_SDPA_APPEND:
        written = tensor_bytes(d.outputs[0])
        for source, pool in zip(inputs[1:3], d.outputs[1:]):
            written += _elements(source) * pool.dtype.byte_size
        cost = replace(cost, read_bytes=cost.read_bytes + _bytes(inputs[1:3]), write_bytes=written)
    return cost


def quantized_route_index(input_count: int) -> Optional[int]:
    """routed.rs:6-12: where the index operand of a routed quantised product sits."""
    return {5: 4, 6: 4, 8: 7}.get(input_count)


def per_expert_bytes(weights: int, experts: int) -> Optional[int]:
    """routed.rs:14-16."""
    if experts == 0 or weights % experts:
        return None
    return weights // experts


def _routed(d: Dispatch, cost: KernelCost) -> Optional[KernelCost]:
    """routed.rs:19-91 for the quantised forms this backend executes."""
    inputs = d.inputs[:len(d.inputs) - d.n_extras]
    if d.op.kind == OpKind.QUANT_EMBED:
        row = per_expert_bytes(_bytes(inputs[:3]), inputs[0].shape[0])
        if row is None:
            return None
        weights = row * _elements(inputs[3])
        return replace(cost, weight_bytes=weights, read_bytes=weights + tensor_bytes(inputs[3]))
    if d.op.kind != OpKind.GATHER_QUANT_MATMUL:
        return cost
    index = quantized_route_index(len(inputs))
    if index is None:
        return None
    x, packed, indices = inputs[0].shape, inputs[1].shape, inputs[index].shape
    if len(inputs) == 6:            # weighted sum: x [R, k, K]
        flops = 2 * x[0] * x[1] * x[2] * packed[1]
    else:                           # projection (x2 for the pair): x [R, K]
        flops = 2 * x[0] * indices[1] * x[1] * packed[1] * (2 if len(inputs) == 8 else 1)
    weights = _bytes(inputs[1:index])
    experts = packed[0]
    per_expert = per_expert_bytes(weights, experts)
    if per_expert is None:
        return None
    routes = _elements(inputs[index])
    assigned = per_expert * routes
    return replace(cost, flops=flops, weight_bytes=assigned,
                   read_bytes=cost.read_bytes - weights + assigned,
                   minimum_weight_bytes=per_expert * min(indices[-1], experts),
                   maximum_weight_bytes=per_expert * min(experts, routes))


def of(dispatch: Dispatch) -> Optional[KernelCost]:
    """`KernelCost::of` (cost.rs:111-153) for the ops of the ragged forward step; None for the ops
    the reference has no rule for (the packed ragged batch: see ragged_attention_cost)."""
    kind = dispatch.op.kind
    if kind in (OpKind.PAGED_ATTENTION_RAGGED, OpKind.ROUTE_PACK, OpKind.FILL_SEEDED):
        return None
    cost = KernelCost(read_bytes=_bytes(dispatch.inputs), write_bytes=_bytes(dispatch.outputs))
    inputs = dispatch.inputs[:len(dispatch.inputs) - dispatch.n_extras]
    if kind == OpKind.MATMUL:
        left, right = inputs[0].shape, inputs[1].shape
        batch = left[0] if len(left) == 3 else 1
        cost = replace(cost, flops=2 * batch * left[-2] * left[-1] * right[-1],
                       weight_bytes=tensor_bytes(inputs[1]))
    elif kind == OpKind.QUANT_MATMUL:
        rows, inner = inputs[0].shape
        cost = replace(cost, flops=2 * rows * inner * inputs[1].shape[0],
                       weight_bytes=_bytes(inputs[1:4]))
    cost = _routed(dispatch, _attention(dispatch, cost))
    if cost is None or any(getattr(cost, f.name) > U64_MAX for f in fields(cost)):
        return None
    return cost


def ragged_attention_cost(query_heads: int, kv_heads: int, width: int, value_width: int,
                          counts: Sequence[int], starts: Sequence[int], page_tokens: int,
                          activation_bytes: int, pool_bytes: int, activity: bool = True) -> KernelCost:
    """The packed ragged batch priced as what it replaces, lane by lane: two
    Op::PagedCopy{IntoPages} of the lane's new key and value rows and one causal Op::PagedSdpa
    through them (engines/qwen38/src/attention/batch.rs:37-53) - for a lane with one row the same
    bytes as Op::PagedSdpaAppend plus the metadata of the copies.  `counts[l]` new rows at
    position `starts[l]`; lanes without rows cost nothing."""
    total = KernelCost()
    activity_bytes = 4 if activity else 0
    for count, start in zip(counts, starts):
        if count == 0:
            continue
        for row_width in (width, value_width):
            rows = count * kv_heads * row_width
            total = total.checked_add(replace(
                _metadata(start, count, page_tokens, activity_bytes),
                write_bytes=rows * pool_bytes).checked_add(KernelCost(read_bytes=rows * activation_bytes)))
        key_length = start + count
        pairs = count * (start + 1) + count * (count - 1) // 2
        kv = kv_heads * key_length * (width + value_width) * pool_bytes
        attention = KernelCost(
            flops=2 * query_heads * pairs * (width + value_width), sfu_ops=query_heads * (pairs + count),
            scalar_ops=query_heads * pairs * 5 + query_heads * count, kv_bytes=kv,
            read_bytes=query_heads * count * width * activation_bytes + kv,
            write_bytes=query_heads * count * value_width * activation_bytes)
        total = total.checked_add(attention).checked_add(
            _metadata(0, key_length, page_tokens, activity_bytes))
    return total


def traffic(cost: KernelCost, maximum_reuse: bool) -> Optional[int]:
    """roofline.rs:144-156: operand traffic at one end of the expert-reuse interval."""
    if cost.maximum_weight_bytes == 0:
        weights = cost.weight_bytes
    else:
        weights = cost.minimum_weight_bytes if maximum_reuse else cost.maximum_weight_bytes
    if cost.read_bytes < cost.weight_bytes:
        return None
    total = cost.read_bytes - cost.weight_bytes + weights + cost.write_bytes
    return total if total <= U64_MAX else None


def distinct_expert_traffic(dispatch: Dispatch, distinct: int) -> Optional[int]:
    """Traffic of a routed quantised product whose routes were seen to touch `distinct` experts:
    the measured point inside the reference's [minimum, maximum] interval (a profiler's duty,
    cost.rs:48-51).  None when `distinct` lies outside what the shape allows."""
    cost = of(dispatch)
    if cost is None or cost.maximum_weight_bytes == 0:
        return None
    inputs = dispatch.inputs[:len(dispatch.inputs) - dispatch.n_extras]
    index = quantized_route_index(len(inputs))
    per_expert = per_expert_bytes(_bytes(inputs[1:index]), inputs[1].shape[0])
    weights = per_expert * distinct
    if not cost.minimum_weight_bytes <= weights <= cost.maximum_weight_bytes and distinct != 0:
        return None
    return cost.read_bytes - cost.weight_bytes + weights + cost.write_bytes


@dataclass(frozen=True)
class Ceilings:
    """roofline.rs `Ceilings`: device rates a cost is priced against."""
    read_bytes_per_second: float
    copy_bytes_per_second: float
    flops_per_second: float
    dispatch_seconds: float

    @staticmethod
    def new(read, copy, flops, dispatch) -> Optional["Ceilings"]:
        values = (read, copy, flops, dispatch)
        if not all(math.isfinite(v) and v > 0.0 for v in values):
            return None
        return Ceilings(*values)


@dataclass(frozen=True)
class ResourceTimes:
    """roofline.rs `ResourceTimes`: competing bounds, never added."""
    memory: float
    compute: float
    dispatch: float

    def seconds(self) -> float:
        return max(self.memory, self.compute, self.dispatch)

    def bound(self) -> str:
        if self.dispatch >= max(self.memory, self.compute):
            return "dispatch-floor"
        return "memory" if self.memory >= self.compute else "compute"

    def target_seconds(self, utilization: float) -> Optional[float]:
        if not (math.isfinite(utilization) and 0.0 < utilization <= 1.0):
            return None
        target = max(max(self.memory, self.compute) / utilization, self.dispatch)
        return target if math.isfinite(target) else None


def limits(cost: KernelCost, dispatches: int, ceilings: Ceilings) -> Optional[ResourceTimes]:
    """roofline.rs:158-178: memory, matrix-product and dependent-dispatch bounds of a cost."""
    total = traffic(cost, True)
    if total is None or total < cost.write_bytes:
        return None
    read = total - cost.write_bytes
    times = ResourceTimes(
        memory=max(read / ceilings.read_bytes_per_second, total / ceilings.copy_bytes_per_second),
        compute=cost.flops / ceilings.flops_per_second,
        dispatch=dispatches * ceilings.dispatch_seconds)
    if not all(math.isfinite(v) for v in (times.memory, times.compute, times.dispatch)):
        return None
    return times


# MI355X published ceilings: HBM3E 8 TB/s; dense bf16 matrix cores 2.5 PFLOP/s.
MI355X = Ceilings(8.0e12, 8.0e12, 2.5e15, 2.0e-6)
