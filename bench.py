#!/usr/bin/env python3
"""Headline benchmark: decode tokens/s of the 4-bit Qwen3-Coder-30B-A3B-shaped ragged continuous
batch on one MI355X (BASELINE.json metric, config 3).

A step = one forward step of the whole batch: 128 decode lanes (contexts log-uniform over
256..32768, non-contiguous block tables, page size 16), 48 MoE layers, lm_head and greedy argmax,
recorded once as a command list and replayed; every step 8 sequences retire and 8 are admitted.
Weights and K/V pools are synthetic, generated on the device, resident in HBM before timing.

Prints one JSON line with the throughput, the roofline of the dominant kernel (paged attention,
HBM-bound) measured with HIP events on the backend's stream inside the timed region, and the CPU
baseline (the single-threaded oracle on a bounded sample of the same workload).
"""
import argparse
import json
import math
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

from forja_amd import cost as costs  # noqa: E402
from forja_amd.core import CommandList, DType, Op  # noqa: E402
from forja_amd.hip_backend import HipBackend  # noqa: E402
from forja_amd.model import (QWEN3_CODER_30B_A3B, QWEN3_0_6B, DecodeSession, Model,  # noqa: E402
                             ModelConfig)

HBM_PEAK_GBPS = 8000.0
TRAFFIC_SUMMARY = os.path.join(ROOT, "profiles", "c3_decode_step_hbm_traffic.txt")


def measured_traffic_ratio():
    """HBM bytes moved by ragged_attention_mfma_kernel per algorithmic byte on the timed workload,
    as the hardware counters gave it (rocprofv3 --pmc FETCH_SIZE and WRITE_SIZE over the same
    launches, each scaled by what the counter reads for a 1 GiB copy): read from the tracked
    summary of that measurement.  None when the summary is not there."""
    import re
    try:
        match = re.search(r"ratio ([0-9.]+)", open(TRAFFIC_SUMMARY).read())
    except OSError:
        return None
    return float(match.group(1)) if match else None


KC_ATTENTION, KC_MOE, KC_QMM = 3, 2, 1
KC_ATTENTION_KERNEL, KC_MOE_KERNEL, KC_QMM_KERNEL = 4, 5, 6
ATTENTION_TIMER_STRIDE = 6   # launches of the dominant kernel per HIP-event timing in the timed region


def log_uniform(rng, lo, hi, count):
    return np.exp(rng.uniform(math.log(lo), math.log(hi), count)).astype(np.int64)


class Workload:
    """Config 3: 128 decode lanes, 8 retire + 8 admit per step."""

    def __init__(self, backend, config: ModelConfig, lanes, ctx_lo, ctx_hi, churn, seed, layers=None,
                 capacity_factor=1.45, router_noise_seed=None):
        self.rng = np.random.default_rng(seed)
        self.lanes, self.ctx_lo, self.ctx_hi, self.churn = lanes, ctx_lo, ctx_hi, churn
        contexts = log_uniform(self.rng, ctx_lo, ctx_hi, lanes)
        pt = config.page_tokens
        expected_tokens = lanes * (ctx_hi - ctx_lo) / math.log(ctx_hi / ctx_lo)
        capacity_tokens = max(int(expected_tokens * capacity_factor), int(contexts.sum() * 1.1))
        self.capacity_pages = capacity_tokens // pt + 2 * lanes
        table_pages = (ctx_hi + 4096 + pt) // pt
        self.model = Model(backend, config, seed=seed, layers=layers)
        self.session = DecodeSession(self.model, contexts, seed=seed, physical_pages=self.capacity_pages,
                                     table_pages=table_pages, router_noise_seed=router_noise_seed)
        self.next_lane = 0

    def churn_lanes(self):
        s = self.session
        pt = self.model.config.page_tokens
        for _ in range(self.churn):
            lane = self.next_lane
            self.next_lane = (self.next_lane + 1) % self.lanes
            s.cache.retire(lane)
            # admit a new sequence whose cache fits the free pages (redraw otherwise)
            for _attempt in range(16):
                context = int(log_uniform(self.rng, self.ctx_lo, self.ctx_hi, 1)[0])
                if (context + 64) // pt + 2 < len(s.cache.free) - 4 * self.lanes:
                    break
            else:
                context = self.ctx_lo
            s.contexts[lane] = context
            s.cache.ensure(lane, context + 1)
            s.cache.upload_tables([lane])


def attention_launch_cost(config, contexts):
    """Logical work of one layer's decode attention over lanes at `contexts` (one new row each), by
    the reference's accounting (crates/forja-core/src/cost/attention.rs:5-129): K/V rows once per
    kv head, query and output rows, the appended rows, 12 bytes per page touched."""
    width = config.head_dim
    pool_bytes = config.kv_dtype.byte_size
    return costs.ragged_attention_cost(config.q_heads, config.kv_heads, width, width, [1] * len(contexts),
                                       [int(v) for v in contexts], config.page_tokens,
                                       config.activation_dtype.byte_size, pool_bytes)


def step_costs(model, buffers_session, distinct_experts=None):
    """Logical traffic of the weights one decode step reads, dispatch by dispatch
    (crates/forja-core/src/cost.rs:111-153, cost/routed.rs:19-91): dense products with scales and
    biases; routed products at `distinct_experts` experts per layer when given, else at the
    reference's bounds (minimum: top-k experts, maximum: min(experts, routes))."""
    dense = routed_min = routed_max = routed_seen = 0
    for dispatch in buffers_session.commands.dispatches:
        cost = costs.of(dispatch)
        if cost is None:
            continue
        if cost.maximum_weight_bytes:
            routed_min += costs.traffic(cost, True)
            routed_max += costs.traffic(cost, False)
            if distinct_experts is not None:
                seen = costs.distinct_expert_traffic(dispatch, int(round(distinct_experts)))
                routed_seen += seen if seen is not None else costs.traffic(cost, False)
        elif cost.weight_bytes:
            dense += costs.traffic(cost, True)
    return {"dense": dense, "routed_minimum": routed_min, "routed_maximum": routed_max,
            "routed_seen": routed_seen if distinct_experts is not None else None}


def cpu_baseline(config, seed, sample_lanes, ctx_lo, ctx_hi):
    """Times the CPU oracle (single thread, as the reference backend is single-threaded) on one
    decoder layer over `sample_lanes` lanes of the same workload plus the lm_head on 2 rows, and
    extrapolates linearly in layers and rows to a full step."""
    from oracle.cpu_backend import CpuBackend
    rng = np.random.default_rng(seed)
    contexts = log_uniform(rng, ctx_lo, ctx_hi, 128)[:sample_lanes]
    cpu = CpuBackend(threads=1)
    model = Model(cpu, config, seed=seed, layers=1)
    session = DecodeSession(model, contexts, seed=seed)
    # time the layer: everything except lm_head/argmax, obtained by timing the full single-layer
    # step and a separate lm_head-only dispatch
    started = time.perf_counter()
    session.step()
    step_seconds = time.perf_counter() - started
    b = session.buffers
    head = CommandList()
    head.dispatch(Op.quant_matmul(4, 64), [b.normalized[0].narrow(0, 0, 2), *model.lm_head.triple],
                  b.logits.narrow(0, 0, 2))
    started = time.perf_counter()
    cpu.submit(head).wait()
    head_seconds = time.perf_counter() - started
    head_full_sample = head_seconds * sample_lanes / 2.0
    layer_seconds = max(step_seconds - head_full_sample, 1e-9)
    scale_rows = 128.0 / sample_lanes
    full_step = config.layers * layer_seconds * scale_rows + head_seconds * 64.0
    return {
        "value": 128.0 / full_step, "unit": "tok/s", "cores": 1, "kind": "port",
        "sample": (f"1 of {config.layers} layers x {sample_lanes} of 128 lanes (contexts "
                   f"{int(contexts.min())}..{int(contexts.max())}) + lm_head on 2 rows, timed "
                   f"{step_seconds + head_seconds:.1f} s; step time extrapolated linearly in "
                   f"layers and rows"),
        "extrapolated_ms_per_step": full_step * 1e3,
    }


def moe_block_c2(backend, model, tokens=256, seed=77):
    """BASELINE config 2 on the model's own expert weights, one pass per layer so that no weight
    is read twice: top-8 of N(0,1) router logits (softmax-normalised), routed gate/up + SwiGLU,
    routed down + weighted combine.  Returns the per-layer device times and bytes."""
    c = model.config
    x = backend.alloc(DType.BF16, (tokens, c.hidden))
    logits = backend.alloc(DType.BF16, (tokens, c.experts))
    weights = backend.alloc(DType.BF16, (tokens, c.top_k))
    indices = backend.alloc(DType.U32, (tokens, c.top_k))
    activated = backend.alloc(DType.BF16, (tokens, c.top_k, c.expert_intermediate))
    out = backend.alloc(DType.BF16, (tokens, c.hidden))
    fill = CommandList()
    fill.dispatch(Op.fill_seeded(2, seed, 1), [], x)
    fill.dispatch(Op.fill_seeded(2, seed, 2), [], logits)
    backend.submit(fill).wait()
    gq4 = Op.gather_quant_matmul(4, 64)
    commands = CommandList()
    for layer in model.layers:
        commands.dispatch_many(Op.top_k(c.top_k, True), [logits], [weights, indices])
        commands.dispatch_epilogue(gq4, [x, *layer.gate.triple, *layer.up.triple, indices],
                                   activated, model.swiglu_epilogue, [])
        commands.dispatch(gq4, [activated, *layer.down.triple, indices, weights], out)
    encoded = backend.encode(commands)
    backend.submit(encoded).wait()                      # warm-up pass
    backend.profile_enable(2)
    backend.profile_reset()
    backend.submit(encoded).wait()
    block_ns, _ = backend.profile_read(KC_MOE)
    kernel_ns, launches = backend.profile_read(KC_MOE_KERNEL)
    topk_ns, _ = backend.profile_read(0)
    backend.profile_enable(0)
    chosen = np.frombuffer(backend.read(indices), np.uint32)
    distinct = len(np.unique(chosen))
    layers = len(model.layers)
    per_expert = (model.layers[0].gate.weight_bytes + model.layers[0].up.weight_bytes +
                  model.layers[0].down.weight_bytes) / c.experts
    block_bytes = distinct * per_expert + tokens * c.hidden * 2 * 2
    block_us = (block_ns + topk_ns) / layers / 1e3
    for tensor in (x, logits, weights, indices, activated, out):
        backend.release(tensor)
    return {
        "workload": (f"BASELINE config 2: {tokens} decode tokens, {c.experts} experts top-{c.top_k} "
                     f"from N(0,1) router logits, expert SwiGLU {c.hidden}x{c.expert_intermediate}, "
                     f"one pass over each of {layers} layers' expert weights"),
        "distinct_experts": distinct, "us_per_block": block_us,
        "us_routed_kernels_per_block": kernel_ns / layers / 1e3,
        "algorithmic_mb_per_block": block_bytes / 1e6,
        "achieved_gbps": block_bytes / (block_us * 1e-6) / 1e9,
        "frac_of_hbm_peak": block_bytes / (block_us * 1e-6) / 1e9 / HBM_PEAK_GBPS,
        "frac_of_hbm_peak_kernels_only": block_bytes / (kernel_ns / layers * 1e-9) / 1e9 / HBM_PEAK_GBPS,
    }


MFMA_BF16_PEAK_TFLOPS = 2500.0


def prefill_gemm_c4(backend, rows=8256, seed=91, layers=4, repeats=5):
    """The quantised projections of BASELINE config 4 layers (dense 27B-class shape) over the
    8192-token prefill chunk plus its 64 decode rows: stacked qkv, o, stacked gate/up, down, in the
    order and rhythm of a prefill: the four products of a layer one after the other, `layers`
    layers with weights of their own (no product finds its weights in a cache), the whole sequence
    `repeats` times back to back after one warm-up pass, with no host wait in between.  (The device
    is power-limited under this load: its clock settles near 1.5-1.7 GHz a few milliseconds into a
    stream of such products, and isolated launches with the host waiting in between measure 10 %
    lower.)  Device time per product from the per-dispatch timeline of the profiled submissions."""
    from forja_amd.model import DENSE_27B, QuantLinear
    c = DENSE_27B
    qkv_width = (c.q_heads + 2 * c.kv_heads) * c.head_dim
    shapes = [("qkv", qkv_width, c.hidden), ("o_proj", c.hidden, c.q_heads * c.head_dim),
              ("gate_up", 2 * c.intermediate, c.hidden), ("down", c.hidden, c.intermediate)]
    inputs = {k: backend.alloc(DType.BF16, (rows, k)) for k in sorted({k for _, _, k in shapes})}
    outputs = {n: backend.alloc(DType.BF16, (rows, n)) for n in sorted({n for _, n, _ in shapes})}
    fill = CommandList()
    for index, x in enumerate(inputs.values()):
        fill.dispatch(Op.fill_seeded(2, seed, 5 + index), [], x)
    weights = []
    for layer in range(layers):
        for index, (name, n, k) in enumerate(shapes):
            linear = QuantLinear(backend, n, k)
            linear.fill(fill, seed, 100 * layer + 10 * index)
            weights.append((name, n, k, linear))
    backend.submit(fill).wait()
    commands = CommandList()
    for name, n, k, linear in weights:
        commands.dispatch(Op.quant_matmul(4, 64), [inputs[k], *linear.triple], outputs[n])
    encoded = backend.encode(commands)
    backend.submit(encoded).wait()     # warm-up: every weight's kept operand exists
    submissions = [backend.submit_profiled(encoded) for _ in range(repeats)]
    for submission in submissions:
        submission.wait()
    spans = {}
    for submission in submissions:
        for first, _, _, start, end in submission.profile():
            spans.setdefault(weights[first][0], []).append(end - start)
    products, total_flops, total_ns = {}, 0.0, 0.0
    for name, n, k in shapes:
        per_launch = float(np.mean(spans[name]))
        flops = 2.0 * rows * n * k
        products[name] = {"n": n, "k": k, "us": per_launch / 1e3, "launches": len(spans[name]),
                          "tflops": flops / (per_launch * 1e-9) / 1e12}
        total_flops += flops
        total_ns += per_launch
    for tensor in (*inputs.values(), *outputs.values()):
        backend.release(tensor)
    for _, _, _, linear in weights:
        for tensor in linear.triple:
            backend.release(tensor)
    achieved = total_flops / (total_ns * 1e-9) / 1e12 if total_ns else 0.0
    return {
        "workload": (f"BASELINE config 4 layer projections: {rows} rows (8192-token prefill chunk + "
                     f"64 decode rows), hidden {c.hidden}, intermediate {c.intermediate}, MLX-4bit; "
                     f"the products of {layers} layers back to back, {repeats} times"),
        "roofline": {"bound": "mfma", "achieved": achieved, "peak": MFMA_BF16_PEAK_TFLOPS,
                     "unit": "TFLOP/s", "frac": achieved / MFMA_BF16_PEAK_TFLOPS,
                     "kernel": "gemm_q4_kernel, with prepare_rows_kernel (and prepare_extras_kernel on a weight's first use)"},
        "ms_per_layer_projections": total_ns / 1e6, "products": products,
    }


def prefill_layer_c4(backend, seed=95, repeats=8):
    """One whole BASELINE config 4 decoder layer over the packed batch (6 prompts of 512..3072
    tokens summing to 8192, plus 64 decode rows): norms, stacked qkv, qk-norm + rope, paged
    attention, o, gate/up, SwiGLU, down with residual.  Device time of the step from the
    submission's events; flops = projections + attention."""
    from forja_amd.model import DENSE_27B, Model, PackedStep
    c = DENSE_27B
    rng = np.random.default_rng(seed)
    prompts = [512, 768, 1024, 1280, 1536, 3072]
    contexts = [0] * len(prompts) + [int(v) for v in rng.integers(128, 4097, 64)]
    counts = prompts + [1] * 64
    model = Model(backend, c, seed=seed, layers=1)
    step = PackedStep(model, contexts, counts, seed=seed, head=False)
    step.run()
    # the layer `repeats` times back to back, as the layers of a prefill follow each other
    submissions = [backend.submit(step.encoded) for _ in range(repeats)]
    for submission in submissions:
        submission.wait()
    seconds = sum(submission.gpu_time_ns() for submission in submissions) / repeats * 1e-9
    rows = step.tokens
    qkv_width = (c.q_heads + 2 * c.kv_heads) * c.head_dim
    weights = qkv_width * c.hidden + c.hidden * c.q_heads * c.head_dim + 3 * c.intermediate * c.hidden
    pairs = sum(n * ctx + n * (n + 1) // 2 for ctx, n in zip(contexts, counts))
    flops = 2.0 * rows * weights + 2.0 * c.q_heads * pairs * 2 * c.head_dim
    return {"rows": rows, "ms_per_layer": seconds * 1e3, "flops_per_layer": flops,
            "roofline": {"bound": "mfma", "achieved": flops / seconds / 1e12,
                         "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s",
                         "frac": flops / seconds / 1e12 / MFMA_BF16_PEAK_TFLOPS},
            "prefill_tok_per_s_64_layers": rows / (seconds * c.layers)}


def packed_step_c1(backend, seed=97, repeats=3):
    """BASELINE config 1: the whole Qwen3-0.6B-shaped model (28 layers, vocabulary 151936) over a
    packed 2048-token batch of 48 decode rows (contexts uniform 128..4096) and prefill chunks of
    256, 384, 512 and 848 tokens; logits and greedy tokens for every row.  Device time of the
    step from the submission's events."""
    from forja_amd.model import PackedStep
    c = QWEN3_0_6B
    rng = np.random.default_rng(seed)
    contexts = [int(v) for v in rng.integers(128, 4097, 48)] + [0, 0, 0, 0]
    counts = [1] * 48 + [256, 384, 512, 848]
    model = Model(backend, c, seed=seed)
    step = PackedStep(model, contexts, counts, seed=seed, head=True)
    step.run()
    # the step `repeats` times back to back, as the steps of a server follow each other
    submissions = [backend.submit(step.encoded) for _ in range(repeats)]
    for submission in submissions:
        submission.wait()
    seconds = sum(submission.gpu_time_ns() for submission in submissions) / repeats * 1e-9
    # what bounds it: the matrix work of 2048 rows (projections, lm_head, attention pairs), and the
    # bytes that must move whatever the rows (weights once, the KV the decode rows and chunks read)
    rows = step.tokens
    qkv_width = (c.q_heads + 2 * c.kv_heads) * c.head_dim
    per_layer = qkv_width * c.hidden + c.hidden * c.q_heads * c.head_dim + 3 * c.intermediate * c.hidden
    pairs = sum(n * ctx + n * (n + 1) // 2 for ctx, n in zip(contexts, counts))
    flops = 2.0 * rows * (c.layers * per_layer + c.vocab * c.hidden) + c.layers * 2.0 * c.q_heads * pairs * 2 * c.head_dim
    weight_bytes = (c.layers * per_layer + c.vocab * c.hidden) * 0.5625
    kv_bytes = sum(ctx + n for ctx, n in zip(contexts, counts)) * c.kv_bytes_per_token   # (all layers)
    return {"workload": "BASELINE config 1: 28 layers, 48 decode rows + prefill chunks 256/384/512/848 "
                        "packed into 2048 tokens, lm_head and argmax on every row",
            "tokens": step.tokens, "ms_per_step": seconds * 1e3, "tok_per_s": step.tokens / seconds,
            "roofline": {"bound": "mfma", "achieved": flops / seconds / 1e12, "peak": MFMA_BF16_PEAK_TFLOPS,
                         "unit": "TFLOP/s", "frac": flops / seconds / 1e12 / MFMA_BF16_PEAK_TFLOPS,
                         "flops_per_step": flops,
                         "hbm_floor_ms": (weight_bytes + kv_bytes) / (HBM_PEAK_GBPS * 1e9) * 1e3,
                         "mfma_floor_ms": flops / (MFMA_BF16_PEAK_TFLOPS * 1e12) * 1e3,
                         "note": "a 0.6B model at 2048 rows: 161 kernels of 20-120 us each, none long "
                                 "enough to fill the device; neither floor is near"}}


def lane_by_lane_step(workload, backend, steps=8, warmup=2):
    """The bench's decode step recorded the way the engines record it (per lane one
    PagedSdpaAppend and one Copy per layer, engines/qwen3-coder/src/lib.rs:917-935) on the same
    lanes and storage: the library fuses each layer's run into one ragged launch.  One more step
    with the fusion switched off gives the dispatch-by-dispatch time."""
    session = workload.session
    session.record_lane_by_lane()

    def timed(count):
        backend.synchronize()
        begin = time.perf_counter()
        submissions = []
        for _ in range(count):
            workload.churn_lanes()
            submissions.append(session.submit_lane_step())
        backend.synchronize()
        elapsed = time.perf_counter() - begin
        device_ns = 0
        for submission in submissions:
            submission.wait()
            device_ns += submission.gpu_time_ns()
            submission.free()
        return elapsed / count * 1e3, device_ns / count / 1e6

    before = backend.fusion_stats()
    timed(warmup)
    wall_ms, device_ms = timed(steps)
    runs, replaced = (after - start for after, start in zip(backend.fusion_stats(), before))
    backend.fusion_enable(False)
    serial_wall_ms, serial_device_ms = timed(1)
    backend.fusion_enable(True)
    lanes = len(session.contexts)
    return {"workload": "the timed decode step recorded lane by lane (standard ops only)",
            "dispatches_per_step": len(session.lane_commands),
            "fused_runs_per_step": runs / (steps + warmup),
            "dispatches_replaced_per_step": replaced / (steps + warmup),
            "ms_per_step": wall_ms, "device_ms_per_step": device_ms,
            "decode_tokens_per_s": lanes / (wall_ms * 1e-3),
            "unfused_ms_per_step": serial_wall_ms, "unfused_device_ms_per_step": serial_device_ms}


class _FixedLanes:
    """A decode session without churn, in the shape lane_by_lane_step drives."""

    def __init__(self, session):
        self.session = session

    def churn_lanes(self):
        pass


def engine_dtype_step(backend, workload, seed, ctx_lo, ctx_hi, lanes=8):
    """The qwen3-coder engine's own regime: decode batches of at most 8 lanes recorded lane by lane,
    f32 activations, an f16 KV cache and an 8-bit router (engines/qwen3-coder/src/lib.rs:296-437),
    on a second full-depth model of the timed config; beside it the same 8 lanes in the bench's
    bf16 dtypes on the timed model.  The f32 products run on the vector ALUs, attention on the
    matrix cores in f16."""
    from dataclasses import replace
    config = workload.model.config
    rng = np.random.default_rng(seed + 5)
    contexts = log_uniform(rng, ctx_lo, ctx_hi, lanes)
    pt = config.page_tokens
    pages = int(contexts.sum() * 1.1) // pt + 8 * lanes
    table_pages = (ctx_hi + 4096 + pt) // pt
    results = {}
    for name, model in (("bf16", workload.model), ("f32_activations_f16_cache_q8_router", None)):
        if model is None:
            mixed = replace(config, activation_dtype=DType.F32, kv_dtype=DType.F16, router_bits=8)
            model = Model(backend, mixed, seed=seed + 6, layers=workload.model.n_layers)
        session = DecodeSession(model, contexts, seed=seed + 7, physical_pages=pages, table_pages=table_pages)
        timing = lane_by_lane_step(_FixedLanes(session), backend, steps=6, warmup=2)
        results[name] = {key: timing[key] for key in ("dispatches_per_step", "fused_runs_per_step", "ms_per_step",
                                                      "device_ms_per_step", "decode_tokens_per_s",
                                                      "unfused_device_ms_per_step")}
    results["workload"] = ("%d decode lanes, contexts log-uniform %d-%d, full depth, recorded lane by lane"
                           % (lanes, ctx_lo, ctx_hi))
    return results


def stream_read_rate(backend, rows=4096, width=1 << 20, repeats=3):
    """What a plain read-only stream sustains on this device: a row-wise argmax over 8 GiB of
    bf16 (16-byte loads, one workgroup per row).  The practical ceiling the HBM-bound kernels are
    up against, next to the nominal one."""
    source = backend.alloc(DType.BF16, (rows, width))
    result = backend.alloc(DType.U32, (rows,))
    commands = CommandList()
    commands.dispatch(Op.argmax(), [source], result)
    encoded = backend.encode(commands)
    backend.submit(encoded).wait()
    backend.profile_enable(2)
    backend.profile_reset()
    for _ in range(repeats):
        backend.submit(encoded).wait()
    ns, _ = backend.profile_read(0)
    backend.profile_enable(0)
    backend.release(source)
    backend.release(result)
    return 2.0 * rows * width * repeats / (ns * 1e-9) / 1e9


def mfma_sustained_rates():
    """What the matrix cores sustain from registers on this device (v_mfma_f32_32x32x16_f16, one
    wave per SIMD, ~60 ms): with all-zero operands and with random ones.  The second is the
    practical ceiling of the prefill GEMM: operand bits that toggle cost power, and the device
    lowers its clock to stay inside its limit.  None when the probe library is not built."""
    import ctypes
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "forja_amd", "libforja_probes.so")
    if not os.path.exists(path):
        return None
    lib = ctypes.CDLL(path)
    lib.fh_probe_mfma_f16_tflops.restype = ctypes.c_double
    lib.fh_probe_mfma_f16_tflops.argtypes = [ctypes.c_int, ctypes.c_int]
    return {"zeros_tflops": lib.fh_probe_mfma_f16_tflops(200000, 0),
            "random_tflops": lib.fh_probe_mfma_f16_tflops(200000, 1)}


def prefill_attention_c4(backend, seed=93, repeats=3):
    """Paged attention of one BASELINE config 4 layer: an 8192-token chunk packed from 6 prompts
    (512..3072 tokens, from empty contexts) plus 64 decode rows (contexts uniform 128..4096), 40
    query / 8 kv heads of 128, bf16 pools of 16-token pages behind shuffled block tables."""
    from forja_amd.model import DENSE_27B
    c = DENSE_27B
    rng = np.random.default_rng(seed)
    prompts = [512, 768, 1024, 1280, 1536, 3072]
    contexts = [0] * len(prompts) + [int(v) for v in rng.integers(128, 4097, 64)]
    counts = prompts + [1] * 64
    lanes, tokens, pt = len(counts), sum(counts), c.page_tokens
    pages_of = [(ctx + n + pt - 1) // pt for ctx, n in zip(contexts, counts)]
    table_pages = max(pages_of)
    physical = sum(pages_of) + 7
    order = rng.permutation(physical)
    tables = np.zeros((lanes, table_pages, 2), np.uint32)
    tables[:, :, 1] = 0xffffffff
    cursor = 0
    for lane, n_pages in enumerate(pages_of):
        pages = order[cursor:cursor + n_pages]
        cursor += n_pages
        tables[lane, :n_pages, 0] = pages
        tables[lane, :n_pages, 1] = 11 + pages
    generations = (11 + np.arange(physical)).astype(np.uint32)
    cu = np.concatenate([[0], np.cumsum(counts)]).astype(np.uint32)

    def up(array, dtype, shape):
        tensor = backend.alloc(dtype, shape)
        backend.write(tensor, np.ascontiguousarray(array).tobytes())
        return tensor
    t_tables = up(tables, DType.U32, tables.shape)
    t_generations = up(generations, DType.U32, (physical,))
    t_cu = up(cu, DType.U32, (lanes + 1,))
    t_starts = up(np.array(contexts, np.uint32), DType.U32, (lanes,))
    t_activity = up(np.ones(lanes, np.uint32), DType.U32, (lanes,))
    q = backend.alloc(DType.BF16, (tokens, c.q_heads, c.head_dim))
    k_new = backend.alloc(DType.BF16, (tokens, c.kv_heads, c.head_dim))
    v_new = backend.alloc(DType.BF16, (tokens, c.kv_heads, c.head_dim))
    out = backend.alloc(DType.BF16, (tokens, c.q_heads, c.head_dim))
    keys = backend.alloc(DType.BF16, (physical, pt, c.kv_heads, c.head_dim))
    values = backend.alloc(DType.BF16, (physical, pt, c.kv_heads, c.head_dim))
    fill = CommandList()
    for stream, tensor in enumerate((q, k_new, v_new, keys, values)):
        fill.dispatch(Op.fill_seeded(2, seed, 20 + stream), [], tensor)
    backend.submit(fill).wait()
    commands = CommandList()
    commands.dispatch_many(Op.paged_attention_ragged(1.0 / math.sqrt(c.head_dim), pt),
                           [q, k_new, v_new, t_tables, t_generations, t_cu, t_starts, t_activity],
                           [out, keys, values])
    encoded = backend.encode(commands)
    backend.submit(encoded).wait()
    backend.profile_enable(2)
    backend.profile_reset()
    for _ in range(repeats):
        backend.submit(encoded).wait()
    op_ns, _ = backend.profile_read(KC_ATTENTION)
    kernel_ns, _ = backend.profile_read(KC_ATTENTION_KERNEL)
    backend.profile_enable(0)
    pairs = sum(n * ctx + n * (n + 1) // 2 for ctx, n in zip(contexts, counts))
    flops = 2.0 * c.q_heads * pairs * 2 * c.head_dim
    for tensor in (t_tables, t_generations, t_cu, t_starts, t_activity, q, k_new, v_new, out, keys, values):
        backend.release(tensor)
    return {"tokens": tokens, "lanes": lanes, "query_key_pairs": pairs, "flops": flops,
            "us_op": op_ns / repeats / 1e3, "us_kernel": kernel_ns / repeats / 1e3,
            "tflops": flops / (op_ns / repeats * 1e-9) / 1e12}


def decode_attention_f16_cache(backend, config, seed=99, repeats=5):
    """One layer's decode attention of the timed workload's shape (128 lanes, contexts log-uniform
    256..32768) with the dtypes the qwen3-coder engine records: f32 query and new rows, an f16 KV
    cache, f32 output; one row per lane promised, so the kernel stores the new rows itself."""
    rng = np.random.default_rng(seed)
    lanes, pt = 128, config.page_tokens
    contexts = log_uniform(rng, 256, 32768, lanes)
    pages_of = [(int(ctx) + 1 + pt - 1) // pt for ctx in contexts]
    table_pages, physical = max(pages_of), sum(pages_of) + 7
    order = rng.permutation(physical)
    tables = np.zeros((lanes, table_pages, 2), np.uint32)
    tables[:, :, 1] = 0xffffffff
    cursor = 0
    for lane, n_pages in enumerate(pages_of):
        pages = order[cursor:cursor + n_pages]
        cursor += n_pages
        tables[lane, :n_pages, 0] = pages
        tables[lane, :n_pages, 1] = 11 + pages

    def up(array, shape):
        tensor = backend.alloc(DType.U32, shape)
        backend.write(tensor, np.ascontiguousarray(array, dtype=np.uint32).tobytes())
        return tensor
    metadata = [up(tables, tables.shape), up(11 + np.arange(physical), (physical,)),
                up(np.arange(lanes + 1), (lanes + 1,)), up(np.array(contexts), (lanes,))]
    q = backend.alloc(DType.F32, (lanes, config.q_heads, config.head_dim))
    k_new = backend.alloc(DType.F32, (lanes, config.kv_heads, config.head_dim))
    v_new = backend.alloc(DType.F32, (lanes, config.kv_heads, config.head_dim))
    out = backend.alloc(DType.F32, (lanes, config.q_heads, config.head_dim))
    keys = backend.alloc(DType.F16, (physical, pt, config.kv_heads, config.head_dim))
    values = backend.alloc(DType.F16, (physical, pt, config.kv_heads, config.head_dim))
    fill = CommandList()
    for stream, tensor in enumerate((q, k_new, v_new, keys, values)):
        fill.dispatch(Op.fill_seeded(2, seed, 30 + stream), [], tensor)
    backend.submit(fill).wait()
    commands = CommandList()
    commands.dispatch_many(Op.paged_attention_ragged(1.0 / math.sqrt(config.head_dim), pt, one_row_per_lane=True),
                           [q, k_new, v_new, *metadata], [out, keys, values])
    encoded = backend.encode(commands)
    backend.submit(encoded).wait()
    backend.profile_enable(2)
    backend.profile_reset()
    for _ in range(repeats):
        backend.submit(encoded).wait()
    op_ns, _ = backend.profile_read(KC_ATTENTION)
    kernel_ns, _ = backend.profile_read(KC_ATTENTION_KERNEL)
    backend.profile_enable(0)
    for tensor in (*metadata, q, k_new, v_new, out, keys, values):
        backend.release(tensor)
    kv_bytes = sum(int(ctx) + 1 for ctx in contexts) * config.kv_heads * config.head_dim * 2 * 2
    gbps = kv_bytes / (kernel_ns / repeats)
    return {"workload": "one layer's decode attention, 128 lanes, contexts log-uniform 256-32768, f32 rows, "
                        "f16 KV cache, f32 output",
            "us_op": op_ns / repeats / 1e3, "us_kernel": kernel_ns / repeats / 1e3,
            "algorithmic_bytes": kv_bytes, "achieved_gbps": gbps, "frac_of_hbm_peak": gbps / HBM_PEAK_GBPS}


def decode_gemv(backend, model, row_counts=(1, 4, 8, 128), seed=83):
    """The quantised GEMV of small decode batches (the reference's own regime: at most 8 lanes) and
    the same products at the timed batch's 128 rows, product by product on cold weights: every
    layer's stacked qkv, o_proj and (4-bit) router in turn, and lm_head
    over four copies of its weights (one copy fits the 256 MB of cache in front of HBM).  Times
    are device time of back-to-back launches (one submission, no timers between them); bytes are
    the reference's logical traffic of the dispatch (weights with scales and biases, rows in and
    out)."""
    from forja_amd.model import QuantLinear
    c = model.config
    heads = [model.lm_head]
    fill = CommandList()
    for copy in range(3):
        extra = QuantLinear(backend, c.vocab, c.hidden)
        extra.fill(fill, seed, 40 + 3 * copy)
        heads.append(extra)
    backend.submit(fill).wait()
    groups = [("qkv", [layer.qkv for layer in model.layers]),
              ("o_proj", [layer.o_proj for layer in model.layers])]
    if c.moe and model.layers[0].router.bits == 4:
        groups.append(("router", [layer.router for layer in model.layers]))
    groups.append(("lm_head", heads))
    q4 = Op.quant_matmul(4, 64)
    results = {}
    for rows in row_counts:
        per_product = {}
        for name, linears in groups:
            x = backend.alloc(DType.BF16, (rows, linears[0].k))
            out = backend.alloc(DType.BF16, (rows, linears[0].n))
            fill = CommandList()
            fill.dispatch(Op.fill_seeded(2, seed, 60), [], x)
            backend.submit(fill).wait()
            commands = CommandList()
            for linear in linears:
                commands.dispatch(q4, [x, *linear.triple], out)
            encoded = backend.encode(commands)
            backend.submit(encoded).wait()
            nanoseconds, repeats = 0, 3
            for _ in range(repeats):
                submission = backend.submit(encoded)
                submission.wait()
                nanoseconds += submission.gpu_time_ns()
                submission.free()
            per_launch = nanoseconds / repeats / len(linears)
            logical = costs.traffic(costs.of(commands.dispatches[0]), True)
            per_product[name] = {"n": linears[0].n, "k": linears[0].k, "us": per_launch / 1e3,
                                 "logical_mb": logical / 1e6,
                                 "achieved_gbps": logical / per_launch,
                                 "frac_of_hbm_peak": logical / per_launch / HBM_PEAK_GBPS}
            backend.release(x)
            backend.release(out)
        results["rows_%d" % rows] = per_product
    for linear in heads[1:]:
        for tensor in linear.triple:
            backend.release(tensor)
    results["workload"] = ("dense 4-bit products of a decode batch of 1, 4, 8 and 128 rows at the timed "
                           "model's shapes, cold weights, back-to-back launches")
    return results


def main():
    parser = argparse.ArgumentParser()
    parser.add_argument("--gpus", type=int, default=1)
    parser.add_argument("--steps", type=int, default=64)
    parser.add_argument("--warmup", type=int, default=4)
    parser.add_argument("--seed", type=int, default=20261)
    parser.add_argument("--layers", type=int, default=None, help="debug: fewer layers")
    parser.add_argument("--lanes", type=int, default=128)
    parser.add_argument("--no-cpu-baseline", action="store_true")
    parser.add_argument("--cpu-sample-lanes", type=int, default=8)
    parser.add_argument("--no-lane-by-lane", action="store_true",
                        help="skip the lane-by-lane recording of the step (its unfused leg is one "
                             "submission of ~37k kernel launches, more than a counter-collecting "
                             "profiler run should be given)")
    parser.add_argument("--no-profile", action="store_true",
                        help="skip the HIP-event kernel timing inside the timed region")
    parser.add_argument("--headline-only", action="store_true",
                        help="the timed step, its roofline and the per-op breakdown; none of the "
                             "secondary workloads, no CPU baseline")
    parser.add_argument("--prefill-only", action="store_true",
                        help="only run the config 4 prefill projection measurement and exit")
    parser.add_argument("--gemm-only", action="store_true",
                        help="only the projections of one config 4 layer (the prefill GEMM), for counter runs")
    parser.add_argument("--gemv-only", action="store_true",
                        help="only run the small-batch GEMV measurement (on --layers layers, default 8) "
                             "and exit")
    parser.add_argument("--moe-only", action="store_true",
                        help="only run the config 2 MoE block measurement (on --layers layers' "
                             "experts, default 8) and exit")
    parser.add_argument("--calibrate-copy", type=int, default=0, metavar="MIB",
                        help="only run 8 plain copies of MIB mebibytes (a known-size kernel to "
                             "scale hardware traffic counters by) and exit")
    args = parser.parse_args()
    if args.calibrate_copy:
        backend = HipBackend(0)
        elements = args.calibrate_copy * (1 << 20) // 4
        source = backend.alloc(DType.U32, [elements])
        target = backend.alloc(DType.U32, [elements])
        for _ in range(8):
            commands = CommandList()
            commands.dispatch(Op.copy(), [source], target)
            backend.submit(commands).wait()
        print(json.dumps({"copy_bytes_read": elements * 4, "copy_bytes_written": elements * 4,
                          "kernel": "copy_flat_kernel", "launches": 8}))
        return
    if args.gemm_only:
        print(json.dumps({"prefill_gemm_c4": prefill_gemm_c4(HipBackend(0))}))
        return
    if args.gemv_only:
        backend = HipBackend(0)
        model = Model(backend, QWEN3_CODER_30B_A3B, seed=args.seed, layers=args.layers or 8)
        print(json.dumps({"decode_gemv": decode_gemv(backend, model)}))
        return
    if args.moe_only:
        backend = HipBackend(0)
        model = Model(backend, QWEN3_CODER_30B_A3B, seed=args.seed, layers=args.layers or 8)
        print(json.dumps({"moe_block_c2": moe_block_c2(backend, model)}))
        return
    if args.prefill_only:
        backend = HipBackend(0)
        print(json.dumps({"mfma_f16_sustained": mfma_sustained_rates(),
                          "prefill_gemm_c4": prefill_gemm_c4(backend),
                          "prefill_attention_c4": prefill_attention_c4(backend),
                          "prefill_layer_c4": prefill_layer_c4(backend),
                          "packed_step_c1": packed_step_c1(backend)}))
        return
    if args.gpus != 1:
        print("bench.py: this build runs the ragged forward step on ONE MI355X; collectives and "
              "sharding are not part of it, so --gpus must be 1", file=sys.stderr)
        sys.exit(2)

    config = QWEN3_CODER_30B_A3B
    ctx_lo, ctx_hi, churn = 256, 32768, 8
    default_workload = args.layers is None and args.lanes == 128 and args.seed == 20261
    backend = HipBackend(0)
    info = backend.device_info()
    # Config 3 routes "as in config 2": top-8 of the softmax of N(0,1) router logits, seeded per
    # layer.  (Under the prescribed weight law alone every token picks the same few experts; that
    # variant is reported beside the headline as `c3_weight_law_routing`.)
    workload = Workload(backend, config, args.lanes, ctx_lo, ctx_hi, churn, args.seed, layers=args.layers,
                        router_noise_seed=args.seed + 1)
    session = workload.session
    n_layers = workload.model.n_layers
    backend.synchronize()

    def run_step(encoded=None):
        contexts = session.contexts.copy()
        submission = session.submit_step(encoded)
        workload.churn_lanes()
        return submission, contexts

    def timed_steps(count, encoded=None, on_step=None):
        backend.synchronize()
        started = time.perf_counter()
        submissions = []
        for _ in range(count):
            submission, contexts = run_step(encoded)
            if on_step:
                on_step(contexts)
            submissions.append(submission)
        backend.synchronize()
        elapsed = time.perf_counter() - started
        device_ns = 0
        for submission in submissions:
            submission.wait()            # surfaces any device error flag
            device_ns += submission.gpu_time_ns()
            submission.free()
        return elapsed, device_ns

    def traced_distinct_experts(router_noise_seed):
        """Distinct experts per layer on one more (untimed) step that copies out every layer's
        choices: the routed kernels read the weights of the experts chosen, nothing else."""
        from forja_amd.model import record_step
        trace = backend.alloc(DType.U32, (n_layers, args.lanes, config.top_k))
        traced = CommandList()
        record_step(workload.model, session.cache, session.buffers, traced, feed_back=True,
                    route_trace=trace, one_row_per_lane=True, router_noise_seed=router_noise_seed)
        session.prepare_step()
        backend.submit(traced).wait()
        session.contexts += 1
        chosen = np.frombuffer(backend.read(trace), np.uint32).reshape(n_layers, args.lanes * config.top_k)
        backend.release(trace)
        return np.array([len(np.unique(layer)) for layer in chosen])

    timed_steps(args.warmup)
    if not args.no_profile:
        # inside the timed region only the dominant kernel is timed, one launch in six (every layer
        # launches it on the same lanes; a timed launch costs the stream two event records, about
        # 6 us between kernels before and after it: 0.56 ms of a step with all 48 timed)
        backend.profile_select(1 << KC_ATTENTION_KERNEL)
        backend.profile_sample(ATTENTION_TIMER_STRIDE)
        backend.profile_enable(1)
        backend.profile_reset()

    attention = {"bytes": 0, "kv_bytes": 0}

    def account(contexts):
        launch = attention_launch_cost(config, contexts)
        attention["bytes"] += costs.traffic(launch, True) * n_layers
        attention["kv_bytes"] += launch.kv_bytes * n_layers
    elapsed, device_ns = timed_steps(args.steps, on_step=account)

    tokens = args.lanes * args.steps
    result = {
        "metric": "decode tok/s, 4-bit 30B-A3B ragged batch; % HBM roofline; prefill % MFMA",
        "value": tokens / elapsed, "unit": "tok/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": elapsed / args.steps * 1e3,
        "device_ms_per_step": device_ns / args.steps / 1e6,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16",
        "data": "synthetic",
        "config": {
            "workload": ("BASELINE config 3: Qwen3-Coder-30B-A3B-shaped full model, "
                         f"{n_layers} layers, MLX-4bit random weights, {args.lanes} decode "
                         f"lanes, contexts log-uniform {ctx_lo}-{ctx_hi}, paged bf16 KV page 16, "
                         f"non-contiguous block tables, {churn} retire+admit per step, MoE routed as "
                         "in config 2 (top-8 of softmax of seeded N(0,1) router logits)"),
            "lanes": args.lanes, "layers": n_layers, "page_tokens": config.page_tokens,
            "dispatches_per_step": session.dispatches, "device": info["family"],
        },
    }
    attention_per_step = attention["bytes"] / args.steps
    distinct = None
    if not args.no_profile:
        ns, launches = backend.profile_read(KC_ATTENTION_KERNEL)
        backend.profile_sample(1)
        kernel_bytes = attention["bytes"] / (args.steps * n_layers)   # per launch = per layer per step
        average = ns / max(launches, 1) * 1e-9
        achieved = kernel_bytes / average / 1e9 if average > 0 else 0.0
        ratio = measured_traffic_ratio() if default_workload else None
        result["roofline"] = {
            "bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBPS, "unit": "GB/s",
            "frac": achieved / HBM_PEAK_GBPS,
            "traffic": kernel_bytes * ratio if ratio else None,
            "kernel": "ragged_attention_mfma_kernel", "launches": launches,
            "launches_in_timed_region": args.steps * n_layers,
            "avg_launch_us": average * 1e6, "algorithmic_bytes_per_launch": kernel_bytes,
            "kv_bytes_per_launch": attention["kv_bytes"] / max(launches, 1),
        }
        # Secondary kernels from a few extra steps with every kernel class timed, then a per-op
        # breakdown with every dispatch timed (neither is part of `value`).
        secondary_steps = 4
        backend.profile_select(0xffffffff)
        backend.profile_reset()
        for _ in range(secondary_steps):
            submission, _ = run_step()
            submission.wait()
            submission.free()
        moe_ns, moe_launches = backend.profile_read(KC_MOE_KERNEL)
        qmm_ns, qmm_launches = backend.profile_read(KC_QMM_KERNEL)
        secondary = {}
        if moe_launches:
            distinct = traced_distinct_experts(session.router_noise_seed)
            weights = step_costs(workload.model, session, float(distinct.mean()))
            moe_bytes = weights["routed_seen"] * secondary_steps / moe_launches
            secondary["routed_qmm_kernel"] = {
                "avg_launch_us": moe_ns / moe_launches / 1e3,
                "achieved_gbps": moe_bytes / (moe_ns / moe_launches * 1e-9) / 1e9,
                "frac": moe_bytes / (moe_ns / moe_launches * 1e-9) / 1e9 / HBM_PEAK_GBPS,
                "distinct_experts_per_layer": {"mean": float(distinct.mean()),
                                               "min": int(distinct.min()), "max": int(distinct.max()),
                                               "of": config.experts},
                "note": ("bytes = logical traffic of the routed products at the distinct experts the "
                         "router chose (measured on one traced step), per projection launch")}
        if qmm_launches:
            qmm_bytes = step_costs(workload.model, session)["dense"] * secondary_steps / qmm_launches
            secondary["dense_qmm_kernel"] = {
                "avg_launch_us": qmm_ns / qmm_launches / 1e3,
                "achieved_gbps": qmm_bytes / (qmm_ns / qmm_launches * 1e-9) / 1e9,
                "frac": qmm_bytes / (qmm_ns / qmm_launches * 1e-9) / 1e9 / HBM_PEAK_GBPS}
        result["secondary_kernels"] = secondary
        backend.profile_enable(2)
        backend.profile_reset()
        extra = 4
        for _ in range(extra):
            submission, _ = run_step()
            submission.wait()
            submission.free()
        breakdown = {}
        for name, kc in (("attention_ops", KC_ATTENTION), ("routed_matmul_ops", KC_MOE),
                         ("dense_matmul_ops", KC_QMM), ("other_ops", 0)):
            class_ns, _ = backend.profile_read(kc)
            breakdown[name] = class_ns / 1e6 / extra
        result["gpu_ms_per_step_by_op"] = breakdown
        backend.profile_enable(0)
    weights = step_costs(workload.model, session, float(distinct.mean()) if distinct is not None else None)
    routed = weights["routed_seen"] if weights["routed_seen"] is not None else weights["routed_maximum"]
    step_bytes = attention_per_step + weights["dense"] + routed
    result["step_algorithmic_gb"] = step_bytes / 1e9
    result["step_algorithmic_gb_by_part"] = {"attention": attention_per_step / 1e9, "dense_products": weights["dense"] / 1e9,
                                            "routed_products": routed / 1e9,
                                            "routed_products_reference_bounds": [weights["routed_minimum"] / 1e9,
                                                                                 weights["routed_maximum"] / 1e9]}
    result["step_hbm_fraction_of_peak"] = step_bytes / (elapsed / args.steps) / 1e9 / HBM_PEAK_GBPS
    if not args.no_profile and not args.headline_only:
        if config.moe:
            # The same step with the routing the prescribed weights give by themselves.
            plain = session.encode_variant(None)
            timed_steps(2, plain)
            plain_elapsed, plain_device_ns = timed_steps(16, plain)
            plain_distinct = traced_distinct_experts(None)
            plain_weights = step_costs(workload.model, session, float(plain_distinct.mean()))
            result["c3_weight_law_routing"] = {
                "workload": "the timed step with the router logits the prescribed random weights produce",
                "value": args.lanes * 16 / plain_elapsed, "unit": "tok/s",
                "ms_per_step": plain_elapsed / 16 * 1e3, "device_ms_per_step": plain_device_ns / 16 / 1e6,
                "distinct_experts_per_layer": float(plain_distinct.mean()),
                "step_algorithmic_gb": (attention_per_step + plain_weights["dense"] + plain_weights["routed_seen"]) / 1e9}
        if not args.no_lane_by_lane:
            result["lane_by_lane_step"] = lane_by_lane_step(workload, backend)
        result["roofline"]["measured_stream_read_gbps"] = stream_read_rate(backend)
        result["roofline"]["frac_of_measured_stream_read"] = (
            result["roofline"]["achieved"] / result["roofline"]["measured_stream_read_gbps"])
        sustained = mfma_sustained_rates()
        gemm = prefill_gemm_c4(backend)
        if sustained:
            gemm["roofline"]["measured_mfma_f16"] = sustained
            gemm["roofline"]["frac_of_measured_random_data_mfma"] = (
                gemm["roofline"]["achieved"] / sustained["random_tflops"])
        result["secondary_workloads"] = {"prefill_gemm_c4": gemm,
                                         "prefill_attention_c4": prefill_attention_c4(backend),
                                         "prefill_layer_c4": prefill_layer_c4(backend),
                                         "packed_step_c1": packed_step_c1(backend),
                                         "decode_attention_f16_cache": decode_attention_f16_cache(backend, config),
                                         "decode_gemv": decode_gemv(backend, workload.model)}
        if config.moe:
            result["secondary_workloads"]["moe_block_c2"] = moe_block_c2(backend, workload.model)
            if not args.no_lane_by_lane:
                result["secondary_workloads"]["engine_dtype_step"] = engine_dtype_step(
                    backend, workload, args.seed, ctx_lo, ctx_hi)
    if not args.no_cpu_baseline and not args.headline_only:
        result["cpu_baseline"] = cpu_baseline(config, args.seed, args.cpu_sample_lanes, ctx_lo, ctx_hi)
    print(json.dumps(result))


if __name__ == "__main__":
    main()
