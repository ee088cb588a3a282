"""Records the ragged continuous-batch forward step of a Qwen3-style decoder as a command list,
the way the reference engines do (engines/qwen3-coder/src/lib.rs:886-947 `forward_batch`,
:339-375 `project_decode_rows`, :505-603 `SparseMoe`, :2094-2192 embedding / lm_head / argmax),
against any object with the `Backend` methods (alloc / view / write / submit).

It owns no compute: every tensor operation is a dispatch executed by the backend.  Per-lane
`PagedSdpaAppend` dispatches are replaced by the one packed ragged-attention dispatch.
Weights are synthetic (seeded on the device with FILL_SEEDED): MLX-4bit packed words uniform over
u32, bf16 scale ~ U(0.001, 0.02), bf16 bias ~ U(-0.1, 0.1); norm weights ~ U(0.9, 1.1).

A second weight law, "zero_mean", exists for tests only: bias = -7.5 * scale + U(-0.02, 0.02) (-127.5 * scale
for 8-bit weights), so that a dequantised weight scale * (q - 7.5) + noise has no common sign.  Under the prescribed law
every weight has a positive mean about as large as its spread, one direction swamps the hidden
state and every lane emits the same token at every step; under the zero-mean law tokens depend on
the lane's context, its attention and its routing.
"""
from __future__ import annotations

import math
from dataclasses import dataclass, field
from typing import List, Optional

import numpy as np

from . import programs
from .core import CommandList, DType, Layout, Op, Slice, Tensor

GROUP = 64
BITS = 4


@dataclass
class ModelConfig:
    name: str
    hidden: int
    layers: int
    q_heads: int
    kv_heads: int
    head_dim: int
    vocab: int
    intermediate: int = 0          # dense SwiGLU width (0 for MoE models)
    experts: int = 0
    top_k: int = 0
    expert_intermediate: int = 0
    rms_eps: float = 1e-6
    rope_theta: float = 1e6
    page_tokens: int = 16
    # The qwen38 engine records bf16 activations over a bf16 cache, the qwen3-coder engine f32
    # activations over an f16 cache with an 8-bit router (engines/qwen3-coder/src/lib.rs:296-437).
    activation_dtype: DType = DType.BF16
    kv_dtype: DType = DType.BF16
    router_bits: int = 4

    @property
    def moe(self) -> bool:
        return self.experts > 0

    @property
    def kv_bytes_per_token(self) -> int:
        return self.layers * 2 * self.kv_heads * self.head_dim * self.kv_dtype.byte_size


QWEN3_0_6B = ModelConfig("qwen3-0.6b-shaped", hidden=1024, layers=28, q_heads=16, kv_heads=8,
                         head_dim=128, vocab=151936, intermediate=3072)
QWEN3_CODER_30B_A3B = ModelConfig("qwen3-coder-30b-a3b-shaped", hidden=2048, layers=48, q_heads=32,
                                  kv_heads=4, head_dim=128, vocab=151936, experts=128, top_k=8,
                                  expert_intermediate=768, rope_theta=1e7)
DENSE_27B = ModelConfig("dense-27b-shaped", hidden=5120, layers=64, q_heads=40, kv_heads=8,
                        head_dim=128, vocab=151936, intermediate=17408)


class QuantLinear:
    """packed u32 [N, K/8] (or [E, N, K/8]), bf16 scales/biases [.., N, K/64]."""

    def __init__(self, backend, n: int, k: int, experts: int = 0, bits: int = BITS):
        lead = (experts,) if experts else ()
        self.n, self.k, self.experts, self.bits = n, k, experts, bits
        self.packed = backend.alloc(DType.U32, lead + (n, k * bits // 32))
        self.scales = backend.alloc(DType.BF16, lead + (n, k // GROUP))
        self.biases = backend.alloc(DType.BF16, lead + (n, k // GROUP))

    def fill(self, commands: CommandList, seed: int, stream: int, center=None, noise=None):
        """`center`: the prepared program bias = noise - 7.5 * scale of the zero-mean law, with
        `noise` a scratch tensor of the biases' shape."""
        commands.dispatch(Op.fill_seeded(0, seed, stream), [], self.packed)
        commands.dispatch(Op.fill_seeded(1, seed, stream + 1, lo=0.001, hi=0.02), [], self.scales)
        if center is None:
            commands.dispatch(Op.fill_seeded(1, seed, stream + 2, lo=-0.1, hi=0.1), [], self.biases)
            return
        commands.dispatch(Op.fill_seeded(1, seed, stream + 2, lo=-0.02, hi=0.02), [], noise)
        commands.dispatch_kernel(center, [self.scales, noise], [self.biases])

    @property
    def triple(self):
        return [self.packed, self.scales, self.biases]

    @property
    def weight_bytes(self) -> int:
        count = (self.experts or 1) * self.n
        return count * (self.k * self.bits // 8 + 2 * (self.k // GROUP) * 2)


@dataclass
class LayerWeights:
    input_norm: Tensor
    qkv: QuantLinear
    qk_norm: Tensor            # [Hq+Hkv, D]: q_norm rows then k_norm rows (stack_decode_norm)
    o_proj: QuantLinear
    post_norm: Tensor
    router: Optional[QuantLinear] = None
    gate: Optional[QuantLinear] = None
    up: Optional[QuantLinear] = None
    down: Optional[QuantLinear] = None
    gate_up: Optional[QuantLinear] = None   # dense: stacked gate and up


def strided(tensor: Tensor, offset: int, shape, strides) -> Tensor:
    """A view with explicit element strides into the tensor's buffer."""
    return tensor.with_layout(Layout(tensor.dtype, offset, tuple(shape), tuple(strides),
                                     tensor.layout.buffer_len))


class Model:
    def __init__(self, backend, config: ModelConfig, seed: int = 1234, layers: Optional[int] = None,
                 weight_law: str = "baseline"):
        """`weight_law`: "baseline" (the prescribed synthetic law) or "zero_mean" (tests only)."""
        assert weight_law in ("baseline", "zero_mean")
        self.backend, self.config, self.seed = backend, config, seed
        c = config
        self.n_layers = c.layers if layers is None else layers
        self._stream = 0
        self._center = {bits: backend.prepare_program(programs.centered_bias_elements(bits))
                        for bits in {BITS, c.router_bits}} if weight_law == "zero_mean" else None
        self._noise: List[Tensor] = []
        fill = CommandList()
        self.embed = self._linear(fill, c.vocab, c.hidden)
        self.layers: List[LayerWeights] = []
        for _ in range(self.n_layers):
            lw = LayerWeights(
                input_norm=self._norm(fill, (c.hidden,)),
                qkv=self._linear(fill, (c.q_heads + 2 * c.kv_heads) * c.head_dim, c.hidden),
                qk_norm=self._norm(fill, (c.q_heads + c.kv_heads, c.head_dim)),
                o_proj=self._linear(fill, c.hidden, c.q_heads * c.head_dim),
                post_norm=self._norm(fill, (c.hidden,)))
            if c.moe:
                lw.router = self._linear(fill, c.experts, c.hidden, bits=c.router_bits)
                lw.gate = self._linear(fill, c.expert_intermediate, c.hidden, c.experts)
                lw.up = self._linear(fill, c.expert_intermediate, c.hidden, c.experts)
                lw.down = self._linear(fill, c.hidden, c.expert_intermediate, c.experts)
            else:
                lw.gate_up = self._linear(fill, 2 * c.intermediate, c.hidden)
                lw.down = self._linear(fill, c.hidden, c.intermediate)
            self.layers.append(lw)
        self.final_norm = self._norm(fill, (c.hidden,))
        self.lm_head = self._linear(fill, c.vocab, c.hidden)
        backend.submit(fill).wait()
        for noise in self._noise:
            backend.release(noise)
        self._noise = []
        self.rms_norm = backend.prepare_program(programs.rms_norm_rows(c.rms_eps))
        self.residual_norm = backend.prepare_program(programs.residual_norm_rows(c.rms_eps))
        self.qk_norm_rope = backend.prepare_program(
            programs.qk_norm_rope_rows(float(c.head_dim), c.rms_eps, c.rope_theta))
        self.silu_mul = backend.prepare_program(programs.silu_mul_elements())
        self.swiglu_epilogue = backend.prepare_epilogue(programs.silu_mul_elements())
        self.add_epilogue = backend.prepare_epilogue(programs.add_elements())

    # ---- construction helpers
    def _next_stream(self, count: int) -> int:
        first = self._stream
        self._stream += count
        return first

    def _linear(self, fill, n, k, experts=0, bits=BITS) -> QuantLinear:
        linear = QuantLinear(self.backend, n, k, experts, bits)
        noise = None
        if self._center is not None:
            noise = self.backend.alloc(DType.BF16, linear.biases.shape)
            self._noise.append(noise)
        linear.fill(fill, self.seed, self._next_stream(3),
                    self._center[bits] if self._center is not None else None, noise)
        return linear

    def _norm(self, fill, shape) -> Tensor:
        tensor = self.backend.alloc(DType.BF16, shape)
        fill.dispatch(Op.fill_seeded(1, self.seed, self._next_stream(1), lo=0.9, hi=1.1), [], tensor)
        if self.config.activation_dtype == DType.BF16:
            return tensor
        # the seeded uniform fill is defined for bf16: widen its values into the activations' dtype
        wide = self.backend.alloc(self.config.activation_dtype, shape)
        fill.dispatch(Op.copy(), [tensor], wide)
        return wide

    def weight_bytes_per_step(self, rows: int) -> dict:
        """Algorithmic weight bytes one decode step reads (packed + scales + biases), by class."""
        c = self.config
        dense = sum(l.qkv.weight_bytes + l.o_proj.weight_bytes for l in self.layers)
        dense += self.lm_head.weight_bytes
        routed = 0
        for l in self.layers:
            if c.moe:
                dense += l.router.weight_bytes
                routed += l.gate.weight_bytes + l.up.weight_bytes + l.down.weight_bytes
            else:
                dense += l.gate_up.weight_bytes + l.down.weight_bytes
        return {"dense": dense, "routed_all_experts": routed}


class KvCache:
    """Host-side page bookkeeping for one serving slot, as `forja-host` keeps it
    (crates/forja-host/src/lib.rs:4430-4500): per layer one K and one V pool
    [P, page_tokens, Hkv, D], one generations tensor shared by all planes, one table per lane."""

    def __init__(self, backend, config: ModelConfig, layers: int, lanes: int, physical_pages: int,
                 table_pages: int, seed: int, fill_pools: bool = True):
        c = config
        self.backend, self.config = backend, config
        self.lanes, self.physical_pages, self.table_pages = lanes, physical_pages, table_pages
        shape = (physical_pages, c.page_tokens, c.kv_heads, c.head_dim)
        self.keys = [backend.alloc(c.kv_dtype, shape) for _ in range(layers)]
        self.values = [backend.alloc(c.kv_dtype, shape) for _ in range(layers)]
        if fill_pools:
            fill = CommandList()
            for layer in range(layers):
                fill.dispatch(Op.fill_seeded(2, seed, 1000 + 2 * layer), [], self.keys[layer])
                fill.dispatch(Op.fill_seeded(2, seed, 1001 + 2 * layer), [], self.values[layer])
            backend.submit(fill).wait()
        self.generation_values = (11 + np.arange(physical_pages)).astype(np.uint32)
        self.generations = backend.alloc(DType.U32, (physical_pages,))
        backend.write(self.generations, self.generation_values.tobytes())
        self.table_values = np.zeros((lanes, table_pages, 2), np.uint32)
        self.table_values[:, :, 1] = 0xffffffff           # poison: never dereferenced
        self.tables = backend.alloc(DType.U32, (lanes, table_pages, 2))
        self.free = list(range(physical_pages))
        self.lane_pages: List[List[int]] = [[] for _ in range(lanes)]

    def shuffle_free(self, rng):
        order = rng.permutation(len(self.free))
        self.free = [self.free[i] for i in order]

    def ensure(self, lane: int, tokens: int):
        """Grows lane's table to cover `tokens` tokens."""
        need = (tokens + self.config.page_tokens - 1) // self.config.page_tokens
        pages = self.lane_pages[lane]
        while len(pages) < need:
            page = self.free.pop()
            self.table_values[lane, len(pages)] = (page, self.generation_values[page])
            pages.append(page)

    def retire(self, lane: int):
        for page in self.lane_pages[lane]:
            self.free.append(page)
        self.lane_pages[lane] = []
        self.table_values[lane, :, 0] = 0
        self.table_values[lane, :, 1] = 0xffffffff

    def upload_tables(self, lanes=None):
        if lanes is None:
            self.backend.write(self.tables, self.table_values.tobytes())
            return
        for lane in lanes:
            self.backend.write(self.tables.narrow(0, lane, 1), self.table_values[lane].tobytes())


class StepBuffers:
    """Activations and per-lane metadata of one packed batch of `tokens` rows over `lanes` lanes."""

    def __init__(self, backend, config: ModelConfig, tokens: int, lanes: int, head: bool = True):
        c = config
        qkv_width = (c.q_heads + 2 * c.kv_heads) * c.head_dim
        a = lambda *shape: backend.alloc(c.activation_dtype, shape)
        self.tokens, self.lanes = tokens, lanes
        self.ids = backend.alloc(DType.U32, (tokens,))
        self.positions = backend.alloc(DType.F32, (tokens,))     # rope positions, one per row
        self.cu_seqlens = backend.alloc(DType.U32, (lanes + 1,))
        self.q_starts = backend.alloc(DType.U32, (lanes,))
        self.activity = backend.alloc(DType.U32, (lanes,))
        self.hidden = [a(tokens, c.hidden), a(tokens, c.hidden)]
        self.normalized = [a(tokens, c.hidden), a(tokens, c.hidden)]
        self.qkv = a(tokens, qkv_width)
        self.qk = a(tokens, c.q_heads + c.kv_heads, c.head_dim)
        self.attended = a(tokens, c.q_heads, c.head_dim)
        self.projected = a(tokens, c.hidden)
        if c.moe:
            self.router_logits = a(tokens, c.experts)
            self.route_weights = a(tokens, c.top_k)
            self.route_indices = backend.alloc(DType.U32, (tokens, c.top_k))
            self.activated = a(tokens, c.top_k, c.expert_intermediate)
        else:
            self.gate_up = a(tokens, 2 * c.intermediate)
            self.activated = a(tokens, c.intermediate)
        self.logits = a(tokens, c.vocab) if head else None
        self.next_tokens = backend.alloc(DType.U32, (tokens,))


def seeded_router_logits(model: Model, buffers: StepBuffers, seed: int) -> Tensor:
    """[layers, tokens, experts] N(0,1) values, stream 7000 + layer of `seed`, filled on first use
    and kept with the step's buffers."""
    kept = getattr(buffers, "seeded_logits", None)
    if kept is not None and kept[0] == seed:
        return kept[1]
    c, backend = model.config, model.backend
    noise = backend.alloc(c.activation_dtype, (model.n_layers, buffers.tokens, c.experts))
    fill = CommandList()
    for layer in range(model.n_layers):
        fill.dispatch(Op.fill_seeded(2, seed, 7000 + layer), [],
                      noise.narrow(0, layer, 1).reshape((buffers.tokens, c.experts)))
    backend.submit(fill).wait()
    buffers.seeded_logits = (seed, noise)
    return noise


def record_step(model: Model, cache: KvCache, buffers: StepBuffers, commands: CommandList,
                feed_back: bool = False, route_trace: Optional[Tensor] = None,
                head: bool = True, lane_starts=None, lane_sites: Optional[list] = None,
                one_row_per_lane: bool = False, router_noise_seed: Optional[int] = None) -> None:
    """Appends one forward step over the packed batch to `commands`.  With `feed_back` the greedy
    tokens are copied into the id buffer for the next step (device to device).  `route_trace`
    (u32 [layers, tokens, top_k]) receives a copy of every layer's expert choices, for
    diagnostics.  Without `head` the step stops after the last layer's norm (no lm_head).

    With `lane_starts` (one cached-token count per lane, one query row per lane) attention is
    recorded the way the engines record a decode batch (engines/qwen3-coder/src/lib.rs:917-935):
    per lane one Op::PagedSdpaAppend on the lane's rows of q/k/v with the lane's table and a row of
    its own for the result, followed by the Op::Copy of that row into the packed activation.  The
    start is an attribute of the op; `lane_sites` receives (dispatch index, lane) of every such
    dispatch so that a replay can patch it.  `one_row_per_lane` passes the packed op the promise
    that the batch is a decode batch (every lane at most one row).

    `router_noise_seed`: every layer's top-k reads seeded N(0,1) logits (a stream per layer, filled
    once into a tensor of their own when the step is recorded) instead of what the router product,
    which still runs, has written: the routing law of the single-block configuration ("top-8 of
    softmax of N(0,1) router logits"), under which nearly every expert is touched; under the
    prescribed weight law alone all tokens choose the same few experts."""
    c, b = model.config, buffers
    tokens = b.tokens
    heads = c.q_heads + c.kv_heads
    half = c.head_dim // 2
    qkv_width = (c.q_heads + 2 * c.kv_heads) * c.head_dim
    scale = 1.0 / math.sqrt(c.head_dim)
    q4 = Op.quant_matmul(BITS, GROUP)
    gq4 = Op.gather_quant_matmul(BITS, GROUP)

    def norm_weight(weight: Tensor) -> Tensor:
        return weight.broadcast((tokens, c.hidden))

    hidden, other = b.hidden
    normalized, normalized_next = b.normalized
    commands.dispatch(Op.quant_embed(BITS, GROUP), [*model.embed.triple, b.ids], hidden)
    commands.dispatch_kernel(model.rms_norm, [hidden, norm_weight(model.layers[0].input_norm)],
                             [normalized])
    # views that do not change from layer to layer
    qk_in = strided(b.qkv, 0, (tokens, heads, c.head_dim), (qkv_width, c.head_dim, 1))
    v_new = strided(b.qkv, heads * c.head_dim, (tokens, c.kv_heads, c.head_dim),
                    (qkv_width, c.head_dim, 1))
    positions = strided(b.positions, 0, (tokens, heads, half), (1, 0, 0))
    q = b.qk.narrow(1, 0, c.q_heads)
    k_new = b.qk.narrow(1, c.q_heads, c.kv_heads)
    attention_inputs_tail = [cache.tables, cache.generations, b.cu_seqlens, b.q_starts, b.activity]
    for index, layer in enumerate(model.layers):
        commands.dispatch(q4, [normalized, *layer.qkv.triple], b.qkv)
        qk_weight = layer.qk_norm.broadcast((tokens, heads, c.head_dim))
        commands.dispatch_kernel(
            model.qk_norm_rope,
            [qk_in.narrow(2, 0, half), qk_in.narrow(2, half, half), qk_weight.narrow(2, 0, half),
             qk_weight.narrow(2, half, half), positions],
            [b.qk.narrow(2, 0, half), b.qk.narrow(2, half, half)])
        if lane_starts is None:
            commands.dispatch_many(Op.paged_attention_ragged(scale, c.page_tokens, one_row_per_lane),
                                   [q, k_new, v_new, *attention_inputs_tail],
                                   [b.attended, cache.keys[index], cache.values[index]])
        else:
            table_pages = cache.tables.shape[1]
            for lane in range(tokens):
                row = b.lane_rows.narrow(0, lane, 1)
                if lane_sites is not None:
                    lane_sites.append((len(commands), lane))
                commands.dispatch_many(
                    Op.paged_sdpa_append(scale, int(lane_starts[lane]), c.page_tokens),
                    [q.narrow(0, lane, 1).permute([1, 0, 2]), k_new.narrow(0, lane, 1),
                     v_new.narrow(0, lane, 1),
                     cache.tables.narrow(0, lane, 1).reshape((table_pages, 2)), cache.generations,
                     b.activity.narrow(0, lane, 1)],
                    [row.permute([1, 0, 2]), cache.keys[index], cache.values[index]])
                commands.dispatch(Op.copy(), [row.reshape((1, c.q_heads * c.head_dim))],
                                  b.attended.narrow(0, lane, 1).reshape((1, c.q_heads * c.head_dim)))
        commands.dispatch(q4, [b.attended.reshape((tokens, c.q_heads * c.head_dim)),
                               *layer.o_proj.triple], b.projected)
        commands.dispatch_kernel(model.residual_norm,
                                 [hidden, b.projected, norm_weight(layer.post_norm)],
                                 [other, normalized_next])
        hidden, other = other, hidden
        normalized, normalized_next = normalized_next, normalized
        if c.moe:
            commands.dispatch(Op.quant_matmul(c.router_bits, GROUP), [normalized, *layer.router.triple],
                              b.router_logits)
            logits = b.router_logits
            if router_noise_seed is not None:
                logits = seeded_router_logits(model, b, router_noise_seed).narrow(0, index, 1).reshape(
                    (tokens, c.experts))
            commands.dispatch_many(Op.top_k(c.top_k, True), [logits],
                                   [b.route_weights, b.route_indices])
            if route_trace is not None:
                commands.dispatch(Op.copy(), [b.route_indices],
                                  route_trace.narrow(0, index, 1).reshape((tokens, c.top_k)))
            commands.dispatch_epilogue(gq4, [normalized, *layer.gate.triple, *layer.up.triple,
                                             b.route_indices], b.activated, model.swiglu_epilogue, [])
            commands.dispatch_epilogue(gq4, [b.activated, *layer.down.triple, b.route_indices,
                                             b.route_weights], other, model.add_epilogue, [hidden])
        else:
            commands.dispatch(q4, [normalized, *layer.gate_up.triple], b.gate_up)
            commands.dispatch_kernel(model.silu_mul,
                                     [b.gate_up.narrow(1, 0, c.intermediate),
                                      b.gate_up.narrow(1, c.intermediate, c.intermediate)],
                                     [b.activated])
            commands.dispatch_epilogue(q4, [b.activated, *layer.down.triple], other,
                                       model.add_epilogue, [hidden])
        hidden, other = other, hidden
        following = model.layers[index + 1].input_norm if index + 1 < len(model.layers) \
            else model.final_norm
        commands.dispatch_kernel(model.rms_norm, [hidden, norm_weight(following)], [normalized_next])
        normalized, normalized_next = normalized_next, normalized
    if not head:
        return
    commands.dispatch(q4, [normalized, *model.lm_head.triple], b.logits)
    commands.dispatch(Op.argmax(), [b.logits], b.next_tokens)
    if feed_back:
        commands.dispatch(Op.copy(), [b.next_tokens], b.ids)


class DecodeSession:
    """A continuous batch of decode lanes: owns the cache bookkeeping and the per-step metadata the
    host uploads between steps (positions, query starts, tables), and replays one encoded command
    list per step.  Greedy tokens are fed back on the device."""

    def __init__(self, model: Model, contexts, seed: int = 7, headroom_tokens: int = 64,
                 physical_pages: Optional[int] = None, table_pages: Optional[int] = None,
                 fill_pools: bool = True, lane_by_lane: bool = False,
                 router_noise_seed: Optional[int] = None):
        c = model.config
        backend = model.backend
        self.model = model
        self.contexts = np.array(contexts, dtype=np.int64)
        lanes = len(contexts)
        pt = c.page_tokens
        if table_pages is None:
            table_pages = int((self.contexts.max() + headroom_tokens + pt) // pt)
        if physical_pages is None:
            physical_pages = int(((self.contexts + headroom_tokens + pt) // pt).sum() + 8)
        self.cache = KvCache(backend, c, model.n_layers, lanes, physical_pages, table_pages, seed,
                             fill_pools=fill_pools)
        rng = np.random.default_rng(seed)
        self.rng = rng
        self.cache.shuffle_free(rng)                       # non-contiguous block tables
        for lane in range(lanes):
            self.cache.ensure(lane, int(self.contexts[lane]) + 1)
        self.cache.upload_tables()
        self.buffers = StepBuffers(backend, c, lanes, lanes)
        b = self.buffers
        backend.write(b.cu_seqlens, np.arange(lanes + 1, dtype=np.uint32).tobytes())
        backend.write(b.activity, np.ones(lanes, dtype=np.uint32).tobytes())
        first_ids = rng.integers(0, c.vocab, lanes).astype(np.uint32)
        backend.write(b.ids, first_ids.tobytes())
        self.router_noise_seed = router_noise_seed
        commands = CommandList()
        record_step(model, self.cache, b, commands, feed_back=True, one_row_per_lane=True,
                    router_noise_seed=router_noise_seed)
        self.commands = commands
        self.encoded = backend.encode(commands) if hasattr(backend, "encode") else commands
        self.dispatches = len(commands)
        self.lane_commands = self.lane_encoded = None
        if lane_by_lane:
            self.record_lane_by_lane()

    def record_lane_by_lane(self):
        """Records the same step lane by lane, as the engines record it, on the same storage."""
        if self.lane_encoded is not None:
            return
        c, b, backend = self.model.config, self.buffers, self.model.backend
        b.lane_rows = backend.alloc(c.activation_dtype, (len(self.contexts), c.q_heads, c.head_dim))
        self.lane_sites = []
        self.lane_commands = CommandList()
        record_step(self.model, self.cache, b, self.lane_commands, feed_back=True,
                    lane_starts=self.contexts, lane_sites=self.lane_sites,
                    router_noise_seed=self.router_noise_seed)
        self.lane_encoded = backend.encode(self.lane_commands) if hasattr(backend, "encode") \
            else self.lane_commands
        self._site_index = np.array([site for site, _ in self.lane_sites])
        self._site_lane = np.array([lane for _, lane in self.lane_sites])

    def submit_lane_step(self):
        """Like submit_step, through the lane-by-lane recording: the query starts are attributes of
        the per-lane dispatches, patched into the encoded list before it is submitted."""
        self.prepare_step()
        backend = self.model.backend
        if hasattr(backend, "patch_query_starts"):
            backend.patch_query_starts(self.lane_encoded, self._site_index,
                                       self.contexts[self._site_lane])
        else:   # a backend without an encoded form: record the step again with this step's starts
            self.lane_encoded = CommandList()
            record_step(self.model, self.cache, self.buffers, self.lane_encoded, feed_back=True,
                        lane_starts=self.contexts)
        submission = backend.submit(self.lane_encoded)
        self.contexts += 1
        return submission

    def upload_positions(self):
        b, backend = self.buffers, self.model.backend
        backend.write(b.q_starts, self.contexts.astype(np.uint32).tobytes())
        backend.write(b.positions, self.contexts.astype(np.float32).tobytes())

    def prepare_step(self):
        """Makes room for this step's token in every lane and uploads the step's metadata."""
        grown = []
        for lane in range(len(self.contexts)):
            before = len(self.cache.lane_pages[lane])
            self.cache.ensure(lane, int(self.contexts[lane]) + 1)
            if len(self.cache.lane_pages[lane]) != before:
                grown.append(lane)
        if grown:
            self.cache.upload_tables(grown)
        self.upload_positions()

    def encode_variant(self, router_noise_seed: Optional[int]):
        """The same step on the same storage recorded with another routing law."""
        commands = CommandList()
        record_step(self.model, self.cache, self.buffers, commands, feed_back=True,
                    one_row_per_lane=True, router_noise_seed=router_noise_seed)
        backend = self.model.backend
        return backend.encode(commands) if hasattr(backend, "encode") else commands

    def submit_step(self, encoded=None):
        """Uploads this step's metadata and enqueues the step; returns the submission."""
        self.prepare_step()
        submission = self.model.backend.submit(self.encoded if encoded is None else encoded)
        self.contexts += 1
        return submission

    def step(self, lane_by_lane: bool = False) -> np.ndarray:
        submission = self.submit_lane_step() if lane_by_lane else self.submit_step()
        submission.wait()
        raw = self.model.backend.read(self.buffers.next_tokens)
        return np.frombuffer(raw, dtype=np.uint32).copy()

    def replace_lane(self, lane: int, context: int):
        """Retires the lane's sequence and admits a new one with `context` cached tokens."""
        self.cache.retire(lane)
        self.contexts[lane] = context
        self.cache.ensure(lane, context + 1)
        self.cache.upload_tables([lane])

    def kv_bytes_this_step(self) -> int:
        """Algorithmic K/V bytes the next step's attention reads: (context+1) rows per lane."""
        return int((self.contexts + 1).sum()) * self.model.config.kv_bytes_per_token \
            * self.model.n_layers // self.model.config.layers


class PackedStep:
    """One forward step over a packed batch that mixes prefill chunks and decode rows: lane l has
    `contexts[l]` cached tokens and contributes `counts[l]` new rows (BASELINE configs 1 and 4).
    Owns the cache, the buffers and the recorded command list; `run()` executes it once."""

    def __init__(self, model: Model, contexts, counts, seed: int = 7, head: bool = True,
                 fill_pools: bool = True):
        c, backend = model.config, model.backend
        self.model = model
        contexts = np.array(contexts, dtype=np.int64)
        counts = np.array(counts, dtype=np.int64)
        lanes, tokens, pt = len(contexts), int(counts.sum()), c.page_tokens
        pages = (contexts + counts + pt - 1) // pt
        self.cache = KvCache(backend, c, model.n_layers, lanes, int(pages.sum()) + 8,
                             int(pages.max()) + 1, seed, fill_pools=fill_pools)
        rng = np.random.default_rng(seed)
        self.cache.shuffle_free(rng)
        for lane in range(lanes):
            self.cache.ensure(lane, int(contexts[lane] + counts[lane]))
        self.cache.upload_tables()
        self.buffers = b = StepBuffers(backend, c, tokens, lanes, head=head)
        cu = np.concatenate([[0], np.cumsum(counts)]).astype(np.uint32)
        positions = np.concatenate([contexts[lane] + np.arange(counts[lane]) for lane in range(lanes)])
        backend.write(b.cu_seqlens, cu.tobytes())
        backend.write(b.activity, np.ones(lanes, dtype=np.uint32).tobytes())
        backend.write(b.q_starts, contexts.astype(np.uint32).tobytes())
        backend.write(b.positions, positions.astype(np.float32).tobytes())
        backend.write(b.ids, rng.integers(0, c.vocab, tokens).astype(np.uint32).tobytes())
        self.commands = CommandList()
        record_step(model, self.cache, b, self.commands, head=head)
        self.encoded = backend.encode(self.commands) if hasattr(backend, "encode") else self.commands
        self.tokens, self.lanes = tokens, lanes

    def run(self):
        submission = self.model.backend.submit(self.encoded)
        submission.wait()
        return submission
