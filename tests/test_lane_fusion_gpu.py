"""A decode batch recorded the way the engines record it (engines/qwen3-coder/src/lib.rs:917-935):
per lane one Op::PagedSdpaAppend on narrowed rows of the packed q/k/v, with the lane's own table
allocation (crates/forja-host/src/lib.rs:4466-4480) and a fresh output row
(crates/forja-sdk/src/paged.rs:525-528), each followed by the Op::Copy of that row into the packed
activation.  The library executes such a run as one ragged launch; these tests hold the result to
the CPU oracle's serial execution and to the library's own dispatch-by-dispatch execution."""
import math

import numpy as np
import pytest

from forja_amd.core import BackendError, CommandList, DType, Op, Status, INTO_PAGES
from oracle import cpu_backend as orc
from tests.helpers import assert_close, normal_bf16, to_f32, upload

pytestmark = pytest.mark.gpu

WIDTH = 128


def run(backend, commands):
    backend.submit(commands).wait()


class LaneBatch:
    """Storage of a decode batch: packed q/k/v rows, one table allocation per lane, shared
    generations and activity, `layers` pairs of pools."""

    def __init__(self, backend, contexts, hq, hkv, pt, seed, layers=1, activity=None, corrupt=None,
                 dtype=DType.BF16, pool_dtype=None):
        pool_dtype = dtype if pool_dtype is None else pool_dtype
        self.backend, self.contexts, self.hq, self.hkv, self.pt = backend, list(contexts), hq, hkv, pt
        lanes = len(contexts)
        pages_needed = [(c + 1 + pt - 1) // pt for c in contexts]
        self.table_pages = max(pages_needed) + 2
        physical = sum(pages_needed) + 3
        rng = np.random.default_rng(seed)
        free = list(rng.permutation(physical))
        self.tables, self.host_tables = [], []
        for lane, need in enumerate(pages_needed):
            table = np.zeros((self.table_pages, 2), np.uint32)
            table[:, 1] = 0xffffffff
            for logical in range(need):
                page = free.pop()
                table[logical] = (page, 11 + page)
            if corrupt is not None and corrupt[0] == lane:
                table[corrupt[1], 1] += 1
            self.tables.append(upload(backend, table, DType.U32))
            self.host_tables.append(table)
        self.spare_pages = free
        self.generations = upload(backend, 11 + np.arange(physical), DType.U32)
        self.activity = None if activity is None else upload(backend, np.array(activity), DType.U32)
        self.q = upload(backend, normal_bf16(seed, 3, (lanes, hq, WIDTH)), dtype)
        self.k = upload(backend, normal_bf16(seed, 4, (lanes, hkv, WIDTH)), dtype)
        self.v = upload(backend, normal_bf16(seed, 5, (lanes, hkv, WIDTH)), dtype)
        self.pools = []
        for layer in range(layers):
            keys = upload(backend, normal_bf16(seed, 10 + 2 * layer, (physical, pt, hkv, WIDTH)), pool_dtype)
            values = upload(backend, normal_bf16(seed, 11 + 2 * layer, (physical, pt, hkv, WIDTH)), pool_dtype)
            self.pools.append((keys, values))
        self.dtype = dtype
        self.lanes = lanes

    def record_layer(self, commands, layer, starts=None, copy_rows=True, lanes=None, idiom="append"):
        """Appends the per-lane dispatches of one layer; returns (packed attended, lane rows).
        idiom "append": Op::PagedSdpaAppend per lane; "copies": two Op::PagedCopy{IntoPages} and
        one Op::PagedSdpa per lane (engines/qwen38/src/attention/batch.rs:37-53)."""
        backend, hq = self.backend, self.hq
        starts = self.contexts if starts is None else starts
        scale = 1.0 / math.sqrt(WIDTH)
        attended = backend.alloc(self.dtype, (self.lanes, hq * WIDTH))
        rows = []
        keys, values = self.pools[layer]
        for lane in (range(self.lanes) if lanes is None else lanes):
            row = backend.alloc(self.dtype, (1, hq, WIDTH))
            inputs = [self.q.narrow(0, lane, 1).permute([1, 0, 2]), self.k.narrow(0, lane, 1),
                      self.v.narrow(0, lane, 1), self.tables[lane], self.generations]
            if self.activity is not None:
                inputs.append(self.activity.narrow(0, lane, 1))
            if idiom == "append":
                commands.dispatch_many(Op.paged_sdpa_append(scale, starts[lane], self.pt), inputs,
                                       [row.permute([1, 0, 2]), keys, values])
            else:
                physical, elements = keys.shape[0], self.hkv * WIDTH
                paging = inputs[3:]
                for new_row, pool in ((inputs[1], keys), (inputs[2], values)):
                    commands.dispatch(Op.paged_copy(INTO_PAGES, starts[lane], self.pt),
                                      [new_row.reshape((1, elements)), *paging],
                                      pool.reshape((physical, self.pt, elements)))
                commands.dispatch(Op.paged_sdpa(scale, True, starts[lane], starts[lane] + 1, self.pt),
                                  [inputs[0], keys, values, *paging], row.permute([1, 0, 2]))
            if copy_rows:
                commands.dispatch(Op.copy(), [row.reshape((1, hq * WIDTH))], attended.narrow(0, lane, 1))
            rows.append(row)
        return attended, rows


def check(cpu, hip, cpu_tensors, hip_tensors, exact=(), bar=None):
    """`bar`: the dtype whose tolerance judges the float rows (the reference holds f32 outputs
    attended from f16 pools to the pools' tolerance, crates/forja-metal/tests/paged.rs:982-988)."""
    for index, (a, b) in enumerate(zip(cpu_tensors, hip_tensors)):
        if index in exact:
            assert cpu.read(a) == hip.read(b)
        else:
            assert_close(to_f32(hip.read(b), b.dtype), to_f32(cpu.read(a), a.dtype), bar or b.dtype)


CASES = [
    # contexts, hq, hkv, page_tokens
    ([17, 64, 130, 511], 16, 8, 16),                        # BASELINE config 0
    ([300, 1, 2047, 700, 15, 16, 0], 32, 4, 16),
    ([100, 257, 31], 32, 4, 64),                            # engine page size
    ([3 + (5 * lane) % 28 for lane in range(131)], 16, 2, 16),  # 131 lanes: more than one argument block
]


@pytest.mark.parametrize("idiom", ["append", "copies"])
@pytest.mark.parametrize("contexts,hq,hkv,pt", CASES)
def test_lane_by_lane_batch_equals_serial_execution(cpu, hip, contexts, hq, hkv, pt, idiom):
    """Two layers on the same lanes (the second reuses the gathered metadata), fused on the
    device, serial on the oracle; pools bit for bit, attention rows to the float bar; then the
    library's own serial execution of the same list."""
    outputs = {}
    for name, backend in (("cpu", cpu), ("fused", hip), ("serial", hip)):
        if backend is hip:
            hip.fusion_enable(name == "fused")
        before = hip.fusion_stats()
        batch = LaneBatch(backend, contexts, hq, hkv, pt, seed=71, layers=2)
        commands = CommandList()
        kept = []
        for layer in range(2):
            attended, rows = batch.record_layer(commands, layer, idiom=idiom)
            kept += [attended, rows[0], rows[-1], *batch.pools[layer]]
        run(backend, commands)
        outputs[name] = (backend, kept)
        runs, dispatches = (after - start for after, start in zip(hip.fusion_stats(), before))
        if name == "fused":
            assert (runs, dispatches) == (2, 2 * (2 if idiom == "append" else 4) * len(contexts))
        else:
            assert (runs, dispatches) == (0, 0)
    hip.fusion_enable(True)
    pools = (3, 4, 8, 9)
    check(cpu, hip, outputs["cpu"][1], outputs["fused"][1], exact=pools)
    check(cpu, hip, outputs["cpu"][1], outputs["serial"][1], exact=pools)
    check(hip, hip, outputs["serial"][1], outputs["fused"][1], exact=pools)


@pytest.mark.parametrize("idiom", ["append", "copies"])
@pytest.mark.parametrize("dtype,pool_dtype", [(DType.F32, DType.F16), (DType.F16, DType.F16)])
def test_lane_by_lane_batch_with_f16_pools(cpu, hip, idiom, dtype, pool_dtype):
    """The qwen3-coder engine's dtypes (f32 rows, f16 KV cache) through the fused run: the rows are
    rounded into the pools exactly as serial execution rounds them."""
    contexts = [300, 1, 2047, 700, 15, 16, 0, 64, 63]
    outputs = []
    for backend in (cpu, hip):
        before = hip.fusion_stats()
        batch = LaneBatch(backend, contexts, 32, 4, 64, seed=79, layers=2, dtype=dtype, pool_dtype=pool_dtype)
        batch.k = upload(backend, normal_bf16(79, 6, (len(contexts), 4, WIDTH)) * 1.001, dtype)
        batch.v = upload(backend, normal_bf16(79, 7, (len(contexts), 4, WIDTH)) * 1.001, dtype)
        commands = CommandList()
        kept = []
        for layer in range(2):
            attended, rows = batch.record_layer(commands, layer, idiom=idiom)
            kept += [attended, rows[0], rows[-1], *batch.pools[layer]]
        run(backend, commands)
        outputs.append(kept)
        if backend is hip:
            assert hip.fusion_stats()[0] - before[0] == 2
    check(cpu, hip, outputs[0], outputs[1], exact=(3, 4, 8, 9), bar=pool_dtype)


def test_runs_without_row_copies_and_with_inactive_lanes(cpu, hip):
    results = []
    for backend in (cpu, hip):
        before = hip.fusion_stats()
        batch = LaneBatch(backend, [33, 70, 5, 129], 8, 4, 16, seed=72, activity=[1, 0, 1, 1])
        commands = CommandList()
        _, rows = batch.record_layer(commands, 0, copy_rows=False)
        run(backend, commands)
        results.append(rows + list(batch.pools[0]))
        if backend is hip:
            assert hip.fusion_stats()[0] - before[0] == 1
    check(cpu, hip, results[0], results[1], exact=(4, 5))
    assert not to_f32(hip.read(results[1][1]), DType.BF16).any()


def test_gathered_metadata_follows_a_table_rewritten_between_layers(cpu, hip):
    """Layer 0 and 1 share the gathered tables; then lane 1's table is overwritten on the device
    (its first page moves to a spare physical page) and it gets a new start: the third run must
    see both."""
    contexts = [40, 90, 200, 7]
    results = []
    for backend in (cpu, hip):
        batch = LaneBatch(backend, contexts, 16, 8, 16, seed=73, layers=2)
        commands = CommandList()
        first, _ = batch.record_layer(commands, 0)
        second, _ = batch.record_layer(commands, 1)
        replacement = batch.host_tables[1].copy()
        spare = batch.spare_pages[0]
        replacement[0] = (spare, 11 + spare)
        commands.dispatch(Op.copy(), [upload(backend, replacement, DType.U32)], batch.tables[1])
        moved = list(contexts)
        moved[1] = 70
        third, _ = batch.record_layer(commands, 0, starts=moved)
        run(backend, commands)
        results.append([first, second, third, *batch.pools[0], *batch.pools[1]])
    check(cpu, hip, results[0], results[1], exact=(3, 4, 5, 6))


@pytest.mark.parametrize("idiom,corrupt,expected", [
    ("append", (2, 1), (4, 1)),      # stale history page: lane 2's attention dispatch, page 1
    ("copies", (2, 1), (10, 1)),     # ... which is the third of its four dispatches
    ("copies", (1, 4), (4, 4)),      # stale page under the appended row: lane 1's first copy
])
def test_a_stale_page_is_reported_for_the_dispatch_that_meets_it(hip, idiom, corrupt, expected):
    indices = []
    for fused in (True, False):
        hip.fusion_enable(fused)
        batch = LaneBatch(hip, [33, 70, 50, 5], 8, 4, 16, seed=74, corrupt=corrupt)
        commands = CommandList()
        attended, rows = batch.record_layer(commands, 0, idiom=idiom)
        with pytest.raises(BackendError) as info:
            run(hip, commands)
        assert info.value.status == Status.DEVICE_ERROR_FLAG
        indices.append((info.value.dispatch, info.value.index))
    hip.fusion_enable(True)
    assert indices[0] == indices[1] == expected


def test_runs_that_cannot_be_proved_independent_are_executed_serially(cpu, hip):
    """Lane rows that overlap each other, and an output row inside the packed q allocation: the
    list is valid dispatch by dispatch, so it runs, but not fused."""
    contexts = [20, 45, 9]
    results = []
    for backend in (cpu, hip):
        before = hip.fusion_stats()
        batch = LaneBatch(backend, contexts, 8, 4, 16, seed=75)
        commands = CommandList()
        scale = 1.0 / math.sqrt(WIDTH)
        shared = backend.alloc(DType.BF16, (1, 8, WIDTH))     # every lane writes the same row
        keys, values = batch.pools[0]
        for lane in range(3):
            commands.dispatch_many(
                Op.paged_sdpa_append(scale, contexts[lane], 16),
                [batch.q.narrow(0, lane, 1).permute([1, 0, 2]), batch.k.narrow(0, lane, 1),
                 batch.v.narrow(0, lane, 1), batch.tables[lane], batch.generations],
                [shared.permute([1, 0, 2]), keys, values])
        run(backend, commands)
        results.append([shared, keys, values])
        if backend is hip:
            assert hip.fusion_stats() == before
    check(cpu, hip, results[0], results[1], exact=(1, 2))


@pytest.mark.parametrize("idiom", ["append", "copies"])
@pytest.mark.parametrize("case", ["reader_first", "writer_first", "same_slot"])
def test_tables_that_share_a_tail_page_run_dispatch_by_dispatch(cpu, hip, case, idiom):
    """Two lanes whose tables name the same physical tail page: the slot one lane appends lies in
    the range the other attends (or is the very slot the other appends), so the order of the
    dispatches decides what each lane sees.  Nothing in the tensors shows it; the library finds it
    on the device, in the tables, and executes that run one dispatch at a time: the result is the
    oracle's serial result, pools included, and a batch without the overlap is fused as before."""
    pt = 16
    contexts = {"reader_first": [25, 21, 40], "writer_first": [21, 25, 40], "same_slot": [21, 21, 40]}[case]
    results = []
    for backend in (cpu, hip):
        batch = LaneBatch(backend, contexts, 8, 4, pt, seed=91)
        # lane 1's tail (logical page 1) becomes the physical page that is lane 0's tail
        table = batch.host_tables[1].copy()
        table[1] = batch.host_tables[0][1]
        backend.write(batch.tables[1], table.tobytes())
        before = hip.fusion_stats()
        commands = CommandList()
        attended, rows = batch.record_layer(commands, 0, idiom=idiom)
        run(backend, commands)
        if backend is hip:
            assert hip.fusion_stats() == before          # not fused
        results.append([attended, *rows, *batch.pools[0]])
    pools = (len(results[0]) - 2, len(results[0]) - 1)
    check(cpu, hip, results[0], results[1], exact=pools)
    # the same shapes without the shared page are fused
    batch = LaneBatch(hip, contexts, 8, 4, pt, seed=91)
    before = hip.fusion_stats()
    commands = CommandList()
    batch.record_layer(commands, 0, idiom=idiom)
    run(hip, commands)
    assert hip.fusion_stats()[0] == before[0] + 1


def _random_scenario(rng):
    """A decode batch recorded with random deviations from the regular pattern; every list is
    valid dispatch by dispatch, only some of it can be fused."""
    lanes = int(rng.integers(2, 10))
    return dict(
        contexts=[int(c) for c in rng.integers(0, 200, lanes)],
        hq=int(rng.choice([4, 8, 16])), hkv=int(rng.choice([2, 4])),
        idiom=str(rng.choice(["append", "copies"])),
        copy_rows=bool(rng.integers(0, 2)),
        activity=[int(a) for a in (rng.random(lanes) > 0.2)] if rng.integers(0, 2) else None,
        order=[int(l) for l in (rng.permutation(lanes) if rng.integers(0, 3) == 0 else np.arange(lanes))],
        repeat=bool(rng.integers(0, 4) == 0),          # one lane recorded twice in a row
        shared_row=bool(rng.integers(0, 4) == 0),      # two lanes write the same output row
        f32_rows=bool(rng.integers(0, 4) == 0),        # outputs in another dtype than q
        interloper=bool(rng.integers(0, 3) == 0))      # an unrelated dispatch in the middle


def _record_scenario(backend, scenario, seed):
    batch = LaneBatch(backend, scenario["contexts"], scenario["hq"], scenario["hkv"], 16, seed,
                      activity=scenario["activity"])
    hq, scale = scenario["hq"], 1.0 / math.sqrt(WIDTH)
    row_dtype = DType.F32 if scenario["f32_rows"] else DType.BF16
    attended = backend.alloc(row_dtype, (batch.lanes, hq * WIDTH))
    other = backend.alloc(DType.BF16, (4, 4))
    keys, values = batch.pools[0]
    commands = CommandList()
    rows = {}
    order = list(scenario["order"])
    if scenario["repeat"]:
        order.insert(1, order[0])
    for position, lane in enumerate(order):
        if scenario["shared_row"] and position == 1 and 0 in rows:
            row = rows[0]
        else:
            row = backend.alloc(row_dtype, (1, hq, WIDTH))
        rows[position] = row
        start = scenario["contexts"][lane]
        inputs = [batch.q.narrow(0, lane, 1).permute([1, 0, 2]), batch.k.narrow(0, lane, 1),
                  batch.v.narrow(0, lane, 1), batch.tables[lane], batch.generations]
        if batch.activity is not None:
            inputs.append(batch.activity.narrow(0, lane, 1))
        if scenario["idiom"] == "append":
            commands.dispatch_many(Op.paged_sdpa_append(scale, start, 16), inputs,
                                   [row.permute([1, 0, 2]), keys, values])
        else:
            physical, elements = keys.shape[0], scenario["hkv"] * WIDTH
            for new_row, pool in ((inputs[1], keys), (inputs[2], values)):
                commands.dispatch(Op.paged_copy(INTO_PAGES, start, 16),
                                  [new_row.reshape((1, elements)), *inputs[3:]],
                                  pool.reshape((physical, 16, elements)))
            commands.dispatch(Op.paged_sdpa(scale, True, start, start + 1, 16),
                              [inputs[0], keys, values, *inputs[3:]], row.permute([1, 0, 2]))
        if scenario["copy_rows"]:
            commands.dispatch(Op.copy(), [row.reshape((1, hq * WIDTH))], attended.narrow(0, lane, 1))
        if scenario["interloper"] and position == len(order) // 2:
            commands.dispatch(Op.copy(), [other], backend.alloc(DType.BF16, (4, 4)))
    return commands, [attended, keys, values] + [rows[p] for p in sorted(rows)]


@pytest.mark.parametrize("seed", range(24))
def test_random_recordings_give_the_same_result_fused_and_dispatch_by_dispatch(cpu, hip, seed):
    """Random lane orders, repeated lanes, shared output rows, other output dtypes and foreign
    dispatches in the middle: whatever part of the list the library fuses, pools are bit for bit
    what its own serial execution leaves and rows agree to the float bar; the first eight seeds
    are also held to the oracle."""
    scenario = _random_scenario(np.random.default_rng(1000 + seed))
    results = {}
    for name, backend in (("fused", hip), ("serial", hip)) + ((("cpu", cpu),) if seed < 8 else ()):
        if backend is hip:
            hip.fusion_enable(name == "fused")
        commands, tensors = _record_scenario(backend, scenario, 200 + seed)
        before = hip.fusion_stats()[0]
        run(backend, commands)
        results[name] = tensors
        regular = scenario["order"] == sorted(scenario["order"]) and not scenario["repeat"] \
            and not scenario["shared_row"]
        if name == "fused" and regular:
            assert hip.fusion_stats()[0] > before
    hip.fusion_enable(True)
    check(hip, hip, results["serial"], results["fused"], exact=(1, 2), bar=DType.BF16)
    if "cpu" in results:
        check(cpu, hip, results["cpu"], results["fused"], exact=(1, 2), bar=DType.BF16)


# ---- runs that bring prefill chunks (a sequence's chunk recorded on its own: cache.append, then
# cache.attention over its rows, engines/qwen3-coder/src/lib.rs:685-707) ----

class ChunkBatch:
    """A packed batch of members (start, rows): rows > 1 is a prefill chunk, rows == 1 a decode row.
    `share` = (a, b, pages): member b's first `pages` table entries name member a's physical pages
    (a common prompt prefix, read only)."""

    def __init__(self, backend, members, hq, hkv, pt, seed, layers=1, share=None, corrupt=None,
                 activity=None):
        self.backend, self.members, self.hq, self.hkv, self.pt = backend, list(members), hq, hkv, pt
        pages_needed = [(start + rows + pt - 1) // pt for start, rows in members]
        self.table_pages = max(pages_needed) + 2
        physical = sum(pages_needed) + 3
        rng = np.random.default_rng(seed)
        free = list(rng.permutation(physical))
        self.tables, self.host_tables = [], []
        for index, need in enumerate(pages_needed):
            table = np.zeros((self.table_pages, 2), np.uint32)
            table[:, 1] = 0xffffffff
            for logical in range(need):
                page = free.pop()
                table[logical] = (page, 11 + page)
            self.host_tables.append(table)
        if share is not None:
            a, b, pages = share
            self.host_tables[b][:pages] = self.host_tables[a][:pages]
        if corrupt is not None:
            self.host_tables[corrupt[0]][corrupt[1], 1] += 1
        self.tables = [upload(backend, table, DType.U32) for table in self.host_tables]
        self.generations = upload(backend, 11 + np.arange(physical), DType.U32)
        self.activity = None if activity is None else upload(backend, np.array(activity), DType.U32)
        self.tokens = sum(rows for _, rows in members)
        self.q = upload(backend, normal_bf16(seed, 3, (self.tokens, hq, WIDTH)), DType.BF16)
        self.k = upload(backend, normal_bf16(seed, 4, (self.tokens, hkv, WIDTH)), DType.BF16)
        self.v = upload(backend, normal_bf16(seed, 5, (self.tokens, hkv, WIDTH)), DType.BF16)
        self.pools = []
        for layer in range(layers):
            keys = upload(backend, normal_bf16(seed, 10 + 2 * layer, (physical, pt, hkv, WIDTH)), DType.BF16)
            values = upload(backend, normal_bf16(seed, 11 + 2 * layer, (physical, pt, hkv, WIDTH)), DType.BF16)
            self.pools.append((keys, values))

    def record_layer(self, commands, layer, copy_rows=True, decode_idiom="append"):
        backend, hq, hkv, pt = self.backend, self.hq, self.hkv, self.pt
        scale = 1.0 / math.sqrt(WIDTH)
        attended = backend.alloc(DType.BF16, (self.tokens, hq * WIDTH))
        keys, values = self.pools[layer]
        physical, elements = keys.shape[0], hkv * WIDTH
        outs, first = [], 0
        for index, (start, rows) in enumerate(self.members):
            paging = [self.tables[index], self.generations]
            if self.activity is not None:
                paging.append(self.activity.narrow(0, index, 1))
            q = self.q.narrow(0, first, rows).permute([1, 0, 2])
            k_rows, v_rows = self.k.narrow(0, first, rows), self.v.narrow(0, first, rows)
            if rows == 1 and decode_idiom == "append":
                out = backend.alloc(DType.BF16, (1, hq, WIDTH))
                commands.dispatch_many(Op.paged_sdpa_append(scale, start, pt), [q, k_rows, v_rows, *paging],
                                       [out.permute([1, 0, 2]), keys, values])
                if copy_rows:
                    commands.dispatch(Op.copy(), [out.reshape((1, hq * WIDTH))], attended.narrow(0, first, 1))
            else:
                out = backend.alloc(DType.BF16, (hq, rows, WIDTH))
                for new_rows, pool in ((k_rows, keys), (v_rows, values)):
                    commands.dispatch(Op.paged_copy(INTO_PAGES, start, pt),
                                      [new_rows.reshape((rows, elements)), *paging],
                                      pool.reshape((physical, pt, elements)))
                commands.dispatch(Op.paged_sdpa(scale, True, start, start + rows, pt),
                                  [q, keys, values, *paging], out)
                if copy_rows:
                    commands.dispatch(Op.copy(), [out.permute([1, 0, 2])],
                                      attended.narrow(0, first, rows).reshape((rows, hq, WIDTH)))
            outs.append(out)
            first += rows
        return attended, outs


CHUNK_CASES = [
    # members (start, rows), hq, hkv, page_tokens, share (a, b, pages), dispatches per layer when copies follow
    ([(48, 37), (130, 1), (0, 20), (77, 1)], 8, 4, 16, (0, 1, 3), "append"),
    ([(48, 37), (130, 1), (0, 20), (77, 1)], 8, 4, 16, (0, 1, 3), "copies"),
    ([(0, 300), (64, 129)], 32, 4, 64, None, "append"),                      # chunks only, engine page size
    ([(5, 1), (9, 1), (16, 16), (31, 2), (200, 1)], 16, 2, 16, (2, 4, 1), "append"),
]


@pytest.mark.parametrize("copy_rows", [True, False])
@pytest.mark.parametrize("members,hq,hkv,pt,share,decode_idiom", CHUNK_CASES)
def test_chunks_recorded_per_sequence_run_as_one_ragged_launch(cpu, hip, members, hq, hkv, pt, share,
                                                                decode_idiom, copy_rows):
    """Prefill chunks and decode rows of different sequences, each recorded on its own, two layers
    on the same members: one fused launch per layer on the device, serial on the oracle and in the
    library's own dispatch-by-dispatch execution; pools bit for bit, rows to the float bar."""
    outputs = {}
    for name, backend in (("cpu", cpu), ("fused", hip), ("serial", hip)):
        if backend is hip:
            hip.fusion_enable(name == "fused")
        before = hip.fusion_stats()
        batch = ChunkBatch(backend, members, hq, hkv, pt, seed=171, layers=2, share=share)
        commands = CommandList()
        kept, pools = [], []
        for layer in range(2):
            attended, outs = batch.record_layer(commands, layer, copy_rows=copy_rows, decode_idiom=decode_idiom)
            kept += [attended, *outs] if copy_rows else list(outs)
            pools += [len(kept), len(kept) + 1]
            kept += list(batch.pools[layer])
        recorded = len(commands.dispatches)
        run(backend, commands)
        outputs[name] = kept
        runs, dispatches = (after - start for after, start in zip(hip.fusion_stats(), before))
        assert (runs, dispatches) == ((2, recorded) if name == "fused" else (0, 0))
    hip.fusion_enable(True)
    check(cpu, hip, outputs["cpu"], outputs["fused"], exact=pools)
    check(cpu, hip, outputs["cpu"], outputs["serial"], exact=pools)
    check(hip, hip, outputs["serial"], outputs["fused"], exact=pools)


@pytest.mark.parametrize("case", ["chunk_into_attended_page", "row_into_chunk_page"])
def test_a_chunk_stored_into_a_page_another_member_attends_runs_dispatch_by_dispatch(cpu, hip, case):
    """Two members whose tables name one physical page where one stores rows and the other attends:
    found on the device, executed one dispatch at a time, equal to the oracle's serial result."""
    pt = 16
    members = {"chunk_into_attended_page": [(16, 20), (40, 1)],     # the chunk stores into logical page 1, which the row attends
               "row_into_chunk_page": [(40, 1), (30, 12)]}[case]    # the row's slot lies in a page the chunk attends
    results = []
    for backend in (cpu, hip):
        batch = ChunkBatch(backend, members, 8, 4, pt, seed=173)
        if case == "chunk_into_attended_page":
            batch.host_tables[1][1] = batch.host_tables[0][1]
            backend.write(batch.tables[1], batch.host_tables[1].tobytes())
        else:
            batch.host_tables[1][2] = batch.host_tables[0][2]
            backend.write(batch.tables[1], batch.host_tables[1].tobytes())
        before = hip.fusion_stats()
        commands = CommandList()
        attended, outs = batch.record_layer(commands, 0)
        run(backend, commands)
        if backend is hip:
            assert hip.fusion_stats() == before
        results.append([attended, *outs, *batch.pools[0]])
    pools = (len(results[0]) - 2, len(results[0]) - 1)
    check(cpu, hip, results[0], results[1], exact=pools)


@pytest.mark.parametrize("corrupt,expected", [
    ((0, 1), (2, 1)),     # stale history page of the first chunk: its attention dispatch, page 1
    ((2, 0), (6, 0)),     # stale page under the second chunk's rows: that chunk's first copy
    ((1, 2), (4, 2)),     # stale page under the decode row: its append
])
def test_a_chunk_run_reports_a_stale_page_for_the_dispatch_that_meets_it(hip, corrupt, expected):
    indices = []
    for fused in (True, False):
        hip.fusion_enable(fused)
        batch = ChunkBatch(hip, [(32, 9), (40, 1), (0, 14)], 8, 4, 16, seed=174, corrupt=corrupt)
        commands = CommandList()
        batch.record_layer(commands, 0)
        with pytest.raises(BackendError) as info:
            run(hip, commands)
        assert info.value.status == Status.DEVICE_ERROR_FLAG
        indices.append((info.value.dispatch, info.value.index))
    hip.fusion_enable(True)
    assert indices[0] == indices[1] == expected


def test_chunk_runs_with_inactive_members(cpu, hip):
    results = []
    for backend in (cpu, hip):
        before = hip.fusion_stats()
        batch = ChunkBatch(backend, [(20, 18), (33, 1), (0, 7), (64, 5)], 8, 4, 16, seed=175,
                           activity=[1, 0, 0, 1])
        commands = CommandList()
        attended, outs = batch.record_layer(commands, 0, decode_idiom="copies")
        run(backend, commands)
        results.append([attended, *outs, *batch.pools[0]])
        if backend is hip:
            assert hip.fusion_stats()[0] - before[0] == 1
    pools = (len(results[0]) - 2, len(results[0]) - 1)
    check(cpu, hip, results[0], results[1], exact=pools)


@pytest.mark.parametrize("seed", range(12))
def test_random_chunk_recordings_give_the_same_result_fused_and_dispatch_by_dispatch(cpu, hip, seed):
    """Random mixes of chunks and decode rows, with and without the row copies, inactive members and
    shared prefix pages: pools bit for bit what serial execution leaves, rows to the float bar; the
    first four seeds are also held to the oracle."""
    rng = np.random.default_rng(3000 + seed)
    count = int(rng.integers(2, 7))
    members = []
    for _ in range(count):
        rows = 1 if rng.integers(0, 2) else int(rng.integers(2, 50))
        members.append((int(rng.integers(0, 150)), rows))
    if all(rows == 1 for _, rows in members):
        members[0] = (members[0][0], 9)
    options = dict(hq=int(rng.choice([4, 8, 16])), hkv=int(rng.choice([2, 4])),
                   activity=[int(a) for a in (rng.random(count) > 0.25)] if rng.integers(0, 2) else None,
                   copy_rows=bool(rng.integers(0, 2)), idiom=str(rng.choice(["append", "copies"])))
    share = None
    if count >= 2 and rng.integers(0, 2):
        a, b = (int(v) for v in rng.choice(count, 2, replace=False))
        pages = min(members[a][0], members[b][0]) // 16     # whole pages of history both have
        share = (a, b, pages) if pages else None
    results = {}
    for name, backend in (("fused", hip), ("serial", hip)) + ((("cpu", cpu),) if seed < 4 else ()):
        if backend is hip:
            hip.fusion_enable(name == "fused")
        batch = ChunkBatch(backend, members, options["hq"], options["hkv"], 16, seed=300 + seed,
                           share=share, activity=options["activity"])
        commands = CommandList()
        before = hip.fusion_stats()[0]
        attended, outs = batch.record_layer(commands, 0, copy_rows=options["copy_rows"],
                                            decode_idiom=options["idiom"])
        run(backend, commands)
        results[name] = [*batch.pools[0], attended, *outs] if options["copy_rows"] else [*batch.pools[0], *outs]
        if name == "fused":
            assert hip.fusion_stats()[0] == before + 1
    hip.fusion_enable(True)
    check(hip, hip, results["serial"], results["fused"], exact=(0, 1))
    if "cpu" in results:
        check(cpu, hip, results["cpu"], results["fused"], exact=(0, 1))
