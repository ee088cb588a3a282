"""Op::Sample / Op::SampleMasked on the device against the CPU oracle on identical logits,
parameters and masks: the sampled indices must be the same, row for row.  The oracle's sampling is
pinned by the reference's own tests in tests/test_oracle_golden.py; exp and ln are evaluated the
same way on both sides (f64, rounded once), so nothing here is left to libm rounding."""
import numpy as np
import pytest

from forja_amd.core import BackendError, CommandList, DType, Op, Status
from oracle import cpu_backend as orc
from tests.helpers import normal_bf16, upload

pytestmark = pytest.mark.gpu


def run(backend, commands):
    backend.submit(commands).wait()


def logits_case(rows, width, seed, kind):
    values = normal_bf16(seed, 1, (rows, width)) * 3.0
    if kind == "ties":                      # a handful of distinct values: every cut lands in a tie
        values = np.round(values)
    if kind == "specials":
        rng = np.random.default_rng(seed)
        for special in (np.inf, -np.inf, np.nan, -np.nan):
            values[rng.integers(0, rows, 6), rng.integers(0, width, 6)] = special
    return values.astype(np.float32)


def sample_both(cpu, hip, values, words, position, dtype=DType.BF16, allow=None):
    results = []
    for backend in (cpu, hip):
        logits = upload(backend, values, dtype)
        params = upload(backend, words, DType.U32)
        out = backend.alloc(DType.U32, (values.shape[0],))
        commands = CommandList()
        if allow is None:
            commands.dispatch(Op.sample(position), [logits, params], out)
        else:
            commands.dispatch(Op.sample_masked(position),
                              [logits, params, upload(backend, allow, DType.U32)], out)
        run(backend, commands)
        results.append(np.frombuffer(backend.read(out), np.uint32).copy())
    return results


PARAMETERS = [
    (0.0, 0, 1.0),        # greedy by temperature
    (1.3, 1, 0.4),        # greedy by top_k
    (0.7, 0, 1.0),        # every column competes
    (1.0, 20, 0.8),       # the usual serving setting: few candidates, nucleus cut
    (1.0, 64, 1.0),
    (0.9, 256, 0.95),     # the largest extracted set
    (0.9, 257, 0.95),     # just past it: ordered through the radix passes
    (0.8, 1000, 0.9),
    (1.0, 0, 0.9),        # nucleus cut over the whole row
    (2.0, 5000, 1.0),     # top_k beyond the row for the narrow cases
]


@pytest.mark.parametrize("rows,width,kind", [(5, 7, "plain"), (3, 1025, "ties"), (4, 4097, "specials"),
                                              (8, 151936, "plain"), (2, 151936, "ties"),
                                              (300, 333, "ties")])    # more rows than workgroups
def test_sampled_indices_equal_the_oracle(cpu, hip, rows, width, kind):
    values = logits_case(rows, width, 101, kind)
    for number, (temperature, top_k, top_p) in enumerate(PARAMETERS):
        words = orc.sampling_words(temperature, top_k, top_p, 0xfeedbeefdeadcafe + number)
        for position in (0, 4097):
            expected, actual = sample_both(cpu, hip, values, words, position)
            assert expected.tolist() == actual.tolist(), (temperature, top_k, top_p, position)


@pytest.mark.parametrize("width", [7, 70, 4100])
def test_masked_sampling_equals_the_oracle_and_stays_inside_the_mask(cpu, hip, width):
    rows = 6
    values = logits_case(rows, width, 102, "ties")
    rng = np.random.default_rng(width)
    words_in_mask = (width + 31) // 32
    masks = [rng.integers(0, 2 ** 32, words_in_mask, dtype=np.uint64).astype(np.uint32),
             np.zeros(words_in_mask, np.uint32), np.full(words_in_mask, 0xffffffff, np.uint32)]
    masks[1][words_in_mask // 2] = 1 << 3                      # a single allowed column
    for mask in masks:
        if width % 32:
            mask[-1] &= (1 << (width % 32)) - 1
        for temperature, top_k, top_p in PARAMETERS:
            words = orc.sampling_words(temperature, top_k, top_p, 77)
            expected, actual = sample_both(cpu, hip, values, words, 3, allow=mask)
            assert expected.tolist() == actual.tolist(), (temperature, top_k, top_p)
            for index in actual:
                assert (int(mask[index // 32]) >> (index % 32)) & 1
    full = np.full(words_in_mask, 0xffffffff, np.uint32)
    if width % 32:
        full[-1] &= (1 << (width % 32)) - 1
    words = orc.sampling_words(0.7, 7, 0.9, 0xfeedbeef)
    assert sample_both(cpu, hip, values, words, 9, allow=full)[1].tolist() == \
        sample_both(cpu, hip, values, words, 9)[1].tolist()


def test_f32_f16_and_strided_rows_and_a_single_row(cpu, hip):
    values = logits_case(4, 300, 103, "plain")
    words = orc.sampling_words(0.9, 40, 0.9, 5)
    for dtype in (DType.F32, DType.F16):
        expected, actual = sample_both(cpu, hip, values, words, 1, dtype=dtype)
        assert expected.tolist() == actual.tolist()
    results = []
    for backend in (cpu, hip):
        stored = upload(backend, values.T.copy(), DType.F32)             # [300, 4]: columns are rows
        params = upload(backend, words, DType.U32)
        out = backend.alloc(DType.U32, (4,))
        single = backend.alloc(DType.U32, ())
        commands = CommandList()
        commands.dispatch(Op.sample(2), [stored.permute([1, 0]), params], out)
        commands.dispatch(Op.sample(2), [upload(backend, values[1], DType.F32), params], single)
        run(backend, commands)
        results.append((backend.read(out), backend.read(single)))
    assert results[0] == results[1]
    assert np.frombuffer(results[1][0], np.uint32)[1] == np.frombuffer(results[1][1], np.uint32)[0]


def test_distribution_on_the_device_matches_the_known_probabilities(hip):
    """The reference's chi-squared check (crates/forja-cpu/src/lib.rs:3283-3306) on the device:
    20000 positions of the 4-way case with top_k 3 and top_p 0.95."""
    row = np.array([[2.0, 1.0, 0.0, -1.0]], dtype=np.float32)
    expected = np.array([0.66524094, 0.24472848, 0.09003057, 0.0])
    logits = upload(hip, row, DType.F32)
    params = upload(hip, orc.sampling_words(1.0, 3, 0.95, 94), DType.U32)
    trials = 20_000
    out = hip.alloc(DType.U32, (trials,))
    commands = CommandList()
    for position in range(trials):
        commands.dispatch(Op.sample(position), [logits, params], out.narrow(0, position, 1))
    run(hip, commands)
    counts = np.bincount(np.frombuffer(hip.read(out), np.uint32), minlength=4)
    live = expected > 0
    statistic = (((counts - expected * trials) ** 2)[live] / (expected * trials)[live]).sum()
    assert statistic < 16.3 and counts[3] == 0


def test_refused_live_parameters_and_masks_are_invalid_input(cpu, hip):
    values = np.zeros((2, 7), dtype=np.float32)
    bad_words = [np.array([np.float32("nan").view(np.uint32), 0, np.float32(1).view(np.uint32), 0, 0],
                          dtype=np.uint32),
                 orc.sampling_words(-1.0, 0, 1.0, 0), orc.sampling_words(1.0, 0, 0.0, 0),
                 orc.sampling_words(1.0, 0, 1.5, 0), orc.sampling_words(float("inf"), 0, 1.0, 0)]
    for words in bad_words:
        for backend in (cpu, hip):
            with pytest.raises(BackendError) as info:
                sample_both(backend, backend, values, words, 0)
            assert info.value.status == Status.INVALID_INPUT
    good = orc.sampling_words(1.0, 0, 1.0, 0)
    for mask in ([0], [1 << 7]):
        for backend in (cpu, hip):
            with pytest.raises(BackendError) as info:
                sample_both(backend, backend, values, good, 0, allow=np.array(mask, dtype=np.uint32))
            assert info.value.status == Status.INVALID_INPUT
    assert sample_both(cpu, hip, values, good, 0, allow=np.array([1 << 6], dtype=np.uint32))[1].tolist() == [6, 6]


def test_sample_signatures_are_checked_at_submission(hip):
    logits = hip.alloc(DType.BF16, (2, 40))
    params = hip.alloc(DType.U32, (5,))
    out = hip.alloc(DType.U32, (2,))
    for inputs, output in (([logits, hip.alloc(DType.U32, (4,))], out),
                           ([logits, hip.alloc(DType.F32, (5,))], out),
                           ([hip.alloc(DType.U32, (2, 40)), params], out),
                           ([logits, params], hip.alloc(DType.U32, (3,))),
                           ([logits, params], hip.alloc(DType.F32, (2,)))):
        commands = CommandList()
        commands.dispatch(Op.sample(0), inputs, output)
        with pytest.raises(BackendError) as info:
            hip.submit(commands)
        assert info.value.status == Status.INVALID_INPUT
    commands = CommandList()
    commands.dispatch(Op.sample_masked(0), [logits, params, hip.alloc(DType.U32, (1,))], out)
    with pytest.raises(BackendError):
        hip.submit(commands)                                   # 40 columns need two mask words
