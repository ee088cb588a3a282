"""The boundary as the host really drives it (crates/forja-host/src/lib.rs:8805-8925): one backend
shared by several worker threads that allocate, write, submit, wait and read concurrently, and
`Submission::wait_timeout` (crates/forja-core/src/backend.rs:609-647) per submission."""
import threading

import numpy as np
import pytest

from forja_amd.core import BackendError, CommandList, DType, Op, Status
from tests.helpers import Quantised, assert_close, normal_bf16, to_f32, upload

pytestmark = pytest.mark.gpu


def test_four_host_threads_share_one_backend(cpu, hip):
    """ctypes releases the interpreter lock around every call into the library, so the four
    threads are inside fh_alloc / fh_write / fh_submit / fh_wait / fh_read_tensor at the same
    time.  Every thread's products must equal the oracle's for its own operands."""
    rounds, failures = 12, []

    def products(backend, seed, rows):
        weights = Quantised(seed, 1, (96, 256))
        x = upload(backend, normal_bf16(seed, 2, (rows, 256)), DType.BF16)
        out = backend.alloc(DType.BF16, (rows, 96))
        top_values, top_indices = backend.alloc(DType.BF16, (rows, 4)), backend.alloc(DType.U32, (rows, 4))
        commands = CommandList()
        commands.dispatch(Op.quant_matmul(4, 64), [x, *weights.upload(backend)], out)
        commands.dispatch_many(Op.top_k(4, True), [out], [top_values, top_indices])
        backend.submit(commands).wait()
        return backend.read(out), backend.read(top_indices)

    expected = {(worker, r): products(cpu, 100 * worker + r, 1 + (worker + r) % 9)
                for worker in range(4) for r in range(rounds)}
    barrier = threading.Barrier(4)

    def work(worker):
        try:
            barrier.wait()
            for r in range(rounds):
                out, indices = products(hip, 100 * worker + r, 1 + (worker + r) % 9)
                reference, reference_indices = expected[(worker, r)]
                assert_close(to_f32(out, DType.BF16), to_f32(reference, DType.BF16), DType.BF16)
                same = np.frombuffer(indices, np.uint32) == np.frombuffer(reference_indices, np.uint32)
                assert same.mean() > 0.9
        except BaseException as error:      # reported by the main thread
            failures.append((worker, repr(error)))

    threads = [threading.Thread(target=work, args=(worker,)) for worker in range(4)]
    for thread in threads:
        thread.start()
    for thread in threads:
        thread.join(timeout=120)
    assert not any(thread.is_alive() for thread in threads)
    assert not failures, failures


def long_running(hip, launches):
    """Ordinary long work: row-wise argmax over 1 GiB, `launches` times in one submission."""
    source = hip.alloc(DType.BF16, (2048, 1 << 18))
    result = hip.alloc(DType.U32, (2048,))
    commands = CommandList()
    for _ in range(launches):
        commands.dispatch(Op.argmax(), [source], result)
    return commands, (source, result)


def test_wait_timeout_returns_and_a_later_wait_succeeds(hip):
    commands, tensors = long_running(hip, 200)          # tens of milliseconds of device time
    submission = hip.submit(commands)
    with pytest.raises(BackendError) as info:
        submission.wait(timeout_ns=20_000)              # 20 microseconds
    assert info.value.status == Status.TIMEOUT
    submission.wait()                                   # every kernel runs to its end
    assert submission.gpu_time_ns() > 1_000_000
    for tensor in tensors:
        hip.release(tensor)


def test_waiting_is_per_submission(hip):
    """A short submission followed by a long one: waiting on the first with a deadline far shorter
    than the second's run time succeeds, because later work is not part of its completion."""
    weights = Quantised(7, 1, (64, 128))
    x = upload(hip, normal_bf16(7, 2, (4, 128)), DType.BF16)
    out = hip.alloc(DType.BF16, (4, 64))
    short = CommandList()
    short.dispatch(Op.quant_matmul(4, 64), [x, *weights.upload(hip)], out)
    commands, tensors = long_running(hip, 400)
    hip.synchronize()
    first = hip.submit(short)
    second = hip.submit(commands)
    first.wait(timeout_ns=20_000_000)                   # 20 ms; the second runs for longer
    with pytest.raises(BackendError) as info:
        second.wait(timeout_ns=1_000)
    assert info.value.status == Status.TIMEOUT
    second.wait()
    assert second.gpu_time_ns() > 20_000_000
    assert np.frombuffer(hip.read(out), np.uint16).any()
    for tensor in tensors:
        hip.release(tensor)
