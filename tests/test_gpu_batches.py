"""Submission and completion of batches through the C ABI: the callback form of commit
(metal-compute/src/apple.rs:2202-2233: `on_done(Completed)` once the GPU has finished, buffers handed
back) and batches recorded on several threads at once, whose split-K dispatches share the library's
scratch buffers and must not interleave on the device."""
import threading

import numpy as np
import pytest

from loadngo_amd import compute as C
from oracle import oracle as orc
from tests.gpu_common import THREADS, gpu  # noqa: F401
from tests.helpers import from_bf16_bits, normal_inputs, to_bf16_bits

pytestmark = pytest.mark.gpu
H, G, D = 64, 8, 64


def _decode_case(seed, end):
    q, k, v, sinks = normal_inputs(seed, 1, end, H, G, D, 0.5)
    qb, kb, vb = to_bf16_bits(q), to_bf16_bits(k), to_bf16_bits(v)
    want = orc.attention_f32(from_bf16_bits(qb), from_bf16_bits(kb), from_bf16_bits(vb), sinks, end - 1,
                             threads=THREADS)
    return qb, kb, vb, sinks, want


def _record(gpu, bufs, end):
    batch = gpu.batch(bufs)
    shape = C.GroupedShape(1, end - 1, H, G, D, C.FULL, end, 0.125)
    batch.attention_grouped_with_sinks((C.Slice(0, 0, H * D * 2), C.Slice(1, 0, end * G * D * 2),
                                        C.Slice(2, 0, end * G * D * 2)), C.Slice(4, 0, H * 4),
                                       C.Slice(3, 0, H * D * 2), shape, C.BF16)
    return batch


def test_commit_with_a_callback_hands_back_the_buffers_and_the_gpu_time(gpu):
    end = 3000
    qb, kb, vb, sinks, want = _decode_case(1, end)
    bufs = [gpu.upload(qb), gpu.upload(kb), gpu.upload(vb), gpu.buffer(H * D * 2), gpu.upload(sinks)]
    batch = _record(gpu, bufs, end)
    seen, fired = [], threading.Event()

    def on_done(done):
        seen.append(done)
        fired.set()

    batch.commit(on_done)
    with pytest.raises(C.Dispatch):        # committed: nothing more can be recorded
        batch.barrier()
    assert fired.wait(30), "the completion callback never ran"
    done = batch.wait()                    # returns at once: the batch has finished
    assert len(seen) == 1 and seen[0].buffers == bufs
    assert isinstance(seen[0].gpu_time, float) and 0 < seen[0].gpu_time < 1.0
    assert isinstance(done.gpu_time, float)
    got = from_bf16_bits(bufs[3].read(np.uint16)).reshape(1, H, D)   # readable again: the buffers are back
    assert np.abs(got - want).max() <= 2e-2
    batch.drop()
    for b in bufs:
        b.free()


def test_batches_recorded_and_committed_on_several_threads_at_once(gpu):
    """Each thread runs its own split-K decodes (every dispatch uses the library's shared partials
    and arrival counters) and must get its own answer every time."""
    cases = [_decode_case(10 + i, 20000 + 3000 * i) for i in range(4)]
    errors, lock = [], threading.Lock()

    def work(i):
        try:
            qb, kb, vb, sinks, want = cases[i]
            end = kb.shape[0]
            bufs = [gpu.upload(qb), gpu.upload(kb), gpu.upload(vb), gpu.buffer(H * D * 2), gpu.upload(sinks)]
            for _ in range(25):
                bufs[3].fill(0xFF)
                batch = _record(gpu, bufs, end)
                done = batch.run()
                batch.drop()
                assert not isinstance(done.gpu_time, Exception), done.gpu_time
                got = from_bf16_bits(bufs[3].read(np.uint16)).reshape(1, H, D)
                err = np.abs(got - want).max()
                assert err <= 2e-2, f"thread {i}: {err}"
            for b in bufs:
                b.free()
        except Exception as e:  # noqa: BLE001 - reported to the main thread
            with lock:
                errors.append(repr(e))

    threads = [threading.Thread(target=work, args=(i,)) for i in range(4)]
    for t in threads:
        t.start()
    for t in threads:
        t.join(120)
    assert not errors, errors
