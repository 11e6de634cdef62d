"""Submission and completion of batches through the C ABI: the callback form of commit
(metal-compute/src/apple.rs:2202-2233: `on_done(Completed)` once the GPU has finished, buffers handed
back) and batches recorded on several threads at once, whose split-K dispatches share the library's
scratch buffers and must not interleave on the device."""
import threading

import numpy as np
import pytest

from loadngo_amd import compute as C
from oracle import oracle as orc
from tests.gpu_common import THREADS, gpu, knobs  # noqa: F401
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


def test_a_dispatch_of_more_rows_than_one_grid_dimension_holds(gpu):
    """9,000 sequences of 8 kv heads are 72,000 (row, kv head) pairs, past the 65,535 workgroups one grid dimension
    holds: the dispatch is one-dimensional, so it is accepted and every row comes out right (the reference accepts
    any rows x heads that fit u32, apple.rs:1257-1272). Rows of unequal length: the list of live workgroups
    is found through the table of running counts over 9,001 entries (three levels of the 64-way search)."""
    n, ctx = 9000, 20000
    rng = np.random.default_rng(77)
    k = to_bf16_bits((rng.standard_normal((ctx, G, D)) * 0.5).astype(np.float32))
    v = to_bf16_bits((rng.standard_normal((ctx, G, D)) * 0.5).astype(np.float32))
    q = to_bf16_bits((rng.standard_normal((n, H, D)) * 0.5).astype(np.float32))
    sinks = rng.standard_normal(H).astype(np.float32)
    lens = rng.integers(1, 701, size=n)
    lens[[17, 4000, 4001, 8999]] = [ctx, ctx - 1, 13000, 6500]  # a few long rows: these are cut into chunks, the rest are not
    bufs = [gpu.upload(q), gpu.upload(k), gpu.upload(v), gpu.buffer(q.nbytes), gpu.upload(sinks)]
    bufs[3].fill(0xFF)
    items = [C.DecodeItem(i * H * D * 2, i * H * D * 2, 0, 0, 0, int(lens[i]) - 1, C.FULL, int(lens[i])) for i in range(n)]
    batch = gpu.batch(bufs)
    batch.attention_decode_batched(0, 1, 2, 3, 4, items, H, G, D, 0.125, C.BF16)
    done = batch.run()
    assert not isinstance(done.gpu_time, Exception)
    got = from_bf16_bits(bufs[3].read(np.uint16).reshape(q.shape))
    batch.drop()
    for b in bufs:
        b.free()
    assert not np.isnan(got).any()
    for i in list(rng.integers(0, n, 60)) + [0, n - 1, 17, 4000, 4001, 4002, 8999, 8998, int(np.argmin(lens))]:
        want = orc.attention_bf16(q[i:i + 1], k[:lens[i]], v[:lens[i]], sinks, int(lens[i]) - 1, scale=0.125)
        assert np.abs(got[i] - from_bf16_bits(want[0])).max() < 2e-2, (i, lens[i])


def test_a_row_table_read_from_host_memory_and_one_copied_to_the_device_give_the_same_rows(gpu, knobs):
    """A table of 8 KB or more stays in pinned host memory, where the kernels read it; smaller ones are copied to the
    device ahead of the batch. 300 sequences of unequal length (a 19 KB table and its running counts) both ways, and
    with every table left in host memory (LNG_TABLE_IN_PLACE=1): the same bits, and right against the oracle."""
    n, ctx = 300, 6000
    rng = np.random.default_rng(78)
    k = to_bf16_bits((rng.standard_normal((ctx, G, D)) * 0.5).astype(np.float32))
    v = to_bf16_bits((rng.standard_normal((ctx, G, D)) * 0.5).astype(np.float32))
    q = to_bf16_bits((rng.standard_normal((n, H, D)) * 0.5).astype(np.float32))
    sinks = rng.standard_normal(H).astype(np.float32)
    lens = rng.integers(1, ctx + 1, size=n)
    items = [C.DecodeItem(i * H * D * 2, i * H * D * 2, 0, 0, 0, int(lens[i]) - 1, C.FULL if i % 3 else 128, int(lens[i])) for i in range(n)]
    few = items[:40] # a 2.5 KB table: copied unless every table stays
    results = {}
    for mode in (None, "0", "1"):
        if mode is None:
            knobs.delenv("LNG_TABLE_IN_PLACE", raising=False)
        else:
            knobs.setenv("LNG_TABLE_IN_PLACE", mode)
        bufs = [gpu.upload(q), gpu.upload(k), gpu.upload(v), gpu.buffer(2 * q.nbytes), gpu.upload(sinks)]
        bufs[3].fill(0xFF)
        batch = gpu.batch(bufs)
        batch.attention_decode_batched(0, 1, 2, 3, 4, items, H, G, D, 0.125, C.BF16)
        shifted = [C.DecodeItem(it.q_offset, q.nbytes + it.out_offset, it.k_offset, it.v_offset, it.sinks_offset, it.start, it.window, it.slots)
                   for it in few]
        batch.attention_decode_batched(0, 1, 2, 3, 4, shifted, H, G, D, 0.125, C.BF16)
        done = batch.run()
        assert not isinstance(done.gpu_time, Exception)
        results[mode] = bufs[3].read(np.uint16).reshape(2, n, H, D).copy()
        batch.drop()
        for b in bufs:
            b.free()
    got = results[None]
    assert np.array_equal(got, results["0"]) and np.array_equal(got, results["1"])
    rows = from_bf16_bits(got[0])
    assert np.abs(rows[:40] - from_bf16_bits(got[1, :40])).max() < 2e-2  # split differently, so not the same bits
    assert not np.isnan(rows).any()
    for i in list(rng.integers(0, n, 25)) + [0, n - 1]:
        window = None if i % 3 else 128
        want = orc.attention_bf16(q[i:i + 1], k[:lens[i]], v[:lens[i]], sinks, int(lens[i]) - 1, scale=0.125,
                                  **({} if window is None else {"window": window}))
        assert np.abs(rows[i] - from_bf16_bits(want[0])).max() < 2e-2, (i, lens[i])


def test_many_small_decodes_merged_inside_the_kernel(gpu):
    """The split-K merge inside the decode kernel (small grids: the workgroup that finishes last for a (row, kv
    head) reads the other workgroups' partials) rests on an ordering between workgroups on different XCDs, so it
    is exercised many times, not once: 3,000 decodes of one or two rows over fresh queries and fresh stretches of
    a cache, each compared with the CPU reference; stops at the first mismatch."""
    rng = np.random.default_rng(5)
    total = 1 << 16
    k = to_bf16_bits((rng.standard_normal((total, G, D)) * 0.5).astype(np.float32))
    v = to_bf16_bits((rng.standard_normal((total, G, D)) * 0.5).astype(np.float32))
    kf, vf = from_bf16_bits(k), from_bf16_bits(v)
    sinks = rng.standard_normal(H).astype(np.float32)
    bufs = [gpu.buffer(2 * H * D * 2), gpu.upload(k), gpu.upload(v), gpu.buffer(2 * H * D * 2), gpu.upload(sinks)]
    row = G * D * 2
    for it in range(3000):
        t = 1 + (it & 1)
        ctx = int(rng.integers(300, 6000))
        base = int(rng.integers(0, total - ctx))
        q = to_bf16_bits((rng.standard_normal((t, H, D)) * 0.5).astype(np.float32))
        bufs[0].write(q)
        batch = gpu.batch(bufs)
        shape = C.GroupedShape(t, ctx - t, H, G, D, C.FULL, ctx, 0.125)
        batch.attention_grouped_with_sinks((C.Slice(0, 0, q.nbytes), C.Slice(1, base * row, ctx * row),
                                            C.Slice(2, base * row, ctx * row)), C.Slice(4, 0, H * 4),
                                           C.Slice(3, 0, q.nbytes), shape, C.BF16)
        done = batch.run()
        batch.drop()
        assert not isinstance(done.gpu_time, Exception)
        got = from_bf16_bits(bufs[3].read(np.uint16, count=t * H * D).reshape(t, H, D))
        want = orc.attention_f32(from_bf16_bits(q), kf[base:base + ctx], vf[base:base + ctx], sinks, ctx - t,
                                 scale=0.125, threads=THREADS)
        err = np.abs(got - want).max()
        assert err < 2e-2 and not np.isnan(err), (it, t, ctx, base, err)
    for b in bufs:
        b.free()


@pytest.mark.parametrize("dtype,dim,heads,kv_heads", [(C.BF16, 64, 64, 8), (C.F32, 64, 16, 8), (C.BF16, 128, 16, 8)])
def test_a_table_of_many_short_sequences_takes_the_small_merge_and_the_four_wavefront_build(gpu, dtype, dim, heads, kv_heads):
    """160 sequences of 300..2,400 positions in one dispatch: rows of two to seven chunks, several thousand
    workgroups, merged by the second dispatch (lng_decode_merge_few; the per-kernel times say which kernels ran),
    each sequence against the CPU reference on its own cache."""
    n_seq = 160
    rng = np.random.default_rng(160 + dim)
    lens = rng.integers(300, 2401, size=n_seq)
    offs = np.concatenate([[0], np.cumsum(lens)])
    es = 2 if dtype == C.BF16 else 4
    row = kv_heads * dim
    scale = float(1.0 / np.sqrt(np.float32(dim)))
    k_all = rng.standard_normal((int(offs[-1]), kv_heads, dim), dtype=np.float32) * np.float32(0.7)
    v_all = rng.standard_normal((int(offs[-1]), kv_heads, dim), dtype=np.float32)
    q = rng.standard_normal((n_seq, heads, dim), dtype=np.float32) * np.float32(0.7)
    sinks = rng.standard_normal(heads).astype(np.float32)
    if dtype == C.BF16:
        q, k_all, v_all = to_bf16_bits(q), to_bf16_bits(k_all), to_bf16_bits(v_all)
    bufs = [gpu.upload(q), gpu.upload(k_all), gpu.upload(v_all), gpu.buffer(q.size * es), gpu.upload(sinks)]
    bufs[3].fill(0xFF)
    items = [C.DecodeItem(i * heads * dim * es, i * heads * dim * es, int(offs[i]) * row * es, int(offs[i]) * row * es, 0,
                          int(n) - 1, C.FULL, int(n)) for i, n in enumerate(lens)]
    batch = gpu.batch(bufs)
    try:
        batch.set_timing(True)
        batch.attention_decode_batched(0, 1, 2, 3, 4, items, heads, kv_heads, dim, scale, dtype)
        done = batch.run()
        assert not isinstance(done.gpu_time, Exception), done.gpu_time
        assert batch.kernel_seconds("lng_decode_merge_few")[1] == 1
        if dtype == C.BF16 and dim == 64:
            assert batch.kernel_seconds("lng_decode_bf16_d64_o4")[1] == 1
        out = bufs[3].read(np.uint16 if dtype == C.BF16 else np.float32).reshape(n_seq, heads, dim)
    finally:
        batch.drop()
        for b in bufs:
            b.free()
    for i in range(0, n_seq, 7):
        ks, vs = k_all[offs[i]:offs[i + 1]], v_all[offs[i]:offs[i + 1]]
        if dtype == C.BF16:
            want = from_bf16_bits(orc.attention_bf16(q[i:i + 1], ks, vs, sinks, int(lens[i]) - 1, scale=scale, threads=THREADS))
            assert np.abs(from_bf16_bits(out[i:i + 1]) - want).max() < 2e-2, i
        else:
            want = orc.attention_f32(q[i:i + 1], ks, vs, sinks, int(lens[i]) - 1, scale=scale, threads=THREADS)
            err = np.abs(out[i:i + 1].astype(np.float64) - want) / (np.abs(want) + 1.0)
            assert err.max() <= 1e-5, i


def test_buffers_outlive_a_closed_gpu():
    """Closing a gpu whose buffers are still alive leaves them valid to free (they share the device the way the
    reference's buffers share theirs); the device goes with the last of them."""
    g = C.Gpu()
    a, b = g.upload(np.arange(16, dtype=np.float32)), g.buffer(64)
    batch = g.batch([b])
    g.close()
    batch.drop()
    assert np.array_equal(a.read(np.float32), np.arange(16, dtype=np.float32))
    a.free()
    b.free()


@pytest.mark.parametrize("nbytes", [16, 4096 + 16, 1 << 20, (1 << 24) + 48])
def test_checksum_is_the_xor_of_every_16_byte_word(gpu, nbytes):
    """lng_hip_checksum (the plain streaming read the decode kernels are measured beside) against numpy, at sizes of
    one word, a ragged number of words and many workgroups' worth; the slice may start inside its buffer."""
    rng = np.random.default_rng(nbytes)
    data = rng.integers(0, 2**32, size=nbytes // 4 + 8, dtype=np.uint32)
    src, dst = gpu.upload(data), gpu.buffer(64)
    dst.fill(0xFF)
    batch = gpu.batch([src, dst])
    try:
        batch.checksum(C.Slice(0, 32, nbytes), C.Slice(1, 16, 16))
        with pytest.raises(C.Dispatch):
            batch.checksum(C.Slice(0, 32, nbytes - 8), C.Slice(1, 16, 16))  # not whole 16-byte words
        with pytest.raises(C.Dispatch):
            batch.checksum(C.Slice(0, 0, 64), C.Slice(0, 16, 16))           # the sum over its own source
        done = batch.run()
        assert not isinstance(done.gpu_time, Exception), done.gpu_time
        got = dst.read(np.uint32)
    finally:
        batch.drop()
        src.free()
        dst.free()
    want = np.bitwise_xor.reduce(data[8:8 + nbytes // 4].reshape(-1, 4), axis=0)
    assert (got[4:8] == want).all()
    assert (got[:4] == 0xFFFFFFFF).all() and (got[8:] == 0xFFFFFFFF).all()
