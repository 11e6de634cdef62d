"""GPU parity: the HIP operator, called through the C ABI, against the CPU oracle.

Bars: f32 within 1e-5 relative of the CPU reference restatement (and within the reference's
own 2e-5 / 1e-4 of its float64 definition on its own test shapes); bf16 in/out within 2e-2
max-abs of the CPU reference run on the same bf16 inputs."""
import numpy as np
import pytest

from loadngo_amd import compute as C
from oracle import oracle
from tests.gpu_common import THREADS, gpu, knobs, max_error, reference_case, run_attention  # noqa: F401
from tests.helpers import (FULL, REF_GPT_OSS_CASES, REF_PLAIN_CASES, REF_REJECTED, REF_TILED_CASES,
                           from_bf16_bits, normal_inputs, ring_layout, to_bf16_bits)

pytestmark = pytest.mark.gpu

BF16_TOL = 2e-2  # max-abs, bf16 in/out with f32 accumulation
F32_RTOL = 1e-5  # relative, f32 configuration


def rel_error(got, want):
    e = np.abs(got.astype(np.float64) - want) / (np.abs(want) + 1.0)
    return np.inf if np.isnan(e).any() else float(e.max())


# ---- the reference's own operator tests, f32 -------------------------------------------------
@pytest.mark.parametrize("case,sharp", REF_PLAIN_CASES)
def test_plain_matches_the_float64_definition(gpu, case, sharp):
    q, k, v, kr, vr, shape = reference_case(oracle, case, sharp, False, None, 1.0, C.F32)
    got = run_attention(gpu, q, kr, vr, None, shape, False, C.F32)
    want = oracle.attention_f64(q, k, v, None, shape.start, window=shape.window, scale=1.0, threads=THREADS)
    assert max_error(got, want) < 2e-5, case  # attention_grouped.rs:201


@pytest.mark.parametrize("case,sharp", REF_TILED_CASES)
def test_tiled_matches_the_float64_definition(gpu, case, sharp):
    q, k, v, kr, vr, shape = reference_case(oracle, case, sharp, True, None, 1.0, C.F32)
    # widths 256 and 512 (the reference's tiled kernel is generic in the width): the prompt-pass kernel of that width
    kernel = {256: "lng_prefill_f32_w256", 512: "lng_prefill_f32_w512", 64: None}[shape.dim]
    got = run_attention(gpu, q, kr, vr, None, shape, True, C.F32, expect_kernel=kernel)
    want = oracle.attention_f64(q, k, v, None, shape.start, window=shape.window, scale=1.0, threads=THREADS)
    assert max_error(got, want) < 1e-4, case  # attention_grouped.rs:224


@pytest.mark.parametrize("case,tiled", REF_GPT_OSS_CASES)
@pytest.mark.parametrize("dtype", [C.F32, C.BF16])
def test_sinks_take_probability_without_value_on_gpt_oss_shapes(gpu, case, tiled, dtype):
    t, start, window, slots = case
    sinks = oracle.values(4, 64) * np.float32(3.0)
    q, k, v, kr, vr, shape = reference_case(oracle, (t, start, 64, 8, 64, window, slots), 1.0, tiled, sinks,
                                            0.125, dtype)
    if dtype == C.F32:
        got = run_attention(gpu, q, kr, vr, sinks, shape, tiled, C.F32)
        want = oracle.attention_f64(q, k, v, sinks, start, window=window, scale=0.125, threads=THREADS)
        assert max_error(got, want) < 1e-4, case  # attention_grouped.rs:251
        want32 = oracle.attention_f32(q, k, v, sinks, start, window=window, scale=0.125, threads=THREADS)
        assert rel_error(got, want32) < F32_RTOL
    else:
        got = run_attention(gpu, to_bf16_bits(q), to_bf16_bits(kr), to_bf16_bits(vr), sinks, shape, tiled, C.BF16)
        want = oracle.attention_bf16(to_bf16_bits(q), to_bf16_bits(k), to_bf16_bits(v), sinks, start,
                                     window=window, scale=0.125, threads=THREADS)
        assert max_error(from_bf16_bits(got), from_bf16_bits(want)) < BF16_TOL, case


def test_rejects_shapes_it_cannot_run(gpu):
    """attention_grouped.rs:255-275: four 1 MiB buffers, whole-buffer slices, every shape refused."""
    for case in REF_REJECTED:
        bufs = [gpu.buffer(1 << 20) for _ in range(4)]
        batch = gpu.batch(bufs)
        s = [C.Slice(i, 0, 1 << 20) for i in range(4)]
        with pytest.raises(C.Dispatch):
            batch.attention_grouped(s[0], s[1], s[2], s[3], C.GroupedShape(*case, 1.0))
        assert batch.dispatches() == 0
        batch.drop()
        for b in bufs:
            b.free()


# ---- configuration 1: fp32 plumbing ----------------------------------------------------------
def test_config1_fp32_plumbing_matches_the_cpu_reference(gpu):
    """H=4, G=1, D=64, T=32 causal with sinks, seed 0: every row of the pass against the CPU
    reference's f32 arithmetic, 1e-5 relative; both operator forms."""
    q, k, v, sinks = normal_inputs(0, 32, 32, 4, 1, 64)
    want = oracle.attention_f32(q, k, v, sinks, 0)
    shape = C.GroupedShape(32, 0, 4, 1, 64, FULL, 32, 0.125)
    for tiled in (False, True):
        got = run_attention(gpu, q, k, v, sinks, shape, tiled, C.F32)
        assert rel_error(got, want) < F32_RTOL
    golden = np.load("tests/golden/config1_fp32.npz")
    assert np.array_equal(golden["q"], q) and np.array_equal(golden["sinks"], sinks)
    assert rel_error(run_attention(gpu, q, k, v, sinks, shape, False, C.F32), golden["out"]) < F32_RTOL


# ---- configuration 2: one decoding query over 4096 cached positions, bf16 ---------------------
def test_config2_decode_4096_bf16(gpu):
    q, k, v, sinks = normal_inputs(2, 1, 4096, 64, 8, 64, scale=0.5)
    qb, kb, vb = to_bf16_bits(q), to_bf16_bits(k), to_bf16_bits(v)
    shape = C.GroupedShape(1, 4095, 64, 8, 64, FULL, 4096, 0.125)
    got = run_attention(gpu, qb, kb, vb, sinks, shape, False, C.BF16)
    want = oracle.attention_bf16(qb, kb, vb, sinks, 4095, scale=0.125, threads=THREADS)
    assert max_error(from_bf16_bits(got), from_bf16_bits(want)) < BF16_TOL
    # and much closer than the bar against the float64 definition
    exact = oracle.attention_f64(from_bf16_bits(qb), from_bf16_bits(kb), from_bf16_bits(vb), sinks, 4095,
                                 scale=0.125, threads=THREADS)
    assert max_error(from_bf16_bits(got), exact) < 4e-3


@pytest.mark.parametrize("start,window,slots", [
    (0, FULL, 64), (1, FULL, 64), (31, FULL, 32), (32, FULL, 33), (127, 128, 640), (128, 128, 640),
    (700, 128, 640), (3000, 128, 640), (5000, 128, 129), (130, 7, 12), (4095, FULL, 8192), (8191, FULL, 8192),
    (1000, 1, 5), (999, 1000, 1000), (6001, 4000, 4096),
])
def test_decode_bf16_window_ring_and_edges(gpu, start, window, slots):
    """Decoding at the edges: first token, tile boundaries, windows that wrap the ring, rings not
    a multiple of the tile, a window of one. Rows the operator must not read hold NaN."""
    end = start + 1
    q, k, v, sinks = normal_inputs(start + 17, 1, end, 64, 8, 64, scale=0.5)
    kr, vr = ring_layout(k, 1, start, slots, False), ring_layout(v, 1, start, slots, False)
    # rows of the ring older than the window are poisoned too
    first = 0 if window == FULL else max(0, end - window)
    for p in range(max(0, end - slots), first):
        kr[p % slots] = np.nan
        vr[p % slots] = np.nan
    qb, kb, vb = to_bf16_bits(q), to_bf16_bits(kr), to_bf16_bits(vr)
    shape = C.GroupedShape(1, start, 64, 8, 64, window, slots, 0.125)
    got = run_attention(gpu, qb, kb, vb, sinks, shape, False, C.BF16)
    want = oracle.attention_bf16(qb, to_bf16_bits(k), to_bf16_bits(v), sinks, start, window=window, scale=0.125,
                                 threads=THREADS)
    assert max_error(from_bf16_bits(got), from_bf16_bits(want)) < BF16_TOL
    none = run_attention(gpu, qb, kb, vb, None, shape, False, C.BF16)
    want_none = oracle.attention_bf16(qb, to_bf16_bits(k), to_bf16_bits(v), None, start, window=window,
                                      scale=0.125, threads=THREADS)
    assert max_error(from_bf16_bits(none), from_bf16_bits(want_none)) < BF16_TOL


@pytest.mark.parametrize("heads,kv_heads,dim", [(8, 8, 64), (16, 1, 64), (12, 4, 64), (64, 2, 64), (8, 2, 128),
                                                (4, 4, 32)])
def test_decode_bf16_other_groupings(gpu, heads, kv_heads, dim):
    """Group sizes 1..32 and widths other than 64 (width 32, and groups over 16, take the
    general kernel; width 128 the kernel that walks the head dimension in slices)."""
    start = 777
    q, k, v, sinks = normal_inputs(5, 3, start + 3, heads, kv_heads, dim, scale=0.5)
    qb, kb, vb = to_bf16_bits(q), to_bf16_bits(k), to_bf16_bits(v)
    shape = C.GroupedShape(3, start, heads, kv_heads, dim, 300, start + 3, 0.125)
    got = run_attention(gpu, qb, kb, vb, sinks, shape, False, C.BF16)
    want = oracle.attention_bf16(qb, kb, vb, sinks, start, window=300, scale=0.125, threads=THREADS)
    assert max_error(from_bf16_bits(got), from_bf16_bits(want)) < BF16_TOL


# ---- configuration 3: ragged batch, a full and a sliding layer per sequence -------------------
def test_config3_batched_ragged_decode(gpu):
    rng = np.random.default_rng(3)
    n_seq, heads, kv_heads, dim = 32, 64, 8, 64
    lens = rng.integers(128, 8193, size=n_seq)
    row = kv_heads * dim
    k_all = to_bf16_bits((rng.standard_normal((int(lens.sum()), kv_heads, dim)) * 0.5).astype(np.float32))
    v_all = to_bf16_bits((rng.standard_normal((int(lens.sum()), kv_heads, dim)) * 0.5).astype(np.float32))
    q = to_bf16_bits((rng.standard_normal((2 * n_seq, heads, dim)) * 0.5).astype(np.float32))
    sinks = rng.standard_normal((2, heads)).astype(np.float32)  # one set per layer
    bufs = [gpu.upload(q), gpu.upload(k_all), gpu.upload(v_all), gpu.buffer(q.nbytes), gpu.upload(sinks)]
    bufs[3].fill(0xFF)
    offs = np.concatenate([[0], np.cumsum(lens)[:-1]])
    items, want = [], np.empty_like(q)
    for layer, window in enumerate((FULL, 128)):
        for s in range(n_seq):
            i = layer * n_seq + s
            L = int(lens[s])
            items.append(C.DecodeItem(i * heads * dim * 2, i * heads * dim * 2, int(offs[s]) * row * 2,
                                      int(offs[s]) * row * 2, layer * heads * 4, L - 1, window, L))
            sl = slice(int(offs[s]), int(offs[s]) + L)
            want[i] = oracle.attention_bf16(q[i:i + 1], k_all[sl], v_all[sl], sinks[layer], L - 1, window=window,
                                            scale=0.125, threads=THREADS)[0]
    batch = gpu.batch(bufs)
    batch.attention_decode_batched(0, 1, 2, 3, 4, items, heads, kv_heads, dim, 0.125, C.BF16)
    assert batch.dispatches() == 1
    done = batch.run()
    assert not isinstance(done.gpu_time, Exception)
    got = bufs[3].read(np.uint16).reshape(q.shape)
    batch.drop()
    for b in bufs:
        b.free()
    assert max_error(from_bf16_bits(got), from_bf16_bits(want)) < BF16_TOL


def test_batched_decode_f32_and_errors(gpu):
    heads, kv_heads, dim = 8, 2, 64
    q, k, v, sinks = normal_inputs(21, 2, 50, heads, kv_heads, dim)
    bufs = [gpu.upload(q), gpu.upload(k), gpu.upload(v), gpu.buffer(q.nbytes), gpu.upload(sinks)]
    batch = gpu.batch(bufs)
    step = heads * dim * 4
    items = [C.DecodeItem(0, 0, 0, 0, 0, 39, FULL, 40), C.DecodeItem(step, step, 0, 0, None, 49, 16, 50)]
    batch.attention_decode_batched(0, 1, 2, 3, 4, items, heads, kv_heads, dim, 0.125, C.F32)
    with pytest.raises(C.Dispatch):  # outputs overlap
        batch.attention_decode_batched(0, 1, 2, 3, 4, [items[0], items[0]], heads, kv_heads, dim, 0.125, C.F32)
    with pytest.raises(C.Dispatch):  # cache rows outside the buffer
        batch.attention_decode_batched(0, 1, 2, 3, 4, [C.DecodeItem(0, 0, 0, 0, 0, 99, FULL, 100)], heads, kv_heads,
                                       dim, 0.125, C.F32)
    batch.run()
    got = bufs[3].read(np.float32).reshape(q.shape)
    batch.drop()
    for b in bufs:
        b.free()
    want0 = oracle.attention_f32(q[0:1], k[:40], v[:40], sinks, 39, scale=0.125)[0]
    want1 = oracle.attention_f32(q[1:2], k, v, None, 49, window=16, scale=0.125)[0]
    assert rel_error(got[0], want0) < F32_RTOL and rel_error(got[1], want1) < F32_RTOL


# ---- the glue either side --------------------------------------------------------------------
def test_copy_rows_writes_new_rows_into_a_ring_and_converts(gpu):
    """gpt-oss/src/gpu.rs:744-759: position s goes to row s % slots, in at most two runs; here
    the f32 rows of a projection are rounded into a bf16 cache on the way."""
    slots, width, n, start = 12, 512, 7, 9
    rng = np.random.default_rng(4)
    new = rng.standard_normal((n, width)).astype(np.float32)
    cache = np.zeros((slots, width), np.uint16)
    bufs = [gpu.upload(new), gpu.upload(cache)]
    batch = gpu.batch(bufs)
    done = 0
    while done < n:
        row = (start + done) % slots
        run = min(n - done, slots - row)
        batch.copy_rows((C.Slice(0, done * width * 4, run * width * 4), width),
                        (C.Slice(1, row * width * 2, run * width * 2), width), run, width, C.F32, C.BF16)
        done += run
    with pytest.raises(C.Dispatch):
        batch.copy_rows((C.Slice(0, 0, 4), 1), (C.Slice(1, 0, 2), 1), 0, 1, C.F32, C.BF16)
    with pytest.raises(C.Dispatch):  # stride narrower than the width
        batch.copy_rows((C.Slice(0, 0, 2 * width * 4), width - 1), (C.Slice(1, 0, 2 * width * 2), width), 2, width,
                        C.F32, C.BF16)
    batch.run()
    got = bufs[1].read(np.uint16).reshape(slots, width)
    batch.drop()
    for i in range(n):
        cache[(start + i) % slots] = to_bf16_bits(new[i])
    assert np.array_equal(got, cache)
    for b in bufs:
        b.free()


def test_buffers_belong_to_their_batch_until_it_finishes(gpu):
    a, b = gpu.buffer(1024), gpu.buffer(1024)
    batch = gpu.batch([a, b])
    with pytest.raises(C.Dispatch):
        a.write(np.zeros(4, np.float32))
    with pytest.raises(C.Dispatch):
        gpu.batch([a])
    with pytest.raises(C.Dispatch):
        a.free()
    batch.drop()  # dropped uncommitted: nothing ran, the buffers are back
    a.write(np.arange(256, dtype=np.float32))
    assert np.array_equal(a.read(np.float32), np.arange(256, dtype=np.float32))
    with pytest.raises(C.Alloc):
        gpu.buffer(0)
    res = gpu.resident(np.arange(8, dtype=np.float32))
    batch = gpu.batch([a, b])
    whole = batch.attach(res)
    assert whole == C.Slice(2, 0, 32) and batch.attach(res) == whole
    with pytest.raises(C.Dispatch):  # output in resident memory
        batch.copy_rows((C.Slice(0, 0, 32), 8), (whole, 8), 1, 8)
    with pytest.raises(C.Dispatch):  # output overlaps the input
        batch.copy_rows((C.Slice(0, 0, 32), 8), (C.Slice(0, 16, 32), 8), 1, 8)
    batch.copy_rows((whole, 8), (C.Slice(1, 0, 32), 8), 1, 8)
    seen = []
    batch.commit(lambda done: seen.append(done.gpu_time))
    done = batch.wait()
    assert seen and seen[0] == done.gpu_time and done.gpu_time >= 0.0
    assert np.array_equal(b.read(np.float32, count=8), np.arange(8, dtype=np.float32))
    batch.drop()
    for x in (a, b, res):
        x.free()


def test_synthetic_fill_is_reproducible_on_the_host(gpu):
    n, seed, scale, period = 5000, 77, 0.5, 1024
    buf = gpu.buffer(n * 2)
    f32 = gpu.buffer(n * 4)
    batch = gpu.batch([buf, f32])
    batch.fill_synthetic(C.Slice(0, 0, n * 2), C.BF16, seed, scale, period)
    batch.fill_synthetic(C.Slice(1, 0, n * 4), C.F32, seed, scale, 0)
    batch.run()
    got, got32 = buf.read(np.uint16), f32.read(np.float32)
    batch.drop()
    buf.free()
    f32.free()
    from loadngo_amd.synthetic import synthetic_values
    assert np.array_equal(got32, synthetic_values(n, seed, scale, 0))
    assert np.array_equal(got, to_bf16_bits(synthetic_values(n, seed, scale, period)))
    assert abs(float(got32.std()) - scale) < 0.02 and abs(float(got32.mean())) < 0.03


# ---- prompt passes in bf16 (MFMA kernel) -----------------------------------------------------
@pytest.mark.parametrize("t,start,window,slots,heads,kv_heads", [
    (64, 0, FULL, 64, 64, 8), (33, 5, FULL, 64, 64, 8), (100, 37, FULL, 160, 64, 8), (65, 0, 1, 96, 64, 8),
    (128, 64, 64, 192, 64, 8), (200, 1400, 1024, 1536, 16, 2), (512, 2600, 128, 640, 8, 8), (97, 31, 40, 128, 16, 4),
    (130, 1000, 128, 320, 6, 2), (77, 700, FULL, 4096, 10, 2), (40, 97, 7, 64, 4, 1), (256, 0, 100, 256, 32, 8),
])
def test_prefill_bf16_matches_the_cpu_reference(gpu, t, start, window, slots, heads, kv_heads):
    end = start + t
    q, k, v, sinks = normal_inputs(t + start, t, end, heads, kv_heads, 64, scale=0.5)
    qb, kb, vb = to_bf16_bits(q), to_bf16_bits(k), to_bf16_bits(v)
    kr, vr = ring_layout(kb, t, start, slots, True), ring_layout(vb, t, start, slots, True)
    shape = C.GroupedShape(t, start, heads, kv_heads, 64, window, slots, 0.125)
    want = oracle.attention_bf16(qb, kb, vb, sinks, start, window=window, scale=0.125, threads=THREADS)
    got = run_attention(gpu, qb, kr, vr, sinks, shape, True, C.BF16)
    assert max_error(from_bf16_bits(got), from_bf16_bits(want)) < BF16_TOL
    want_none = oracle.attention_bf16(qb, kb, vb, None, start, window=window, scale=0.125, threads=THREADS)
    none = run_attention(gpu, qb, kr, vr, None, shape, True, C.BF16)
    assert max_error(from_bf16_bits(none), from_bf16_bits(want_none)) < BF16_TOL
    # the row-by-row operator gives the same pass (decode == prefill, row for row)
    krp, vrp = ring_layout(kb, t, start, slots, False), ring_layout(vb, t, start, slots, False)
    plain = run_attention(gpu, qb, krp, vrp, sinks, shape, False, C.BF16)
    assert max_error(from_bf16_bits(plain), from_bf16_bits(want)) < BF16_TOL


@pytest.mark.parametrize("t,start,window,slots,forced", [
    (512, 3584, FULL, 4096, None), (64, 4000, FULL, 4096, None), (33, 5000, 2048, 5056, None), (100, 8000, FULL, 8128, None),
    (512, 1536, FULL, 2048, "7"), (64, 960, FULL, 1024, "64"), (96, 0, FULL, 96, "5"), (160, 2000, 1500, 2176, "3"),
    (64, 4000, 3000, 3072, None), (96, 6000, 4000, 4096, "6"),
    # up to 32 rows: the 32-row form of the kernel, with splits
    (32, 4064, FULL, 4096, None), (20, 5000, FULL, 5024, None), (7, 9000, 4000, 4032, "9"),
])
def test_prefill_bf16_few_query_rows_over_many_keys(gpu, t, start, window, slots, forced, knobs):
    """A chunk of a long prompt (the reference passes 512 rows at a time, engine.rs:51), or a few rows late
    in a long context: too few query tiles to fill the device, so the keys of a tile are split between
    workgroups and merged afterwards. Same bound as the unsplit pass; LNG_PREFILL_SPLITS forces split counts
    that leave some workgroups without a tile, or with edge tiles only."""
    if forced:
        knobs.setenv("LNG_PREFILL_SPLITS", forced)
    heads, kv_heads = 64, 8
    end = start + t
    q, k, v, sinks = normal_inputs(t + start, t, end, heads, kv_heads, 64, scale=0.5)
    qb, kb, vb = to_bf16_bits(q), to_bf16_bits(k), to_bf16_bits(v)
    kr, vr = ring_layout(kb, t, start, slots, True), ring_layout(vb, t, start, slots, True)
    shape = C.GroupedShape(t, start, heads, kv_heads, 64, window, slots, 0.125)
    for sk in (sinks, None):
        want = oracle.attention_bf16(qb, kb, vb, sk, start, window=window, scale=0.125, threads=THREADS)
        got = run_attention(gpu, qb, kr, vr, sk, shape, True, C.BF16)
        assert max_error(from_bf16_bits(got), from_bf16_bits(want)) < BF16_TOL


@pytest.mark.parametrize("t,start,window,slots", [(8, 5000, FULL, 5008), (31, 3000, 2000, 2031), (4, 9000, FULL, 9100),
                                                  (16, 2100, FULL, 2116), (31, 40000, 1100, 1131), (5, 7000, 6999, 7004)])
def test_several_rows_through_the_row_by_row_operator_over_long_caches(gpu, t, start, window, slots, knobs):
    """attention_grouped with a handful of rows over thousands of keys (the tail of a prompt: gpu.rs:760-806
    takes this operator below 32 rows) is served by the prompt-pass kernel, which reads the cache once instead
    of once per row. Same results as row by row (LNG_PLAIN_ROW_BY_ROW) and as the CPU reference; rows of the
    cache outside [first visible, last] hold NaN, as in attention_grouped.rs:57; rings need not be multiples
    of 32 rows here."""
    heads, kv_heads = 64, 8
    end = start + t
    q, k, v, sinks = normal_inputs(t + start, t, end, heads, kv_heads, 64, scale=0.5)
    qb, kb, vb = to_bf16_bits(q), to_bf16_bits(k), to_bf16_bits(v)
    kr, vr = ring_layout(kb, t, start, slots, False), ring_layout(vb, t, start, slots, False)
    first = 0 if window == FULL else max(0, start + 1 - window)
    if slots >= end:                               # flat: poison what no query may see
        kr[:first] = 0x7FC0
        vr[:first] = 0x7FC0
    shape = C.GroupedShape(t, start, heads, kv_heads, 64, window, slots, 0.125)
    want = from_bf16_bits(oracle.attention_bf16(qb, kb, vb, sinks, start, window=window, scale=0.125, threads=THREADS))
    got = from_bf16_bits(run_attention(gpu, qb, kr, vr, sinks, shape, False, C.BF16))
    assert not np.isnan(got).any() and max_error(got, want) < BF16_TOL
    knobs.setenv("LNG_PLAIN_ROW_BY_ROW", "1")
    rows = from_bf16_bits(run_attention(gpu, qb, kr, vr, sinks, shape, False, C.BF16))
    assert max_error(rows, want) < BF16_TOL and np.abs(rows - got).max() < 2.0 ** -6


def long_causal_kernel(knobs, which):
    """"0": one workgroup per (query tile, kv head); "1": workgroups that walk several query tiles; "pair": one
    workgroup per (query tile, kv head, pair of heads), its wavefronts sharing out the keys."""
    knobs.setenv("LNG_PREFILL_STREAM", "0" if which == "pair" else which)
    knobs.setenv("LNG_PREFILL_PAIR", "1" if which == "pair" else "0")


@pytest.mark.parametrize("stream", ["0", "1", "pair"])
@pytest.mark.parametrize("spike_at,sinks_on", [(300, True), (300, False), (5, True), (5, False), (700, True)])
def test_prefill_bf16_with_scores_far_outside_the_usual_range(gpu, spike_at, sinks_on, stream, knobs):
    """Long causal passes first keep the running maximum fixed after one interior tile and check the
    normalisers afterwards. A key whose score is about 10,000 above the rest (2^10000 cannot be held)
    late in the pass must send the workgroup through the pass that tracks the maximum; the same key
    early in the pass, or a cache whose scores all sit far below the first tile's, must not lose anything."""
    long_causal_kernel(knobs, stream)  # every kernel of the long causal pass (see the next test)
    t, heads, kv_heads = 1024, 16, 2
    q, k, v, sinks = normal_inputs(91 + spike_at, t, t, heads, kv_heads, 64, scale=0.5)
    q[:] = np.abs(q) + 1.0                      # every query has a large positive overlap with the spike key
    k[spike_at] = 30.0                          # score = 0.125 * 30 * sum(q) ~ 0.125 * 30 * 64 * 1.4
    if spike_at == 700:                         # and everything before it far below the first tile's scores
        k[64:700] = -k[64:700] - 8.0
    qb, kb, vb = to_bf16_bits(q), to_bf16_bits(k), to_bf16_bits(v)
    shape = C.GroupedShape(t, 0, heads, kv_heads, 64, FULL, t, 0.125)
    sk = sinks if sinks_on else None
    want = oracle.attention_bf16(qb, kb, vb, sk, 0, scale=0.125, threads=THREADS)
    got = run_attention(gpu, qb, kb, vb, sk, shape, True, C.BF16)
    assert max_error(from_bf16_bits(got), from_bf16_bits(want)) < BF16_TOL
    # rows after the spike attend to it alone: their output is its value row
    late = from_bf16_bits(got)[spike_at + 1:]
    assert np.abs(late - from_bf16_bits(vb)[spike_at][None, :, None, :].repeat(heads // kv_heads, 2).reshape(1, heads, 64)).max() < BF16_TOL


@pytest.mark.parametrize("stream", ["0", "1", "pair"])
@pytest.mark.parametrize("case", ["all_far_below", "all_far_above", "huge_sink", "std4", "far_above_then_usual"])
def test_long_causal_passes_with_every_score_far_outside_the_usual_range(gpu, case, stream, knobs):
    """The long causal kernels (both: workgroups that walk several query tiles, and one tile per workgroup) fold
    scale * log2(e) into the queries with one more bf16 rounding and first run with the maximum fixed; with every
    score of a row below -600 or above 600, with sinks of +-300, with Gaussian scores of standard deviation 4
    (sixteen times the benign fills'), and with scores that sit near +600 for the first tiles and near zero after
    them, the range check must send the rows that need it through the tracked pass and the result must stay
    within the bf16 bar of the CPU reference, with and without sinks. The kernel of a workgroup per pair of heads
    (calls of few rows) runs the same scheme and is put through the same cases."""
    long_causal_kernel(knobs, stream)
    t, heads, kv_heads = 1024, 16, 2
    q, k, v, sinks = normal_inputs(17 + len(case), t, t, heads, kv_heads, 64, scale=0.5)
    if case == "all_far_below":   # q . k about -64 * 1.4 * 9 * 8 * 0.125 = -800
        q[:] = np.abs(q) + 1.0
        k[:] = -np.abs(k) * 8.0 - 5.0
    elif case == "all_far_above":
        q[:] = np.abs(q) + 1.0
        k[:] = np.abs(k) * 8.0 + 5.0
    elif case == "huge_sink":
        sinks[:] = 300.0
        sinks[::3] = -300.0
    elif case == "std4":          # q . k * 0.125 has standard deviation 4: q, k of standard deviation 2
        q *= 4.0
        k *= 4.0
    elif case == "far_above_then_usual":
        q[:] = np.abs(q) + 1.0
        k[:192] = np.abs(k[:192]) * 8.0 + 5.0
    qb, kb, vb = to_bf16_bits(q), to_bf16_bits(k), to_bf16_bits(v)
    shape = C.GroupedShape(t, 0, heads, kv_heads, 64, FULL, t, 0.125)
    for sk in (sinks, None):
        want = oracle.attention_bf16(qb, kb, vb, sk, 0, scale=0.125, threads=THREADS)
        got = run_attention(gpu, qb, kb, vb, sk, shape, True, C.BF16,
                            expect_kernel={"0": "lng_prefill_bf16_d64", "1": "lng_prefill_bf16_d64_stream", "pair": "lng_prefill_bf16_d64_pair"}[stream])
        assert max_error(from_bf16_bits(got), from_bf16_bits(want)) < BF16_TOL


@pytest.mark.parametrize("case", ["spike", "all_far_below", "all_far_above", "huge_sink", "usual"])
@pytest.mark.parametrize("window,start", [(128, 0), (100, 777), (33, 64)])
def test_windowed_prefill_with_scores_far_outside_the_usual_range(gpu, case, window, start):
    """Passes under a window (one head per wavefront, the maximum tracked throughout) with a score near 10,000, with
    every score of a row below -600 or above 600, with sinks of +-300: against the CPU reference, with and without
    sinks."""
    t, heads, kv_heads = 500, 16, 2
    end = start + t
    q, k, v, sinks = normal_inputs(5 + window, t, end, heads, kv_heads, 64, scale=0.5)
    if case == "spike":
        q[:] = np.abs(q) + 1.0
        k[start + 300] = 30.0
    elif case == "all_far_below":   # q . k about -64 * 1.4 * 9 * 8 * 0.125 = -800
        q[:] = np.abs(q) + 1.0
        k[:] = -np.abs(k) * 8.0 - 5.0
    elif case == "all_far_above":
        q[:] = np.abs(q) + 1.0
        k[:] = np.abs(k) * 8.0 + 5.0
    elif case == "huge_sink":
        sinks[:] = 300.0
        sinks[::3] = -300.0
    qb, kb, vb = to_bf16_bits(q), to_bf16_bits(k), to_bf16_bits(v)
    slots = end
    kr, vr = ring_layout(kb, t, start, slots, True), ring_layout(vb, t, start, slots, True)
    shape = C.GroupedShape(t, start, heads, kv_heads, 64, window, slots, 0.125)
    for sk in (sinks, None):
        want = oracle.attention_bf16(qb, kb, vb, sk, start, window=window, scale=0.125, threads=THREADS)
        got = run_attention(gpu, qb, kr, vr, sk, shape, True, C.BF16)
        assert max_error(from_bf16_bits(got), from_bf16_bits(want)) < BF16_TOL


@pytest.mark.parametrize("t,start,window,slots,heads,kv_heads", [
    (500, 0, 128, 500, 64, 8),      # the usual window, aligned: three tiles of keys per workgroup
    (333, 4077, 128, 4410, 16, 2),  # an odd start: four tiles
    (200, 1000, 160, 1300, 6, 2),   # the widest window that goes this way; groups of three heads: idle wavefronts
    (97, 31, 40, 128, 16, 4), (65, 3, 1, 96, 8, 8), (130, 1000, 128, 320, 4, 1), (40, 97, 7, 64, 10, 2),
    (31, 900, 100, 160, 64, 8),     # fewer than 32 rows, in a ring that wraps
])
def test_narrow_windows_with_every_row_requested_up_front(gpu, t, start, window, slots, heads, kv_heads, knobs):
    """Windows of up to 160 positions run the kernel that asks for all of a workgroup's K and V rows at its start,
    by loads that write LDS directly into swizzled rows: it is the kernel the dispatch names, it agrees with the CPU
    reference, and it gives the bits of the tile-by-tile kernel (same arithmetic in the same order; a wrong swizzle
    or a row in the wrong place changes them)."""
    end = start + t
    q, k, v, sinks = normal_inputs(11 + window + t, t, end, heads, kv_heads, 64, scale=0.5)
    qb, kb, vb = to_bf16_bits(q), to_bf16_bits(k), to_bf16_bits(v)
    # rows the pass may not read are poisoned (NaN bits): positions before the first query's window, rows never written
    kp, vp = kb.copy(), vb.copy()
    kp[:max(0, start + 1 - window)] = 0x7FC0
    vp[:max(0, start + 1 - window)] = 0x7FC0
    kr, vr = ring_layout(kp, t, start, slots, True, fill=0x7FC0), ring_layout(vp, t, start, slots, True, fill=0x7FC0)
    shape = C.GroupedShape(t, start, heads, kv_heads, 64, window, slots, 0.125)
    want = oracle.attention_bf16(qb, kb, vb, sinks, start, window=window, scale=0.125, threads=THREADS)

    def run(expect):
        rows = (t + 31) // 32 * 32
        qp = np.zeros((rows, heads, 64), dtype=np.uint16)
        qp[:t] = qb
        bufs = [gpu.upload(qp), gpu.upload(kr), gpu.upload(vr), gpu.buffer(qp.nbytes), gpu.upload(sinks)]
        bufs[3].fill(0xFF)
        batch = gpu.batch(bufs)
        try:
            batch.set_timing(True)
            batch.attention_grouped_tiled_with_sinks((C.Slice(0, 0, qp.nbytes), C.Slice(1, 0, kr.nbytes), C.Slice(2, 0, vr.nbytes)),
                                                     C.Slice(4, 0, heads * 4), C.Slice(3, 0, qp.nbytes), shape, C.BF16)
            done = batch.run()
            assert not isinstance(done.gpu_time, Exception), done.gpu_time
            assert batch.kernel_seconds(expect)[1] == 1
            return bufs[3].read(np.uint16).reshape(rows, heads, 64)[:t]
        finally:
            batch.drop()
            for b in bufs:
                b.free()

    got = run("lng_prefill_bf16_d64_h1w")
    assert max_error(from_bf16_bits(got), from_bf16_bits(want)) < BF16_TOL
    knobs.setenv("LNG_PREFILL_UPFRONT", "0")
    tile_by_tile = run("lng_prefill_bf16_d64_h1")
    assert np.array_equal(got, tile_by_tile)


@pytest.mark.parametrize("t,start,heads,kv_heads,sinks_on", [
    (300, 0, 64, 8, True), (1000, 0, 32, 8, True), (777, 1300, 64, 8, False), (64, 0, 16, 2, True), (65, 63, 8, 1, True),
    (130, 4000, 24, 8, True), (2048, 0, 64, 8, True)])
def test_long_causal_pass_on_workgroups_that_walk_several_query_tiles(gpu, t, start, heads, kv_heads, sinks_on, knobs):
    """lng_prefill_bf16_d64_stream (one resident workgroup per compute unit, query tiles dealt out in a snake,
    K/V tiles through three LDS buffers, the interior in matrix and arithmetic phases with the second wavefront of
    every SIMD one phase behind and the normaliser summed by the matrix unit): forced for shapes of every kind it
    takes - a ragged last query tile, positions before the pass, groups that leave wavefronts without a head, fewer
    query tiles than workgroups, no sinks - against the CPU reference, and against the kernel with one workgroup
    per query tile (LNG_PREFILL_STREAM=0), which runs the same arithmetic tile for tile."""
    end = start + t
    q, k, v, sinks = normal_inputs(7 * t + start, t, end, heads, kv_heads, 64, scale=0.5)
    qb, kb, vb = to_bf16_bits(q), to_bf16_bits(k), to_bf16_bits(v)
    kr, vr = ring_layout(kb, t, start, end, True), ring_layout(vb, t, start, end, True)
    shape = C.GroupedShape(t, start, heads, kv_heads, 64, FULL, end, 0.125)
    sk = sinks if sinks_on else None
    knobs.setenv("LNG_PREFILL_STREAM", "1")
    got = from_bf16_bits(run_attention(gpu, qb, kr, vr, sk, shape, True, C.BF16))
    knobs.setenv("LNG_PREFILL_STREAM", "0")
    other = from_bf16_bits(run_attention(gpu, qb, kr, vr, sk, shape, True, C.BF16))
    rows = sorted(set([0, 1, 31, 32, 63, 64, t - 1] + [int(x) for x in np.random.default_rng(t).integers(0, t, 24)]))
    rows = [r for r in rows if r < t]
    want = oracle.attention_rows_f32(from_bf16_bits(qb[rows]), from_bf16_bits(kb), from_bf16_bits(vb), sk,
                                     [start + r for r in rows], scale=0.125, threads=THREADS)
    assert not np.isnan(got).any()
    assert max_error(got[rows], want) < BF16_TOL
    assert np.abs(got - other).max() <= 2.0 ** -7  # a bf16 step or two at |o| < 1


@pytest.mark.parametrize("t,start,heads,kv_heads,window,kernel", [
    (2048, 1000, 64, 8, FULL, "1"), (1000, 0, 32, 8, FULL, "1"), (2048, 1000, 64, 8, 128, "1"), (1000, 37, 24, 4, 100, "1"),
    (512, 1536, 64, 8, FULL, "pair"), (300, 2900, 24, 4, 2500, "pair")])
def test_long_passes_give_the_same_bits_every_launch(gpu, t, start, heads, kv_heads, window, kernel, knobs):
    """The resident kernel's wavefronts pass the tile barrier at two different places of their sequence and share
    three LDS buffers; the kernel for narrow windows and the one of a workgroup per pair of heads read rows that
    other wavefronts' loads wrote straight into LDS (the latter into two buffers in turn, and its wavefronts exchange
    their accumulators through the same memory at the end): 256 launches over the same inputs, each into its own
    output, all bit for bit the first (an LDS row overwritten early or read late would show as a launch that differs)."""
    long_causal_kernel(knobs, kernel)
    dim, per_batch, end = 64, 32, start + t
    rows, krows = (t + 31) // 32 * 32, (end + 31) // 32 * 32
    one = rows * heads * dim * 2
    bufs = [gpu.buffer(one), gpu.buffer(krows * kv_heads * dim * 2), gpu.buffer(krows * kv_heads * dim * 2),
            gpu.buffer(per_batch * one), gpu.upload(np.random.default_rng(1).standard_normal(heads).astype(np.float32))]
    try:
        for i in range(3):
            fill = gpu.batch([bufs[i]])
            fill.fill_synthetic(C.Slice(0, 0, bufs[i].len), C.BF16, 90 + i, 0.5, 0)
            fill.run()
            fill.drop()
        shape = C.GroupedShape(t, start, heads, kv_heads, dim, window, end, 0.125)
        first = None
        for _ in range(8):
            batch = gpu.batch(bufs)
            for j in range(per_batch):
                batch.attention_grouped_tiled_with_sinks(
                    (C.Slice(0, 0, bufs[0].len), C.Slice(1, 0, bufs[1].len), C.Slice(2, 0, bufs[2].len)),
                    C.Slice(4, 0, heads * 4), C.Slice(3, j * one, one), shape, C.BF16)
            done = batch.run()
            batch.drop()
            assert not isinstance(done.gpu_time, Exception), done.gpu_time
            got = bufs[3].read(np.uint16).reshape(per_batch, rows, heads, dim)[:, :t]
            if first is None:
                first = got[0].copy()
                assert not np.isnan(from_bf16_bits(first)).any()
            for j in range(per_batch):
                assert np.array_equal(got[j], first), "launch %d of a batch differs from the first launch" % j
    finally:
        for b in bufs:
            b.free()


@pytest.mark.parametrize("window", [FULL, 128])
def test_config4_prefill_8192_sampled_rows(gpu, window):
    """The 8192-position prompt pass at its real size; a sample of query rows (first, last,
    tile edges, random) is checked against the CPU reference, every head of each."""
    t, heads, kv_heads = 8192, 64, 8
    rng = np.random.default_rng(44)
    qb = to_bf16_bits((rng.standard_normal((t, heads, 64), dtype=np.float32) * 0.5))
    kb = to_bf16_bits((rng.standard_normal((t, kv_heads, 64), dtype=np.float32) * 0.5))
    vb = to_bf16_bits((rng.standard_normal((t, kv_heads, 64), dtype=np.float32) * 0.5))
    sinks = rng.standard_normal(heads).astype(np.float32)
    shape = C.GroupedShape(t, 0, heads, kv_heads, 64, window, t, 0.125)
    got = run_attention(gpu, qb, kb, vb, sinks, shape, True, C.BF16)
    assert not np.isnan(from_bf16_bits(got)).any()
    rows = sorted(set([0, 1, 31, 32, 63, 64, 127, 128, 129, 4095, 4096, 8190, 8191] +
                      [int(x) for x in rng.integers(0, t, 40)]))
    want = oracle.attention_rows_f32(from_bf16_bits(qb[rows]), from_bf16_bits(kb), from_bf16_bits(vb), sinks, rows,
                                     window=window, scale=0.125, threads=THREADS)
    assert max_error(from_bf16_bits(got[rows]), want) < BF16_TOL


@pytest.mark.parametrize("chunk", [512, 96])
def test_config4_prefill_in_calls_of_fewer_rows_equals_the_one_call(gpu, chunk):
    """The 8192-position full-causal pass made the way the reference makes it (engine.rs:51: a run of rows per
    call, each over the cache so far; the keys of a call are split between workgroups and merged) gives the
    rows of the single call: the same softmax summed in another order, both rounded to bf16 once."""
    t, heads, kv_heads = 8192, 64, 8
    rng = np.random.default_rng(45)
    qb = to_bf16_bits((rng.standard_normal((t, heads, 64), dtype=np.float32) * 0.5))
    kb = to_bf16_bits((rng.standard_normal((t, kv_heads, 64), dtype=np.float32) * 0.5))
    vb = to_bf16_bits((rng.standard_normal((t, kv_heads, 64), dtype=np.float32) * 0.5))
    sinks = rng.standard_normal(heads).astype(np.float32)
    one = from_bf16_bits(run_attention(gpu, qb, kb, vb, sinks, C.GroupedShape(t, 0, heads, kv_heads, 64, FULL, t, 0.125), True, C.BF16))
    starts = list(range(0, t, chunk))[-3:] + [0, chunk * 7]     # the last calls (longest caches), the first, one between
    for start in starts:
        n = min(chunk, t - start)
        shape = C.GroupedShape(n, start, heads, kv_heads, 64, FULL, t, 0.125)
        rows = (start + n + 31) // 32 * 32
        part = from_bf16_bits(run_attention(gpu, qb[start:start + n], kb[:rows], vb[:rows], sinks, shape, True, C.BF16))
        assert np.abs(part - one[start:start + n]).max() <= 2.0 ** -7, (start, n)  # a bf16 step or two at |o| < 1


# ---- configuration 5 at its real per-layer size, through a size-independent identity -----------
def test_config5_layer_at_full_size_periodic_identity(gpu):
    """One layer of the long-context stack at its real shape (batch 16, context 131072, 2 GiB of K
    and of V). The cache is filled on the device with a stream that repeats every 1024 positions,
    so every weight of the full-causal layer appears 128 times: the exact result is attention over
    one period with the sink lowered by ln(128) (pinned on the oracle in test_oracle_pinning). The
    128-window layer sees the last 128 positions of a period. Every sequence and head is checked."""
    from loadngo_amd.synthetic import synthetic_values
    batch_size, ctx, heads, kv_heads, dim, period = 16, 131072, 64, 8, 64, 1024
    row = kv_heads * dim
    kbuf, vbuf = gpu.buffer(batch_size * ctx * row * 2), gpu.buffer(batch_size * ctx * row * 2)
    rng = np.random.default_rng(55)
    q = to_bf16_bits((rng.standard_normal((2 * batch_size, heads, dim), dtype=np.float32) * 0.5))
    sinks = rng.standard_normal((2, heads)).astype(np.float32)
    qbuf, obuf, sbuf = gpu.upload(q), gpu.buffer(q.nbytes), gpu.upload(sinks)
    obuf.fill(0xFF)
    bufs = [qbuf, kbuf, vbuf, obuf, sbuf]
    batch = gpu.batch(bufs)
    batch.fill_synthetic(C.Slice(1, 0, kbuf.len), C.BF16, 7, 0.5, period * row)
    batch.fill_synthetic(C.Slice(2, 0, vbuf.len), C.BF16, 8, 0.5, period * row)
    step = heads * dim * 2
    items = []
    for layer, window in enumerate((FULL, 128)):
        for b in range(batch_size):
            i = layer * batch_size + b
            items.append(C.DecodeItem(i * step, i * step, b * ctx * row * 2, b * ctx * row * 2, layer * heads * 4,
                                      ctx - 1, window, ctx))
    batch.attention_decode_batched(0, 1, 2, 3, 4, items[:batch_size], heads, kv_heads, dim, 0.125, C.BF16)
    batch.attention_decode_batched(0, 1, 2, 3, 4, items[batch_size:], heads, kv_heads, dim, 0.125, C.BF16)
    done = batch.run()
    assert not isinstance(done.gpu_time, Exception)
    got = from_bf16_bits(obuf.read(np.uint16).reshape(q.shape))
    batch.drop()
    for b in bufs:
        b.free()
    k1 = to_bf16_bits(synthetic_values(period * row, 7, 0.5).reshape(period, kv_heads, dim))
    v1 = to_bf16_bits(synthetic_values(period * row, 8, 0.5).reshape(period, kv_heads, dim))
    repeats = ctx // period
    lowered = sinks[0] - np.float32(np.log(repeats))
    for b in range(batch_size):
        full = oracle.attention_bf16(q[b:b + 1], k1, v1, lowered, period - 1, scale=0.125, threads=THREADS)
        assert max_error(got[b], from_bf16_bits(full[0])) < BF16_TOL, ("full", b)
        win = oracle.attention_bf16(q[batch_size + b:batch_size + b + 1], k1, v1, sinks[1], period - 1, window=128,
                                    scale=0.125, threads=THREADS)
        assert max_error(got[batch_size + b], from_bf16_bits(win[0])) < BF16_TOL, ("window", b)


@pytest.mark.parametrize("start,window,slots,heads,kv_heads", [
    (131148, FULL, 131149, 64, 8), (200000, 100000, 150016, 64, 8), (70000, FULL, 70001, 64, 8),
    # one kv head: the planner lets the row have more chunks (137 and 256) so that the compute units have work
    (70000, FULL, 70001, 4, 1), (300000, FULL, 300001, 16, 1), (6000, FULL, 6001, 8, 1)])
def test_decode_bf16_one_long_row(gpu, start, window, slots, heads, kv_heads):
    """A single query over a very long cache: the run is cut into chunks (at most 32 unless fewer would leave
    compute units idle, never more than 256: the chunk length grows to respect that) and merged in the kernel
    or by a second dispatch; with a ring that has wrapped and a window that does not start on a tile boundary."""
    dim = 64
    rows = min(slots, start + 1)
    rng = np.random.default_rng(start)
    q = to_bf16_bits(rng.standard_normal((1, heads, dim), dtype=np.float32) * 0.5)
    kr = to_bf16_bits(rng.standard_normal((rows, kv_heads, dim), dtype=np.float32) * 0.5)
    vr = to_bf16_bits(rng.standard_normal((rows, kv_heads, dim), dtype=np.float32) * 0.5)
    sinks = rng.standard_normal(heads).astype(np.float32)
    shape = C.GroupedShape(1, start, heads, kv_heads, dim, window, slots, 0.125)
    got = run_attention(gpu, q, kr, vr, sinks, shape, False, C.BF16)
    # the oracle reads position p from row p % slots of the same ring
    want = oracle.attention_bf16(q, kr, vr, sinks, start, window=window, slots=slots, scale=0.125, threads=THREADS)
    assert max_error(from_bf16_bits(got), from_bf16_bits(want)) < BF16_TOL


# ---- f32 caches (the reference's own element type) at the gpt-oss head width: lng_decode_f32_d64 ----
@pytest.mark.parametrize("t,start,window,slots,heads,kv_heads", [
    (1, 0, FULL, 1, 64, 8), (1, 36, FULL, 37, 64, 8), (1, 4095, FULL, 4096, 64, 8), (1, 5000, 128, 200, 64, 8),
    (1, 70000, FULL, 70001, 64, 8), (1, 200000, 100000, 150016, 16, 2), (3, 2000, FULL, 2003, 8, 8), (7, 900, 33, 41, 6, 2),
    (1, 70000, FULL, 70001, 4, 1), (1, 300000, FULL, 300001, 16, 1),
    (31, 100, FULL, 131, 5, 1), (2, 9000, 1, 3, 64, 8), (5, 260, 300, 305, 24, 8), (1, 5000, FULL, 5001, 32, 2),
    (3, 700, 100, 128, 12, 1), (2, 40, 17, 19, 16, 1), (1, 31, FULL, 32, 64, 8), (1, 0, FULL, 1, 64, 8),
])
def test_decode_f32_at_head_width_64(gpu, t, start, window, slots, heads, kv_heads, knobs):
    """The row-by-row operator on f32 caches: groupings up to 16 heads per kv head, one chunk and many
    (merged by a second dispatch), rings that have wrapped, windows that start inside a tile, with and without
    sinks; rows the operator must not read hold NaN (attention_grouped.rs:57). Within 1e-5 (relative to
    1 + |x|) of the CPU reference, and the generic kernel (LNG_F32_GENERIC) agrees."""
    end = start + t
    rng = np.random.default_rng(start + t)
    q = (rng.standard_normal((t, heads, 64)) * 0.7).astype(np.float32)
    first = 0 if window == FULL else max(0, start + 1 - window)
    kept = max(first, end - slots)
    k = np.full((end, kv_heads, 64), np.nan, np.float32)
    v = np.full((end, kv_heads, 64), np.nan, np.float32)
    k[kept:] = (rng.standard_normal((end - kept, kv_heads, 64)) * 0.7).astype(np.float32)
    v[kept:] = rng.standard_normal((end - kept, kv_heads, 64)).astype(np.float32)
    shape = C.GroupedShape(t, start, heads, kv_heads, 64, window, slots, 0.125)
    kr, vr = ring_layout(k, t, start, slots, False), ring_layout(v, t, start, slots, False)
    kz, vz = np.nan_to_num(k), np.nan_to_num(v)     # the oracle multiplies unseen rows by zero weights
    for sinks in (rng.standard_normal(heads).astype(np.float32), None):
        want = oracle.attention_f32(q, kz, vz, sinks, start, window=window, slots=None, scale=0.125, threads=THREADS)
        got = run_attention(gpu, q, kr, vr, sinks, shape, False, C.F32)
        assert rel_error(got, want) <= F32_RTOL
        knobs.setenv("LNG_F32_GENERIC", "1")
        generic = run_attention(gpu, q, kr, vr, sinks, shape, False, C.F32)
        knobs.delenv("LNG_F32_GENERIC")
        assert rel_error(generic, want) <= F32_RTOL


# ---- prompt passes in f32 (f32 matrix-instruction kernel) -------------------------------------
@pytest.mark.parametrize("t,start,window,slots,heads,kv_heads,forced", [
    (64, 0, FULL, 64, 64, 8, None), (33, 5, FULL, 64, 64, 8, None), (100, 37, FULL, 160, 16, 2, None), (65, 0, 1, 96, 64, 8, None),
    (128, 64, 64, 192, 64, 8, None), (200, 1400, 1024, 1536, 16, 2, None), (512, 2600, 128, 640, 8, 8, None),
    (97, 31, 40, 128, 16, 4, None), (130, 1000, 128, 320, 6, 2, None), (77, 700, FULL, 4096, 10, 2, None),
    (40, 97, 7, 64, 4, 1, None), (256, 0, 100, 256, 32, 8, None), (128, 3968, FULL, 4096, 64, 8, None),
    (96, 1952, FULL, 2048, 64, 8, "7"), (64, 960, FULL, 1024, 24, 8, "64"), (96, 0, FULL, 96, 64, 8, "5"),
    (160, 2000, 1500, 2176, 16, 2, "3"),
    # a thousand workgroups and more: the build of the kernel with two workgroups per compute unit
    (4096, 0, 128, 4096, 8, 8, None), (4096, 0, FULL, 4096, 8, 8, None), (2080, 3000, 300, 2400, 32, 8, None),
])
def test_prefill_f32_matches_the_cpu_reference(gpu, t, start, window, slots, heads, kv_heads, forced, knobs):
    """The tiled operator on f32 operands at head width 64 (the reference's own prompt pass, gpu.rs:760-806):
    within 1e-5 (relative to 1 + |x|) of the CPU reference, with and without sinks, rings, windows, ragged
    last tiles, groupings from 1 to 8, keys split between workgroups (by the library's own choice and forced
    through LNG_PREFILL_SPLITS); the generic kernel (LNG_F32_GENERIC) agrees."""
    if forced:
        knobs.setenv("LNG_PREFILL_SPLITS", forced)
    end = start + t
    q, k, v, sinks = normal_inputs(t + start, t, end, heads, kv_heads, 64, scale=0.5)
    kr, vr = ring_layout(k, t, start, slots, True), ring_layout(v, t, start, slots, True)
    shape = C.GroupedShape(t, start, heads, kv_heads, 64, window, slots, 0.125)
    for sk in (sinks, None):
        want = oracle.attention_f32(q, k, v, sk, start, window=window, slots=None, scale=0.125, threads=THREADS)
        got = run_attention(gpu, q, kr, vr, sk, shape, True, C.F32)
        assert rel_error(got, want) <= F32_RTOL
    knobs.setenv("LNG_F32_GENERIC", "1")
    generic = run_attention(gpu, q, kr, vr, None, shape, True, C.F32)
    assert rel_error(generic, want) <= F32_RTOL


@pytest.mark.parametrize("t,start,window,slots", [(8, 5000, FULL, 5008), (31, 3000, 2000, 2031), (16, 2100, FULL, 2116),
                                                  (5, 7000, 6999, 7004)])
def test_several_f32_rows_through_the_row_by_row_operator_over_long_caches(gpu, t, start, window, slots, knobs):
    """attention_grouped on f32 caches with a handful of rows over thousands of keys goes through the f32
    prompt-pass kernel; same results as row by row (LNG_PLAIN_ROW_BY_ROW) and as the CPU reference; cache rows
    outside [first visible, last] hold NaN, and rings need not be multiples of 32 rows."""
    heads, kv_heads = 64, 8
    end = start + t
    q, k, v, sinks = normal_inputs(t + start, t, end, heads, kv_heads, 64, scale=0.5)
    kr, vr = ring_layout(k, t, start, slots, False), ring_layout(v, t, start, slots, False)
    first = 0 if window == FULL else max(0, start + 1 - window)
    if slots >= end:
        kr[:first] = np.nan
        vr[:first] = np.nan
    shape = C.GroupedShape(t, start, heads, kv_heads, 64, window, slots, 0.125)
    want = oracle.attention_f32(q, k, v, sinks, start, window=window, slots=None, scale=0.125, threads=THREADS)
    got = run_attention(gpu, q, kr, vr, sinks, shape, False, C.F32)
    assert rel_error(got, want) <= F32_RTOL
    knobs.setenv("LNG_PLAIN_ROW_BY_ROW", "1")
    rows = run_attention(gpu, q, kr, vr, sinks, shape, False, C.F32)
    assert rel_error(rows, want) <= F32_RTOL


@pytest.mark.parametrize("scale", [-0.125, 0.0])
def test_scales_that_are_not_positive(gpu, scale):
    """GroupedShape.scale is 1/sqrt(dim) in every caller, but the operator takes any float: a negative or zero
    scale (which the matrix kernels, taking maxima of unscaled products, do not handle) still gives the CPU
    reference's result, in both element types, prompt pass and decode."""
    heads, kv_heads = 16, 2
    for t, start in ((96, 32), (1, 700)):
        end = start + t
        q, k, v, sinks = normal_inputs(t + start, t, end, heads, kv_heads, 64, scale=0.5)
        tiled = t >= 32
        slots = (end + 31) // 32 * 32
        kr, vr = ring_layout(k, t, start, slots, tiled), ring_layout(v, t, start, slots, tiled)
        shape = C.GroupedShape(t, start, heads, kv_heads, 64, FULL, slots, scale)
        want = oracle.attention_f32(q, k, v, sinks, start, window=FULL, slots=None, scale=scale, threads=THREADS)
        assert rel_error(run_attention(gpu, q, kr, vr, sinks, shape, tiled, C.F32), want) <= F32_RTOL
        qb, kb, vb = to_bf16_bits(q), to_bf16_bits(k), to_bf16_bits(v)
        krb, vrb = ring_layout(kb, t, start, slots, tiled), ring_layout(vb, t, start, slots, tiled)
        wantb = oracle.attention_bf16(qb, kb, vb, sinks, start, window=FULL, scale=scale, threads=THREADS)
        gotb = run_attention(gpu, qb, krb, vrb, sinks, shape, tiled, C.BF16)
        assert max_error(from_bf16_bits(gotb), from_bf16_bits(wantb)) < BF16_TOL


# ---- head widths 128, 256 and 512: K and V read once per kv head, the head dimension walked in slices of 64 ----
WIDE_CASES = [
    # the reference's other user of the operator: 32 heads over 16 kv heads of width 256 (decider/src/gpu.rs:878-893)
    (1, 0, FULL, 1, 32, 16, 256), (1, 36, FULL, 37, 32, 16, 256), (1, 4095, FULL, 4096, 32, 16, 256),
    (1, 5000, 128, 200, 32, 16, 256), (1, 9000, FULL, 9001, 32, 16, 256), (4, 700, FULL, 704, 32, 16, 256),
    (1, 33000, FULL, 33001, 8, 4, 256), (1, 50000, 30000, 32768, 16, 1, 256),
    (3, 2000, FULL, 2003, 8, 8, 128), (7, 900, 33, 41, 6, 2, 128), (1, 40000, FULL, 40001, 16, 1, 128),
    (1, 131, FULL, 132, 64, 8, 128), (2, 31, FULL, 33, 5, 1, 128),
    (2, 9000, 1, 3, 8, 2, 512), (1, 9000, FULL, 9001, 8, 2, 512), (5, 260, 300, 305, 24, 8, 512),
    (1, 20000, 7000, 8192, 4, 1, 512), (1, 63, FULL, 64, 16, 1, 512),
]


@pytest.mark.parametrize("dtype", [C.BF16, C.F32])
@pytest.mark.parametrize("t,start,window,slots,heads,kv_heads,dim", WIDE_CASES)
def test_decode_at_head_widths_128_256_512(gpu, dtype, t, start, window, slots, heads, kv_heads, dim, knobs):
    """The row-by-row operator at the wider heads: one chunk and many (merged by a second dispatch), rings that
    have wrapped, windows that start inside a tile, groups of 1..16, with and without sinks; rows the operator must
    not read hold NaN (attention_grouped.rs:57). To the bars of the width-64 kernels against the CPU reference, and
    the kernel of one wavefront per (row, head) (LNG_WIDE_GENERIC) agrees."""
    end = start + t
    rng = np.random.default_rng(start + t + dim)
    scale = float(1.0 / np.sqrt(np.float32(dim)))
    q = rng.standard_normal((t, heads, dim), dtype=np.float32) * np.float32(0.7)
    first = 0 if window == FULL else max(0, start + 1 - window)
    kept = max(first, end - slots)
    k = np.full((end, kv_heads, dim), np.nan, np.float32)
    v = np.full((end, kv_heads, dim), np.nan, np.float32)
    k[kept:] = rng.standard_normal((end - kept, kv_heads, dim), dtype=np.float32) * np.float32(0.7)
    v[kept:] = rng.standard_normal((end - kept, kv_heads, dim), dtype=np.float32)
    shape = C.GroupedShape(t, start, heads, kv_heads, dim, window, slots, scale)
    kr, vr = ring_layout(k, t, start, slots, False), ring_layout(v, t, start, slots, False)
    kz, vz = np.nan_to_num(k), np.nan_to_num(v)     # the oracle multiplies unseen rows by zero weights
    if dtype == C.BF16:
        q, kr, vr, kz, vz = (to_bf16_bits(x) for x in (q, kr, vr, kz, vz))
    for sinks in (rng.standard_normal(heads).astype(np.float32), None):
        if dtype == C.F32:
            want = oracle.attention_f32(q, kz, vz, sinks, start, window=window, scale=scale, threads=THREADS)
            err = lambda got: rel_error(got, want)  # noqa: E731
            bar = F32_RTOL
        else:
            want = from_bf16_bits(oracle.attention_bf16(q, kz, vz, sinks, start, window=window, scale=scale, threads=THREADS))
            err = lambda got: max_error(from_bf16_bits(got), want)  # noqa: E731
            bar = BF16_TOL
        got = run_attention(gpu, q, kr, vr, sinks, shape, False, dtype)
        assert err(got) <= bar
        knobs.setenv("LNG_WIDE_GENERIC", "1")
        generic = run_attention(gpu, q, kr, vr, sinks, shape, False, dtype)
        knobs.delenv("LNG_WIDE_GENERIC")
        assert err(generic) <= bar


def test_ragged_table_of_sequences_at_head_width_256(gpu):
    """attention_decode_batched at 32 heads over 16 kv heads of width 256: sequences of very different
    lengths in one dispatch (live workgroups only), each against the CPU reference on its own cache."""
    heads, kv_heads, dim = 32, 16, 256
    lens = [1, 40, 129, 700, 5000, 12000, 33, 2048]
    rng = np.random.default_rng(256)
    row = kv_heads * dim
    offs = np.concatenate([[0], np.cumsum(lens)])
    k_all = to_bf16_bits(rng.standard_normal((int(offs[-1]), kv_heads, dim), dtype=np.float32) * np.float32(0.7))
    v_all = to_bf16_bits(rng.standard_normal((int(offs[-1]), kv_heads, dim), dtype=np.float32))
    q = to_bf16_bits(rng.standard_normal((len(lens), heads, dim), dtype=np.float32) * np.float32(0.7))
    sinks = rng.standard_normal(heads).astype(np.float32)
    scale = float(1.0 / np.sqrt(np.float32(dim)))
    bufs = [gpu.upload(q), gpu.upload(k_all), gpu.upload(v_all), gpu.buffer(q.nbytes), gpu.upload(sinks)]
    bufs[3].fill(0xFF)
    items = [C.DecodeItem(i * heads * dim * 2, i * heads * dim * 2, int(offs[i]) * row * 2, int(offs[i]) * row * 2, 0,
                          n - 1, FULL, n) for i, n in enumerate(lens)]
    batch = gpu.batch(bufs)
    try:
        batch.attention_decode_batched(0, 1, 2, 3, 4, items, heads, kv_heads, dim, scale, C.BF16)
        done = batch.run()
        assert not isinstance(done.gpu_time, Exception), done.gpu_time
        out = bufs[3].read(np.uint16).reshape(len(lens), heads, dim)
    finally:
        batch.drop()
        for b in bufs:
            b.free()
    for i, n in enumerate(lens):
        ks, vs = k_all[offs[i]:offs[i + 1]], v_all[offs[i]:offs[i + 1]]
        want = oracle.attention_bf16(q[i:i + 1], ks, vs, sinks, n - 1, scale=scale, threads=THREADS)
        assert max_error(from_bf16_bits(out[i:i + 1]), from_bf16_bits(want)) < BF16_TOL, (i, n)
