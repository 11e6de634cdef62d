"""Prompt passes at head widths 128, 256 and 512 on the MI355X, through the C ABI, against the CPU oracle.

The reference's tiled kernel is generic in the head width (kernels.metal:588-720); its own tiled tests are at
widths 256 and 512 (attention_grouped.rs:210-221; run in tests/test_gpu_attention.py with the kernel's name
asserted). Here: seeded random shapes at every width, both element types, groups of 1..16, windows, rings that
have wrapped, passes split between workgroups, and the row-by-row operator with several rows over a long cache.
Tolerances: f32 1e-5 relative (|err| / (|want| + 1)); bf16 2e-2 max-abs, or one bf16 step of the expected value where
that is more (values of 4 and above, which windows of one or two keys over N(0,1) values do produce)."""
import numpy as np
import pytest

from loadngo_amd import compute as C
from oracle import oracle
from tests.gpu_common import THREADS, gpu, knobs, max_error, run_attention  # noqa: F401
from tests.helpers import FULL, from_bf16_bits, ring_layout, to_bf16_bits

pytestmark = pytest.mark.gpu

F32_RTOL = 1e-5
BF16_TOL = 2e-2


def rel_error(got, want):
    e = np.abs(got.astype(np.float64) - want) / (np.abs(want) + 1.0)
    return np.inf if np.isnan(e).any() else float(e.max())


def inputs(t, start, window, slots, heads, kv_heads, dim, tiled, seed):
    """q [t][H][D]; k, v for every absolute position with NaN where the operator may not read (rows before the
    first visible position or fallen out of the ring); their ring layouts; zero-filled twins for the oracle."""
    end = start + t
    rng = np.random.default_rng(seed)
    q = rng.standard_normal((t, heads, dim), dtype=np.float32) * np.float32(0.7)
    first = 0 if window == FULL else max(0, start + 1 - window)
    kept = max(first, end - slots)
    k = np.full((end, kv_heads, dim), np.nan, np.float32)
    v = np.full((end, kv_heads, dim), np.nan, np.float32)
    k[kept:] = rng.standard_normal((end - kept, kv_heads, dim), dtype=np.float32) * np.float32(0.7)
    v[kept:] = rng.standard_normal((end - kept, kv_heads, dim), dtype=np.float32)
    kr, vr = ring_layout(k, t, start, slots, tiled, fill=np.nan), ring_layout(v, t, start, slots, tiled, fill=np.nan)
    sinks = rng.standard_normal(heads).astype(np.float32)
    return q, kr, vr, np.nan_to_num(k), np.nan_to_num(v), sinks


def check(gpu, dtype, q, kr, vr, kz, vz, sinks, shape, tiled, kernel):
    if dtype == C.F32:
        want = oracle.attention_f32(q, kz, vz, sinks, shape.start, window=shape.window, scale=shape.scale, threads=THREADS)
        got = run_attention(gpu, q, kr, vr, sinks, shape, tiled, C.F32, expect_kernel=kernel)
        assert rel_error(got, want) <= F32_RTOL
    else:
        qb, krb, vrb, kzb, vzb = (to_bf16_bits(x) for x in (q, kr, vr, kz, vz))
        want = from_bf16_bits(oracle.attention_bf16(qb, kzb, vzb, sinks, shape.start, window=shape.window, scale=shape.scale,
                                                    threads=THREADS))
        got = run_attention(gpu, qb, krb, vrb, sinks, shape, tiled, C.BF16, expect_kernel=kernel)
        have = from_bf16_bits(got).astype(np.float64)
        assert not np.isnan(have).any()
        assert (np.abs(have - want) <= np.maximum(BF16_TOL, np.abs(want) * 2.0 ** -7)).all(), max_error(from_bf16_bits(got), want)
    return got


# (t, start, window, slots, heads, kv_heads, dim, forced splits)
WIDE_PASSES = [
    # the reference's other model: 32 heads over 16 kv heads of width 256, window 1024 in a ring of 1536
    (512, 2600, 1024, 1536, 32, 16, 256, None), (200, 1400, 1024, 1536, 32, 16, 256, None), (512, 0, 1024, 1536, 32, 16, 256, None),
    # width 512, groups of 8: two workgroups per kv head
    (512, 0, FULL, 512, 32, 4, 512, None), (77, 700, FULL, 4096, 32, 4, 512, None), (33, 5, FULL, 64, 32, 4, 512, None),
    # width 128; groups of 1, 3, 5, 16; rows that are no multiple of anything; windows that start inside a tile
    (130, 0, FULL, 160, 8, 8, 128, None), (97, 333, 100, 512, 6, 2, 128, None), (64, 1000, FULL, 1088, 10, 2, 128, None),
    (40, 97, 7, 64, 16, 1, 128, None), (300, 200, FULL, 512, 16, 1, 256, None), (257, 31, 129, 416, 3, 3, 512, None),
    # passes split between workgroups, some splits left without a tile or with edge tiles only
    (64, 960, FULL, 1024, 8, 2, 256, "8"), (96, 0, FULL, 96, 4, 4, 128, "5"), (160, 2000, 1500, 2176, 4, 1, 512, "3"),
    (32, 4064, FULL, 4096, 32, 16, 256, None), (100, 3000, FULL, 3104, 32, 4, 512, None),
]


@pytest.mark.parametrize("dtype", [C.F32, C.BF16])
@pytest.mark.parametrize("t,start,window,slots,heads,kv_heads,dim,forced", WIDE_PASSES)
def test_prompt_passes_at_head_widths_128_256_512(gpu, dtype, t, start, window, slots, heads, kv_heads, dim, forced, knobs):
    """The tiled operator at the wider heads, with and without sinks, to the bars of the width-64 kernels; rows
    the operator must not read hold NaN. The kernel of that width is the one that ran."""
    if forced:
        knobs.setenv("LNG_PREFILL_SPLITS", forced)
    scale = float(1.0 / np.sqrt(np.float32(dim)))
    q, kr, vr, kz, vz, sinks = inputs(t, start, window, slots, heads, kv_heads, dim, True, t + start + dim)
    shape = C.GroupedShape(t, start, heads, kv_heads, dim, window, slots, scale)
    kernel = "lng_prefill_%s_w%d" % ("f32" if dtype == C.F32 else "bf16", dim)
    for sk in (sinks, None):
        check(gpu, dtype, q, kr, vr, kz, vz, sk, shape, True, kernel)


@pytest.mark.parametrize("dtype", [C.F32, C.BF16])
@pytest.mark.parametrize("t,start,window,slots,heads,kv_heads,dim", [
    (8, 5000, FULL, 5008, 32, 16, 256), (31, 3000, 2000, 2031, 32, 4, 512), (16, 2100, FULL, 2116, 8, 2, 128),
])
def test_several_rows_at_the_wider_heads_through_the_row_by_row_operator(gpu, dtype, t, start, window, slots, heads, kv_heads,
                                                                         dim, knobs):
    """attention_grouped with a handful of rows over thousands of keys takes the prompt-pass kernel of its width
    (the cache is read once, not once per row); the decode kernels (LNG_WIDE_ROW_BY_ROW) give the same rows to the
    same bar."""
    scale = float(1.0 / np.sqrt(np.float32(dim)))
    q, kr, vr, kz, vz, sinks = inputs(t, start, window, slots, heads, kv_heads, dim, False, t + start)
    shape = C.GroupedShape(t, start, heads, kv_heads, dim, window, slots, scale)
    kernel = "lng_prefill_%s_w%d" % ("f32" if dtype == C.F32 else "bf16", dim)
    check(gpu, dtype, q, kr, vr, kz, vz, sinks, shape, False, kernel)
    knobs.setenv("LNG_WIDE_ROW_BY_ROW", "1")
    check(gpu, dtype, q, kr, vr, kz, vz, sinks, shape, False, "lng_decode_%s_w%d" % ("f32" if dtype == C.F32 else "bf16", dim))


def test_a_pass_in_chunks_equals_the_pass_in_one_call(gpu):
    """512 rows in one call and in calls of 128, 65 and 319 rows (each over the cache so far) give the same
    rows to the f32 bar: the reference feeds a prompt in pieces (engine.rs:51)."""
    heads, kv_heads, dim, start, t = 32, 16, 256, 700, 512
    scale = float(1.0 / np.sqrt(np.float32(dim)))
    end = start + t
    rng = np.random.default_rng(11)
    q = rng.standard_normal((t, heads, dim), dtype=np.float32) * np.float32(0.7)
    k = rng.standard_normal((end, kv_heads, dim), dtype=np.float32) * np.float32(0.7)
    v = rng.standard_normal((end, kv_heads, dim), dtype=np.float32)
    sinks = rng.standard_normal(heads).astype(np.float32)
    window = 1024
    want = oracle.attention_f32(q, k, v, sinks, start, window=window, scale=scale, threads=THREADS)
    done = 0
    for n in (128, 65, 319):
        s = start + done
        shape = C.GroupedShape(n, s, heads, kv_heads, dim, window, s + n + 31 & ~31, scale)
        kr = ring_layout(k[:s + n], n, s, shape.slots, True)
        vr = ring_layout(v[:s + n], n, s, shape.slots, True)
        got = run_attention(gpu, q[done:done + n], kr, vr, sinks, shape, True, C.F32, expect_kernel="lng_prefill_f32_w256")
        assert rel_error(got, want[done:done + n]) <= F32_RTOL
        done += n
    assert done == t


@pytest.mark.parametrize("dtype", [C.F32, C.BF16])
def test_random_prompt_passes_at_the_wider_heads(gpu, dtype, knobs):
    """Seeded random shapes at widths 128, 256 and 512: groups of 1..16 (one, two and four heads per workgroup, idle
    wavefronts, several workgroups per kv head), 1..300 rows after up to 3,000 cached positions, windows of every size
    against flat caches and rings that wrap at every phase, the library's own split count and forced ones. Every shape
    the reference's rules accept must run on the kernel of its width and meet the bar."""
    rng = np.random.default_rng(4242 + dtype)
    ran = 0
    for _ in range(36):
        dim = int(rng.choice([128, 256, 512]))
        kv_heads = int(rng.choice([1, 2, 3, 4] if dim < 512 else [1, 2]))
        group = int(rng.choice([1, 2, 3, 4, 5, 8, 16]))
        heads = kv_heads * group
        t = int(rng.choice([32, 33, 63, 64, 65, 100, 129, 300]))
        start = int(rng.choice([0, 1, 31, 64, 500, 1000, 3000]))
        window = [FULL, FULL, 1, 33, 64, 100, 1025][int(rng.integers(7))]
        end = start + t
        if rng.integers(0, 2):
            slots = end + int(rng.integers(0, 70))
        else:
            slots = ((window if window != FULL else end) + t + int(rng.integers(0, 100)) + 31) // 32 * 32
        forced = [None, None, "2", "3", "8"][int(rng.integers(5))]
        if forced:
            knobs.setenv("LNG_PREFILL_SPLITS", forced)
        else:
            knobs.delenv("LNG_PREFILL_SPLITS", raising=False)
        if not oracle.accepts(t, start, heads, kv_heads, dim, window, slots, True):
            continue
        scale = float(1.0 / np.sqrt(np.float32(dim)))
        q, kr, vr, kz, vz, sinks = inputs(t, start, window, slots, heads, kv_heads, dim, True, 9000 + ran)
        shape = C.GroupedShape(t, start, heads, kv_heads, dim, window, slots, scale)
        kernel = "lng_prefill_%s_w%d" % ("f32" if dtype == C.F32 else "bf16", dim)
        try:
            check(gpu, dtype, q, kr, vr, kz, vz, sinks if rng.integers(0, 3) else None, shape, True, kernel)
        except AssertionError as e:
            raise AssertionError(f"t={t} start={start} H={heads} G={kv_heads} D={dim} window={window} slots={slots} "
                                 f"splits={forced}: {e}") from e
        ran += 1
    assert ran >= 25, ran
