"""The prompt-pass kernel of one workgroup per (64 query rows, kv head, pair of query heads) on the MI355X, through
the C ABI, against the CPU oracle: lng_prefill_bf16_d64_pair, which serves calls with too few rows to give every
compute unit a (query tile, kv head) of its own - the reference feeds a prompt 512 rows at a time (engine.rs:51).
Its wavefronts deal out the keys among themselves and put their states together in LDS, so besides the shapes of
the other prompt-pass tests this covers: runs of 1..9 sub-tiles of 64 keys (wavefronts with nothing to do, with only
an edge sub-tile, with one more than the others), windows whose edge and diagonal fall to different wavefronts,
rings, odd groups (a pair with one head), and which calls the library gives to it. bf16 bar: 2e-2 max-abs."""
import numpy as np
import pytest

from loadngo_amd import compute as C
from oracle import oracle
from tests.gpu_common import THREADS, gpu, knobs, max_error, run_attention  # noqa: F401
from tests.helpers import FULL, from_bf16_bits, normal_inputs, ring_layout, to_bf16_bits

pytestmark = pytest.mark.gpu
BF16_TOL = 2e-2
PAIR = "lng_prefill_bf16_d64_pair"


def case(t, start, window, slots, heads, kv_heads, seed=0):
    end = start + t
    q, k, v, sinks = normal_inputs(seed + t + start + heads, t, end, heads, kv_heads, 64, scale=0.5)
    qb, kb, vb = to_bf16_bits(q), to_bf16_bits(k), to_bf16_bits(v)
    kr, vr = ring_layout(kb, t, start, slots, True), ring_layout(vb, t, start, slots, True)
    first = 0 if window == FULL else max(0, start + 1 - window)
    if slots >= end:  # flat: poison what no query may see
        kr[:first] = 0x7FC0
        vr[:first] = 0x7FC0
    return qb, kb, vb, kr, vr, sinks, C.GroupedShape(t, start, heads, kv_heads, 64, window, slots, 0.125)


@pytest.mark.parametrize("t,start,window,slots,heads,kv_heads", [
    # the reference's chunks of a prompt: first, second, a middle one, the last of 8,192 positions
    (512, 0, FULL, 512, 64, 8), (512, 512, FULL, 1024, 64, 8), (512, 1536, FULL, 2048, 64, 8), (512, 7680, FULL, 8192, 64, 8),
    # one sub-tile; rows that are no multiple of anything; runs of 5 and 9 sub-tiles
    (64, 0, FULL, 64, 64, 8), (100, 37, FULL, 160, 64, 8), (33, 300, FULL, 352, 64, 8), (63, 513, FULL, 576, 16, 2),
    # groups of 6, 5, 7 and 1 (the last pair has one head), 8 kv heads of one head each
    (300, 1000, FULL, 1312, 24, 4), (130, 500, FULL, 640, 10, 2), (65, 4000, FULL, 4096, 7, 1), (512, 300, FULL, 832, 8, 8),
    # windows wider than the narrow kernels take, flat and in rings that have wrapped
    (256, 3000, 2000, 3264, 64, 8), (256, 3000, 1500, 1792, 64, 8), (200, 900, 1100, 1120, 16, 2), (77, 5000, 4097, 4224, 64, 8),
    (1024, 0, FULL, 1024, 16, 2),
])
def test_head_pair_kernel_matches_the_cpu_reference(gpu, t, start, window, slots, heads, kv_heads, knobs):
    knobs.setenv("LNG_PREFILL_STREAM", "0")
    knobs.setenv("LNG_PREFILL_PAIR", "1")
    qb, kb, vb, kr, vr, sinks, shape = case(t, start, window, slots, heads, kv_heads)
    for sk in (sinks, None):
        want = from_bf16_bits(oracle.attention_bf16(qb, kb, vb, sk, start, window=window, scale=0.125, threads=THREADS))
        got = from_bf16_bits(run_attention(gpu, qb, kr, vr, sk, shape, True, C.BF16, expect_kernel=PAIR))
        assert not np.isnan(got).any() and max_error(got, want) < BF16_TOL


@pytest.mark.parametrize("t,start,window,slots", [(100, 3000, FULL, 3100), (63, 2500, 2000, 2063), (40, 5000, FULL, 5040), (333, 700, FULL, 1033)])
def test_the_row_by_row_operator_on_the_head_pair_kernel(gpu, t, start, window, slots, knobs):
    """attention_grouped with tens of rows over thousands of keys goes to a prompt-pass kernel as well (the cache is read
    once, not once per row); its caches are not padded to 32 rows and hold NaN wherever the operator may not read
    (attention_grouped.rs:57), its queries and outputs have exactly t rows."""
    knobs.setenv("LNG_PREFILL_STREAM", "0")
    knobs.setenv("LNG_PREFILL_PAIR", "1")
    heads, kv_heads = 64, 8
    end = start + t
    q, k, v, sinks = normal_inputs(3 * t + start, t, end, heads, kv_heads, 64, scale=0.5)
    qb, kb, vb = to_bf16_bits(q), to_bf16_bits(k), to_bf16_bits(v)
    kr, vr = ring_layout(kb, t, start, slots, False), ring_layout(vb, t, start, slots, False)
    first = 0 if window == FULL else max(0, start + 1 - window)
    if slots >= end:
        kr[:first] = 0x7FC0
        vr[:first] = 0x7FC0
    shape = C.GroupedShape(t, start, heads, kv_heads, 64, window, slots, 0.125)
    want = from_bf16_bits(oracle.attention_bf16(qb, kb, vb, sinks, start, window=window, scale=0.125, threads=THREADS))
    got = from_bf16_bits(run_attention(gpu, qb, kr, vr, sinks, shape, False, C.BF16, expect_kernel=PAIR))
    assert not np.isnan(got).any() and max_error(got, want) < BF16_TOL


def test_random_shapes_on_the_head_pair_kernel(gpu, knobs):
    """Seeded random shapes: 33..700 rows after 0..5,000 cached positions, 1..8 kv heads (3, 5 and 6 among them) with
    groups of 1..8, windows above 1,024 or none, flat caches and rings at every phase, both operators (tiled: padded
    caches; row by row: NaN wherever it may not read), with and without sinks."""
    knobs.setenv("LNG_PREFILL_STREAM", "0")
    knobs.setenv("LNG_PREFILL_PAIR", "1")
    rng = np.random.default_rng(20250)
    ran = 0
    for _ in range(60):
        kv_heads = int(rng.choice([1, 2, 3, 4, 5, 6, 8]))
        heads = kv_heads * int(rng.integers(1, 9))
        t = int(rng.choice([33, 64, 65, 127, 128, 200, 256, 511, 600, 700]))
        start = int(rng.choice([0, 1, 17, 63, 64, 191, 256, 257, 1000, 2049, 5000]))
        window = [FULL, FULL, 1025, 1500, 4000][int(rng.integers(5))]
        tiled = bool(rng.integers(0, 2))
        end = start + t
        if rng.integers(0, 2):
            slots = end + int(rng.integers(0, 70))
        else:
            slots = ((window if window != FULL else end) + t + int(rng.integers(0, 100)) + 31) // 32 * 32
        if not oracle.accepts(t, start, heads, kv_heads, 64, window, slots, tiled):
            continue
        q, k, v, sinks = normal_inputs(ran + t + start + heads, t, end, heads, kv_heads, 64, scale=0.5)
        qb, kb, vb = to_bf16_bits(q), to_bf16_bits(k), to_bf16_bits(v)
        kr, vr = ring_layout(kb, t, start, slots, tiled), ring_layout(vb, t, start, slots, tiled)
        first = 0 if window == FULL else max(0, start + 1 - window)
        if slots >= end:
            kr[:first] = 0x7FC0
            vr[:first] = 0x7FC0
        shape = C.GroupedShape(t, start, heads, kv_heads, 64, window, slots, 0.125)
        sk = sinks if rng.integers(0, 3) else None
        want = from_bf16_bits(oracle.attention_bf16(qb, kb, vb, sk, start, window=window, scale=0.125, threads=THREADS))
        # (the row-by-row operator goes to a prompt-pass kernel only with enough rows x keys: lng_hip.cpp)
        seen = min(end, t + window)
        here = tiled or (seen >= 1024 and t * seen >= 32768)
        got = from_bf16_bits(run_attention(gpu, qb, kr, vr, sk, shape, tiled, C.BF16, expect_kernel=PAIR if here else None))
        assert not np.isnan(got).any() and max_error(got, want) < BF16_TOL, (t, start, window, slots, heads, kv_heads, tiled)
        ran += 1
    assert ran >= 35, ran


def test_head_pair_kernel_counts_the_query_tiles_it_makes_again(gpu, knobs):
    """LNG_COUNT_SECOND_PASSES: a key whose score is about 10,000 above the rest, late in the run, fails the range check
    of the attempts that fix their reference point (the counter moves, per workgroup and failed attempt); benign scores
    never do (the counter stays at zero); both results are right."""
    knobs.setenv("LNG_PREFILL_STREAM", "0")
    knobs.setenv("LNG_PREFILL_PAIR", "1")
    knobs.setenv("LNG_COUNT_SECOND_PASSES", "1")
    t, heads, kv_heads = 1024, 16, 2
    gpu.debug_get("LNG_COUNT_SECOND_PASSES")
    for spike in (False, True):
        q, k, v, sinks = normal_inputs(123, t, t, heads, kv_heads, 64, scale=0.5)
        if spike:
            q[:] = np.abs(q) + 1.0
            k[700] = 30.0
        qb, kb, vb = to_bf16_bits(q), to_bf16_bits(k), to_bf16_bits(v)
        shape = C.GroupedShape(t, 0, heads, kv_heads, 64, FULL, t, 0.125)
        want = from_bf16_bits(oracle.attention_bf16(qb, kb, vb, sinks, 0, scale=0.125, threads=THREADS))
        got = from_bf16_bits(run_attention(gpu, qb, kb, vb, sinks, shape, True, C.BF16, expect_kernel=PAIR))
        assert max_error(got, want) < BF16_TOL
        again = gpu.debug_get("LNG_COUNT_SECOND_PASSES")
        if spike:
            # the query tiles that see key 700 behind interior steps: tiles 11..15 of 16, x 2 kv heads x 4 pairs of heads
            assert again >= 5 * 2 * 4, again
        else:
            assert again == 0, again


@pytest.mark.parametrize("t,start,slots,expect", [
    (512, 3584, 4096, PAIR),                   # a 512-row chunk of a prompt: 64 (query tile, kv head) pairs on 256 units
    (256, 1024, 1280, PAIR), (128, 1920, 2048, PAIR),
    (512, 15872, 16384, "lng_prefill_merge"),  # over 16,384 keys a kv head's K and V outgrow an XCD's L2: keys split
    (256, 7936, 8192, "lng_prefill_merge"),    # half the units and 8,192 keys each: keys split between workgroups
    (32, 4064, 4096, "lng_prefill_merge"),     # up to 32 rows: the 32-row kernel, keys split
])
def test_which_calls_the_library_gives_to_the_head_pair_kernel(gpu, t, start, slots, expect, knobs):
    """The planner's choice, and both choices right: the same call with LNG_PREFILL_PAIR=0 (keys split between
    workgroups, merged by a second dispatch) gives the same rows to a bf16 step."""
    qb, kb, vb, kr, vr, sinks, shape = case(t, start, FULL, slots, 64, 8)
    got = from_bf16_bits(run_attention(gpu, qb, kr, vr, sinks, shape, True, C.BF16, expect_kernel=expect))
    knobs.setenv("LNG_PREFILL_PAIR", "0")
    split = from_bf16_bits(run_attention(gpu, qb, kr, vr, sinks, shape, True, C.BF16, expect_kernel="lng_prefill_bf16_d64" if t > 32 else "lng_prefill_bf16_d64_h1"))
    rows = sorted(set([0, t - 1] + [int(x) for x in np.random.default_rng(t).integers(0, t, 12)]))
    want = oracle.attention_rows_f32(from_bf16_bits(qb[rows]), from_bf16_bits(kb), from_bf16_bits(vb), sinks,
                                     [start + r for r in rows], scale=0.125, threads=THREADS)
    assert max_error(got[rows], want) < BF16_TOL and max_error(split[rows], want) < BF16_TOL
    assert np.abs(got - split).max() <= 2.0 ** -7
