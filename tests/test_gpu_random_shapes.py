"""Seeded random shapes through both operators and both element types against the CPU oracle:
every shape the reference's rules accept (checked with the oracle's restatement of them) must
run and agree; every shape they refuse must be refused. Covers what the hand-picked cases may
miss: odd head counts and groupings, head widths 32..256, windows of every size against rings that
wrap at every phase, one-row and ragged-tail passes."""
import numpy as np
import pytest

from loadngo_amd import compute as C
from oracle import oracle as orc
from tests.gpu_common import THREADS, gpu, knobs, max_error, run_attention  # noqa: F401
from tests.helpers import FULL, from_bf16_bits, ring_layout, to_bf16_bits

pytestmark = pytest.mark.gpu


def _pick(rng, values):
    """One of `values` as the Python object it is (numpy would turn a list holding 2**64 - 1 into floats)."""
    return values[int(rng.integers(len(values)))]


def _random_shape(rng, tiled):
    kv_heads = int(rng.choice([1, 2, 3, 8]))
    group = int(rng.choice([1, 2, 4, 5, 8, 16]))
    dim = int(rng.choice([32, 64, 64, 64, 96, 128, 256]))
    t = int(rng.choice([1, 1, 2, 7, 31, 32, 33, 64, 65, 100]))
    start = int(rng.choice([0, 0, 1, 5, 31, 32, 63, 200, 777]))
    window = _pick(rng, [FULL, FULL, FULL, 1, 2, 7, 31, 32, 33, 128, 500, 0])   # a window of 0 is refused
    end = start + t
    kind = rng.integers(0, 3)
    if kind == 0:
        slots = end                              # flat cache, exactly full
    elif kind == 1:
        slots = end + int(rng.integers(0, 70))   # flat cache with room
    else:                                        # a ring, sometimes too small on purpose
        need = (window if window != FULL else end) + t
        slots = max(1, need + int(rng.integers(-3, 40)))
        if tiled and rng.integers(0, 4):
            slots = (slots + 31) // 32 * 32
    return t, start, kv_heads * group, kv_heads, dim, window, slots


@pytest.mark.parametrize("tiled", [False, True])
@pytest.mark.parametrize("dtype", [C.F32, C.BF16])
def test_random_shapes_agree_with_the_oracle_or_are_refused(gpu, tiled, dtype):
    rng = np.random.default_rng(1234 + 2 * int(tiled) + dtype)
    ran = refused = 0
    for _ in range(40):
        t, start, heads, kv_heads, dim, window, slots = _random_shape(rng, tiled)
        shape = C.GroupedShape(t, start, heads, kv_heads, dim, window, slots, 1.0 / np.sqrt(np.float32(dim)))
        ok = orc.accepts(t, start, heads, kv_heads, dim, window, slots, tiled)
        end = start + t
        q = (rng.standard_normal((t, heads, dim)) * 0.7).astype(np.float32)
        k = (rng.standard_normal((end, kv_heads, dim)) * 0.7).astype(np.float32)
        v = rng.standard_normal((end, kv_heads, dim)).astype(np.float32)
        sinks = rng.standard_normal(heads).astype(np.float32) if rng.integers(0, 3) else None
        if dtype == C.BF16:
            q, k, v = (from_bf16_bits(to_bf16_bits(x)) for x in (q, k, v))
        what = f"t={t} start={start} H={heads} G={kv_heads} D={dim} window={window} slots={slots} tiled={tiled}"
        if not ok:
            rows = max(1, min(slots, end)) if not tiled else max(32, (min(slots, end) + 31) // 32 * 32)
            junk = np.zeros((rows, kv_heads, dim), np.float32)
            cast = (lambda a: a) if dtype == C.F32 else to_bf16_bits
            with pytest.raises(C.Dispatch):
                run_attention(gpu, cast(q), cast(junk), cast(junk), sinks, shape, tiled, dtype)
            refused += 1
            continue
        kr, vr = ring_layout(k, t, start, slots, tiled), ring_layout(v, t, start, slots, tiled)
        want = orc.attention_f32(q, k, v, sinks, start, window=window, slots=None, scale=shape.scale, threads=THREADS)
        if dtype == C.F32:
            got = run_attention(gpu, q, kr, vr, sinks, shape, tiled, dtype)
            err = np.abs(got - want) / (np.abs(want) + 1.0)
            assert not np.isnan(got).any() and err.max() <= 1e-5, f"{what}: {err.max()}"
        else:
            got = from_bf16_bits(run_attention(gpu, to_bf16_bits(q), to_bf16_bits(kr), to_bf16_bits(vr), sinks, shape,
                                               tiled, dtype))
            assert max_error(got, want) <= 2e-2, f"{what}: {max_error(got, want)}"
        ran += 1
    assert ran >= 25 and refused >= 1, (ran, refused)


def test_random_prompt_passes_with_few_rows_over_long_caches(gpu, knobs):
    """bf16, head width 64, 32..600 rows after up to 6,000 cached positions, flat caches and rings, full
    attention and windows above 1,024: the calls whose keys the library splits between workgroups, with the
    library's own split count and with forced ones (including more splits than tiles)."""
    rng = np.random.default_rng(77)
    ran = 0
    for _ in range(40):
        kv_heads = int(rng.choice([1, 2, 4, 8]))
        heads = kv_heads * int(rng.choice([1, 2, 3, 5, 8]))
        t = int(rng.choice([32, 33, 64, 65, 96, 128, 200, 511, 512, 600]))
        start = int(rng.choice([0, 31, 500, 1000, 2047, 3000, 4097, 6000]))
        window = _pick(rng, [FULL, FULL, FULL, 1025, 1500, 3000])
        end = start + t
        if rng.integers(0, 2):
            slots = end + int(rng.integers(0, 70))
        else:
            slots = ((window if window != FULL else end) + t + int(rng.integers(0, 200)) + 31) // 32 * 32
        forced = rng.choice([None, None, "1", "2", "3", "5", "8", "9", "17", "64"])
        if forced:
            knobs.setenv("LNG_PREFILL_SPLITS", str(forced))
        else:
            knobs.delenv("LNG_PREFILL_SPLITS", raising=False)
        if not orc.accepts(t, start, heads, kv_heads, 64, window, slots, True):
            continue
        qb = to_bf16_bits((rng.standard_normal((t, heads, 64)) * 0.7).astype(np.float32))
        kb = to_bf16_bits((rng.standard_normal((end, kv_heads, 64)) * 0.7).astype(np.float32))
        vb = to_bf16_bits((rng.standard_normal((end, kv_heads, 64)) * 0.5).astype(np.float32))
        sinks = rng.standard_normal(heads).astype(np.float32) if rng.integers(0, 3) else None
        shape = C.GroupedShape(t, start, heads, kv_heads, 64, window, slots, 0.125)
        want = from_bf16_bits(orc.attention_bf16(qb, kb, vb, sinks, start, window=window, scale=0.125, threads=THREADS))
        got = from_bf16_bits(run_attention(gpu, qb, ring_layout(kb, t, start, slots, True),
                                           ring_layout(vb, t, start, slots, True), sinks, shape, True, C.BF16))
        what = f"t={t} start={start} H={heads} G={kv_heads} window={window} slots={slots} splits={forced}"
        assert not np.isnan(got).any() and max_error(got, want) <= 2e-2, f"{what}: {max_error(got, want)}"
        ran += 1
    assert ran >= 25, ran
