"""Pins the CPU oracle (oracle/attention_oracle.c) before anything is compared against it.

Each check is chosen so that a plausible mistake fails it: a dropped sink term, a window off
by one, a wrong kv-head index, a wrong ring row, a transposed operand. None of them retypes
the oracle's formula: they use the reference's literal vectors, torch's library attention,
closed forms, and invariants.
"""
import numpy as np
import pytest
import torch

from oracle import oracle
from tests.helpers import (FULL, REF_GPT_OSS_CASES, REF_PLAIN_CASES, REF_REJECTED, REF_TILED_CASES,
                           from_bf16_bits, normal_inputs, ring_layout, to_bf16_bits, xorshift_values)


# ---- bf16 (weights/src/dtype.rs:183-202) --------------------------------------------------
def test_bf16_literal_vectors_of_the_reference():
    def rt(x):
        return float(oracle.bf16_to_f32(oracle.f32_to_bf16(np.float32([x])))[0])

    assert rt(0.9567871) == 0.95703125
    assert rt(0.8925781) == 0.890625
    assert rt(1.0) == 1.0
    assert rt(1.0 + 1.0 / 256.0) == 1.0  # tie: even wins
    assert rt(1.0 + 3.0 / 256.0) == 1.0 + 4.0 / 256.0
    assert np.isnan(rt(np.nan))
    assert rt(np.inf) == np.inf


def test_bf16_every_code_round_trips_and_matches_torch():
    codes = np.arange(65536, dtype=np.uint32).astype(np.uint16)
    wide = oracle.bf16_to_f32(codes)
    assert np.array_equal(wide.view(np.uint32), codes.astype(np.uint32) << 16)
    back = oracle.f32_to_bf16(wide)
    ok = ~np.isnan(wide)
    assert np.array_equal(back[ok], codes[ok])
    # narrowing agrees with torch's cast (the convention dtype.rs names) on random floats
    x = np.random.default_rng(5).standard_normal(200000).astype(np.float32) * 37.0
    want = torch.from_numpy(x).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(oracle.f32_to_bf16(x), want)
    assert np.array_equal(to_bf16_bits(x), want)  # the tests' own numpy helper, same rule


# ---- generator (attention_grouped.rs:25-35) ------------------------------------------------
def test_xorshift_generator_matches_integer_restatement():
    for seed in (1, 2, 3, 4, 12345):
        got = oracle.values(seed, 5000)
        want = xorshift_values(seed, 5000)
        assert np.array_equal(got, want)
    v = oracle.values(1, 100000)
    assert v.min() >= -1.0 and v.max() < 1.0
    assert abs(float(v.mean())) < 0.01  # uniform on [-1, 1)
    # first step from state 1: 1 -> 0x2001 -> 0x2041 -> 0x40822041; top 24 bits are 0
    assert oracle.values(1, 1)[0] == -1.0
    # on the 2^-23 grid
    assert np.all((v.astype(np.float64) + 1.0) * 2**23 % 1 == 0)


# ---- shape acceptance (apple.rs:1243-1272, 1356-1385; tests 255-275) ------------------------
def test_rejects_what_the_reference_rejects():
    for shape in REF_REJECTED:
        assert not oracle.accepts(*shape, tiled=False), shape
    for shape, _ in REF_PLAIN_CASES:
        assert oracle.accepts(*shape, tiled=False), shape
    for shape, _ in REF_TILED_CASES:
        assert oracle.accepts(*shape, tiled=True), shape
    for (t, start, window, slots), tiled in REF_GPT_OSS_CASES:
        assert oracle.accepts(t, start, 64, 8, 64, window, slots, tiled=tiled)
    # tiled: dim need only be a multiple of 16; a wrapping ring must be a multiple of 32
    assert oracle.accepts(32, 0, 4, 4, 48, 8, 64, tiled=True)
    assert not oracle.accepts(32, 0, 4, 4, 40, 8, 64, tiled=True)
    assert not oracle.accepts(40, 97, 4, 1, 64, 7, 60, tiled=True)
    assert oracle.accepts(40, 97, 4, 1, 64, 7, 60, tiled=False)
    # window 0, zero kv heads, zero slots, counts beyond u32
    assert not oracle.accepts(1, 0, 4, 4, 64, 0, 8)
    assert not oracle.accepts(1, 0, 4, 0, 64, 8, 8)
    assert not oracle.accepts(1, 0, 4, 4, 64, 8, 0)
    assert not oracle.accepts(1, 2**32, 4, 4, 64, 8, 2**33)
    assert oracle.accepts(1, 2**32 - 2, 4, 4, 64, 8, 16)


# ---- attention: library routine -------------------------------------------------------------
def sdpa_reference(q, k_all, v_all, sinks, start, window, scale):
    """torch's scaled_dot_product_attention in float64 with an explicit boolean mask; the
    sink is one extra key whose logit is the sink and whose value is zero."""
    t, heads, dim = q.shape
    end, kv_heads, _ = k_all.shape
    group = heads // kv_heads
    qt = torch.from_numpy(q).double().permute(1, 0, 2)  # [H][t][D]
    kt = torch.from_numpy(k_all).double().permute(1, 0, 2).repeat_interleave(group, dim=0)
    vt = torch.from_numpy(v_all).double().permute(1, 0, 2).repeat_interleave(group, dim=0)
    pos = torch.arange(start, start + t)[:, None]
    key = torch.arange(end)[None, :]
    lo = pos + 1 - (end + 1 if window == FULL else window)
    mask = (key <= pos) & (key >= lo)
    if sinks is None:
        out = torch.nn.functional.scaled_dot_product_attention(qt, kt, vt, attn_mask=mask, scale=scale)
    else:
        # extra key column: q . e = sink / scale needs a widened head; build it by hand instead:
        # append one dimension holding 1 to q and sink/scale to the extra key.
        s = torch.from_numpy(sinks).double()
        q1 = torch.cat([qt, torch.ones(heads, t, 1, dtype=torch.float64)], dim=2)
        k1 = torch.cat([kt, torch.zeros(heads, end, 1, dtype=torch.float64)], dim=2)
        sink_key = torch.zeros(heads, 1, dim + 1, dtype=torch.float64)
        sink_key[:, 0, dim] = s / scale
        k1 = torch.cat([k1, sink_key], dim=1)
        v1 = torch.cat([vt, torch.zeros(heads, 1, dim, dtype=torch.float64)], dim=1)
        m1 = torch.cat([mask, torch.ones(t, 1, dtype=torch.bool)], dim=1)
        out = torch.nn.functional.scaled_dot_product_attention(q1, k1, v1, attn_mask=m1, scale=scale)
    return out.permute(1, 0, 2).numpy()


SMALL = [
    # t, start, H, G, D, window, scale
    (1, 0, 4, 1, 64, FULL, 0.125),
    (7, 0, 4, 2, 32, FULL, 1.0),
    (5, 97, 4, 1, 64, 7, 0.125),
    (3, 2, 8, 2, 32, 16, 1.0),
    (9, 150, 16, 2, 64, 128, 0.125),
    (32, 0, 4, 1, 64, FULL, 0.125),  # the fp32 plumbing configuration
    (4, 300, 6, 3, 96, 1, 0.3),
]


@pytest.mark.parametrize("case", SMALL)
@pytest.mark.parametrize("with_sinks", [False, True])
def test_f64_definition_equals_library_attention(case, with_sinks):
    t, start, heads, kv_heads, dim, window, scale = case
    q, k, v, sinks = normal_inputs(11, t, start + t, heads, kv_heads, dim)
    sinks = sinks * 3 if with_sinks else None
    want = sdpa_reference(q, k, v, sinks, start, window, scale)
    got = oracle.attention_f64(q, k, v, sinks, start, window=window, scale=scale)
    assert np.max(np.abs(got - want)) < 2e-6  # f32 output of an f64 computation
    got32 = oracle.attention_f32(q, k, v, sinks, start, window=window, scale=scale)
    assert np.max(np.abs(got32 - want) / (np.abs(want) + 1.0)) < 1e-5


def test_f32_restatement_stays_within_1e5_of_the_f64_definition_on_reference_cases():
    cases = [c for c in REF_PLAIN_CASES if c[0][0] * c[0][2] * (c[0][1] + c[0][0]) < 3e6]
    assert len(cases) >= 5
    for (t, start, heads, kv_heads, dim, window, slots), sharp in cases:
        end = start + t
        q = (oracle.values(1, t * heads * dim) * np.float32(sharp)).reshape(t, heads, dim)
        k = oracle.values(2, end * kv_heads * dim).reshape(end, kv_heads, dim)
        v = oracle.values(3, end * kv_heads * dim).reshape(end, kv_heads, dim)
        kr, vr = ring_layout(k, t, start, slots, False), ring_layout(v, t, start, slots, False)
        want = oracle.attention_f64(q, k, v, None, start, window=window, scale=1.0)
        got = oracle.attention_f32(q, kr, vr, None, start, window=window, slots=slots, scale=1.0)
        assert not np.isnan(got).any()
        assert np.max(np.abs(got - want)) < 2e-5, (t, start, heads)  # the reference's own bound


# ---- attention: closed forms and invariants --------------------------------------------------
def test_zero_queries_give_the_window_mean_shrunk_by_the_sink():
    t, start, heads, kv_heads, dim, window = 3, 40, 4, 2, 32, 9
    _, k, v, sinks = normal_inputs(3, t, start + t, heads, kv_heads, dim)
    q = np.zeros((t, heads, dim), dtype=np.float32)
    got = oracle.attention_f32(q, k, v, sinks, start, window=window)
    for i in range(t):
        last = start + i
        for h in range(heads):
            mean = v[last + 1 - window:last + 1, h // 2].astype(np.float64).mean(axis=0)
            want = mean * window / (window + np.exp(np.float64(sinks[h])))
            assert np.allclose(got[i, h], want, rtol=1e-5, atol=1e-6)


def test_constant_values_lose_exactly_the_sink_probability():
    t, start, heads, kv_heads, dim = 2, 20, 4, 1, 64
    q, k, _, sinks = normal_inputs(4, t, start + t, heads, kv_heads, dim)
    v = np.full((start + t, kv_heads, dim), 2.5, dtype=np.float32)
    got = oracle.attention_f32(q, k, v, sinks, start, scale=0.125)
    none = oracle.attention_f32(q, k, v, None, start, scale=0.125)
    assert np.allclose(none, 2.5, rtol=1e-6)
    for i in range(t):
        for h in range(heads):
            s = (k[:start + i + 1, 0].astype(np.float64) @ q[i, h].astype(np.float64)) * 0.125
            p_sink = np.exp(sinks[h]) / (np.exp(sinks[h]) + np.exp(s).sum())
            assert np.allclose(got[i, h], 2.5 * (1 - p_sink), rtol=1e-5)


def test_window_of_one_sees_only_itself():
    t, start, heads, kv_heads, dim = 4, 10, 2, 2, 32
    q, k, v, sinks = normal_inputs(6, t, start + t, heads, kv_heads, dim)
    # poison everything but the query's own position
    got = oracle.attention_f32(q, k, v, sinks, start, window=1, scale=0.2)
    for i in range(t):
        for h in range(heads):
            s = float(k[start + i, h].astype(np.float64) @ q[i, h].astype(np.float64)) * 0.2
            want = v[start + i, h] / (1 + np.exp(sinks[h] - s))
            assert np.allclose(got[i, h], want, rtol=1e-5, atol=1e-6)


def test_rows_outside_the_window_are_never_read():
    t, start, heads, kv_heads, dim, window = 3, 50, 4, 2, 32, 8
    q, k, v, sinks = normal_inputs(7, t, start + t, heads, kv_heads, dim)
    clean = oracle.attention_f32(q, k, v, sinks, start, window=window)
    kp, vp = k.copy(), v.copy()
    kp[:start + 1 - window] = np.nan  # first visible key of the first query is start+1-window
    vp[:start + 1 - window] = np.nan
    got = oracle.attention_f32(q, kp, vp, sinks, start, window=window)
    assert np.array_equal(got, clean)
    # one row later and the first query is poisoned: the window is not one narrower
    kp[start + 1 - window] = np.nan
    assert np.isnan(oracle.attention_f32(q, kp, vp, sinks, start, window=window)[0]).all()
    # a future row (beyond the last query) would be read by a non-causal implementation
    k2 = np.concatenate([k, np.full((1, kv_heads, dim), np.nan, np.float32)])
    v2 = np.concatenate([v, np.full((1, kv_heads, dim), np.nan, np.float32)])
    assert np.array_equal(oracle.attention_f32(q, k2, v2, sinks, start, window=window), clean)


def test_result_does_not_depend_on_the_ring_size():
    t, start, heads, kv_heads, dim, window = 5, 97, 4, 1, 64, 7
    q, k, v, sinks = normal_inputs(8, t, start + t, heads, kv_heads, dim)
    flat = oracle.attention_f32(q, k, v, sinks, start, window=window)
    for slots in (12, 13, 31, 64, 102, 500):
        kr = ring_layout(k, t, start, slots, False)
        vr = ring_layout(v, t, start, slots, False)
        if slots > start + t:
            kr = np.concatenate([kr, np.full((slots - start - t,) + kr.shape[1:], np.nan, np.float32)])
            vr = np.concatenate([vr, np.full((slots - start - t,) + vr.shape[1:], np.nan, np.float32)])
        got = oracle.attention_f32(q, kr, vr, sinks, start, window=window, slots=slots)
        assert np.array_equal(got, flat), slots
        got64 = oracle.attention_f64(q, kr, vr, sinks, start, window=window, slots=slots)
        assert np.array_equal(got64, oracle.attention_f64(q, k, v, sinks, start, window=window))
    # the C ring() equals the numpy one
    flat_rows = k.reshape(start + t, -1)
    assert np.array_equal(oracle.ring(flat_rows, t, start, 12, False),
                          ring_layout(flat_rows, t, start, 12, False), equal_nan=True)
    assert np.array_equal(oracle.ring(flat_rows, t, start, 64, True),
                          ring_layout(flat_rows, t, start, 64, True))
    assert np.array_equal(oracle.ring(flat_rows, t, start, 4096, True),
                          ring_layout(flat_rows, t, start, 4096, True))


def test_heads_of_a_group_share_their_kv_head_and_groups_do_not():
    t, start, heads, kv_heads, dim = 1, 30, 8, 2, 32
    q, k, v, sinks = normal_inputs(9, t, start + t, heads, kv_heads, dim)
    q[:] = q[:, :1]  # same query in every head
    sinks[:] = 0.3
    got = oracle.attention_f32(q, k, v, sinks, start)
    for h in range(1, 4):
        assert np.array_equal(got[0, h], got[0, 0])
        assert np.array_equal(got[0, 4 + h], got[0, 4])
    assert not np.allclose(got[0, 0], got[0, 4])
    # head 4 is kv head 1: recompute it alone
    alone = oracle.attention_f32(q[:, 4:5], k[:, 1:2], v[:, 1:2], sinks[4:5], start)
    assert np.array_equal(alone[0, 0], got[0, 4])


def test_each_row_of_a_pass_equals_decoding_that_position():
    t, start, heads, kv_heads, dim, window = 6, 33, 4, 2, 32, 16
    q, k, v, sinks = normal_inputs(10, t, start + t, heads, kv_heads, dim)
    whole = oracle.attention_f32(q, k, v, sinks, start, window=window)
    for i in range(t):
        one = oracle.attention_f32(q[i:i + 1], k[:start + i + 1], v[:start + i + 1], sinks, start + i,
                                   window=window)
        assert np.array_equal(one[0], whole[i])
    rows = oracle.attention_rows_f32(q[[1, 4]], k, v, sinks, [start + 1, start + 4], window=window)
    assert np.array_equal(rows, whole[[1, 4]])


def test_a_very_negative_sink_is_no_sink_and_a_dominant_sink_empties_the_output():
    t, start, heads, kv_heads, dim = 2, 12, 4, 4, 32
    q, k, v, _ = normal_inputs(12, t, start + t, heads, kv_heads, dim)
    none = oracle.attention_f32(q, k, v, None, start)
    low = oracle.attention_f32(q, k, v, np.full(heads, -1e30, np.float32), start)
    assert np.array_equal(none, low)
    high = oracle.attention_f32(q, k, v, np.full(heads, 80.0, np.float32), start)
    assert np.max(np.abs(high)) < 1e-20


def test_periodic_cache_equals_one_period_with_a_lowered_sink():
    """If positions repeat with period P and the context holds m whole periods, every weight
    appears m times: the result is attention over one period with sink - ln(m). This is the
    size-independent property the full-size GPU tests lean on."""
    heads, kv_heads, dim, period, m = 4, 2, 32, 24, 5
    q, k, v, sinks = normal_inputs(13, 1, period, heads, kv_heads, dim)
    kk, vv = np.tile(k, (m, 1, 1)), np.tile(v, (m, 1, 1))
    long = oracle.attention_f64(q, kk, vv, sinks, period * m - 1)
    short = oracle.attention_f64(q, k, v, sinks - np.float32(np.log(m)), period - 1)
    assert np.max(np.abs(long - short)) < 1e-6


def test_bf16_entry_is_widen_compute_round():
    t, start, heads, kv_heads, dim = 3, 70, 8, 2, 64
    q, k, v, sinks = normal_inputs(14, t, start + t, heads, kv_heads, dim, scale=0.5)
    qb, kb, vb = to_bf16_bits(q), to_bf16_bits(k), to_bf16_bits(v)
    got = oracle.attention_bf16(qb, kb, vb, sinks, start, window=32)
    wide = oracle.attention_f32(from_bf16_bits(qb), from_bf16_bits(kb), from_bf16_bits(vb), sinks, start,
                                window=32)
    assert np.array_equal(got, to_bf16_bits(wide))
