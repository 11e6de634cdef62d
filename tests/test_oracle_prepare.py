"""Pins the oracle's restatement of the step before attention (bias, rotation by halves, cache
append: gpt-oss/src/model.rs:427-433, gpu.rs:733-759) against what the mathematics fixes:
complex multiplication in float64, the composition law and norm of a rotation, the identity at
position 0, an independent numpy restatement, and sentinel checks on which cache rows are written.
The reference's end-to-end fixture pins the same functions through tests/test_tiny_model.py."""
import numpy as np
import pytest

from oracle import oracle as orc
from oracle import tiny_model as tm


def _inv_freq(half, theta=150000.0):
    return theta ** (-np.arange(half, dtype=np.float64) / half)


def test_table_is_cos_sin_of_position_times_frequency_scaled():
    inv = _inv_freq(16)
    table = orc.rope_table(inv, 1.3465735902799727, 37, 9)
    angle = (37 + np.arange(9))[:, None] * inv[None, :]
    assert table.shape == (9, 16, 2)
    np.testing.assert_array_equal(table[..., 0], (np.cos(angle) * 1.3465735902799727).astype(np.float32))
    np.testing.assert_array_equal(table[..., 1], (np.sin(angle) * 1.3465735902799727).astype(np.float32))


def test_rotation_is_complex_multiplication_of_first_half_with_second_half():
    rng = np.random.default_rng(1)
    rows, heads, dim = 5, 3, 32
    x = rng.standard_normal((rows, heads * dim)).astype(np.float32)
    table = orc.rope_table(_inv_freq(dim // 2), 1.0, 11, rows)
    got = orc.rotate_halves(x, table, heads, dim).reshape(rows, heads, dim)
    xs = x.reshape(rows, heads, dim).astype(np.float64)
    z = (xs[..., :dim // 2] + 1j * xs[..., dim // 2:]) * (table[:, None, :, 0].astype(np.float64)
                                                          + 1j * table[:, None, :, 1].astype(np.float64))
    np.testing.assert_allclose(got[..., :dim // 2], z.real, rtol=0, atol=1e-6)
    np.testing.assert_allclose(got[..., dim // 2:], z.imag, rtol=0, atol=1e-6)


def test_position_zero_only_scales_and_rotations_compose_and_keep_the_norm():
    rng = np.random.default_rng(2)
    heads, dim = 2, 64
    inv = _inv_freq(dim // 2)
    x = rng.standard_normal((1, heads * dim)).astype(np.float32)
    np.testing.assert_array_equal(orc.rotate_halves(x, orc.rope_table(inv, 1.25, 0, 1), heads, dim),
                                  x * np.float32(1.25))
    once = orc.rotate_halves(orc.rotate_halves(x, orc.rope_table(inv, 1.0, 5, 1), heads, dim),
                             orc.rope_table(inv, 1.0, 9, 1), heads, dim)
    both = orc.rotate_halves(x, orc.rope_table(inv, 1.0, 14, 1), heads, dim)
    np.testing.assert_allclose(once, both, rtol=0, atol=2e-6)
    pairs = lambda a: np.hypot(a.reshape(heads, 2, dim // 2)[:, 0], a.reshape(heads, 2, dim // 2)[:, 1])
    scaled = orc.rotate_halves(x, orc.rope_table(inv, 1.5, 123, 1), heads, dim)
    np.testing.assert_allclose(pairs(scaled), 1.5 * pairs(x), rtol=1e-6)


def test_partial_rotation_leaves_the_tail_of_each_head_alone():
    rng = np.random.default_rng(3)
    rows, heads, dim, rotary = 4, 2, 32, 16
    x = rng.standard_normal((rows, heads * dim)).astype(np.float32)
    table = orc.rope_table(_inv_freq(rotary // 2), 1.0, 3, rows)
    got = orc.rotate_halves(x, table, heads, dim, rotary).reshape(rows, heads, dim)
    xs = x.reshape(rows, heads, dim)
    np.testing.assert_array_equal(got[..., rotary:], xs[..., rotary:])
    want = tm.rotate_halves(np.ascontiguousarray(xs[..., :rotary]).reshape(rows, heads * rotary), table, heads, rotary)
    np.testing.assert_array_equal(got[..., :rotary].reshape(rows, -1), want)


def test_add_rows_broadcasts_a_bias_or_adds_row_by_row():
    rng = np.random.default_rng(4)
    dst = rng.standard_normal((6, 10)).astype(np.float32)
    bias = rng.standard_normal(10).astype(np.float32)
    np.testing.assert_array_equal(orc.add_rows(dst, bias, 0), dst + bias)
    src = rng.standard_normal((6, 12)).astype(np.float32)
    np.testing.assert_array_equal(orc.add_rows(dst, src, 12), dst + src[:, :10])


@pytest.mark.parametrize("bf16", [False, True])
@pytest.mark.parametrize("n,start,slots", [(1, 0, 8), (5, 6, 8), (8, 13, 8), (3, 100, 640), (7, 0, 7)])
def test_prepare_is_bias_rotation_and_a_ring_append(n, start, slots, bf16):
    rng = np.random.default_rng(n * 1000 + start)
    heads, kv_heads, dim = 4, 2, 32
    q = rng.standard_normal((n, heads * dim)).astype(np.float32)
    k = rng.standard_normal((n, kv_heads * dim)).astype(np.float32)
    v = rng.standard_normal((n, kv_heads * dim)).astype(np.float32)
    qb, kb, vb = (rng.standard_normal(w).astype(np.float32) for w in (heads * dim, kv_heads * dim, kv_heads * dim))
    table = orc.rope_table(_inv_freq(dim // 2), 1.2, start, n)
    sentinel = 0x7FC1 if bf16 else np.float32(-777.0)
    kind = np.uint16 if bf16 else np.float32
    kc = np.full((slots, kv_heads * dim), sentinel, dtype=kind)
    vc = np.full((slots, kv_heads * dim), sentinel, dtype=kind)
    q_out = orc.prepare(q, k, v, qb, kb, vb, table, kc, vc, start, heads, kv_heads, dim, bf16=bf16)
    cast = (lambda a: orc.f32_to_bf16(a)) if bf16 else (lambda a: a)
    np.testing.assert_array_equal(q_out, cast(tm.rotate_halves(q + qb, table, heads, dim)))
    want_k, want_v = cast(tm.rotate_halves(k + kb, table, kv_heads, dim)), cast(v + vb)
    written = set()
    for r in range(n):
        slot = (start + r) % slots
        written.add(slot)
        np.testing.assert_array_equal(kc[slot], want_k[r])
        np.testing.assert_array_equal(vc[slot], want_v[r])
    for slot in set(range(slots)) - written:
        assert (kc[slot] == sentinel).all() and (vc[slot] == sentinel).all()
    # without biases
    q2 = orc.prepare(q, k, v, None, None, None, table, kc, vc, start, heads, kv_heads, dim, bf16=bf16)
    np.testing.assert_array_equal(q2, cast(tm.rotate_halves(q, table, heads, dim)))


def test_rms_norm_is_the_cpu_models_and_has_unit_mean_square():
    """model.rs:274-280: against an independent numpy restatement bit for bit, the strided form
    leaves the other columns alone, and with unit weights the result has mean square 1 - eps-ish."""
    rng = np.random.default_rng(6)
    rows, d, stride = 7, 2880, 2890
    v = rng.standard_normal((rows, stride)).astype(np.float32) * np.float32(3.0)
    w = (1 + 0.1 * rng.standard_normal(d)).astype(np.float32)
    got = orc.rms_norm_rows(v, w, d, 1e-5)
    assert np.array_equal(got[:, :d], tm.rms_norm(v[:, :d], w, 1e-5))
    assert np.array_equal(got[:, d:], v[:, d:])
    unit = orc.rms_norm_rows(v, np.ones(d, np.float32), d, 1e-5)[:, :d].astype(np.float64)
    np.testing.assert_allclose((unit ** 2).mean(axis=1), 1.0, rtol=1e-5)
    # scaling the input changes nothing but what eps contributes
    np.testing.assert_allclose(orc.rms_norm_rows(v * 8, w, d, 0.0)[:, :d], orc.rms_norm_rows(v, w, d, 0.0)[:, :d],
                               rtol=3e-7, atol=0)
