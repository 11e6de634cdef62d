"""GPU parity of the step before attention (biases, rotation by halves, cache append:
gpt-oss/src/gpu.rs:733-759), through the C ABI, bit for bit against the CPU oracle: the f32
arithmetic is the same sequence of individually rounded operations, and bf16 outputs are the
round-to-nearest-even of those f32 results."""
import numpy as np
import pytest

from loadngo_amd import compute as C
from oracle import oracle as orc
from tests.gpu_common import gpu  # noqa: F401
from tests.helpers import xorshift_values

pytestmark = pytest.mark.gpu


def _inv_freq(half, theta=150000.0):
    return theta ** (-np.arange(half, dtype=np.float64) / half)


def _run(gpu, arrays, record, read):
    """Uploads `arrays`, records with record(batch), returns [read buffers as uint8]."""
    bufs = [gpu.upload(a) for a in arrays]
    batch = gpu.batch(bufs)
    try:
        record(batch)
        done = batch.run()
        assert not isinstance(done.gpu_time, Exception), done.gpu_time
        return [bufs[i].read(np.uint8) for i in read]
    finally:
        batch.drop()
        for b in bufs:
            b.free()


def test_add_rows_adds_a_bias_or_a_strided_source(gpu):
    rng = np.random.default_rng(1)
    rows, width = 37, 520
    dst = rng.standard_normal((rows, width)).astype(np.float32)
    bias = rng.standard_normal(width).astype(np.float32)
    src = rng.standard_normal((rows, width + 8)).astype(np.float32)

    def record(batch):
        batch.add_rows(C.Slice(0, 0, dst.nbytes), (C.Slice(1, 0, bias.nbytes), 0), rows, width)
        batch.add_rows(C.Slice(0, 0, dst.nbytes), (C.Slice(2, 0, ((rows - 1) * (width + 8) + width) * 4), width + 8),
                       rows, width)
        # apple.rs:1893-1897
        for bad in [(0, width, 0), (rows, 0, 0), (rows, width, width - 1)]:
            with pytest.raises(C.Dispatch):
                batch.add_rows(C.Slice(0, 0, dst.nbytes), (C.Slice(1, 0, bias.nbytes), bad[2]), bad[0], bad[1])
        with pytest.raises(C.Dispatch):  # output overlaps the input
            batch.add_rows(C.Slice(0, 0, dst.nbytes), (C.Slice(0, 0, dst.nbytes), width), rows, width)

    (got,) = _run(gpu, [dst, bias, src], record, [0])
    want = orc.add_rows(orc.add_rows(dst, bias, 0), src, width + 8)
    assert np.array_equal(got.view(np.float32).reshape(rows, width), want)


@pytest.mark.parametrize("rows,heads,dim,rotary", [(1, 64, 64, 64), (9, 8, 64, 64), (40, 4, 32, 32), (5, 3, 48, 16),
                                                   (3, 2, 6, 2)])
def test_rotate_halves_matches_the_cpu_rotation_bit_for_bit(gpu, rows, heads, dim, rotary):
    rng = np.random.default_rng(rows * 100 + dim)
    x = rng.standard_normal((rows, heads * dim)).astype(np.float32)
    table = orc.rope_table(_inv_freq(rotary // 2), 1.3465736, 1234, rows)
    assert np.array_equal(table, C.rope_table(_inv_freq(rotary // 2), 1.3465736, 1234, rows))

    def record(batch):
        xs, ts = C.Slice(0, 0, x.nbytes), C.Slice(1, 0, table.nbytes)
        if rotary == dim:
            batch.rotate_halves(xs, ts, rows, (heads, dim))
        else:
            batch.rotate_halves_partial(xs, ts, rows, (heads, dim, rotary))
        # apple.rs:1936-1940
        for bad in [(0, heads, dim, rotary), (rows, 0, dim, rotary), (rows, heads, dim, 0),
                    (rows, heads, dim, dim + 2), (rows, heads, dim + 1, dim + 1)]:
            with pytest.raises(C.Dispatch):
                batch.rotate_halves_partial(xs, ts, *bad[:1], bad[1:])

    (got,) = _run(gpu, [x, table], record, [0])
    want = orc.rotate_halves(x, table, heads, dim, rotary)
    assert np.array_equal(got.view(np.float32).reshape(rows, -1), want)


def _prepare_case(gpu, n, start, slots, heads, kv_heads, dim, rotary, bf16, biases=True, shift=0, seed=0):
    """One sequence through lng_hip_prepare_attention; `shift` moves every slice off 16-byte
    alignment (the one-element-per-thread kernel)."""
    rng = np.random.default_rng(seed + n * 7 + start)
    qw, kw = heads * dim, kv_heads * dim
    q = rng.standard_normal((n, qw)).astype(np.float32)
    k = rng.standard_normal((n, kw)).astype(np.float32)
    v = rng.standard_normal((n, kw)).astype(np.float32)
    qb, kb, vb = ((rng.standard_normal(w).astype(np.float32) if biases else None) for w in (qw, kw, kw))
    table = orc.rope_table(_inv_freq(rotary // 2), 1.3465736, start, n)
    kind, es = (np.uint16, 2) if bf16 else (np.float32, 4)
    sentinel = 0x7FC1 if bf16 else np.float32(-777.0)
    kc = np.full((slots, kw), sentinel, dtype=kind)
    vc = np.full((slots, kw), sentinel, dtype=kind)
    want_kc, want_vc = kc.copy(), vc.copy()
    want_q = orc.prepare(q, k, v, qb, kb, vb, table, want_kc, want_vc, start, heads, kv_heads, dim, rotary, bf16)

    def padded(a, unit):  # `shift` bytes of padding in front
        raw = np.zeros(shift + a.nbytes, np.uint8)
        raw[shift:] = a.reshape(-1).view(np.uint8)
        return raw
    ins = [q, k, v, table, np.full((n, qw), sentinel, dtype=kind), kc, vc]
    ins += [a if a is not None else np.zeros(4, np.float32) for a in (qb, kb, vb)]
    arrays = [padded(a, 4) for a in ins]
    item = C.PrepareItem(q_offset=shift, k_offset=shift, v_offset=shift, table_offset=shift, q_out_offset=shift,
                         k_cache_offset=shift, v_cache_offset=shift, n=n, start=start, slots=slots)

    def record(batch):
        bias = [C.Slice(7 + i, shift, w * 4) if biases else None for i, w in enumerate((qw, kw, kw))]
        batch.prepare_attention(dict(q=0, k=1, v=2, table=3, q_out=4, k_cache=5, v_cache=6), [item], heads, kv_heads,
                                dim, rotary, C.BF16 if bf16 else C.F32, *bias)

    got_q, got_k, got_v = _run(gpu, arrays, record, [4, 5, 6])
    for got, want, name in ((got_q, want_q, "q"), (got_k, want_kc, "k cache"), (got_v, want_vc, "v cache")):
        got = got[shift:].view(kind).reshape(want.shape)
        assert np.array_equal(got, want), f"{name}: {np.argwhere(got != want)[:4]}"


@pytest.mark.parametrize("bf16", [True, False])
@pytest.mark.parametrize("n,start,slots", [(1, 0, 640), (1, 3000, 640), (9, 700, 640), (512, 2600, 640),
                                           (300, 200, 4096), (640, 5, 640), (33, 0, 33)])
def test_prepare_gpt_oss_shapes_match_the_oracle_bit_for_bit(gpu, n, start, slots, bf16):
    _prepare_case(gpu, n, start, slots, 64, 8, 64, 64, bf16)


@pytest.mark.parametrize("heads,kv_heads,dim,rotary,shift", [(4, 2, 32, 32, 0), (4, 2, 32, 32, 8), (3, 1, 48, 16, 0),
                                                             (2, 2, 6, 2, 0), (5, 5, 20, 12, 0), (64, 8, 64, 64, 8),
                                                             (32, 16, 256, 256, 0)])
def test_prepare_other_shapes_alignments_and_partial_rotation(gpu, heads, kv_heads, dim, rotary, shift):
    for bf16 in (False, True):
        _prepare_case(gpu, 11, 95, 16, heads, kv_heads, dim, rotary, bf16, shift=shift)
    _prepare_case(gpu, 4, 2, 9, heads, kv_heads, dim, rotary, True, biases=False, shift=shift)


def test_prepare_many_sequences_in_one_dispatch(gpu):
    """One decoding step of 16 sequences at different positions (and one with 3 rows), each with
    its own caches: every item is what a single-sequence call computes."""
    heads, kv_heads, dim = 64, 8, 64
    qw, kw = heads * dim, kv_heads * dim
    rng = np.random.default_rng(5)
    seqs = 16
    ns = [1] * (seqs - 1) + [3]
    starts = [int(s) for s in rng.integers(0, 5000, seqs)]
    slots = [640 if i % 2 == 0 else 5008 for i in range(seqs)]
    inv = _inv_freq(dim // 2)
    rows = sum(ns)
    q = rng.standard_normal((rows, qw)).astype(np.float32)
    k = rng.standard_normal((rows, kw)).astype(np.float32)
    v = rng.standard_normal((rows, kw)).astype(np.float32)
    qb, kb, vb = (rng.standard_normal(w).astype(np.float32) for w in (qw, kw, kw))
    table = np.concatenate([orc.rope_table(inv, 1.3465736, starts[i], ns[i]) for i in range(seqs)])
    cache_rows = sum(slots)
    kc = np.full((cache_rows, kw), 0x7FC1, np.uint16)
    vc = np.full((cache_rows, kw), 0x7FC1, np.uint16)
    want_kc, want_vc, want_q = kc.copy(), vc.copy(), np.zeros((rows, qw), np.uint16)
    items, row, crow = [], 0, 0
    for i in range(seqs):
        n = ns[i]
        items.append(C.PrepareItem(q_offset=row * qw * 4, k_offset=row * kw * 4, v_offset=row * kw * 4,
                                   table_offset=row * dim * 4, q_out_offset=row * qw * 2,
                                   k_cache_offset=crow * kw * 2, v_cache_offset=crow * kw * 2, n=n, start=starts[i],
                                   slots=slots[i]))
        want_q[row:row + n] = orc.prepare(q[row:row + n], k[row:row + n], v[row:row + n], qb, kb, vb, table[row:row + n],
                                          want_kc[crow:crow + slots[i]], want_vc[crow:crow + slots[i]], starts[i],
                                          heads, kv_heads, dim, bf16=True)
        row += n
        crow += slots[i]

    def record(batch):
        bias = [C.Slice(7 + i, 0, w * 4) for i, w in enumerate((qw, kw, kw))]
        batch.prepare_attention(dict(q=0, k=1, v=2, table=3, q_out=4, k_cache=5, v_cache=6), items, heads, kv_heads,
                                dim, dim, C.BF16, *bias)

    got_q, got_k, got_v = _run(gpu, [q, k, v, table, np.zeros((rows, qw), np.uint16), kc, vc, qb, kb, vb], record,
                               [4, 5, 6])
    assert np.array_equal(got_q.view(np.uint16).reshape(rows, qw), want_q)
    assert np.array_equal(got_k.view(np.uint16).reshape(cache_rows, kw), want_kc)
    assert np.array_equal(got_v.view(np.uint16).reshape(cache_rows, kw), want_vc)


def test_prepare_refuses_what_it_cannot_do_before_recording(gpu):
    heads, kv_heads, dim = 4, 2, 32
    qw, kw = heads * dim, kv_heads * dim
    n, slots = 4, 8
    bufs = [gpu.buffer(n * qw * 4), gpu.buffer(n * kw * 4), gpu.buffer(n * kw * 4), gpu.buffer(n * dim * 4),
            gpu.buffer(n * qw * 4), gpu.buffer(slots * kw * 4), gpu.buffer(slots * kw * 4)]
    res = gpu.resident(np.zeros(slots * kw, np.float32))
    batch = gpu.batch(bufs)
    names = dict(q=0, k=1, v=2, table=3, q_out=4, k_cache=5, v_cache=6)
    good = dict(q_offset=0, k_offset=0, v_offset=0, table_offset=0, q_out_offset=0, k_cache_offset=0, v_cache_offset=0,
                n=n, start=3, slots=slots)

    def refuse(buffers=names, dtype=C.F32, rotary=dim, **change):
        with pytest.raises(C.Dispatch):
            batch.prepare_attention(buffers, [C.PrepareItem(**{**good, **change})], heads, kv_heads, dim, rotary, dtype)

    refuse(n=0)
    refuse(slots=0)
    refuse(n=4, slots=3)                       # two new rows would share a cache row
    refuse(rotary=dim + 2)
    refuse(rotary=3)
    refuse(rotary=0)
    refuse(q_offset=4)                         # runs past the buffer
    refuse(table_offset=4)                     # table pairs are 8-byte aligned
    refuse(buffers={**names, "q_out": 0})      # output over an input
    refuse(buffers={**names, "v_cache": 5})    # two outputs over each other
    refuse(buffers={**names, "k_cache": batch.attach(res).buffer})  # resident output
    refuse(buffers={**names, "q": 99})
    assert batch.dispatches() == 0
    batch.prepare_attention(names, [C.PrepareItem(**good)], heads, kv_heads, dim, dim, C.F32)
    assert batch.dispatches() == 1
    batch.drop()
    for b in bufs:
        b.free()
    res.free()


def test_strided_rmsnorm_and_row_copy_touch_only_their_columns(gpu):
    """metal-compute/tests/glue.rs:241-297: rows of 20 floats, the first 12 normalised in place, columns
    12..20 copied elsewhere first; bound 2e-6 * (1 + |want|) against the float64 mean of squares."""
    rows, d, stride = 9, 12, 20
    v = xorshift_values(20, rows * stride)
    w = xorshift_values(21, d)

    def record(batch):
        batch.copy_rows((C.Slice(0, d * 4, ((rows - 1) * stride + 8) * 4), stride),
                        (C.Slice(2, 0, ((rows - 1) * 16 + 8) * 4), 16), rows, 8)
        batch.rmsnorm_rows((C.Slice(0, 0, ((rows - 1) * stride + d) * 4), C.Slice(1, 0, d * 4)), rows, (d, stride), 1e-5)
        for bad in [(0, d, stride), (rows, 0, stride), (rows, d, d - 1)]:   # apple.rs:1740-1744
            with pytest.raises(C.Dispatch):
                batch.rmsnorm_rows((C.Slice(0, 0, ((rows - 1) * stride + d) * 4), C.Slice(1, 0, d * 4)), bad[0],
                                   (bad[1], bad[2]), 1e-5)

    got, copied = _run(gpu, [v, w, np.zeros(rows * 16, np.float32)], record, [0, 2])
    got = got.view(np.float32).reshape(rows, stride)
    vv = v.reshape(rows, stride)
    want = vv.copy()
    ss = (vv[:, :d].astype(np.float64) ** 2).sum(axis=1)
    inv = (1.0 / np.sqrt(ss / d + 1e-5)).astype(np.float32)
    want[:, :d] = w[None, :] * vv[:, :d] * inv[:, None]
    assert (np.abs(got - want) <= 2e-6 * (1 + np.abs(want))).all()
    assert np.array_equal(got[:, d:], vv[:, d:])
    copied = copied.view(np.float32).reshape(rows, 16)
    assert np.array_equal(copied[:, :8], vv[:, d:d + 8])
    # and the CPU model's form of the same operator
    assert (np.abs(got - orc.rms_norm_rows(vv, w, d, 1e-5)) <= 2e-6 * (1 + np.abs(want))).all()


@pytest.mark.parametrize("rows,d", [(37, 2880), (1, 2880), (5, 256), (5, 257), (3, 4096), (3, 4100), (2, 12288)])
def test_rmsnorm_at_the_model_width(gpu, rows, d):
    """Rows of 257..4096 floats take a workgroup each, other widths a wavefront: both sides of both limits."""
    rng = np.random.default_rng(8)
    v = (rng.standard_normal((rows, d)) * 4).astype(np.float32)
    w = (1 + 0.1 * rng.standard_normal(d)).astype(np.float32)
    (got,) = _run(gpu, [v, w], lambda b: b.rmsnorm_rows((C.Slice(0, 0, v.nbytes), C.Slice(1, 0, w.nbytes)), rows,
                                                        (d, d), 1e-5), [0])
    want = orc.rms_norm_rows(v, w, d, 1e-5)
    assert (np.abs(got.view(np.float32).reshape(rows, d) - want) <= 2e-6 * (1 + np.abs(want))).all()


def test_glue_adds_and_rotates_as_the_reference_defines(gpu):
    """metal-compute/tests/q8_0_and_gpt_oss_glue.rs:212-300, the rotation and the row add with the
    reference's inputs and bounds (1e-6 against float64; the add exact)."""
    rows, heads, dim, width = 3, 4, 64, 96
    x = xorshift_values(1, rows * heads * dim)
    bias = xorshift_values(2, width)
    h = xorshift_values(3, rows * width)
    angle = np.arange(rows * dim // 2, dtype=np.float64) * 0.37
    table = np.stack([np.cos(angle).astype(np.float32) * np.float32(1.3),
                      np.sin(angle).astype(np.float32) * np.float32(1.3)], axis=-1).reshape(-1)

    def record(batch):
        f = lambda b, n: C.Slice(b, 0, n * 4)
        batch.rotate_halves(f(0, x.size), f(1, table.size), rows, (heads, dim))
        batch.add_rows(f(2, h.size), (f(3, width), 0), rows, width)

    rotated, added = _run(gpu, [x, table, h, bias], record, [0, 2])
    rotated = rotated.view(np.float32).reshape(rows, heads, dim).astype(np.float64)
    xs = x.reshape(rows, heads, dim).astype(np.float64)
    cs = table.reshape(rows, 1, dim // 2, 2).astype(np.float64)
    a, b = xs[..., :dim // 2], xs[..., dim // 2:]
    assert np.abs(rotated[..., :dim // 2] - (a * cs[..., 0] - b * cs[..., 1])).max() < 1e-6
    assert np.abs(rotated[..., dim // 2:] - (b * cs[..., 0] + a * cs[..., 1])).max() < 1e-6
    assert np.array_equal(added.view(np.float32), (h.reshape(rows, width) + bias[None, :]).reshape(-1))
