"""The reference's end-to-end golden (gpt-oss/tests/tiny_oracle.rs:10-40: transformers' logits of a
4-layer gpt-oss over 40 positions, within 2e-3) with the HIP library doing the step before attention
and attention itself, through the C ABI, the way gpt-oss/src/gpu.rs:703-806 records them: caches on
the device, sliding layers in rings of window + chunk rows, one token at a time and in prompt chunks.
Everything else of the model is the numpy restatement in oracle/tiny_model.py."""
import os

import numpy as np
import pytest

from loadngo_amd import compute as C
from oracle import oracle as orc
from oracle import tiny_model as tm
from tests.gpu_common import gpu  # noqa: F401
from tests.helpers import from_bf16_bits

pytestmark = pytest.mark.gpu
FIXTURE = os.path.join(os.path.dirname(__file__), "golden", "tiny")
TOLERANCE = 2e-3  # tiny_oracle.rs:10


class DeviceSession:
    def __init__(self, gpu, model, chunk, dtype, tiled):
        m = self.m = model
        self.gpu, self.chunk, self.dtype, self.tiled = gpu, chunk, dtype, tiled
        self.es = 4 if dtype == C.F32 else 2
        self.qw, self.kw = m.heads * m.dim, m.kv_heads * m.dim
        pad = (chunk + 31) // 32 * 32
        # gpu.rs:567-578: sliding layers hold (window + chunk) rounded up to 32 rows, full layers the context
        self.slots = [((m.window + chunk + 31) // 32 * 32) if m.is_sliding(l) else 64 for l in range(m.layers_n)]
        self.q = gpu.buffer(pad * self.qw * 4)
        self.k = gpu.buffer(chunk * self.kw * 4)
        self.v = gpu.buffer(chunk * self.kw * 4)
        self.table = gpu.buffer(chunk * m.dim * 4)
        self.q_out = gpu.buffer(pad * self.qw * self.es)
        self.att = gpu.buffer(pad * self.qw * self.es)
        self.q_out.fill(0)  # rows past n of a padded prompt pass must be finite (apple.rs:1386-1395)
        self.caches = []
        for l in range(m.layers_n):
            pair = (gpu.buffer(self.slots[l] * self.kw * self.es), gpu.buffer(self.slots[l] * self.kw * self.es))
            for b in pair:
                b.fill(0 if tiled else 0xFF)  # NaN where the plain operator must never read
            self.caches.append(pair)
        self.weights = [[gpu.resident(model.layers[l][n]) for n in ("q_bias", "k_bias", "v_bias", "sinks")]
                        for l in range(m.layers_n)]
        self.n = 0

    def prepare(self, l, q, k, v, start):
        m, n = self.m, q.shape[0]
        self.n = n
        self.q.write(q)
        self.k.write(k)
        self.v.write(v)
        self.table.write(C.rope_table(m.inv_freq, m.rope_scale, start, n))
        kc, vc = self.caches[l]
        batch = self.gpu.batch([self.q, self.k, self.v, self.table, self.q_out, kc, vc, self.att])
        qb, kb, vb, sinks = (batch.attach(r) for r in self.weights[l])
        item = C.PrepareItem(n=n, start=start, slots=self.slots[l])
        batch.prepare_attention(dict(q=0, k=1, v=2, table=3, q_out=4, k_cache=5, v_cache=6), [item], m.heads,
                                m.kv_heads, m.dim, m.dim, self.dtype, qb, kb, vb)
        window = m.window if m.is_sliding(l) else C.FULL
        shape = C.GroupedShape(n, start, m.heads, m.kv_heads, m.dim, window, self.slots[l], 1.0 / np.sqrt(np.float32(m.dim)))
        end, slots = start + n, self.slots[l]
        if self.tiled and n >= 32:  # gpu.rs:777-793
            pad = (n + 31) // 32 * 32
            rows = slots if slots < end else (end + 31) // 32 * 32
            batch.attention_grouped_tiled_with_sinks(
                (C.Slice(4, 0, pad * self.qw * self.es), C.Slice(5, 0, rows * self.kw * self.es),
                 C.Slice(6, 0, rows * self.kw * self.es)), sinks, C.Slice(7, 0, pad * self.qw * self.es), shape,
                self.dtype)
        else:                       # gpu.rs:794-805
            rows = min(slots, end)
            batch.attention_grouped_with_sinks(
                (C.Slice(4, 0, n * self.qw * self.es), C.Slice(5, 0, rows * self.kw * self.es),
                 C.Slice(6, 0, rows * self.kw * self.es)), sinks, C.Slice(7, 0, n * self.qw * self.es), shape,
                self.dtype)
        done = batch.run()
        assert not isinstance(done.gpu_time, Exception), done.gpu_time
        batch.drop()

    def attention(self, l, start, n, window):
        if self.dtype == C.F32:
            return self.att.read(np.float32, count=n * self.qw).reshape(n, self.qw)
        return from_bf16_bits(self.att.read(np.uint16, count=n * self.qw)).reshape(n, self.qw)

    def close(self):
        for b in [self.q, self.k, self.v, self.table, self.q_out, self.att] + [b for p in self.caches for b in p] + \
                [r for w in self.weights for r in w]:
            b.free()


@pytest.fixture(scope="module")
def model():
    return tm.TinyModel(os.path.join(FIXTURE, "model.gguf"))


@pytest.mark.parametrize("chunk,tiled", [(1, False), (7, False), (40, False), (40, True), (32, True)])
def test_every_position_matches_transformers_in_f32(gpu, model, chunk, tiled):
    ids, want = tm.load_fixture(FIXTURE)
    s = DeviceSession(gpu, model, chunk, C.F32, tiled)
    try:
        got = model.forward(ids, s.prepare, s.attention, chunk=chunk)
    finally:
        s.close()
    worst = np.abs(got - want).max(axis=1)
    assert worst.max() < TOLERANCE, f"position {worst.argmax()}: max error {worst.max()}"


class Bf16Shadow:
    """The CPU oracle with bf16 q, k, v and output decides what the model sees; the device session is
    fed the same projections layer by layer and each of its attention outputs is held against the
    oracle's. (End to end in bf16 the logits of this random model are not a usable yardstick: a
    rounding difference can flip a near-tie in the expert router and move a logit by 0.9.)"""

    def __init__(self, device):
        self.dev, m = device, device.m
        self.k = [np.zeros((s, m.kv_heads * m.dim), np.uint16) for s in device.slots]
        self.v = [np.zeros((s, m.kv_heads * m.dim), np.uint16) for s in device.slots]
        self.worst = 0.0

    def prepare(self, l, q, k, v, start):
        m, layer = self.dev.m, self.dev.m.layers[l]
        self.dev.prepare(l, q, k, v, start)
        table = orc.rope_table(m.inv_freq, m.rope_scale, start, q.shape[0])
        self.q = orc.prepare(q, k, v, layer["q_bias"], layer["k_bias"], layer["v_bias"], table, self.k[l], self.v[l],
                             start, m.heads, m.kv_heads, m.dim, bf16=True)

    def attention(self, l, start, n, window):
        m, slots = self.dev.m, self.dev.slots[l]
        want = from_bf16_bits(orc.attention_bf16(self.q.reshape(n, m.heads, m.dim),
                                                 self.k[l].reshape(slots, m.kv_heads, m.dim),
                                                 self.v[l].reshape(slots, m.kv_heads, m.dim), m.layers[l]["sinks"],
                                                 start, window=window, slots=slots)).reshape(n, -1)
        got = self.dev.attention(l, start, n, window)
        self.worst = max(self.worst, float(np.abs(got - want).max()))
        assert not np.isnan(got).any()
        return want


@pytest.mark.parametrize("chunk,tiled", [(1, False), (40, False), (40, True)])
def test_bf16_session_follows_the_bf16_oracle_layer_by_layer(gpu, model, chunk, tiled):
    ids, _ = tm.load_fixture(FIXTURE)
    s = DeviceSession(gpu, model, chunk, C.BF16, tiled)
    shadow = Bf16Shadow(s)
    try:
        model.forward(ids, shadow.prepare, shadow.attention, chunk=chunk)
    finally:
        s.close()
    assert shadow.worst <= 2e-2, shadow.worst


class DeviceBlocks:
    """Every layer's whole attention block recorded in one batch, as gpt-oss/src/gpu.rs:703-827 records it:
    H -> X, RMS norm, the three Q8_0 projections, biases + rotation + cache append (one dispatch here), attention,
    output projection, its bias, the residual add into H. The host only uploads H and the rotary table and reads
    H back (the experts stay in numpy)."""

    def __init__(self, gpu, model, chunk, tiled, qkv_together=False):
        m = self.m = model
        self.gpu, self.chunk, self.tiled, self.qkv_together = gpu, chunk, tiled, qkv_together
        self.qw, self.kw = m.heads * m.dim, m.kv_heads * m.dim
        self.pad = pad = (chunk + 31) // 32 * 32
        self.slots = [((m.window + chunk + 31) // 32 * 32) if m.is_sliding(l) else 64 for l in range(m.layers_n)]
        f = lambda n: gpu.buffer(n * 4)
        self.H, self.X, self.TMP = f(pad * m.hidden), f(pad * m.hidden), f(pad * m.hidden)
        self.Q, self.K, self.V = f(pad * self.qw), f(pad * self.kw), f(pad * self.kw)
        self.QR, self.ATT, self.TABLE = f(pad * self.qw), f(pad * self.qw), f(pad * m.dim)
        for b in (self.X, self.QR, self.ATT):
            b.fill(0)  # padded rows of a tiled pass must be finite
        self.caches = []
        for l in range(m.layers_n):
            pair = (f(self.slots[l] * self.kw), f(self.slots[l] * self.kw))
            for b in pair:
                b.fill(0 if tiled else 0xFF)
            self.caches.append(pair)
        self.res = []
        for l in range(m.layers_n):
            layer, r = m.layers[l], {}
            for part in ("q", "k", "v", "output"):
                raw, rows, cols = m.q8_raw[f"blk.{l}.attn_{part}.weight"]
                codes, scales = C.split_q8_0_blocks(raw)
                r[part] = (gpu.resident(codes), gpu.resident(scales), rows, cols)
            for name in ("attn_norm", "q_bias", "k_bias", "v_bias", "o_bias", "sinks"):
                r[name] = gpu.resident(layer[name])
            self.res.append(r)

    def block(self, l, h, start):
        m, n, r = self.m, h.shape[0], self.res[l]
        hidden, qw, kw = m.hidden, self.qw, self.kw
        self.H.write(h)
        self.TABLE.write(C.rope_table(m.inv_freq, m.rope_scale, start, n))
        kc, vc = self.caches[l]
        bufs = [self.H, self.X, self.Q, self.K, self.V, self.TABLE, self.QR, kc, vc, self.ATT, self.TMP]
        H, X, Q, K, V, TABLE, QR, KC, VC, ATT, TMP = range(11)
        batch = self.gpu.batch(bufs)
        rows_of = lambda b, w, count=n: C.Slice(b, 0, count * w * 4)
        tiled = self.tiled and n >= 32
        n_run = (n + 31) // 32 * 32 if tiled else n

        def mul(part, x, y):  # gpu.rs:119-137
            codes, scales, rows, cols = r[part]
            mat = (batch.attach(codes), batch.attach(scales))
            xs, ys = rows_of(x, cols, n_run), rows_of(y, rows, n_run)
            if n == 1:
                batch.gemv_q8_0(mat, xs, ys, rows, cols)
            elif tiled and rows % 64 == 0:
                batch.gemm_q8_0_tiled(mat, xs, ys, rows, cols, n_run, (cols, rows))
            else:
                batch.gemm_q8_0(mat, xs, ys, rows, cols, n_run, (cols, rows))

        fused = self.qkv_together == "fused"  # norm folded into the projections, bias and residual into the output projection
        if not fused:
            batch.copy_rows((rows_of(H, hidden), hidden), (rows_of(X, hidden), hidden), n, hidden)
            batch.rmsnorm_rows((rows_of(X, hidden), batch.attach(r["attn_norm"])), n, (hidden, hidden), m.eps)
        if fused:
            mats = []
            for part, y in (("q", Q), ("k", K), ("v", V)):
                codes, scales, rows, cols = r[part]
                mats.append(((batch.attach(codes), batch.attach(scales)), rows_of(y, rows), rows))
            batch.gemm_q8_0_many_normed(mats, rows_of(H, hidden), (batch.attach(r["attn_norm"]), m.eps), hidden, n, hidden)
        elif self.qkv_together:  # the three projections as one call (one dispatch below 32 positions)
            mats = []
            for part, y in (("q", Q), ("k", K), ("v", V)):
                codes, scales, rows, cols = r[part]
                mats.append(((batch.attach(codes), batch.attach(scales)), rows_of(y, rows, n_run), rows))
            batch.gemm_q8_0_many(mats, rows_of(X, cols, n_run), cols, n_run, cols)
        else:
            mul("q", X, Q)
            mul("k", X, K)
            mul("v", X, V)
        item = C.PrepareItem(n=n, start=start, slots=self.slots[l])
        batch.prepare_attention(dict(q=Q, k=K, v=V, table=TABLE, q_out=QR, k_cache=KC, v_cache=VC), [item], m.heads,
                                m.kv_heads, m.dim, m.dim, C.F32, batch.attach(r["q_bias"]), batch.attach(r["k_bias"]),
                                batch.attach(r["v_bias"]))
        window = m.window if m.is_sliding(l) else C.FULL
        slots, end = self.slots[l], start + n
        shape = C.GroupedShape(n, start, m.heads, m.kv_heads, m.dim, window, slots, 1.0 / np.sqrt(np.float32(m.dim)))
        sinks = batch.attach(r["sinks"])
        if tiled:
            rows = slots if slots < end else (end + 31) // 32 * 32
            batch.attention_grouped_tiled_with_sinks((rows_of(QR, qw, n_run), rows_of(KC, kw, rows), rows_of(VC, kw, rows)),
                                                     sinks, rows_of(ATT, qw, n_run), shape, C.F32)
        else:
            rows = min(slots, end)
            batch.attention_grouped_with_sinks((rows_of(QR, qw), rows_of(KC, kw, rows), rows_of(VC, kw, rows)), sinks,
                                               rows_of(ATT, qw), shape, C.F32)
        if fused:
            codes, scales, rows, cols = r["output"]
            batch.gemm_q8_0_residual((batch.attach(codes), batch.attach(scales)), rows_of(ATT, cols), batch.attach(r["o_bias"]),
                                     rows_of(H, hidden), rows, cols, n, (cols, hidden))
        else:
            mul("output", ATT, TMP)
            batch.add_rows(rows_of(TMP, hidden), (batch.attach(r["o_bias"]), 0), n, hidden)
            batch.add_rows(rows_of(H, hidden), (rows_of(TMP, hidden), hidden), n, hidden)
        done = batch.run()
        assert not isinstance(done.gpu_time, Exception), done.gpu_time
        batch.drop()
        return self.H.read(np.float32, count=n * hidden).reshape(n, hidden)

    def close(self):
        for b in [self.H, self.X, self.TMP, self.Q, self.K, self.V, self.QR, self.ATT, self.TABLE] + \
                [b for p in self.caches for b in p]:
            b.free()
        for r in self.res:
            for v in r.values():
                for b in (v[:2] if isinstance(v, tuple) else (v,)):
                    b.free()


@pytest.mark.parametrize("chunk,tiled,qkv_together", [(1, False, False), (9, False, False), (40, False, False), (40, True, False),
                                                      (1, False, True), (9, False, True), (40, True, True),
                                                      (1, False, "fused"), (9, False, "fused")])
def test_whole_attention_blocks_on_the_device_match_transformers(gpu, model, chunk, tiled, qkv_together):
    ids, want = tm.load_fixture(FIXTURE)
    s = DeviceBlocks(gpu, model, chunk, tiled, qkv_together)
    try:
        got = model.forward(ids, None, None, chunk=chunk, block=s.block)
    finally:
        s.close()
    worst = np.abs(got - want).max(axis=1)
    assert worst.max() < TOLERANCE, f"position {worst.argmax()}: max error {worst.max()}"


@pytest.mark.parametrize("chunk,back", [(5, 5), (5, 3), (8, 8)])
def test_truncating_a_session_and_feeding_it_again_gives_the_same_logits(gpu, model, chunk, back):
    """`Session::truncate` (model.rs:203-213; gpu.rs:403-409: at most one chunk back, which the rings of
    window + chunk rows still hold): after 40 positions the session goes back `back` positions and the
    same tokens are fed again over the same device caches."""
    ids, want = tm.load_fixture(FIXTURE)
    s = DeviceSession(gpu, model, chunk, C.F32, False)
    try:
        got = model.forward(ids, s.prepare, s.attention, chunk=chunk)
        again = model.forward(ids[40 - back:], s.prepare, s.attention, chunk=chunk, first=40 - back)
    finally:
        s.close()
    assert np.abs(got - want).max() < TOLERANCE
    assert np.abs(again - want[40 - back:]).max() < TOLERANCE
    assert np.abs(again - got[40 - back:]).max() < 1e-5
