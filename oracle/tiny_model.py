"""TEST INFRASTRUCTURE - a numpy restatement of the reference's whole gpt-oss forward pass.

Only tests may import this file. It exists so that the attention path (the CPU oracle, or the
HIP library behind the C ABI) can be driven by the one end-to-end golden the reference holds:
`gpt-oss/tests/fixtures/tiny/{model.gguf,oracle.json,logits.f32}`, transformers' logits for a
random 4-layer gpt-oss with a sliding window of 8 over 40 positions, which
`gpt-oss/tests/tiny_oracle.rs:10-40` requires the forward pass to meet within 2e-3.

Everything around attention follows the reference's CPU model:

* GGUF header and tensor table: `weights/src/gguf.rs:259-353` (little-endian; magic, version,
  counts, metadata, tensor descriptions, data aligned to `general.alignment` or 32).
* Q8_0 blocks (f16 scale + 32 signed bytes): `weights/src/q8_0.rs:80-97`.
* ggml MXFP4 blocks (E8M0 scale byte + 16 bytes, low nibbles = elements 0-15, high nibbles =
  elements 16-31; E2M1 codes): `weights/src/mxfp4.rs:16-42,119-151`.
* Shape from metadata: `gpt-oss/src/config.rs:38-99`; YaRN frequencies: `config.rs:105-133`.
* RMS norm: `model.rs:274-280`; rotation by halves: `model.rs:389-404`; the layer loop:
  `model.rs:408-478`; routing and experts: `model.rs:482-548`.

Attention itself (`model.rs:434-464`) is NOT restated here: `forward` takes it as a callable,
and so it takes the step before it (bias, rotation, cache append), so that a test can put the
C oracle or the device kernels in those two places.
"""
import json
import struct

import numpy as np

FULL = 2**64 - 1

_SCALAR = {0: "<B", 1: "<b", 2: "<H", 3: "<h", 4: "<I", 5: "<i", 6: "<f", 7: "<?",
           10: "<Q", 11: "<q", 12: "<d"}
# ggml type id -> (elements per block, bytes per block), gguf.rs:108-127
_BLOCK = {0: (1, 4), 1: (1, 2), 8: (32, 34), 30: (1, 2), 39: (32, 17)}
F32, Q8_0, MXFP4 = 0, 8, 39


class _Cursor:
    def __init__(self, data):
        self.data, self.at = data, 0

    def unpack(self, fmt):
        (value,) = struct.unpack_from(fmt, self.data, self.at)
        self.at += struct.calcsize(fmt)
        return value

    def string(self):
        n = self.unpack("<Q")
        text = bytes(self.data[self.at:self.at + n]).decode("utf-8")
        self.at += n
        return text

    def value(self, kind):
        if kind == 8:
            return self.string()
        if kind == 9:
            element, n = self.unpack("<I"), self.unpack("<Q")
            return [self.value(element) for _ in range(n)]
        return self.unpack(_SCALAR[kind])


def read_gguf(path):
    """(metadata, tensors): tensors maps a name to (dims, ggml type id, bytes)."""
    data = memoryview(open(path, "rb").read())
    at = _Cursor(data)
    if bytes(data[:4]) != b"GGUF":
        raise ValueError("not a GGUF file")
    at.at = 4
    version = at.unpack("<I")
    if version not in (2, 3):
        raise ValueError(f"GGUF version {version}")
    n_tensors, n_meta = at.unpack("<Q"), at.unpack("<Q")
    meta = {}
    for _ in range(n_meta):
        key = at.string()
        meta[key] = at.value(at.unpack("<I"))
    align = int(meta.get("general.alignment", 32))
    described = []
    for _ in range(n_tensors):
        name = at.string()
        dims = [at.unpack("<Q") for _ in range(at.unpack("<I"))]
        described.append((name, dims, at.unpack("<I"), at.unpack("<Q")))
    start = -(-at.at // align) * align
    tensors = {}
    for name, dims, kind, relative in described:
        per, size = _BLOCK[kind]
        n = int(np.prod(dims)) // per * size
        tensors[name] = (dims, kind, bytes(data[start + relative:start + relative + n]))
    return meta, tensors


def dequant_q8_0(raw, rows, cols):
    """element = d * q, exact in f32 (q8_0.rs:80-97)."""
    blocks = np.frombuffer(raw, dtype=np.uint8).reshape(rows, cols // 32, 34)
    d = blocks[:, :, :2].copy().view("<f2").astype(np.float32)          # [rows][blocks][1]
    q = blocks[:, :, 2:].view(np.int8).astype(np.float32)
    return (d * q).reshape(rows, cols)


_E2M1 = np.array([0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0], dtype=np.float32)


def dequant_mxfp4(raw, rows, cols):
    """element = 2^(scale - 127) * E2M1(code) (mxfp4.rs:16-42, ggml block order 119-151)."""
    blocks = np.frombuffer(raw, dtype=np.uint8).reshape(rows, cols // 32, 17)
    scale = blocks[:, :, :1].astype(np.int32)
    if (scale == 255).any():
        raise ValueError("NaN scale")
    power = np.ldexp(np.float32(1.0), scale - 127).astype(np.float32)
    codes = np.concatenate([blocks[:, :, 1:] & 0x0F, blocks[:, :, 1:] >> 4], axis=2)
    value = _E2M1[codes & 7] * np.where(codes & 8, np.float32(-1.0), np.float32(1.0))
    return (value * power).astype(np.float32).reshape(rows, cols)


def _matrix(kind, raw, rows, cols):
    if kind == F32:
        return np.frombuffer(raw, dtype="<f4").reshape(rows, cols).copy()
    if kind == Q8_0:
        return dequant_q8_0(raw, rows, cols)
    if kind == MXFP4:
        return dequant_mxfp4(raw, rows, cols)
    raise ValueError(f"matrices of ggml type {kind}")


def _mul(w, x):
    """rows of x through W: f64 accumulation, f32 result (the reference sums in f32 or f64
    depending on the format; both are far inside the fixture's 2e-3)."""
    return (x.astype(np.float64) @ w.astype(np.float64).T).astype(np.float32)


def rms_norm(x, weight, eps):
    """model.rs:274-280: the mean square in f64, the scale as one f32, x * scale * w in f32."""
    mean = (x.astype(np.float64) ** 2).mean(axis=-1, keepdims=True)
    scale = (1.0 / np.sqrt(mean + np.float64(np.float32(eps)))).astype(np.float32)
    return x * scale * weight


class TinyModel:
    def __init__(self, path):
        meta, t = read_gguf(path)
        g = lambda key: meta["gpt-oss." + key]
        if meta.get("general.architecture") != "gpt-oss" or g("rope.scaling.type") != "yarn":
            raise ValueError("not a YaRN gpt-oss file")
        self.layers_n = g("block_count")
        self.hidden = g("embedding_length")
        self.heads = g("attention.head_count")
        self.kv_heads = g("attention.head_count_kv")
        self.dim = g("attention.key_length")
        self.experts = g("expert_count")
        self.used = g("expert_used_count")
        self.expert_hidden = g("expert_feed_forward_length")
        self.window = g("attention.sliding_window")
        self.eps = g("attention.layer_norm_rms_epsilon")
        self.theta = float(g("rope.freq_base"))
        self.original = float(g("rope.scaling.original_context_length"))
        self.factor = float(g("rope.scaling.factor"))
        self.vocab = t["token_embd.weight"][0][1]
        self.inv_freq, self.rope_scale = self._rope()

        def vector(name, n):
            dims, kind, raw = t[name]
            assert kind == F32 and int(np.prod(dims)) == n, name
            return np.frombuffer(raw, dtype="<f4").copy()

        self.q8_raw = {}  # tensor name -> (ggml Q8_0 block bytes, rows, cols), for tests of Q8_0 products

        def matrix(name, rows, cols):
            dims, kind, raw = t[name]
            assert dims == [cols, rows], (name, dims)
            if kind == Q8_0:
                self.q8_raw[name] = (raw, rows, cols)
            return _matrix(kind, raw, rows, cols)

        def experts(name, rows, cols):
            dims, kind, raw = t[name]
            assert dims == [cols, rows, self.experts], (name, dims)
            each = len(raw) // self.experts
            return [_matrix(kind, raw[e * each:(e + 1) * each], rows, cols) for e in range(self.experts)]

        qw, kw = self.heads * self.dim, self.kv_heads * self.dim
        self.embedding = matrix("token_embd.weight", self.vocab, self.hidden)
        self.output = matrix("output.weight", self.vocab, self.hidden)
        self.output_norm = vector("output_norm.weight", self.hidden)
        self.layers = []
        for l in range(self.layers_n):
            n = lambda part: f"blk.{l}.{part}"
            self.layers.append(dict(
                attn_norm=vector(n("attn_norm.weight"), self.hidden),
                q=matrix(n("attn_q.weight"), qw, self.hidden),
                k=matrix(n("attn_k.weight"), kw, self.hidden),
                v=matrix(n("attn_v.weight"), kw, self.hidden),
                o=matrix(n("attn_output.weight"), self.hidden, qw),
                q_bias=vector(n("attn_q.bias"), qw), k_bias=vector(n("attn_k.bias"), kw),
                v_bias=vector(n("attn_v.bias"), kw), o_bias=vector(n("attn_output.bias"), self.hidden),
                sinks=vector(n("attn_sinks.weight"), self.heads),
                ffn_norm=vector(n("post_attention_norm.weight"), self.hidden),
                router=matrix(n("ffn_gate_inp.weight"), self.experts, self.hidden),
                router_bias=vector(n("ffn_gate_inp.bias"), self.experts),
                gate=experts(n("ffn_gate_exps.weight"), self.expert_hidden, self.hidden),
                up=experts(n("ffn_up_exps.weight"), self.expert_hidden, self.hidden),
                down=experts(n("ffn_down_exps.weight"), self.hidden, self.expert_hidden),
                gate_bias=vector(n("ffn_gate_exps.bias"), self.experts * self.expert_hidden)
                .reshape(self.experts, -1),
                up_bias=vector(n("ffn_up_exps.bias"), self.experts * self.expert_hidden)
                .reshape(self.experts, -1),
                down_bias=vector(n("ffn_down_exps.bias"), self.experts * self.hidden)
                .reshape(self.experts, -1),
            ))

    def _rope(self):
        """config.rs:105-133 (ramp bounds 32 and 1 rotations over the original context)."""
        dim, half = float(self.dim), self.dim // 2
        correction = lambda rot: dim * np.log(self.original / (rot * 2.0 * np.pi)) / (2.0 * np.log(self.theta))
        low, high = max(correction(32.0), 0.0), min(correction(1.0), dim - 1.0)
        if low == high:
            high += 0.001
        i = np.arange(half, dtype=np.float64)
        freq = self.theta ** (2.0 * i / dim)
        ramp = np.clip((i - low) / (high - low), 0.0, 1.0)
        inv = (1.0 / (self.factor * freq)) * ramp + (1.0 / freq) * (1.0 - ramp)
        scale = 1.0 if self.factor <= 1.0 else 0.1 * np.log(self.factor) + 1.0
        return inv, scale

    def is_sliding(self, layer):
        return layer % 2 == 0  # config.rs:101-103

    def rope_table(self, start, n):
        """[n][dim/2][2] f32 (cos, sin) * rope_scale for positions start..start+n, as the
        reference's GPU path tabulates them (gpu.rs:690-697); same numbers as model.rs:393-398."""
        angle = (start + np.arange(n, dtype=np.float64))[:, None] * self.inv_freq[None, :]
        return np.stack([(np.cos(angle) * self.rope_scale).astype(np.float32),
                         (np.sin(angle) * self.rope_scale).astype(np.float32)], axis=-1)

    def experts_out(self, layer, x):
        """model.rs:482-548 for one row x."""
        router = _mul(layer["router"], x[None, :])[0] + layer["router_bias"]
        order = sorted(range(self.experts), key=lambda e: (-router[e], e))[:self.used]
        w = np.exp(router[order] - router[order[0]]).astype(np.float32)
        w = w / w.sum(dtype=np.float32)
        out = np.zeros(self.hidden, dtype=np.float32)
        for e, weight in zip(order, w):
            g = np.minimum(_mul(layer["gate"][e], x[None, :])[0] + layer["gate_bias"][e], np.float32(7.0))
            u = np.clip(_mul(layer["up"][e], x[None, :])[0] + layer["up_bias"][e], np.float32(-7.0), np.float32(7.0))
            hidden = (u + np.float32(1.0)) * g / (np.float32(1.0) + np.exp(np.float32(-1.702) * g))
            y = _mul(layer["down"][e], hidden[None, :].astype(np.float32))[0] + layer["down_bias"][e]
            out += weight * y
        return out

    def forward(self, ids, prepare, attention, chunk=1, project=None, block=None, first=0):
        """Logits [len(ids)][vocab]. Positions are fed `chunk` at a time (1 = `Model::step`,
        model.rs:408-478; more = a prompt pass, gpu.rs:703-827). ids[0] sits at position `first`
        (a session that was truncated to `first` positions, model.rs:203-213, and is fed again).

        prepare(l, q, k, v, start) -> None: q [n][heads*dim], k, v [n][kv_heads*dim] are the raw
            projections of layer l for positions start..start+n; it must add the biases, rotate
            q and k, and append k and v to layer l's cache, keeping q for `attention`.
        attention(l, start, n, window) -> [n][heads*dim] f32: layer l's attention output for the
            rows `prepare` was just given.
        block(l, h, start) -> [n][hidden] f32, optional: the whole attention block of layer l
            (gpu.rs:703-827 up to the residual add: norm, projections, biases, rotation, cache append,
            attention, output projection and bias, h + result) in place of everything above.
        project(name, x) -> [n][rows] f32, optional: the product with the Q8_0 tensor `name`
            (blk.{l}.attn_{q,k,v,output}.weight; its blocks are in self.q8_raw) instead of this
            file's dequantise-and-multiply.
        """
        def mul(l, part, x):
            name = f"blk.{l}.attn_{part}.weight"
            if project is not None and name in self.q8_raw:
                return np.asarray(project(name, np.ascontiguousarray(x, dtype=np.float32)), dtype=np.float32)
            return _mul(self.layers[l][{"output": "o"}.get(part, part)], x)

        logits = np.zeros((len(ids), self.vocab), dtype=np.float32)
        for at in range(0, len(ids), chunk):
            tokens = ids[at:at + chunk]
            start = first + at
            n = len(tokens)
            h = self.embedding[tokens].copy()
            for l, layer in enumerate(self.layers):
                if block is not None:
                    h = np.asarray(block(l, np.ascontiguousarray(h, dtype=np.float32), start), dtype=np.float32)
                else:
                    x = rms_norm(h, layer["attn_norm"], self.eps)
                    prepare(l, mul(l, "q", x), mul(l, "k", x), mul(l, "v", x), start)
                    window = self.window if self.is_sliding(l) else FULL
                    attended = np.asarray(attention(l, start, n, window), dtype=np.float32).reshape(n, -1)
                    h = h + (mul(l, "output", attended) + layer["o_bias"])
                x = rms_norm(h, layer["ffn_norm"], self.eps)
                h = h + np.stack([self.experts_out(layer, x[i]) for i in range(n)])
            logits[at:at + n] = _mul(self.output, rms_norm(h, self.output_norm, self.eps))
        return logits


def rotate_halves(x, table, heads, dim):
    """model.rs:389-404 on rows: x [n][heads*dim], table [n][dim/2][2]; element i of a head's
    first half turns with element i of its second half; every product and difference rounds
    to f32 on its own."""
    n, half = x.shape[0], dim // 2
    x = x.reshape(n, heads, dim)
    cos, sin = table[:, None, :, 0], table[:, None, :, 1]
    a, b = x[:, :, :half], x[:, :, half:]
    out = np.empty_like(x)
    out[:, :, :half] = (a * cos).astype(np.float32) - (b * sin).astype(np.float32)
    out[:, :, half:] = (b * cos).astype(np.float32) + (a * sin).astype(np.float32)
    return out.reshape(n, heads * dim)


def load_fixture(directory):
    """(ids, want[positions][vocab]) of a `tiny` fixture directory."""
    meta = json.load(open(f"{directory}/oracle.json"))
    want = np.fromfile(f"{directory}/logits.f32", dtype="<f4").reshape(meta["positions"], meta["vocab"])
    return meta["ids"], want
