"""TEST INFRASTRUCTURE — NOT PRODUCT CODE.

ctypes access to ``liblng_oracle.so`` (built from ``attention_oracle.c``, which cites the
reference lines each function restates). Only ``tests/``, ``__graft_entry__.smoke`` and the
``cpu_baseline`` leg of ``bench.py`` import this module; ``loadngo_amd`` never does.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liblng_oracle.so")
FULL = 2**64 - 1  # GroupedShape.window = usize::MAX: every earlier position is visible

_u64 = ctypes.c_uint64
_fp = ctypes.POINTER(ctypes.c_float)
_hp = ctypes.POINTER(ctypes.c_uint16)


def build():
    """Compiles the oracle with the committed Makefile."""
    subprocess.check_call(["make", "-C", _HERE, "-B", "liblng_oracle.so"], stdout=subprocess.DEVNULL)


def _load():
    if not os.path.exists(_LIB_PATH):
        build()
    lib = ctypes.CDLL(_LIB_PATH)
    lib.lng_oracle_bf16_to_f32.restype = ctypes.c_float
    lib.lng_oracle_bf16_to_f32.argtypes = [ctypes.c_uint16]
    lib.lng_oracle_f32_to_bf16.restype = ctypes.c_uint16
    lib.lng_oracle_f32_to_bf16.argtypes = [ctypes.c_float]
    lib.lng_oracle_widen.argtypes = [_hp, _fp, ctypes.c_size_t]
    lib.lng_oracle_narrow.argtypes = [_fp, _hp, ctypes.c_size_t]
    lib.lng_oracle_values.argtypes = [_u64, ctypes.c_size_t, _fp]
    lib.lng_oracle_ring_rows.restype = ctypes.c_size_t
    lib.lng_oracle_ring_rows.argtypes = [_u64, _u64, _u64, ctypes.c_int]
    lib.lng_oracle_ring.restype = ctypes.c_size_t
    lib.lng_oracle_ring.argtypes = [_fp, ctypes.c_size_t, _u64, _u64, _u64, ctypes.c_int, _fp]
    lib.lng_oracle_accepts.restype = ctypes.c_int
    lib.lng_oracle_accepts.argtypes = [_u64] * 7 + [ctypes.c_int]
    attn = [_fp, _fp, _fp, _fp, _fp] + [_u64] * 7 + [ctypes.c_float, ctypes.c_int]
    lib.lng_oracle_attention_f32.argtypes = attn
    lib.lng_oracle_attention_f64.argtypes = attn
    lib.lng_oracle_attention_bf16.argtypes = (
        [_hp, _hp, _hp, _fp, _hp] + [_u64] * 8 + [ctypes.c_float, ctypes.c_int]
    )
    lib.lng_oracle_attention_rows_f32.argtypes = (
        [_fp, _fp, _fp, _fp, _fp, ctypes.POINTER(_u64)] + [_u64] * 6 + [ctypes.c_float, ctypes.c_int]
    )
    _dp = ctypes.POINTER(ctypes.c_double)
    lib.lng_oracle_add_rows.argtypes = [_fp, _fp, _u64, _u64, _u64]
    lib.lng_oracle_rope_table.argtypes = [_fp, _dp, _u64, ctypes.c_double, _u64, _u64]
    lib.lng_oracle_rotate_halves.argtypes = [_fp, _fp, _u64, _u64, _u64, _u64]
    lib.lng_oracle_prepare.argtypes = [_fp] * 7 + [ctypes.c_void_p] * 3 + [_u64] * 7 + [ctypes.c_int]
    _bp = ctypes.POINTER(ctypes.c_int8)
    lib.lng_oracle_f16_to_f32.restype = ctypes.c_float
    lib.lng_oracle_f16_to_f32.argtypes = [ctypes.c_uint16]
    lib.lng_oracle_q8_split_blocks.argtypes = [ctypes.POINTER(ctypes.c_uint8), ctypes.c_size_t, _bp, _hp]
    lib.lng_oracle_q8_mul.argtypes = [_bp, _hp, _fp, _fp] + [_u64] * 5
    lib.lng_oracle_q8_mul_f64.argtypes = [_bp, _hp, _fp, ctypes.POINTER(ctypes.c_double)] + [_u64] * 5
    lib.lng_oracle_rms_norm_rows.argtypes = [_fp, _fp, _u64, _u64, _u64, ctypes.c_float]
    return lib


_lib = _load()


def _f(a):
    return a.ctypes.data_as(_fp)


def _h(a):
    return a.ctypes.data_as(_hp)


def bf16_to_f32(bits):
    """weights/src/dtype.rs:95-97. ``bits``: uint16 array or scalar."""
    a = np.ascontiguousarray(bits, dtype=np.uint16)
    out = np.empty(a.shape, dtype=np.float32)
    _lib.lng_oracle_widen(_h(a.reshape(-1)), _f(out.reshape(-1)), a.size)
    return out


def f32_to_bf16(values):
    """weights/src/dtype.rs:101-109. Returns uint16 bit patterns."""
    a = np.ascontiguousarray(values, dtype=np.float32)
    out = np.empty(a.shape, dtype=np.uint16)
    _lib.lng_oracle_narrow(_f(a.reshape(-1)), _h(out.reshape(-1)), a.size)
    return out


def values(seed, n):
    """metal-compute/tests/attention_grouped.rs:25-35."""
    out = np.empty(n, dtype=np.float32)
    _lib.lng_oracle_values(seed, n, _f(out))
    return out


def ring(all_rows, t, start, slots, tiled):
    """metal-compute/tests/attention_grouped.rs:47-63. ``all_rows``: [start+t][row] f32."""
    all_rows = np.ascontiguousarray(all_rows, dtype=np.float32)
    row = all_rows.shape[1]
    rows = _lib.lng_oracle_ring_rows(t, start, slots, int(tiled))
    out = np.empty((rows, row), dtype=np.float32)
    _lib.lng_oracle_ring(_f(all_rows), row, t, start, slots, int(tiled), _f(out))
    return out


def accepts(t, start, heads, kv_heads, dim, window, slots, tiled=False):
    """metal-compute/src/apple.rs:1243-1272 and 1356-1385."""
    for value in (t, start, heads, kv_heads, dim, window, slots):  # ctypes would wrap 2**64 to 0 without a word
        assert 0 <= int(value) < 2**64 and int(value) == value, value
    return bool(_lib.lng_oracle_accepts(t, start, heads, kv_heads, dim, window, slots, int(tiled)))


def _attention(fn, q, k, v, sinks, start, window, slots, scale, threads):
    q = np.ascontiguousarray(q, dtype=np.float32)
    k = np.ascontiguousarray(k, dtype=np.float32)
    v = np.ascontiguousarray(v, dtype=np.float32)
    t, heads, dim = q.shape
    kv_heads = k.shape[1]
    assert k.shape == v.shape and k.shape[2] == dim
    assert k.shape[0] >= min(slots, start + t), "cache holds too few rows"
    out = np.empty_like(q)
    s = None if sinks is None else np.ascontiguousarray(sinks, dtype=np.float32)
    fn(_f(q), _f(k), _f(v), None if s is None else _f(s), _f(out), t, start, heads, kv_heads, dim,
       window, slots, scale, threads)
    return out


def attention_f32(q, k, v, sinks, start, window=FULL, slots=None, scale=None, threads=1):
    """gpt-oss/src/model.rs:434-464 over q [t][H][D], k/v [rows][G][D] (row = pos % slots)."""
    slots = k.shape[0] if slots is None else slots
    scale = 1.0 / np.sqrt(np.float32(q.shape[2])) if scale is None else scale
    return _attention(_lib.lng_oracle_attention_f32, q, k, v, sinks, start, window, slots,
                      float(scale), threads)


def attention_f64(q, k, v, sinks, start, window=FULL, slots=None, scale=None, threads=1):
    """metal-compute/tests/attention_grouped.rs:65-100."""
    slots = k.shape[0] if slots is None else slots
    scale = 1.0 / np.sqrt(np.float32(q.shape[2])) if scale is None else scale
    return _attention(_lib.lng_oracle_attention_f64, q, k, v, sinks, start, window, slots,
                      float(scale), threads)


def attention_bf16(q, k, v, sinks, start, window=FULL, slots=None, scale=None, threads=1):
    """bf16 bit patterns in and out (uint16 arrays), f32 arithmetic of model.rs:434-464."""
    q = np.ascontiguousarray(q, dtype=np.uint16)
    k = np.ascontiguousarray(k, dtype=np.uint16)
    v = np.ascontiguousarray(v, dtype=np.uint16)
    t, heads, dim = q.shape
    rows, kv_heads, _ = k.shape
    slots = rows if slots is None else slots
    scale = 1.0 / np.sqrt(np.float32(dim)) if scale is None else scale
    assert rows >= min(slots, start + t), "cache holds too few rows"
    out = np.empty_like(q)
    s = None if sinks is None else np.ascontiguousarray(sinks, dtype=np.float32)
    _lib.lng_oracle_attention_bf16(_h(q), _h(k), _h(v), None if s is None else _f(s), _h(out), rows,
                                   t, start, heads, kv_heads, dim, window, slots, float(scale),
                                   threads)
    return out


def attention_rows_f32(q, k, v, sinks, positions, window=FULL, slots=None, scale=None, threads=1):
    """Row i of q attends from absolute position positions[i] (a sample of a long pass)."""
    q = np.ascontiguousarray(q, dtype=np.float32)
    k = np.ascontiguousarray(k, dtype=np.float32)
    v = np.ascontiguousarray(v, dtype=np.float32)
    n, heads, dim = q.shape
    kv_heads = k.shape[1]
    slots = k.shape[0] if slots is None else slots
    scale = 1.0 / np.sqrt(np.float32(dim)) if scale is None else scale
    pos = np.ascontiguousarray(positions, dtype=np.uint64)
    assert pos.shape == (n,)
    out = np.empty_like(q)
    s = None if sinks is None else np.ascontiguousarray(sinks, dtype=np.float32)
    _lib.lng_oracle_attention_rows_f32(_f(q), _f(k), _f(v), None if s is None else _f(s), _f(out),
                                       pos.ctypes.data_as(ctypes.POINTER(_u64)), n, heads, kv_heads,
                                       dim, window, slots, float(scale), threads)
    return out


def add_rows(dst, src, src_stride):
    """dst[r] + src[r * src_stride:][:width] (a stride of 0 adds one row to every row)."""
    out = np.ascontiguousarray(dst, dtype=np.float32).copy()
    src = np.ascontiguousarray(src, dtype=np.float32)
    rows, width = out.shape
    _lib.lng_oracle_add_rows(_f(out), _f(src), rows, width, src_stride)
    return out


def rope_table(inv_freq, scale, start, n):
    """[n][half][2] f32: (cos, sin) of position * inv_freq, times scale."""
    inv = np.ascontiguousarray(inv_freq, dtype=np.float64)
    table = np.empty((n, len(inv), 2), dtype=np.float32)
    _lib.lng_oracle_rope_table(_f(table), inv.ctypes.data_as(ctypes.POINTER(ctypes.c_double)), len(inv),
                               float(scale), start, n)
    return table


def rotate_halves(x, table, heads, dim, rotary=None):
    """x [rows][heads*dim] rotated by table [rows][rotary/2][2]."""
    out = np.ascontiguousarray(x, dtype=np.float32).copy()
    table = np.ascontiguousarray(table, dtype=np.float32)
    _lib.lng_oracle_rotate_halves(_f(out), _f(table), out.shape[0], heads, dim, rotary or dim)
    return out


def prepare(q, k, v, q_bias, k_bias, v_bias, table, k_cache, v_cache, start, heads, kv_heads, dim,
            rotary=None, bf16=False):
    """The step before attention on n rows; writes rows (start + r) % slots of k_cache / v_cache
    in place (f32 arrays, or uint16 bf16 bit arrays when bf16) and returns the prepared queries."""
    q, k, v = (np.ascontiguousarray(a, dtype=np.float32) for a in (q, k, v))
    table = np.ascontiguousarray(table, dtype=np.float32)
    n, slots = q.shape[0], k_cache.shape[0]
    want = np.uint16 if bf16 else np.float32
    assert k_cache.dtype == want and v_cache.dtype == want
    assert k_cache.flags.c_contiguous and v_cache.flags.c_contiguous
    q_out = np.empty((n, heads * dim), dtype=want)
    bias = [None if b is None else np.ascontiguousarray(b, dtype=np.float32) for b in (q_bias, k_bias, v_bias)]
    _lib.lng_oracle_prepare(_f(q), _f(k), _f(v), *[None if b is None else _f(b) for b in bias], _f(table),
                            q_out.ctypes.data, k_cache.ctypes.data, v_cache.ctypes.data, n, start, slots,
                            heads, kv_heads, dim, rotary or dim, int(bf16))
    return q_out


def f16_to_f32(bits):
    """binary16 bit patterns (uint16 array) widened to f32."""
    b = np.ascontiguousarray(bits, dtype=np.uint16)
    return np.array([_lib.lng_oracle_f16_to_f32(int(v)) for v in b.reshape(-1)], dtype=np.float32).reshape(b.shape)


def q8_split_blocks(raw):
    """ggml Q8_0 blocks (bytes) -> (codes int8 [32 * blocks], scales uint16 [blocks])."""
    raw = np.ascontiguousarray(np.frombuffer(raw, dtype=np.uint8) if isinstance(raw, (bytes, bytearray, memoryview)) else raw,
                               dtype=np.uint8)
    assert raw.size % 34 == 0, "whole Q8_0 blocks"
    n = raw.size // 34
    codes, scales = np.empty(32 * n, np.int8), np.empty(n, np.uint16)
    _lib.lng_oracle_q8_split_blocks(raw.ctypes.data_as(ctypes.POINTER(ctypes.c_uint8)), n,
                                    codes.ctypes.data_as(ctypes.POINTER(ctypes.c_int8)), _h(scales))
    return codes, scales


def _q8(fn, kind, codes, scales, x, rows, cols, y_stride):
    codes = np.ascontiguousarray(codes, dtype=np.int8)
    scales = np.ascontiguousarray(scales, dtype=np.uint16)
    x = np.ascontiguousarray(x, dtype=np.float32)
    assert codes.size == rows * cols and scales.size == rows * cols // 32 and cols % 32 == 0
    n, x_stride = x.shape
    assert x_stride >= cols
    y_stride = rows if y_stride is None else y_stride
    y = np.zeros((n, y_stride), dtype=kind)
    fn(codes.ctypes.data_as(ctypes.POINTER(ctypes.c_int8)), _h(scales), _f(x),
       y.ctypes.data_as(ctypes.POINTER(ctypes.c_double if kind == np.float64 else ctypes.c_float)),
       rows, cols, n, x_stride, y_stride)
    return y


def q8_mul(codes, scales, x, rows, cols, y_stride=None):
    """y[p] = W x[p], f32 as the reference's CPU product: x is [n][x_stride >= cols]."""
    return _q8(_lib.lng_oracle_q8_mul, np.float32, codes, scales, x, rows, cols, y_stride)


def q8_mul_f64(codes, scales, x, rows, cols, y_stride=None):
    """The same product by its float64 definition."""
    return _q8(_lib.lng_oracle_q8_mul_f64, np.float64, codes, scales, x, rows, cols, y_stride)


def rms_norm_rows(v, w, d=None, eps=1e-5):
    """The first d floats of each row of v [rows][stride] normalised and weighted (a copy)."""
    out = np.ascontiguousarray(v, dtype=np.float32).copy()
    w = np.ascontiguousarray(w, dtype=np.float32)
    rows, stride = out.shape
    d = stride if d is None else d
    _lib.lng_oracle_rms_norm_rows(_f(out), _f(w), rows, d, stride, float(eps))
    return out
