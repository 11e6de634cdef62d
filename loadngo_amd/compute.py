"""Host-side mirror of loadngo's ``metal-compute`` operator interface for the attention
path, over the C ABI of ``liblng_hip.so`` (``include/lng_hip.h``).

Names, argument meaning and error behaviour follow metal-compute/src/apple.rs and lib.rs:
``Gpu`` (apple.rs:105), ``Buffer`` (391), ``Resident`` (465), ``Slice`` (507), ``Batch`` (541),
``GroupedShape`` (598), ``Completed`` (536), ``Error`` (lib.rs:41-53). Device memory is not
CPU-visible here, so ``Buffer.as_f32()`` style access is ``Buffer.write`` / ``Buffer.read``.

There is no CPU fallback: without the built library, or without a HIP device, construction
fails (``Error.Compile`` / ``Error.NoDevice``).
"""
import ctypes
import os
import threading

import numpy as np

FULL = 2**64 - 1  # GroupedShape.window = usize::MAX
NO_SINKS = 2**64 - 1
F32, BF16 = 0, 1

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "liblng_hip.so")


class Error(Exception):
    """metal-compute/src/lib.rs:41-53."""


class NoDevice(Error):
    pass


class Compile(Error):
    pass


class Alloc(Error):
    pass


class Dispatch(Error):
    pass


class GpuFailure(Error):  # Error::Gpu
    pass


Error.NoDevice, Error.Compile, Error.Alloc, Error.Dispatch, Error.Gpu = (
    NoDevice, Compile, Alloc, Dispatch, GpuFailure)
_ERRORS = {-1: NoDevice, -2: Compile, -3: Alloc, -4: Dispatch, -5: GpuFailure}


class _Slice(ctypes.Structure):
    _fields_ = [("buffer", ctypes.c_uint64), ("offset", ctypes.c_uint64), ("len", ctypes.c_uint64)]


class _Shape(ctypes.Structure):
    _fields_ = [(n, ctypes.c_uint64) for n in ("t", "start", "heads", "kv_heads", "dim", "window", "slots")]
    _fields_.append(("scale", ctypes.c_float))


class _Item(ctypes.Structure):
    _fields_ = [(n, ctypes.c_uint64) for n in
                ("q_offset", "out_offset", "k_offset", "v_offset", "sinks_offset", "start", "window", "slots")]


_PREPARE_FIELDS = ("q_offset", "k_offset", "v_offset", "table_offset", "q_out_offset", "k_cache_offset",
                   "v_cache_offset", "n", "start", "slots")


class _PrepareItem(ctypes.Structure):
    _fields_ = [(n, ctypes.c_uint64) for n in _PREPARE_FIELDS]


class _PrepareBuffers(ctypes.Structure):
    _fields_ = [(n, ctypes.c_uint64) for n in ("q", "k", "v", "table", "q_out", "k_cache", "v_cache")] + \
               [(n, ctypes.POINTER(_Slice)) for n in ("q_bias", "k_bias", "v_bias")]


class _Q8Matrix(ctypes.Structure):
    _fields_ = [("codes", _Slice), ("scales", _Slice), ("y", _Slice), ("rows", ctypes.c_uint64)]


class _Completed(ctypes.Structure):
    _fields_ = [("status", ctypes.c_int), ("gpu_seconds", ctypes.c_double), ("message", ctypes.c_char_p)]


_ON_DONE = ctypes.CFUNCTYPE(None, ctypes.POINTER(_Completed), ctypes.c_void_p)

# Every symbol include/lng_hip.h declares: (restype, argtypes)
_P = ctypes.c_void_p
_U64 = ctypes.c_uint64
SYMBOLS = {
    "lng_hip_last_error": (ctypes.c_char_p, []),
    "lng_hip_open": (ctypes.c_int, [ctypes.c_int, ctypes.POINTER(_P)]),
    "lng_hip_close": (None, [_P]),
    "lng_hip_device_name": (ctypes.c_int, [_P, ctypes.c_char_p, ctypes.c_size_t]),
    "lng_hip_debug_set": (ctypes.c_int, [_P, ctypes.c_char_p, ctypes.c_char_p]),
    "lng_hip_debug_get": (ctypes.c_int, [_P, ctypes.c_char_p, ctypes.POINTER(ctypes.c_uint64)]),
    "lng_hip_buffer": (ctypes.c_int, [_P, ctypes.c_size_t, ctypes.POINTER(_P)]),
    "lng_hip_resident": (ctypes.c_int, [_P, _P, ctypes.c_size_t, ctypes.POINTER(_P)]),
    "lng_hip_buffer_free": (ctypes.c_int, [_P]),
    "lng_hip_buffer_len": (ctypes.c_size_t, [_P]),
    "lng_hip_buffer_device_ptr": (_P, [_P]),
    "lng_hip_upload": (ctypes.c_int, [_P, ctypes.c_size_t, _P, ctypes.c_size_t]),
    "lng_hip_download": (ctypes.c_int, [_P, ctypes.c_size_t, _P, ctypes.c_size_t]),
    "lng_hip_fill": (ctypes.c_int, [_P, ctypes.c_size_t, ctypes.c_int, ctypes.c_size_t]),
    "lng_hip_batch": (ctypes.c_int, [_P, ctypes.POINTER(_P), ctypes.c_size_t, ctypes.POINTER(_P)]),
    "lng_hip_batch_attach": (ctypes.c_int, [_P, _P, ctypes.POINTER(_Slice)]),
    "lng_hip_batch_dispatches": (ctypes.c_size_t, [_P]),
    "lng_hip_batch_barrier": (ctypes.c_int, [_P]),
    "lng_hip_batch_commit": (ctypes.c_int, [_P, _ON_DONE, _P]),
    "lng_hip_batch_wait": (ctypes.c_int, [_P, ctypes.POINTER(ctypes.c_double)]),
    "lng_hip_batch_drop": (None, [_P]),
    "lng_hip_batch_set_timing": (ctypes.c_int, [_P, ctypes.c_int]),
    "lng_hip_batch_kernel_seconds": (ctypes.c_int, [_P, ctypes.c_char_p, ctypes.POINTER(ctypes.c_double),
                                                    ctypes.POINTER(ctypes.c_size_t)]),
    "lng_hip_check_grouped": (ctypes.c_int, [ctypes.POINTER(_Shape), ctypes.c_int]),
    "lng_hip_attention_grouped": (ctypes.c_int, [_P, _Slice, _Slice, _Slice, _Slice, ctypes.POINTER(_Slice),
                                                 ctypes.POINTER(_Shape), ctypes.c_int]),
    "lng_hip_attention_grouped_tiled": (ctypes.c_int, [_P, _Slice, _Slice, _Slice, _Slice, ctypes.POINTER(_Slice),
                                                       ctypes.POINTER(_Shape), ctypes.c_int]),
    "lng_hip_attention_grouped_static": (ctypes.c_int, [_P, _P, _P, _P, _P, _P, _P, ctypes.POINTER(_Shape), ctypes.c_int]),
    "lng_hip_copy_rows": (ctypes.c_int, [_P, _Slice, _U64, ctypes.c_int, _Slice, _U64, ctypes.c_int, _U64, _U64]),
    "lng_hip_attention_decode_batched": (ctypes.c_int, [_P, _U64, _U64, _U64, _U64, _U64, ctypes.POINTER(_Item),
                                                        ctypes.c_size_t, _U64, _U64, _U64, ctypes.c_float,
                                                        ctypes.c_int]),
    "lng_hip_fill_synthetic": (ctypes.c_int, [_P, _Slice, ctypes.c_int, _U64, ctypes.c_float, _U64]),
    "lng_hip_checksum": (ctypes.c_int, [_P, _Slice, _Slice]),
    "lng_hip_rmsnorm_rows": (ctypes.c_int, [_P, _Slice, _Slice, _U64, _U64, _U64, ctypes.c_float]),
    "lng_hip_add_rows": (ctypes.c_int, [_P, _Slice, _Slice, _U64, _U64, _U64]),
    "lng_hip_rotate_halves": (ctypes.c_int, [_P, _Slice, _Slice, _U64, _U64, _U64, _U64]),
    "lng_hip_gemv_q8_0": (ctypes.c_int, [_P, _Slice, _Slice, _Slice, _Slice, _U64, _U64]),
    "lng_hip_gemm_q8_0": (ctypes.c_int, [_P, _Slice, _Slice, _Slice, _Slice, _U64, _U64, _U64, _U64, _U64]),
    "lng_hip_gemm_q8_0_tiled": (ctypes.c_int, [_P, _Slice, _Slice, _Slice, _Slice, _U64, _U64, _U64, _U64, _U64]),
    "lng_hip_gemm_q8_0_bf16": (ctypes.c_int, [_P, _Slice, _Slice, _Slice, _Slice, _U64, _U64, _U64, _U64, _U64]),
    "lng_hip_gemm_q8_0_many": (ctypes.c_int, [_P, ctypes.POINTER(_Q8Matrix), ctypes.c_size_t, _Slice, _U64, _U64, _U64]),
    "lng_hip_gemm_q8_0_many_normed": (ctypes.c_int, [_P, ctypes.POINTER(_Q8Matrix), ctypes.c_size_t, _Slice, _Slice,
                                                     ctypes.c_float, _U64, _U64, _U64]),
    "lng_hip_gemm_q8_0_residual": (ctypes.c_int, [_P, _Slice, _Slice, _Slice, ctypes.c_int, ctypes.POINTER(_Slice), _Slice,
                                                  _U64, _U64, _U64, _U64, _U64]),
    "lng_hip_prepare_attention": (ctypes.c_int, [_P, ctypes.POINTER(_PrepareBuffers), ctypes.POINTER(_PrepareItem),
                                                 ctypes.c_size_t, _U64, _U64, _U64, _U64, ctypes.c_int]),
}

_lib = None
_lib_lock = threading.Lock()


def library():
    """The loaded C-ABI library. Raises ``Compile`` when it has not been built."""
    global _lib
    with _lib_lock:
        if _lib is None:
            if not os.path.exists(LIB_PATH):
                raise Compile("liblng_hip.so is not built: run `python -m loadngo_amd.build`")
            lib = ctypes.CDLL(LIB_PATH)
            for name, (restype, argtypes) in SYMBOLS.items():
                fn = getattr(lib, name)
                fn.restype = restype
                fn.argtypes = argtypes
            _lib = lib
    return _lib


def _check(rc):
    if rc != 0:
        message = library().lng_hip_last_error().decode("utf-8", "replace")
        raise _ERRORS.get(rc, Error)(message)


def _u64(name, value):
    """ctypes wraps integers modulo 2**64 without a word (2**64 becomes 0): counts are checked here instead."""
    if not isinstance(value, (int, np.integer)) or isinstance(value, bool) or not 0 <= int(value) < 2**64:
        raise ValueError("%s = %r is not an integer in 0 .. 2**64 - 1" % (name, value))
    return int(value)


class Slice:
    """apple.rs:507-521: bytes ``offset..offset+len`` of the batch's buffer number ``buffer``."""

    __slots__ = ("buffer", "offset", "len")

    def __init__(self, buffer, offset, len):
        self.buffer, self.offset, self.len = buffer, offset, len

    def _c(self):
        return _Slice(*[_u64(n, getattr(self, n)) for n in self.__slots__])

    def __repr__(self):
        return "Slice(buffer=%d, offset=%d, len=%d)" % (self.buffer, self.offset, self.len)

    def __eq__(self, other):
        return (self.buffer, self.offset, self.len) == (other.buffer, other.offset, other.len)


class GroupedShape:
    """apple.rs:598-614."""

    __slots__ = ("t", "start", "heads", "kv_heads", "dim", "window", "slots", "scale")

    def __init__(self, t, start, heads, kv_heads, dim, window, slots, scale):
        self.t, self.start, self.heads, self.kv_heads = t, start, heads, kv_heads
        self.dim, self.window, self.slots, self.scale = dim, window, slots, scale

    def _c(self):
        return _Shape(*[_u64(n, getattr(self, n)) for n in self.__slots__[:7]], self.scale)

    def __repr__(self):
        return "GroupedShape(%s)" % ", ".join("%s=%r" % (n, getattr(self, n)) for n in self.__slots__)


def check_grouped(shape, tiled=False):
    """The shape rules alone (apple.rs:1243-1272, 1356-1385); raises ``Dispatch``. No device needed."""
    _check(library().lng_hip_check_grouped(ctypes.byref(shape._c()), int(tiled)))


class DecodeItem:
    """One decoding query of a batched dispatch: byte offsets into the named buffers."""

    __slots__ = ("q_offset", "out_offset", "k_offset", "v_offset", "sinks_offset", "start", "window", "slots")

    def __init__(self, q_offset, out_offset, k_offset, v_offset, sinks_offset, start, window, slots):
        self.q_offset, self.out_offset, self.k_offset, self.v_offset = q_offset, out_offset, k_offset, v_offset
        self.sinks_offset = NO_SINKS if sinks_offset is None else sinks_offset
        self.start, self.window, self.slots = start, window, slots


def decode_items(items):
    """A prepared table of ``DecodeItem`` for ``Batch.attention_decode_batched`` (built once,
    reused every step)."""
    return (_Item * len(items))(*[
        _Item(*[_u64(n, getattr(i, n)) for n in DecodeItem.__slots__]) for i in items])


class PrepareItem:
    """One sequence of ``Batch.prepare_attention``: byte offsets of its ``n`` projection rows, of its
    rotary table rows, of its prepared queries and of row 0 of its caches; its first new position
    and the rows its caches hold."""

    __slots__ = _PREPARE_FIELDS

    def __init__(self, **fields):
        for name in _PREPARE_FIELDS:
            setattr(self, name, fields.pop(name, 0))
        if fields:
            raise TypeError("unknown fields: %s" % sorted(fields))


def prepare_items(items):
    """A prepared table of ``PrepareItem`` (built once, reused while the offsets hold)."""
    return (_PrepareItem * len(items))(*[_PrepareItem(*[_u64(n, getattr(i, n)) for n in _PREPARE_FIELDS]) for i in items])


def split_q8_0_blocks(raw):
    """ggml ``Q8_0`` blocks (2-byte binary16 scale, then 32 signed bytes) as the two arrays the
    kernels take: the codes in order (int8) and the scales in order (uint16 bit patterns). Moves bytes
    only (weights/src/q8_0.rs:17-31 ``split_blocks``)."""
    blocks = np.frombuffer(raw, dtype=np.uint8) if isinstance(raw, (bytes, bytearray, memoryview)) else np.asarray(raw, np.uint8)
    if blocks.size % 34 != 0:
        raise ValueError("whole Q8_0 blocks")
    blocks = blocks.reshape(-1, 34)
    return (np.ascontiguousarray(blocks[:, 2:]).view(np.int8).reshape(-1),
            np.ascontiguousarray(blocks[:, :2]).view("<u2").reshape(-1))


def rope_table(inv_freq, scale, start, n):
    """``[n][len(inv_freq)][2]`` f32 pairs ``(cos, sin) * scale`` of ``position * inv_freq`` for positions
    ``start..start+n``, computed in f64 as the reference's host does every pass (gpt-oss/src/gpu.rs:690-697)."""
    angle = (start + np.arange(n, dtype=np.float64))[:, None] * np.asarray(inv_freq, dtype=np.float64)[None, :]
    return np.stack([(np.cos(angle) * scale).astype(np.float32), (np.sin(angle) * scale).astype(np.float32)], axis=-1)


class Completed:
    """apple.rs:536-539: the batch's buffers, and the GPU time or why it failed."""

    def __init__(self, buffers, gpu_time):
        self.buffers = buffers
        self.gpu_time = gpu_time  # seconds (float) or an Error instance


class Buffer:
    """apple.rs:391-430, in device memory."""

    resident = False

    def __init__(self, gpu, handle, len):
        self._gpu, self._h, self.len = gpu, handle, len

    def __len__(self):
        return self.len

    def device_ptr(self):
        return library().lng_hip_buffer_device_ptr(self._h)

    def write(self, array, offset=0):
        """``as_bytes_mut()[offset..].copy_from_slice(array bytes)``."""
        a = np.ascontiguousarray(array)
        _check(library().lng_hip_upload(self._h, offset, a.ctypes.data_as(_P), a.nbytes))

    def read(self, dtype=np.uint8, offset=0, count=None):
        """``as_bytes()[offset..]`` viewed as ``dtype``."""
        dtype = np.dtype(dtype)
        nbytes = self.len - offset if count is None else count * dtype.itemsize
        out = np.empty(nbytes // dtype.itemsize, dtype=dtype)
        _check(library().lng_hip_download(self._h, offset, out.ctypes.data_as(_P), out.nbytes))
        return out

    def fill(self, byte, offset=0, len=None):
        _check(library().lng_hip_fill(self._h, offset, byte, self.len - offset if len is None else len))

    def free(self):
        if self._h:
            _check(library().lng_hip_buffer_free(self._h))
            self._h = None

    def __del__(self):
        try:
            if self._h and library():
                library().lng_hip_buffer_free(self._h)
                self._h = None
        except Exception:
            pass


class Resident(Buffer):
    """apple.rs:465-503: read-only memory that many batches may read at once."""

    resident = True


class Gpu:
    """apple.rs:100-389."""

    def __init__(self, device=0):
        lib = library()
        handle = _P()
        _check(lib.lng_hip_open(device, ctypes.byref(handle)))
        self._h = handle

    @classmethod
    def new(cls):
        return cls()

    def name(self):
        buf = ctypes.create_string_buffer(128)
        _check(library().lng_hip_device_name(self._h, buf, 128))
        return buf.value.decode()

    def debug_set(self, name, value):
        """A development switch by its environment name (``include/lng_hip.h`` lists them; not part of the
        interface); ``value`` None puts the default back. The environment itself is read once, at open."""
        _check(library().lng_hip_debug_set(self._h, name.encode(), None if value is None else str(value).encode()))

    def debug_get(self, name):
        """A development counter by name (waits for submitted work; the counter goes back to zero)."""
        value = ctypes.c_uint64()
        _check(library().lng_hip_debug_get(self._h, name.encode(), ctypes.byref(value)))
        return value.value

    def buffer(self, len):
        h = _P()
        _check(library().lng_hip_buffer(self._h, len, ctypes.byref(h)))
        return Buffer(self, h, len)

    def resident(self, data):
        a = np.ascontiguousarray(data)
        h = _P()
        _check(library().lng_hip_resident(self._h, a.ctypes.data_as(_P), a.nbytes, ctypes.byref(h)))
        return Resident(self, h, a.nbytes)

    def upload(self, array):
        """A buffer holding ``array`` (the tests' ``upload`` helper, attention_grouped.rs:37-41)."""
        a = np.ascontiguousarray(array)
        b = self.buffer(max(a.nbytes, 4))
        if a.nbytes:
            b.write(a)
        return b

    def batch(self, buffers, dispatch="serial"):
        return Batch(self, list(buffers))

    def attention_grouped_static(self, q, k, v, out, sinks, shape, dtype=F32, stream=None):
        """The plain operator on raw device addresses (``Buffer.device_ptr()`` plus a byte offset), launched at
        once on ``stream`` (a hipStream_t as an integer; None: the default stream) without allocating anything;
        no counterpart in the reference. Returns without waiting."""
        _check(library().lng_hip_attention_grouped_static(self._h, stream, q, k, v, out, sinks or None,
                                                          ctypes.byref(shape._c()), dtype))

    def close(self):
        if self._h:
            library().lng_hip_close(self._h)
            self._h = None


class Batch:
    """apple.rs:541-2240: one recorded submission. Dispatches run in order."""

    def __init__(self, gpu, buffers):
        self._gpu = gpu
        self.buffers = buffers
        self._residents = []
        arr = (_P * max(len(buffers), 1))(*[b._h for b in buffers])
        h = _P()
        _check(library().lng_hip_batch(gpu._h, arr, len(buffers), ctypes.byref(h)))
        self._h = h
        self._callback = None
        self._committed = False

    def dispatches(self):
        return library().lng_hip_batch_dispatches(self._h)

    def attach(self, resident):
        s = _Slice()
        _check(library().lng_hip_batch_attach(self._h, resident._h, ctypes.byref(s)))
        if resident not in self._residents:
            self._residents.append(resident)
        return Slice(s.buffer, s.offset, s.len)

    def barrier(self):
        _check(library().lng_hip_batch_barrier(self._h))

    def attention_grouped(self, q, k, v, out, shape, dtype=F32):
        _check(library().lng_hip_attention_grouped(self._h, q._c(), k._c(), v._c(), out._c(), None,
                                                   ctypes.byref(shape._c()), dtype))

    def attention_grouped_with_sinks(self, qkv, sinks, out, shape, dtype=F32):
        q, k, v = qkv
        _check(library().lng_hip_attention_grouped(self._h, q._c(), k._c(), v._c(), out._c(),
                                                   ctypes.byref(sinks._c()), ctypes.byref(shape._c()), dtype))

    def attention_grouped_tiled(self, q, k, v, out, shape, dtype=F32):
        _check(library().lng_hip_attention_grouped_tiled(self._h, q._c(), k._c(), v._c(), out._c(), None,
                                                         ctypes.byref(shape._c()), dtype))

    def attention_grouped_tiled_with_sinks(self, qkv, sinks, out, shape, dtype=F32):
        q, k, v = qkv
        _check(library().lng_hip_attention_grouped_tiled(self._h, q._c(), k._c(), v._c(), out._c(),
                                                         ctypes.byref(sinks._c()), ctypes.byref(shape._c()), dtype))

    def copy_rows(self, src, dst, rows, width, src_dtype=F32, dst_dtype=None):
        """``copy_rows((src, src_stride), (dst, dst_stride), rows, width)`` (apple.rs:1762)."""
        (s, s_stride), (d, d_stride) = src, dst
        dst_dtype = src_dtype if dst_dtype is None else dst_dtype
        _check(library().lng_hip_copy_rows(self._h, s._c(), s_stride, src_dtype, d._c(), d_stride, dst_dtype,
                                           rows, width))

    def attention_decode_batched(self, q_buffer, k_buffer, v_buffer, out_buffer, sinks_buffer, items, heads,
                                 kv_heads, dim, scale, dtype=BF16):
        arr = items if isinstance(items, ctypes.Array) else decode_items(items)
        _check(library().lng_hip_attention_decode_batched(self._h, q_buffer, k_buffer, v_buffer, out_buffer,
                                                          sinks_buffer, arr, len(items), heads, kv_heads, dim,
                                                          scale, dtype))

    def rmsnorm_rows(self, v_w, rows, d_stride, eps):
        """``rmsnorm_rows((v, w), rows, (d, stride), eps)`` (apple.rs:1733), f32, in place."""
        (v, w), (d, stride) = v_w, d_stride
        _check(library().lng_hip_rmsnorm_rows(self._h, v._c(), w._c(), rows, d, stride, eps))

    def add_rows(self, dst, src, rows, width):
        """``add_rows(dst, (src, src_stride), rows, width)`` (apple.rs:1886), f32."""
        s, s_stride = src
        _check(library().lng_hip_add_rows(self._h, dst._c(), s._c(), s_stride, rows, width))

    def rotate_halves(self, x, table, rows, heads_dim):
        """``rotate_halves(x, table, rows, (heads, dim))`` (apple.rs:1916), f32, in place."""
        heads, dim = heads_dim
        _check(library().lng_hip_rotate_halves(self._h, x._c(), table._c(), rows, heads, dim, dim))

    def rotate_halves_partial(self, x, table, rows, heads_dim_rotary):
        """``rotate_halves_partial(x, table, rows, (heads, dim, rotary))`` (apple.rs:1929)."""
        heads, dim, rotary = heads_dim_rotary
        _check(library().lng_hip_rotate_halves(self._h, x._c(), table._c(), rows, heads, dim, rotary))

    def prepare_attention(self, buffers, items, heads, kv_heads, dim, rotary=None, out_dtype=BF16,
                          q_bias=None, k_bias=None, v_bias=None):
        """Biases, rotation, narrowing and cache append of gpt-oss/src/gpu.rs:733-759 in one dispatch.
        ``buffers`` maps q, k, v, table, q_out, k_cache, v_cache to buffer numbers of this batch;
        the biases are slices (or None)."""
        held = [None if b is None else b._c() for b in (q_bias, k_bias, v_bias)]
        pb = _PrepareBuffers(*[buffers[n] for n in ("q", "k", "v", "table", "q_out", "k_cache", "v_cache")],
                             *[None if h is None else ctypes.pointer(h) for h in held])
        arr = items if isinstance(items, ctypes.Array) else prepare_items(items)
        _check(library().lng_hip_prepare_attention(self._h, ctypes.byref(pb), arr, len(arr), heads, kv_heads, dim,
                                                   dim if rotary is None else rotary, out_dtype))

    def gemv_q8_0(self, matrix, x, y, rows, cols):
        """``gemv_q8_0((codes, scales), x, y, rows, cols)`` (apple.rs:1812)."""
        codes, scales = matrix
        _check(library().lng_hip_gemv_q8_0(self._h, codes._c(), scales._c(), x._c(), y._c(), rows, cols))

    def gemm_q8_0(self, matrix, x, y, rows, cols, n, strides):
        """``gemm_q8_0((codes, scales), x, y, rows, cols, n, (x_stride, y_stride))`` (apple.rs:1833)."""
        codes, scales = matrix
        _check(library().lng_hip_gemm_q8_0(self._h, codes._c(), scales._c(), x._c(), y._c(), rows, cols, n,
                                           strides[0], strides[1]))

    def gemm_q8_0_tiled(self, matrix, x, y, rows, cols, n, strides):
        """``gemm_q8_0_tiled(...)`` (apple.rs:1857): needs rows % 64, cols % 32 and n % 32 == 0."""
        codes, scales = matrix
        _check(library().lng_hip_gemm_q8_0_tiled(self._h, codes._c(), scales._c(), x._c(), y._c(), rows, cols, n,
                                                 strides[0], strides[1]))

    def gemm_q8_0_bf16(self, matrix, x, y, rows, cols, n, strides):
        """The Q8_0 product of bf16 positions (no counterpart in the reference): x is [n][x_stride] bf16, y f32."""
        codes, scales = matrix
        _check(library().lng_hip_gemm_q8_0_bf16(self._h, codes._c(), scales._c(), x._c(), y._c(), rows, cols, n,
                                                strides[0], strides[1]))

    def gemm_q8_0_many(self, matrices, x, cols, n, x_stride):
        """Up to four Q8_0 products of the same positions (no counterpart in the reference, which records one
        per matrix: gpu.rs:724-732): ``matrices`` is a list of ``((codes, scales), y, rows)``, each y dense
        [n][rows]; one dispatch below 32 positions."""
        arr = (_Q8Matrix * len(matrices))()
        for slot, ((codes, scales), y, rows) in zip(arr, matrices):
            slot.codes, slot.scales, slot.y, slot.rows = codes._c(), scales._c(), y._c(), rows
        _check(library().lng_hip_gemm_q8_0_many(self._h, arr, len(matrices), x._c(), cols, n, x_stride))

    def gemm_q8_0_many_normed(self, matrices, x, norm, cols, n, x_stride):
        """``gemm_q8_0_many`` of the RMS-normalised positions (``norm`` = (weights slice, eps)); x is not changed.
        Replaces copy_rows + rmsnorm_rows + the products of gpu.rs:712-732; fewer than 32 positions."""
        arr = (_Q8Matrix * len(matrices))()
        for slot, ((codes, scales), y, rows) in zip(arr, matrices):
            slot.codes, slot.scales, slot.y, slot.rows = codes._c(), scales._c(), y._c(), rows
        w, eps = norm
        _check(library().lng_hip_gemm_q8_0_many_normed(self._h, arr, len(matrices), x._c(), w._c(), eps, cols, n, x_stride))

    def gemm_q8_0_residual(self, matrix, x, bias, h, rows, cols, n, strides, x_dtype=F32):
        """h += W x + bias in one dispatch, bit for bit gemm_q8_0 + add_rows(bias) + add_rows(residual) of
        gpu.rs:807-827; x f32 or bf16; fewer than 32 positions. ``strides`` = (x_stride, h_stride)."""
        codes, scales = matrix
        held = None if bias is None else bias._c()
        _check(library().lng_hip_gemm_q8_0_residual(self._h, codes._c(), scales._c(), x._c(), x_dtype,
                                                    None if held is None else ctypes.pointer(held), h._c(), rows, cols, n,
                                                    strides[0], strides[1]))

    def fill_synthetic(self, dst, dtype, seed, scale=1.0, period=0):
        _check(library().lng_hip_fill_synthetic(self._h, dst._c(), dtype, seed, scale, period))

    def checksum(self, src, dst):
        """XOR of every 16-byte word of ``src`` into the 16 bytes of ``dst`` (a plain streaming read)."""
        _check(library().lng_hip_checksum(self._h, src._c(), dst._c()))

    def set_timing(self, enabled=True):
        """Record an event after every kernel so ``kernel_seconds`` can report per-kernel time."""
        _check(library().lng_hip_batch_set_timing(self._h, int(enabled)))

    def kernel_seconds(self, kernel):
        """(total seconds, launches) of the kernel named ``kernel`` in this finished batch."""
        seconds, launches = ctypes.c_double(), ctypes.c_size_t()
        _check(library().lng_hip_batch_kernel_seconds(self._h, kernel.encode(), ctypes.byref(seconds),
                                                      ctypes.byref(launches)))
        return seconds.value, launches.value

    def commit(self, on_done=None):
        """apple.rs:2202: submits; ``on_done(Completed)`` runs on a library thread when the GPU
        has finished (a Rust caller re-posts it to its proactor)."""
        if on_done is not None:
            def trampoline(done, _user):
                d = done.contents
                if d.status == 0:
                    gpu_time = d.gpu_seconds
                else:
                    gpu_time = _ERRORS.get(d.status, Error)((d.message or b"").decode("utf-8", "replace"))
                on_done(Completed(self.buffers, gpu_time))
            self._callback = _ON_DONE(trampoline)
        else:
            self._callback = ctypes.cast(None, _ON_DONE)
        self._committed = True
        _check(library().lng_hip_batch_commit(self._h, self._callback, None))

    def wait(self):
        """Blocks until a committed batch has finished; returns ``Completed``."""
        seconds = ctypes.c_double()
        rc = library().lng_hip_batch_wait(self._h, ctypes.byref(seconds))
        if rc == -5:
            return Completed(self.buffers, GpuFailure(library().lng_hip_last_error().decode()))
        _check(rc)
        return Completed(self.buffers, seconds.value)

    def run(self):
        """commit + wait: what the reference's tests do with their proactor loop
        (attention_grouped.rs:11-23)."""
        self.commit()
        return self.wait()

    def drop(self):
        if self._h:
            library().lng_hip_batch_drop(self._h)
            self._h = None

    def __del__(self):
        try:
            self.drop()
        except Exception:
            pass
