"""The entry point that allocates nothing (lng_hip_attention_grouped_static), through the C ABI, against
the existing entry point it is a variant of (lng_hip_attention_grouped) and against the CPU oracle.

Bars: bf16 in/out within 2e-2 max-abs; f32 within 1e-5 relative. Two calls in a row share the fixed
scratch array, the second with a smaller input: what the first one left there must not show."""
import ctypes

import numpy as np
import pytest

from loadngo_amd import compute as C
from oracle import oracle
from tests.gpu_common import THREADS, gpu, max_error, run_attention  # noqa: F401
from tests.helpers import FULL, from_bf16_bits, normal_inputs, to_bf16_bits

pytestmark = pytest.mark.gpu

BF16_TOL = 2e-2
F32_RTOL = 1e-5


def rel_error(got, want):
    e = np.abs(got.astype(np.float64) - want) / (np.abs(want) + 1.0)
    return np.inf if np.isnan(e).any() else float(e.max())


def _hip():
    """The HIP runtime itself, for a stream of the caller's own (the library never makes one for this entry point)."""
    return ctypes.CDLL("libamdhip64.so")


def static_call(gpu, q, k, v, sinks, shape, dtype, stream=None, q_shift=0):
    """Uploads, calls the static entry point on the default stream (or on `stream`, a hipStream_t), downloads (the
    blocking copy is ordered after the kernels on the default stream; the caller synchronises its own). `q_shift`
    puts the queries that many bytes into their buffer. Returns out [t][H][D]."""
    es = 4 if dtype == C.F32 else 2
    qb = gpu.buffer(q.nbytes + q_shift)
    qb.write(q, offset=q_shift)
    bufs = [qb, gpu.upload(k), gpu.upload(v), gpu.buffer(q.size * es), gpu.upload(sinks)]
    bufs[3].fill(0xFF)
    try:
        gpu.attention_grouped_static(bufs[0].device_ptr() + q_shift, bufs[1].device_ptr(), bufs[2].device_ptr(),
                                     bufs[3].device_ptr(), bufs[4].device_ptr(), shape, dtype, stream=stream)
        if stream is not None:
            assert _hip().hipStreamSynchronize(ctypes.c_void_p(stream)) == 0
        out = bufs[3].read(np.float32 if dtype == C.F32 else np.uint16)
    finally:
        for b in bufs:
            b.free()
    return out.reshape(q.shape)


# (t, context, window): one long row in many chunks, then fewer and shorter rows; several rows; a window
CALLS_BF16 = [(1, 16384, FULL), (1, 700, FULL), (3, 4096, FULL), (1, 4096, 128), (1, 131, FULL)]
CALLS_F32 = [(1, 8192, FULL), (2, 900, FULL), (1, 3000, 128)]


@pytest.mark.parametrize("dtype,calls", [(C.BF16, CALLS_BF16), (C.F32, CALLS_F32)])
def test_static_entry_point_matches_the_batch_entry_point_on_calls_in_a_row(gpu, dtype, calls):
    heads, kv_heads, dim = 64, 8, 64
    for n, (t, ctx, window) in enumerate(calls):
        start = ctx - t
        q, k, v, sinks = normal_inputs(100 + n, t, ctx, heads, kv_heads, dim, scale=0.5)
        shape = C.GroupedShape(t, start, heads, kv_heads, dim, window, ctx, 0.125)
        if dtype == C.BF16:
            qd, kd, vd = to_bf16_bits(q), to_bf16_bits(k), to_bf16_bits(v)
        else:
            qd, kd, vd = q, k, v
        got = static_call(gpu, qd, kd, vd, sinks, shape, dtype)
        ref = run_attention(gpu, qd, kd, vd, sinks, shape, False, dtype)
        if dtype == C.BF16:
            want = oracle.attention_bf16(qd, kd, vd, sinks, start, window=window, scale=0.125, threads=THREADS)
            assert max_error(from_bf16_bits(got), from_bf16_bits(ref)) < BF16_TOL, (t, ctx, window)
            assert max_error(from_bf16_bits(got), from_bf16_bits(want)) < BF16_TOL, (t, ctx, window)
        else:
            want = oracle.attention_f32(q, k, v, sinks, start, window=window, scale=0.125, threads=THREADS)
            assert rel_error(got, ref.astype(np.float64)) < F32_RTOL, (t, ctx, window)
            assert rel_error(got, want.astype(np.float64)) < F32_RTOL, (t, ctx, window)


@pytest.mark.parametrize("dtype", [C.BF16, C.F32])
def test_static_entry_point_takes_other_head_widths(gpu, dtype):
    """Width 256 (32 heads over 16 kv heads) in many chunks and then in one, sharing the fixed array (partials of
    `dim` floats per slot); width 96 runs on the kernel without scratch."""
    for t, ctx, heads, kv_heads, dim in [(1, 20000, 32, 16, 256), (2, 300, 32, 16, 256), (2, 300, 8, 2, 96)]:
        q, k, v, sinks = normal_inputs(7 + ctx, t, ctx, heads, kv_heads, dim, scale=0.5)
        shape = C.GroupedShape(t, ctx - t, heads, kv_heads, dim, FULL, ctx, 0.1)
        if dtype == C.BF16:
            qd, kd, vd = to_bf16_bits(q), to_bf16_bits(k), to_bf16_bits(v)
            got = static_call(gpu, qd, kd, vd, sinks, shape, dtype)
            want = oracle.attention_bf16(qd, kd, vd, sinks, ctx - t, window=FULL, scale=0.1, threads=THREADS)
            assert max_error(from_bf16_bits(got), from_bf16_bits(want)) < BF16_TOL, (t, ctx, dim)
        else:
            got = static_call(gpu, q, k, v, sinks, shape, dtype)
            want = oracle.attention_f32(q, k, v, sinks, ctx - t, window=FULL, scale=0.1, threads=THREADS)
            assert rel_error(got, want.astype(np.float64)) < F32_RTOL, (t, ctx, dim)


@pytest.mark.parametrize("dtype", [C.BF16, C.F32])
def test_static_entry_point_on_every_kernel_family_and_on_a_stream_of_the_callers(gpu, dtype):
    """Widths 128 and 512 in many chunks, a group of 32 query heads (the kernel of one workgroup per (row, head)), queries
    off a 16-byte boundary (the same kernel), then two calls in a row on a stream the caller made, the second with the
    smaller input; each against the CPU oracle."""
    stream = ctypes.c_void_p()
    assert _hip().hipStreamCreate(ctypes.byref(stream)) == 0
    try:
        cases = [(1, 9000, 8, 2, 128, None, 0), (2, 5000, 16, 4, 512, None, 0), (1, 600, 32, 1, 64, None, 0),
                 (1, 3000, 64, 8, 64, None, 4), (1, 12000, 64, 8, 64, stream.value, 0), (1, 500, 64, 8, 64, stream.value, 0)]
        for n, (t, ctx, heads, kv_heads, dim, on, shift) in enumerate(cases):
            scale = float(1.0 / np.sqrt(np.float32(dim)))
            q, k, v, sinks = normal_inputs(40 + n, t, ctx, heads, kv_heads, dim, scale=0.5)
            shape = C.GroupedShape(t, ctx - t, heads, kv_heads, dim, FULL, ctx, scale)
            if dtype == C.BF16:
                qd, kd, vd = to_bf16_bits(q), to_bf16_bits(k), to_bf16_bits(v)
                got = static_call(gpu, qd, kd, vd, sinks, shape, dtype, stream=on, q_shift=shift)
                want = oracle.attention_bf16(qd, kd, vd, sinks, ctx - t, window=FULL, scale=scale, threads=THREADS)
                assert max_error(from_bf16_bits(got), from_bf16_bits(want)) < BF16_TOL, (t, ctx, heads, dim)
            else:
                got = static_call(gpu, q, k, v, sinks, shape, dtype, stream=on, q_shift=shift)
                want = oracle.attention_f32(q, k, v, sinks, ctx - t, window=FULL, scale=scale, threads=THREADS)
                assert rel_error(got, want.astype(np.float64)) < F32_RTOL, (t, ctx, heads, dim)
    finally:
        assert _hip().hipStreamDestroy(stream) == 0


def test_static_entry_point_refuses_what_does_not_fit_or_is_malformed(gpu):
    heads, kv_heads, dim = 64, 8, 64
    buf = gpu.buffer(1 << 20)
    p = buf.device_ptr()
    try:
        # 33 rows of 64 heads: past the stated limit of rows x heads <= 2048 (refused before anything is launched)
        big = C.GroupedShape(33, 1000, heads, kv_heads, dim, FULL, 2048, 0.125)
        with pytest.raises(C.Dispatch) as e:
            gpu.attention_grouped_static(p, p + 4096, p + 8192, p + 12288, None, big, C.BF16)
        assert "fixed scratch array" in str(e.value)
        # wider heads take proportionally more of the array: 16 rows of 64 heads of width 128 is the limit
        with pytest.raises(C.Dispatch) as e:
            gpu.attention_grouped_static(p, p + 4096, p + 8192, p + 12288, None,
                                         C.GroupedShape(17, 1000, heads, kv_heads, 128, FULL, 2048, 0.125), C.BF16)
        assert "fixed scratch array" in str(e.value)
        ok = C.GroupedShape(1, 10, heads, kv_heads, dim, FULL, 11, 0.125)
        with pytest.raises(C.Dispatch):  # the reference's shape rules
            gpu.attention_grouped_static(p, p + 65536, p + 131072, p + 262144, None,
                                         C.GroupedShape(1, 0, 6, 4, 64, 8, 8, 1.0), C.BF16)
        with pytest.raises(C.Dispatch):  # the output overlaps the queries
            gpu.attention_grouped_static(p, p + 65536, p + 131072, p + 64, None, ok, C.BF16)
        with pytest.raises(C.Dispatch):  # no address
            gpu.attention_grouped_static(None, p + 65536, p + 131072, p + 262144, None, ok, C.BF16)
        with pytest.raises(C.Dispatch):  # misaligned
            gpu.attention_grouped_static(p + 1, p + 65536, p + 131072, p + 262144, None, ok, C.BF16)
    finally:
        buf.free()
