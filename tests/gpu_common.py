"""Helpers of the GPU parity tests: everything goes through the C ABI (loadngo_amd.compute)."""
import numpy as np
import pytest

from loadngo_amd import compute as C
from tests.helpers import from_bf16_bits, ring_layout, to_bf16_bits

THREADS = 8  # oracle threads: spreads (query, head) pairs, arithmetic per pair unchanged


@pytest.fixture(scope="session")
def gpu():
    g = C.Gpu()  # raises without the built library or without a device: no fallback
    yield g
    g.close()


class _Knobs:
    """Development switches of the session's device for one test (``lng_hip_debug_set``); the library reads the
    environment only when a device is opened, so tests that pick a kernel go through this. Defaults come back at
    the end of the test."""

    def __init__(self, gpu):
        self._gpu, self._touched = gpu, set()

    def setenv(self, name, value):
        self._touched.add(name)
        self._gpu.debug_set(name, value)

    def delenv(self, name, raising=True):
        self._touched.add(name)
        self._gpu.debug_set(name, None)

    def restore(self):
        for name in self._touched:
            self._gpu.debug_set(name, None)


@pytest.fixture
def knobs(gpu):
    k = _Knobs(gpu)
    yield k
    k.restore()


def run_attention(gpu, q, k_ring, v_ring, sinks, shape, tiled, dtype, poison_out=True, expect_kernel=None):
    """One dispatch as the reference's test harness lays it out (attention_grouped.rs:102-158):
    five buffers (q, k, v, out, sinks), slices over all of each. q is [t][H][D]; for the tiled
    operator it is zero-padded to t rounded up to 32 rows. Returns out[:t] (f32 or bf16 bits).
    ``expect_kernel``: the name of a kernel the dispatch must have launched exactly once."""
    t, heads, dim = q.shape
    es = 4 if dtype == C.F32 else 2
    rows = (t + 31) // 32 * 32 if tiled else t
    qp = np.zeros((rows, heads, dim), dtype=q.dtype)
    qp[:t] = q
    out_len = rows * heads * dim * es
    bufs = [gpu.upload(qp), gpu.upload(k_ring), gpu.upload(v_ring), gpu.buffer(out_len),
            gpu.upload(sinks if sinks is not None else np.zeros(1, np.float32))]
    if poison_out:
        bufs[3].fill(0xFF)  # NaN pattern in both f32 and bf16: unwritten outputs show
    batch = gpu.batch(bufs)
    if expect_kernel:
        batch.set_timing(True)
    qs, ks, vs, os_ = (C.Slice(0, 0, qp.nbytes), C.Slice(1, 0, k_ring.nbytes), C.Slice(2, 0, v_ring.nbytes),
                       C.Slice(3, 0, out_len))
    try:
        if sinks is None:
            (batch.attention_grouped_tiled if tiled else batch.attention_grouped)(qs, ks, vs, os_, shape, dtype)
        else:
            ss = C.Slice(4, 0, shape.heads * 4)
            (batch.attention_grouped_tiled_with_sinks if tiled else batch.attention_grouped_with_sinks)(
                (qs, ks, vs), ss, os_, shape, dtype)
        done = batch.run()
        assert not isinstance(done.gpu_time, Exception), done.gpu_time
        if expect_kernel:
            assert batch.kernel_seconds(expect_kernel)[1] == 1, expect_kernel
        out = bufs[3].read(np.float32 if dtype == C.F32 else np.uint16)
    finally:
        batch.drop()
        for b in bufs:
            b.free()
    return out.reshape(rows, heads, dim)[:t]


def reference_case(oracle, case, sharp, tiled, sinks, scale, dtype):
    """Inputs of one reference test case (attention_grouped.rs:102-135): q = values(1)*sharp,
    k = values(2), v = values(3) over every absolute position, laid into the ring."""
    t, start, heads, kv_heads, dim, window, slots = case
    end = start + t
    q = (oracle.values(1, t * heads * dim) * np.float32(sharp)).reshape(t, heads, dim)
    k = oracle.values(2, end * kv_heads * dim).reshape(end, kv_heads, dim)
    v = oracle.values(3, end * kv_heads * dim).reshape(end, kv_heads, dim)
    shape = C.GroupedShape(t, start, heads, kv_heads, dim, window, slots, scale)
    if dtype == C.BF16:
        q, k, v = (from_bf16_bits(to_bf16_bits(x)) for x in (q, k, v))  # exactly representable
    kr, vr = ring_layout(k, t, start, slots, tiled), ring_layout(v, t, start, slots, tiled)
    return q, k, v, kr, vr, shape


def max_error(got, want):
    """attention_grouped.rs:151-157: a NaN counts as infinite error."""
    e = np.abs(got.astype(np.float64) - want.astype(np.float64))
    return np.inf if np.isnan(e).any() else float(e.max())
