"""Shared input builders for the parity tests (numpy only; no oracle, no product code)."""
import numpy as np

FULL = 2**64 - 1

# metal-compute/tests/attention_grouped.rs:187-199 — (t, start, H, G, D, window, slots), sharp
REF_PLAIN_CASES = [
    ((1, 0, 32, 4, 512, FULL, 1), 1.0),
    ((1, 700, 32, 4, 512, FULL, 701), 0.05),
    ((37, 300, 32, 4, 512, FULL, 337), 0.05),
    ((1, 3000, 32, 16, 256, 1024, 1536), 0.08),
    ((200, 1400, 32, 16, 256, 1024, 1536), 0.08),
    ((512, 0, 32, 16, 256, 1024, 1536), 0.08),
    ((5, 97, 4, 1, 64, 7, 12), 3.0),
    ((3, 2, 8, 2, 32, 16, 40), 1.0),
]
# metal-compute/tests/attention_grouped.rs:210-221
REF_TILED_CASES = [
    ((512, 0, 32, 4, 512, FULL, 512), 0.05),
    ((77, 700, 32, 4, 512, FULL, 4096), 0.05),
    ((33, 5, 32, 4, 512, FULL, 40), 0.05),
    ((512, 2600, 32, 16, 256, 1024, 1536), 0.08),
    ((200, 1400, 32, 16, 256, 1024, 1536), 0.08),
    ((512, 0, 32, 16, 256, 1024, 1536), 0.08),
    ((40, 97, 4, 1, 64, 7, 64), 3.0),
]
# metal-compute/tests/attention_grouped.rs:239-249 — ((t, start, window, slots), tiled); H=64 G=8 D=64
REF_GPT_OSS_CASES = [
    ((1, 0, 128, 640), False),
    ((1, 3000, 128, 640), False),
    ((9, 700, 128, 640), False),
    ((512, 0, 128, 640), True),
    ((512, 2600, 128, 640), True),
    ((1, 4095, FULL, 4096), False),
    ((300, 200, FULL, 4096), True),
]
# metal-compute/tests/attention_grouped.rs:258-264
REF_REJECTED = [
    (1, 0, 6, 4, 64, 8, 8),
    (1, 0, 4, 4, 48, 8, 8),
    (1, 0, 4, 4, 544, 8, 8),
    (4, 100, 4, 4, 64, 8, 10),
    (0, 0, 4, 4, 64, 8, 8),
]


def xorshift_values(seed, n):
    """The reference tests' generator (attention_grouped.rs:25-35), vectorised with numpy
    integer arithmetic only: uniform on a 2^-23 grid in [-1, 1)."""
    top = np.empty(n, dtype=np.uint32)
    mask = (1 << 64) - 1
    s = (seed | 1) & mask
    for i in range(n):
        s ^= (s << 13) & mask
        s ^= s >> 7
        s ^= (s << 17) & mask
        top[i] = s >> 40
    return top.astype(np.float32) / np.float32(1 << 23) - np.float32(1.0)


def ring_layout(all_rows, t, start, slots, tiled, fill=None):
    """attention_grouped.rs:47-63 in numpy: position p goes to row p % slots; other rows are
    NaN for the plain operator, zero for the tiled one."""
    end = start + t
    if not tiled:
        rows = min(slots, end)
    elif slots < end:
        rows = slots
    else:
        rows = (end + 31) // 32 * 32
    if fill is None:
        fill = 0.0 if tiled else np.nan
    if all_rows.dtype == np.uint16 and isinstance(fill, float):
        fill = 0x7FC0 if np.isnan(fill) else 0  # bf16 bit patterns: quiet NaN or zero
    out = np.full((rows,) + all_rows.shape[1:], fill, dtype=all_rows.dtype)
    for p in range(max(0, end - slots), end):
        out[p % slots] = all_rows[p]
    return out


def to_bf16_bits(x):
    """f32 -> bf16 bit patterns, round to nearest even (numpy integer arithmetic)."""
    b = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32)
    nan = np.isnan(x)
    bias = np.uint32(0x7FFF) + ((b >> np.uint32(16)) & np.uint32(1))
    r = ((b + bias) >> np.uint32(16)).astype(np.uint16)
    r[nan] = ((b[nan] >> np.uint32(16)) | np.uint32(0x40)).astype(np.uint16)
    return r


def from_bf16_bits(b):
    return (np.ascontiguousarray(b, dtype=np.uint16).astype(np.uint32) << np.uint32(16)).view(np.float32)


def normal_inputs(seed, t, end, heads, kv_heads, dim, scale=1.0):
    """Seeded N(0,1)*scale q [t][H][D], k/v for every absolute position [end][G][D], sinks [H]."""
    rng = np.random.default_rng(seed)
    q = (rng.standard_normal((t, heads, dim)) * scale).astype(np.float32)
    k = (rng.standard_normal((end, kv_heads, dim)) * scale).astype(np.float32)
    v = (rng.standard_normal((end, kv_heads, dim)) * scale).astype(np.float32)
    sinks = rng.standard_normal(heads).astype(np.float32)
    return q, k, v, sinks


# metal-compute/tests/q8_0_and_gpt_oss_glue.rs:58-65: exact binary16 scales of either sign
Q8_TEST_SCALES = [(0x3800, 0.5), (0x2000, 0.0078125), (0xB600, -0.375), (0x3C00, 1.0), (0x1400, 0.0009765625),
                  (0x4100, 2.5)]
# q8_0_and_gpt_oss_glue.rs:160-168: (rows, cols, positions, kind)
REF_Q8_CASES = [(4096, 2880, 1, "gemv"), (512, 2880, 1, "gemv"), (37, 96, 1, "gemv"), (512, 2880, 5, "gemm"),
                (37, 96, 13, "gemm"), (2880, 4096, 32, "tiled"), (512, 2880, 96, "tiled")]


def q8_test_matrix(rows, cols, seed):
    """q8_0_and_gpt_oss_glue.rs:56-84 `q8_matrix`: (codes int8, scale bits uint16, elements f64 [rows][cols])."""
    v = xorshift_values(seed, rows * cols)
    codes = (v * np.float32(127.9)).astype(np.int32).astype(np.int8)  # `as i8` truncates toward zero
    sv = xorshift_values(seed + 1, rows * cols // 32)
    pick = ((((sv + np.float32(1.0)) * np.float32(3.0)).astype(np.int64)) + np.arange(len(sv))) % 6
    bits = np.array([Q8_TEST_SCALES[i][0] for i in pick], dtype=np.uint16)
    scale = np.array([Q8_TEST_SCALES[i][1] for i in pick], dtype=np.float64)
    elements = codes.astype(np.float64).reshape(rows, cols // 32, 32) * scale.reshape(rows, cols // 32, 1)
    return codes, bits, elements.reshape(rows, cols)
