"""Host restatement of the device's synthetic-data generator (``lng_hip_fill_synthetic``),
integer for integer, so a test or benchmark can know any element of a device-filled buffer."""
import numpy as np

SYNTH_STD = np.float32(37837.227)  # sqrt(4 * (65536**2 - 1) / 12)


def synthetic_values(n, seed, scale=1.0, period=0, first=0):
    """Elements first..first+n of the stream ``(seed, period)`` as f32."""
    i = np.arange(first, first + n, dtype=np.uint64)
    if period:
        i = i % np.uint64(period)
    with np.errstate(over="ignore"):
        z = i + np.uint64(seed) * np.uint64(0x9E3779B97F4A7C15)
        z = (z ^ (z >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)
        z = (z ^ (z >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)
        z = z ^ (z >> np.uint64(31))
    m = np.uint64(0xFFFF)
    s = ((z & m) + ((z >> np.uint64(16)) & m) + ((z >> np.uint64(32)) & m) + (z >> np.uint64(48))).astype(np.int64)
    factor = np.float32(scale) / SYNTH_STD
    return (s - 131070).astype(np.float32) * factor


def bf16_bits(x):
    """f32 -> bf16 bit patterns (uint16), round to nearest even."""
    b = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32)
    bias = np.uint32(0x7FFF) + ((b >> np.uint32(16)) & np.uint32(1))
    return ((b + bias) >> np.uint32(16)).astype(np.uint16)


def bf16_widen(bits):
    """bf16 bit patterns -> f32 (exact)."""
    return (np.ascontiguousarray(bits, dtype=np.uint16).astype(np.uint32) << np.uint32(16)).view(np.float32)
