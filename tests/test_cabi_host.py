"""CPU-side checks of the C-ABI library: it loads, exports everything include/lng_hip.h
declares, and applies the reference's shape rules without a device. No compute calls."""
import ctypes
import os
import re

import numpy as np
import pytest

from loadngo_amd import compute as C
from oracle import oracle
from tests.helpers import FULL, REF_GPT_OSS_CASES, REF_PLAIN_CASES, REF_REJECTED, REF_TILED_CASES, normal_inputs

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_library_exports_every_declared_symbol():
    header = open(os.path.join(ROOT, "include", "lng_hip.h")).read()
    declared = set(re.findall(r"\b(lng_hip_\w+)\s*\(", header))
    assert len(declared) >= 20
    lib = ctypes.CDLL(C.LIB_PATH)
    for name in declared:
        assert hasattr(lib, name), name
    assert declared == set(C.SYMBOLS), declared ^ set(C.SYMBOLS)


def test_struct_layouts_match_the_header():
    assert ctypes.sizeof(C._Slice) == 24
    assert ctypes.sizeof(C._Shape) == 64 and C._Shape.scale.offset == 56
    assert ctypes.sizeof(C._Item) == 64
    assert ctypes.sizeof(C._Completed) == 24


def test_shape_rules_match_the_reference_lists():
    for case in REF_REJECTED:
        with pytest.raises(C.Dispatch):
            C.check_grouped(C.GroupedShape(*case, 1.0), tiled=False)
    for case, _ in REF_PLAIN_CASES:
        C.check_grouped(C.GroupedShape(*case, 1.0), tiled=False)
    for case, _ in REF_TILED_CASES:
        C.check_grouped(C.GroupedShape(*case, 1.0), tiled=True)
    for (t, start, window, slots), tiled in REF_GPT_OSS_CASES:
        C.check_grouped(C.GroupedShape(t, start, 64, 8, 64, window, slots, 0.125), tiled=tiled)


def test_shape_rules_agree_with_the_oracle_on_random_shapes():
    rng = np.random.default_rng(1)
    pick = lambda xs: int(xs[rng.integers(len(xs))])  # noqa: E731
    agree = refused = 0
    for _ in range(4000):
        case = (pick([0, 1, 2, 31, 32, 40, 512]), pick([0, 1, 5, 97, 700, 2**32 - 1, 2**32]),
                pick([1, 4, 6, 8, 64]), pick([0, 1, 2, 4, 8]), pick([0, 16, 32, 48, 64, 512, 544]),
                pick([0, 1, 7, 128, FULL]), pick([0, 1, 8, 10, 12, 64, 640, 2**33]))
        for tiled in (False, True):
            want = oracle.accepts(*case, tiled=tiled)
            try:
                C.check_grouped(C.GroupedShape(*case, 1.0), tiled=tiled)
                got = True
            except C.Dispatch as e:
                got = False
                assert "grouped attention shape" in str(e) or "does not fit in u32" in str(e)
            assert got == want, (case, tiled)
            agree += 1
            refused += not got
    assert refused > 1000 and agree - refused > 300


def test_opening_a_gpu_without_a_device_fails_loudly():
    try:
        gpu = C.Gpu()
    except C.NoDevice:
        return                      # the product has no CPU path to fall back to
    gpu.close()
    pytest.skip("a GPU is present")


def test_golden_config1_is_what_the_oracle_computes():
    g = np.load(os.path.join(ROOT, "tests", "golden", "config1_fp32.npz"))
    q, k, v, sinks = normal_inputs(0, 32, 32, 4, 1, 64)
    for name, arr in (("q", q), ("k", k), ("v", v), ("sinks", sinks)):
        assert np.array_equal(g[name], arr), name
    assert g["out"].shape == (32, 4, 64)
    assert np.array_equal(oracle.attention_f32(q, k, v, sinks, 0), g["out"])
    want = oracle.attention_f64(q, k, v, sinks, 0)
    assert np.max(np.abs(g["out"] - want) / (np.abs(want) + 1)) < 1e-5


def test_synthetic_generator_has_unit_variance_and_period():
    from loadngo_amd.synthetic import synthetic_values
    x = synthetic_values(200000, 9)
    assert abs(float(x.std()) - 1.0) < 0.01 and abs(float(x.mean())) < 0.01
    p = synthetic_values(3000, 9, 0.5, period=1000)
    assert np.array_equal(p[:1000], p[1000:2000]) and np.array_equal(p[:1000], p[2000:])
    assert np.array_equal(synthetic_values(10, 9, first=5), x[5:15])
