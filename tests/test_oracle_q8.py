"""Pins the oracle's Q8_0 functions: binary16 widening against numpy over every code, the
reference's own known-answer blocks (weights/src/q8_0.rs:141-175), the split layout against the
tiny fixture's tensors decoded independently, the f32 product against the float64 definition at
the shapes and bound of the reference's GPU test (q8_0_and_gpt_oss_glue.rs:155-177), the float64
definition against numpy, and the whole tiny-model golden with the oracle product in place."""
import os

import numpy as np
import pytest

from oracle import oracle as orc
from oracle import tiny_model as tm
from tests.helpers import REF_Q8_CASES, q8_test_matrix, xorshift_values
from tests.test_tiny_model import FIXTURE, TOLERANCE, OracleSession


def test_binary16_widening_matches_numpy_for_every_code():
    bits = np.arange(65536, dtype=np.uint16)
    got, want = orc.f16_to_f32(bits), bits.view(np.float16).astype(np.float32)
    finite = ~np.isnan(want)
    assert np.array_equal(got.view(np.uint32)[finite], want.view(np.uint32)[finite])
    assert np.isnan(got[~finite]).all()


def _block(d, q):
    return np.uint16(d).tobytes() + bytes((q(i) & 0xFF) for i in range(32))


def test_reference_known_answer_blocks():
    """q8_0.rs:141-175: 0x3800 is 0.5, 0xC000 is -2.0."""
    raw = (_block(0x3800, lambda i: i - 16) + _block(0xC000, lambda i: 127 if i % 2 == 0 else -128)
           + _block(0x0000, lambda i: 5) + _block(0x3C00, lambda i: i))
    codes, scales = orc.q8_split_blocks(raw)
    w = (codes.astype(np.float32).reshape(4, 32) * orc.f16_to_f32(scales)[:, None]).reshape(2, 64)
    assert (w[0, 0], w[0, 31], w[0, 32], w[0, 33]) == (-8.0, 7.5, -254.0, 256.0)
    assert (w[1, :32] == 0).all() and w[1, 63] == 31.0
    assert np.array_equal(w, tm.dequant_q8_0(raw, 2, 64))
    x = np.sin(np.arange(64, dtype=np.float32) * np.float32(0.37)).astype(np.float32)
    y = orc.q8_mul(codes, scales, x[None, :], 2, 64)[0]
    want = w.astype(np.float64) @ x.astype(np.float64)
    assert (np.abs(y - want) < 1e-4 * np.maximum(np.abs(want), 1.0)).all()


def test_split_layout_matches_the_fixture_tensors_decoded_independently():
    model = tm.TinyModel(os.path.join(FIXTURE, "model.gguf"))
    assert len(model.q8_raw) == 2 + 4 * model.layers_n
    for name, (raw, rows, cols) in model.q8_raw.items():
        codes, scales = orc.q8_split_blocks(raw)
        blocks = np.frombuffer(raw, np.uint8).reshape(-1, 34)
        assert np.array_equal(codes.reshape(-1, 32), blocks[:, 2:].view(np.int8))
        assert np.array_equal(scales, blocks[:, :2].copy().view("<u2")[:, 0])
        w = codes.astype(np.float32).reshape(rows, cols // 32, 32) * orc.f16_to_f32(scales).reshape(rows, -1, 1)
        assert np.array_equal(w.reshape(rows, cols), tm.dequant_q8_0(raw, rows, cols)), name


@pytest.mark.parametrize("rows,cols,n,kind", REF_Q8_CASES)
def test_f32_product_meets_the_reference_bound_against_float64(rows, cols, n, kind):
    codes, bits, elements = q8_test_matrix(rows, cols, 7 + rows)
    x = xorshift_values(11, n * cols).reshape(n, cols)
    want = x.astype(np.float64) @ elements.T                          # numpy, from the elements' values
    by_def = orc.q8_mul_f64(codes, bits, x, rows, cols)
    assert np.abs(by_def - want).max() <= 1e-12 * np.abs(want).max()
    got = orc.q8_mul(codes, bits, x, rows, cols)
    assert np.abs(got - want).max() / np.abs(want).max() < 1e-5       # q8_0_and_gpt_oss_glue.rs:171


def test_strides_leave_gaps_alone():
    rows, cols, n = 64, 96, 3
    codes, bits, elements = q8_test_matrix(rows, cols, 3)
    x = np.full((n, cols + 8), np.nan, np.float32)
    x[:, :cols] = xorshift_values(5, n * cols).reshape(n, cols)
    y = orc.q8_mul(codes, bits, x, rows, cols, y_stride=rows + 5)
    assert (y[:, rows:] == 0).all()
    assert np.allclose(y[:, :rows], x[:, :cols].astype(np.float64) @ elements.T, rtol=0, atol=1e-3)


def test_tiny_model_golden_with_the_oracle_products():
    model = tm.TinyModel(os.path.join(FIXTURE, "model.gguf"))
    ids, want = tm.load_fixture(FIXTURE)
    split = {name: orc.q8_split_blocks(raw) + (rows, cols) for name, (raw, rows, cols) in model.q8_raw.items()}

    def project(name, x):
        codes, scales, rows, cols = split[name]
        return orc.q8_mul(codes, scales, x, rows, cols)

    s = OracleSession(model)
    got = model.forward(ids, s.prepare, s.attention, chunk=5, project=project)
    assert np.abs(got - want).max() < TOLERANCE
