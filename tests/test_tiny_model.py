"""The reference's end-to-end golden (gpt-oss/tests/tiny_oracle.rs:10-40) with the attention
oracle in the attention block's place: every position's logits within 2e-3 of transformers'.

This pins the C oracle (sinks, window, layer parity, grouped heads) against numbers the
reference holds, through a whole model."""
import os

import numpy as np
import pytest

from oracle import oracle as orc
from oracle import tiny_model as tm

FIXTURE = os.path.join(os.path.dirname(__file__), "golden", "tiny")
TOLERANCE = 2e-3  # tiny_oracle.rs:10


class OracleSession:
    """Flat caches as model.rs:188-192, attention by the C oracle."""

    def __init__(self, model, slots=None, fn=None):
        self.m, self.slots = model, slots
        self.fn = fn or orc.attention_f32
        rows = slots or 64
        self.k = [np.full((rows, model.kv_heads * model.dim), np.nan, np.float32) for _ in range(model.layers_n)]
        self.v = [np.full((rows, model.kv_heads * model.dim), np.nan, np.float32) for _ in range(model.layers_n)]
        self.q = None

    def prepare(self, l, q, k, v, start):
        m, layer = self.m, self.m.layers[l]
        table = orc.rope_table(m.inv_freq, m.rope_scale, start, q.shape[0])
        self.q = orc.prepare(q, k, v, layer["q_bias"], layer["k_bias"], layer["v_bias"], table,
                             self.k[l], self.v[l], start, m.heads, m.kv_heads, m.dim)

    def attention(self, l, start, n, window):
        m = self.m
        rows = self.k[l].shape[0]
        slots = rows if self.slots else None
        end = start + n
        held = rows if self.slots else end
        return self.fn(self.q.reshape(n, m.heads, m.dim),
                       self.k[l][:held].reshape(held, m.kv_heads, m.dim),
                       self.v[l][:held].reshape(held, m.kv_heads, m.dim),
                       m.layers[l]["sinks"], start, window=window,
                       slots=slots if slots else end)


@pytest.fixture(scope="module")
def model():
    return tm.TinyModel(os.path.join(FIXTURE, "model.gguf"))


def test_fixture_has_the_shape_the_reference_states(model):
    # scripts/gpt_oss_tiny_oracle.py:21-24
    assert (model.layers_n, model.hidden, model.heads, model.kv_heads, model.dim) == (4, 128, 4, 2, 32)
    assert (model.experts, model.used, model.expert_hidden, model.vocab, model.window) == (4, 2, 64, 512, 8)
    ids, want = tm.load_fixture(FIXTURE)
    assert len(ids) == 40 and want.shape == (40, 512)


@pytest.mark.parametrize("chunk", [1, 40, 7])
def test_every_position_matches_transformers(model, chunk):
    ids, want = tm.load_fixture(FIXTURE)
    s = OracleSession(model)
    got = model.forward(ids, s.prepare, s.attention, chunk=chunk)
    worst = np.abs(got - want).max(axis=1)
    assert worst.max() < TOLERANCE, f"position {worst.argmax()}: max error {worst.max()}"


def test_a_wrong_window_or_missing_sinks_fails_the_fixture(model):
    """The fixture discriminates: the same pass with the window one off, or without sinks, is
    outside the tolerance, so agreement above is not vacuous."""
    ids, want = tm.load_fixture(FIXTURE)

    def run(mutate):
        s = OracleSession(model)
        attention = lambda l, start, n, window: mutate(s, l, start, n, window)
        return np.abs(model.forward(ids, s.prepare, attention) - want).max()

    off = lambda s, l, start, n, w: s.attention(l, start, n, w if w == tm.FULL else w + 1)
    assert run(off) > TOLERANCE

    def no_sinks(s, l, start, n, w):
        m = s.m
        end = start + n
        return orc.attention_f32(s.q.reshape(n, m.heads, m.dim), s.k[l][:end].reshape(end, m.kv_heads, m.dim),
                                 s.v[l][:end].reshape(end, m.kv_heads, m.dim), None, start, window=w, slots=end)
    assert run(no_sinks) > TOLERANCE

    parity = lambda s, l, start, n, w: s.attention(l, start, n, tm.FULL if w != tm.FULL else s.m.window)
    assert run(parity) > TOLERANCE


def test_ring_caches_give_the_same_logits(model):
    """Sliding layers in a ring of window + chunk rows (gpu.rs:570-574), full layers flat."""
    ids, want = tm.load_fixture(FIXTURE)

    class Ring(OracleSession):
        def __init__(self, model, chunk):
            super().__init__(model)
            ring = model.window + chunk
            for l in range(model.layers_n):
                if model.is_sliding(l):
                    self.k[l] = np.full((ring, model.kv_heads * model.dim), np.nan, np.float32)
                    self.v[l] = np.full((ring, model.kv_heads * model.dim), np.nan, np.float32)

        def attention(self, l, start, n, window):
            m = self.m
            rows = self.k[l].shape[0]
            held = min(rows, start + n) if m.is_sliding(l) else start + n
            return orc.attention_f32(self.q.reshape(n, m.heads, m.dim),
                                     self.k[l][:held].reshape(held, m.kv_heads, m.dim),
                                     self.v[l][:held].reshape(held, m.kv_heads, m.dim),
                                     m.layers[l]["sinks"], start, window=window,
                                     slots=rows if m.is_sliding(l) else start + n)

    for chunk in (1, 5):
        s = Ring(model, chunk)
        got = model.forward(ids, s.prepare, s.attention, chunk=chunk)
        assert np.abs(got - want).max() < TOLERANCE
