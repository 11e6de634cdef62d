"""Configuration 5 as a whole: the 24-layer decode stack at its real size (batch 16, context 131072,
96 GiB of bf16 K/V caches), recorded exactly as bench.py records the step it times, every output row
checked.

The caches are filled on the device with streams that repeat every 1024 positions (a distinct stream
per layer and per K / V, distinct sinks per layer, a distinct query per layer and sequence). Then every
weight of a full-causal layer appears 128 times and the exact result is attention over one period with
the sink lowered by ln(128) (test_oracle_pinning pins that identity on the oracle); a 128-window layer
sees the last 128 positions. A wrong cache for a layer, a 64-bit offset that wraps beyond the first
layers, or (in the window layers, where the sink still carries weight) a wrong per-layer sink offset would
each miss the bar (bf16: 2e-2 max-abs)."""
import numpy as np
import pytest

import bench
from oracle import oracle
from tests.gpu_common import gpu  # noqa: F401

pytestmark = pytest.mark.gpu


def test_config5_whole_stack_every_row(gpu):
    stack = bench.Stack(gpu)  # batch 16, context 131072, 24 layers
    try:
        assert stack.layers * 2 * stack.batch_size * stack.ctx * bench.ROW == 103079215104
        stack.fill_caches(bench.STACK_PERIOD)
        stack.out.fill(0xFF)
        stack.step()
        got = stack.outputs()
        assert np.isfinite(got).all()
        assert stack.check_full_layers_periodic(got, oracle) < 2e-2
        assert stack.check_window_layers(got, oracle, bench.STACK_PERIOD) < 2e-2
        # the checks discriminate between layers: another layer's rows (its caches, its sinks) miss the bar
        other = np.roll(got, 2, axis=0)
        assert stack.check_full_layers_periodic(other, oracle) > 2e-2
        assert stack.check_window_layers(other, oracle, bench.STACK_PERIOD) > 2e-2
    finally:
        stack.free()
