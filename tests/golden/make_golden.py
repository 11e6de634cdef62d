"""Writes tests/golden/config1_fp32.npz: the fp32 plumbing configuration (4 query heads over
1 kv head, head_dim 64, 32 positions, causal, one sink per head, N(0,1) inputs from seed 0)
and the CPU oracle's output for it. The reference is Rust and cannot run here, so the
expected output comes from oracle/attention_oracle.c, which tests/test_oracle_pinning.py pins.

    python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import oracle  # noqa: E402
from tests.helpers import normal_inputs  # noqa: E402

q, k, v, sinks = normal_inputs(0, 32, 32, 4, 1, 64)
out = oracle.attention_f32(q, k, v, sinks, 0)
np.savez(os.path.join(ROOT, "tests", "golden", "config1_fp32.npz"), q=q, k=k, v=v, sinks=sinks, out=out)
print("wrote config1_fp32.npz", out.shape, float(np.abs(out).max()))
