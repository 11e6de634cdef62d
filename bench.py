#!/usr/bin/env python3
"""Benchmark of the gpt-oss attention path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload c5|c3|c2] [--no-extras] [--no-cpu]

A step is one pass of the hot path over one batch of synthetic input resident in HBM. The
headline workload is the long-context decode stack (24 layers alternating 128-token window
and full-causal, batch 16, context 131072, bf16 KV cache of 96 GiB): one step decodes one
token for every sequence through all 24 layers' attention. `value` is the KV-cache GB/s of
the whole step (algorithmic bytes / wall time per step, K steps with nothing recorded between
the kernels); `roofline` is the decode kernel's own bandwidth (algorithmic bytes per launch /
its average launch time, from HIP events recorded after every kernel on the library's stream
during K further steps: those events cost a few microseconds of gap each, so the throughput is
not taken from the instrumented steps). The other configurations (single 4096-token decode, ragged batch of 32,
8192-token prompt passes) are reported under "extra". The CPU baseline is the oracle (a C
restatement of the reference's CPU attention) timed on this host on a bounded sample.

Prints one JSON line.
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

from loadngo_amd import compute as C  # noqa: E402
from loadngo_amd.synthetic import bf16_bits, bf16_widen, synthetic_values  # noqa: E402

H, G, D = 64, 8, 64
SCALE = 0.125
ROW = G * D * 2          # bytes of one cached position of K (or V) in bf16
QO = H * D * 2           # bytes of one query (or output) row
HBM_PEAK_GBS = 8000.0    # MI355X HBM3E
MFMA_BF16_PEAK_TFLOPS = 2500.0  # MI355X dense bf16
MFMA_F32_PEAK_TFLOPS = 157.3    # MI355X f32 matrix
# HBM bytes per launch of the decode kernel on the default stack workload come from rocprofv3 FETCH_SIZE and
# WRITE_SIZE runs scaled by a 1 GiB copy; the figure and the sources it was measured on are kept in
# profiles/decode_stack_c5_hbm_traffic.json and only reported while those sources are unchanged.
TRAFFIC_RECORD = os.path.join(ROOT, "profiles", "decode_stack_c5_hbm_traffic.json")
DECODE_KERNELS = ("lng_decode_bf16_d64", "lng_decode_bf16_d64_o4")
TRAFFIC_SOURCES = ("loadngo_amd/csrc/lng_kernels.hip", "loadngo_amd/csrc/lng_hip.cpp", "loadngo_amd/csrc/lng_kernel_args.h")


def sources_digest():
    """sha256 over the kernel and planner sources the traffic measurement depends on."""
    import hashlib
    h = hashlib.sha256()
    for rel in TRAFFIC_SOURCES:
        with open(os.path.join(ROOT, rel), "rb") as f:
            h.update(f.read())
    return h.hexdigest()


def stack_traffic_per_launch(ctx, batch):
    """The measured HBM bytes per launch, or None when the record is missing, for another workload, or stale."""
    try:
        with open(TRAFFIC_RECORD) as f:
            rec = json.load(f)
    except (OSError, ValueError):
        return None
    if (rec.get("ctx"), rec.get("batch")) != (ctx, batch) or rec.get("sources_sha256") != sources_digest():
        return None
    return rec.get("hbm_bytes_per_launch")


def record_traffic(root, ctx, batch):
    """Writes profiles/decode_stack_c5_hbm_traffic.json from four rocprofv3 counter runs under `root`:
    pmc_c5_FETCH_SIZE, pmc_c5_WRITE_SIZE (this file with --no-extras --no-cpu) and pmc_copy_FETCH_SIZE,
    pmc_copy_WRITE_SIZE (--only copy: a plain copy of 1 GiB, the yardstick each counter is scaled by).
    The record carries a digest of the sources it was measured on; stack_traffic_per_launch ignores it
    once they change."""
    import csv
    import glob

    def per_dispatch(sub, kernel):
        files = glob.glob(os.path.join(root, sub, "**", "*counter_collection.csv"), recursive=True)
        if not files:
            raise SystemExit("no counter_collection.csv under %s" % os.path.join(root, sub))
        by_grid = {}
        for row in csv.DictReader(open(files[0])):
            if row["Kernel_Name"] == kernel:
                by_grid.setdefault(int(row["Grid_Size"]), []).append(float(row["Counter_Value"]))
        return {g: sum(v) / len(v) for g, v in by_grid.items()}

    gib = float(1 << 30)
    scale = {}
    for counter in ("FETCH_SIZE", "WRITE_SIZE"):
        seen = per_dispatch("pmc_copy_" + counter, "lng_copy_rows")
        scale[counter] = gib / (max(seen.values()) * 1024.0)
    total = 0.0
    detail = {}
    for counter in ("FETCH_SIZE", "WRITE_SIZE"):
        for kernel in DECODE_KERNELS + ("lng_decode_merge", "lng_decode_merge_few"):
            for grid, kib in per_dispatch("pmc_c5_" + counter, kernel).items():
                nbytes = kib * 1024.0 * scale[counter]
                detail["%s grid %d %s" % (kernel, grid, counter)] = {"kib_per_dispatch": kib, "bytes": nbytes}
                if kernel in DECODE_KERNELS:
                    total += nbytes / 2.0  # a step has 12 launches of each of the kernel's two grids: the mean over the 24
    try:  # the last commit that touched the measured sources (empty outside a git checkout)
        import subprocess
        commit = subprocess.run(["git", "-C", ROOT, "log", "-1", "--format=%H", "--"] + list(TRAFFIC_SOURCES),
                                capture_output=True, text=True, timeout=20).stdout.strip()
    except (OSError, subprocess.SubprocessError):
        commit = ""
    rec = {"ctx": ctx, "batch": batch, "sources_commit": commit, "sources_sha256": sources_digest(), "hbm_bytes_per_launch": round(total),
           "scale_factor": scale, "per_dispatch": detail,
           "how": "rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE (one counter per run) on `python3 bench.py --no-extras --no-cpu "
                  "--steps 2 --warmup 1`, each scaled by what the counter reads for `python3 bench.py --only copy` (1 GiB in, 1 GiB out)"}
    with open(TRAFFIC_RECORD, "w") as f:
        json.dump(rec, f, indent=1)
        f.write("\n")
    print(json.dumps(rec, indent=1))


METRIC = "decode attn GB/s (% HBM peak) + prefill attn TFLOP/s (% MFMA), gpt-oss shapes"


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def decode_bytes(length, window):
    """Algorithmic bytes of one decoding query over one layer: visible K+V rows, q, out, sinks."""
    visible = length if window == C.FULL else min(length, window)
    return visible * 2 * ROW + 2 * QO + H * 4


def fill(gpu, buf, seed, scale=0.5, period=0):
    batch = gpu.batch([buf])
    batch.fill_synthetic(C.Slice(0, 0, buf.len), C.BF16, seed, scale, period)
    batch.run()
    batch.drop()


# ------------------------------------------------------------------------------------------------
STACK_PERIOD = 1024  # positions after which the checking fill repeats


class Stack:
    """Configuration 5: the 24-layer decode stack, its caches resident. Caches are allocated layer by layer,
    K then V, as gpt-oss/src/gpu.rs:567-578 does; kv_gap_gib = N allocates all K caches, N GiB left unused,
    then all V caches (an experiment on how placement in HBM changes the rate). Cache 2l is layer l's K
    (fill seed 2l + 1), cache 2l + 1 its V (seed 2l + 2); queries are seed 1000; sinks are N(0,1), seed 5."""

    def __init__(self, gpu, batch_size=16, ctx=131072, layers=24, kv_gap_gib=None):
        self.gpu, self.batch_size, self.ctx, self.layers = gpu, batch_size, ctx, layers
        log("allocating %.1f GiB of KV cache" % (layers * 2 * batch_size * ctx * ROW / 2**30))
        self.q = gpu.buffer(layers * batch_size * QO)
        self.out = gpu.buffer(layers * batch_size * QO)
        self.sink_values = np.random.default_rng(5).standard_normal((layers, H)).astype(np.float32)
        self.sinks = gpu.upload(self.sink_values)
        fill(gpu, self.q, 1000)
        self.caches, self.unused = [], []
        if kv_gap_gib is None:
            for l in range(layers):
                self.caches += [gpu.buffer(batch_size * ctx * ROW), gpu.buffer(batch_size * ctx * ROW)]
        else:
            ks = [gpu.buffer(batch_size * ctx * ROW) for _ in range(layers)]
            if kv_gap_gib:
                self.unused.append(gpu.buffer(kv_gap_gib << 30))
            vs = [gpu.buffer(batch_size * ctx * ROW) for _ in range(layers)]
            for l in range(layers):
                self.caches += [ks[l], vs[l]]
        self.bufs = [self.q, self.out, self.sinks] + self.caches
        self.tables = []
        self.step_bytes = 0
        for l in range(layers):
            window = self.window(l)
            items = [C.DecodeItem((l * batch_size + b) * QO, (l * batch_size + b) * QO, b * ctx * ROW, b * ctx * ROW,
                                  l * H * 4, ctx - 1, window, ctx) for b in range(batch_size)]
            self.tables.append(C.decode_items(items))
            self.step_bytes += batch_size * decode_bytes(ctx, window)

    @staticmethod
    def window(layer):
        return 128 if layer % 2 == 0 else C.FULL  # even layers slide (gpt-oss/src/config.rs:99-103)

    def fill_caches(self, period=0):
        """Fills every cache on the device; period (positions) > 0 makes each cache repeat after that many
        positions (the sequences of a cache then hold the same rows)."""
        for i, b in enumerate(self.caches):
            fill(self.gpu, b, i + 1, period=period * G * D)

    def step(self, timing=False):
        """One decoding step: 24 batched-decode dispatches in one batch. Returns (gpu seconds, (decode kernel
        seconds, launches) when timing)."""
        batch = self.gpu.batch(self.bufs)
        if timing:
            batch.set_timing(True)
        for l in range(self.layers):
            batch.attention_decode_batched(0, 3 + 2 * l, 4 + 2 * l, 1, 2, self.tables[l], H, G, D, SCALE, C.BF16)
        batch.commit()
        done = batch.wait()
        if isinstance(done.gpu_time, Exception):
            raise done.gpu_time
        ks = (0.0, 0)
        if timing:  # both builds of the decode kernel (the second one serves dispatches of many short chunks: none in this stack)
            per = [batch.kernel_seconds(name) for name in DECODE_KERNELS]
            ks = (sum(p[0] for p in per), sum(p[1] for p in per))
        batch.drop()
        return done.gpu_time, ks

    def outputs(self):
        """[layers][batch][H][D] f32 of what the last step wrote."""
        return bf16_widen(self.out.read(np.uint16)).reshape(self.layers, self.batch_size, H, D)

    def queries(self):
        return bf16_bits(synthetic_values(self.layers * self.batch_size * H * D, 1000, 0.5)).reshape(
            self.layers, self.batch_size, H, D)

    def check_window_layers(self, got, oracle, period=0):
        """Every row of every 128-window layer against the oracle on the host's restatement of the fill (the
        last 128 positions of each sequence: cheap whatever the fill). Returns the largest error."""
        q = self.queries()
        worst = 0.0
        for l in range(0, self.layers, 2):
            for b in range(self.batch_size):
                first = (b * self.ctx + self.ctx - 128) * G * D
                k = bf16_bits(synthetic_values(128 * G * D, 2 * l + 1, 0.5, period * G * D, first)).reshape(128, G, D)
                v = bf16_bits(synthetic_values(128 * G * D, 2 * l + 2, 0.5, period * G * D, first)).reshape(128, G, D)
                want = oracle.attention_bf16(q[l, b:b + 1], k, v, self.sink_values[l], 127, window=128, scale=SCALE)
                err = np.abs(got[l, b] - bf16_widen(want[0]))
                worst = max(worst, float(np.inf if np.isnan(err).any() else err.max()))
        return worst

    def check_full_layers_periodic(self, got, oracle):
        """With the caches filled with period STACK_PERIOD, every weight of a full-causal layer appears
        ctx / STACK_PERIOD times, so the exact result is attention over one period with the sink lowered by
        ln(ctx / STACK_PERIOD) (a property of the softmax, pinned on the oracle by its own tests). Every row of
        every full-causal layer. Returns the largest error."""
        assert self.ctx % STACK_PERIOD == 0
        q = self.queries()
        lowered = self.sink_values - np.float32(np.log(self.ctx // STACK_PERIOD))
        worst = 0.0
        for l in range(1, self.layers, 2):
            k = bf16_bits(synthetic_values(STACK_PERIOD * G * D, 2 * l + 1, 0.5)).reshape(STACK_PERIOD, G, D)
            v = bf16_bits(synthetic_values(STACK_PERIOD * G * D, 2 * l + 2, 0.5)).reshape(STACK_PERIOD, G, D)
            for b in range(self.batch_size):
                want = oracle.attention_bf16(q[l, b:b + 1], k, v, lowered[l], STACK_PERIOD - 1, scale=SCALE, threads=8)
                err = np.abs(got[l, b] - bf16_widen(want[0]))
                worst = max(worst, float(np.inf if np.isnan(err).any() else err.max()))
        return worst

    def free(self):
        for b in self.bufs + self.unused:
            b.free()


def run_stack(gpu, steps, warmup, batch_size=16, ctx=131072, layers=24, kv_gap_gib=None, check=True):
    """Configuration 5, timed; then (outside the timed region) its outputs are checked: the timed step's
    window layers against the oracle on the same fill, and, after refilling the caches with a fill that
    repeats every STACK_PERIOD positions, one more step whose every row - 24 layers x 16 sequences x 64 heads -
    is held to the bf16 bar (2e-2) through the periodic identity."""
    stack = Stack(gpu, batch_size, ctx, layers, kv_gap_gib)
    stack.fill_caches()
    step = stack.step
    step_bytes = stack.step_bytes

    for _ in range(warmup):
        step(False)
    # timed region: K steps, nothing recorded between the kernels
    t0 = time.perf_counter()
    gpu_s = 0.0
    for _ in range(steps):
        g, _ = step(False)
        gpu_s += g
    wall = time.perf_counter() - t0
    # the same K steps again with an event after every kernel (each event costs a ~5 us gap, which
    # is why the throughput above is not taken from these): per-launch time of the decode kernel
    kern_s = 0.0
    launches = 0
    for _ in range(steps):
        _, (ks, kn) = step(True)
        kern_s += ks
        launches += kn
    checked = None
    if check:
        from oracle import oracle  # the checker only: nothing timed above touches it
        got = stack.outputs()
        assert np.isfinite(got).all(), "the timed step left outputs that are not finite"
        e_window = stack.check_window_layers(got, oracle)
        assert e_window < 2e-2, "window layers of the timed step are %.3g from the oracle" % e_window
        checked = {"window_layers_of_the_timed_step_max_abs_err": e_window}
        if ctx % STACK_PERIOD == 0:
            stack.fill_caches(STACK_PERIOD)
            stack.out.fill(0xFF)
            step(False)
            got = stack.outputs()
            e_full = stack.check_full_layers_periodic(got, oracle)
            e_win2 = stack.check_window_layers(got, oracle, STACK_PERIOD)
            assert e_full < 2e-2 and e_win2 < 2e-2, "the stack is %.3g / %.3g from the oracle" % (e_full, e_win2)
            checked["all_rows_periodic_fill_max_abs_err"] = max(e_full, e_win2)
            checked["rows_checked"] = layers * batch_size * H
        log("stack outputs checked:", checked)
    stack.free()
    per_launch_bytes = step_bytes * steps / launches
    per_launch_s = kern_s / launches
    return {
        "workload": "C5 long-context decode stack: 24 layers (even: 128-token window, odd: full causal), "
                    "batch %d, context %d, 64 q heads / 8 kv heads / head_dim 64, bf16 KV cache %.1f GiB resident"
                    % (batch_size, ctx, layers * 2 * batch_size * ctx * ROW / 2**30),
        "step_bytes": step_bytes,
        "wall_s_per_step": wall / steps,
        "gpu_s_per_step": gpu_s / steps,
        "value_gbs": step_bytes / (wall / steps) / 1e9,
        "tokens_per_s": batch_size / (wall / steps),
        "kernel": "lng_decode_bf16_d64",
        "kernel_launches_per_step": launches // steps,
        "kernel_bytes_per_launch": per_launch_bytes,
        "kernel_s_per_launch": per_launch_s,
        "kernel_gbs": per_launch_bytes / per_launch_s / 1e9,
        "outputs_checked": checked,
    }


def run_single_decode(gpu, steps, warmup, ctx=4096, burst=64):
    """Configuration 2: one query over 4096 cached positions, full-causal layer. 8.4 MB of
    traffic is about a microsecond at HBM speed, so one launch is latency-bound: reported as
    one launch per batch and as `burst` launches back to back in one batch."""
    q, out = gpu.buffer(QO), gpu.buffer(QO)
    k, v = gpu.buffer(ctx * ROW), gpu.buffer(ctx * ROW)
    sinks = gpu.upload(np.random.default_rng(2).standard_normal(H).astype(np.float32))
    for i, b in enumerate((q, k, v)):
        fill(gpu, b, 10 + i)
    bufs = [q, k, v, out, sinks]
    shape = C.GroupedShape(1, ctx - 1, H, G, D, C.FULL, ctx, SCALE)
    sl = (C.Slice(0, 0, QO), C.Slice(1, 0, ctx * ROW), C.Slice(2, 0, ctx * ROW))

    def go(n):
        batch = gpu.batch(bufs)
        for _ in range(n):
            batch.attention_grouped_with_sinks(sl, C.Slice(4, 0, H * 4), C.Slice(3, 0, QO), shape, C.BF16)
        t0 = time.perf_counter()
        done = batch.run()
        wall = time.perf_counter() - t0
        batch.drop()
        return done.gpu_time, wall

    for _ in range(max(warmup, 5)):
        go(1)
    one = sorted(go(1) for _ in range(max(steps, 20)))
    many = sorted(go(burst) for _ in range(max(steps, 5)))
    for b in bufs:
        b.free()
    # the same query over f32 caches (the reference's own element type; not the metric's): lng_decode_f32_d64
    qf, of = gpu.buffer(2 * QO), gpu.buffer(2 * QO)
    kf, vf = gpu.buffer(ctx * 2 * ROW), gpu.buffer(ctx * 2 * ROW)
    for i, b in enumerate((qf, kf, vf)):
        bb = gpu.batch([b])
        bb.fill_synthetic(C.Slice(0, 0, b.len), C.F32, 10 + i, 0.5, 0)
        bb.run()
        bb.drop()
    sinks32 = gpu.upload(np.random.default_rng(2).standard_normal(H).astype(np.float32))

    def go32():
        batch = gpu.batch([qf, kf, vf, of, sinks32])
        batch.attention_grouped_with_sinks((C.Slice(0, 0, 2 * QO), C.Slice(1, 0, ctx * 2 * ROW), C.Slice(2, 0, ctx * 2 * ROW)),
                                           C.Slice(4, 0, H * 4), C.Slice(3, 0, 2 * QO), shape, C.F32)
        done = batch.run()
        batch.drop()
        return done.gpu_time

    for _ in range(5):
        go32()
    f32_us = sorted(go32() for _ in range(max(steps, 20)))[max(steps, 20) // 2] * 1e6
    for b in (qf, of, kf, vf):
        b.free()
    # one sequence late in a long context (the reference's interactive case): bf16, 131,072 cached positions
    far = 131072
    qs, os_ = gpu.buffer(QO), gpu.buffer(QO)
    ks, vs = gpu.buffer(far * ROW), gpu.buffer(far * ROW)
    for i, b in enumerate((qs, ks, vs)):
        fill(gpu, b, 40 + i)
    far_shape = C.GroupedShape(1, far - 1, H, G, D, C.FULL, far, SCALE)

    def go_far():
        batch = gpu.batch([qs, ks, vs, os_, sinks32])
        batch.attention_grouped_with_sinks((C.Slice(0, 0, QO), C.Slice(1, 0, far * ROW), C.Slice(2, 0, far * ROW)),
                                           C.Slice(4, 0, H * 4), C.Slice(3, 0, QO), far_shape, C.BF16)
        done = batch.run()
        batch.drop()
        return done.gpu_time

    for _ in range(3):
        go_far()
    far_s = sorted(go_far() for _ in range(15))[7]
    far_bytes = decode_bytes(far, C.FULL)
    for b in (qs, os_, ks, vs):
        b.free()
    # one f32 layer of a decoding step: 16 sequences at a 32,768-token context (4.3 GB of cache rows)
    n_seq, long_ctx = 16, 32768
    qf, of = gpu.buffer(n_seq * 2 * QO), gpu.buffer(n_seq * 2 * QO)
    kf, vf = gpu.buffer(n_seq * long_ctx * 2 * ROW), gpu.buffer(n_seq * long_ctx * 2 * ROW)
    for i, b in enumerate((qf, kf, vf)):
        bb = gpu.batch([b])
        bb.fill_synthetic(C.Slice(0, 0, b.len), C.F32, 20 + i, 0.5, 0)
        bb.run()
        bb.drop()
    items = C.decode_items([C.DecodeItem(i * 2 * QO, i * 2 * QO, i * long_ctx * 2 * ROW, i * long_ctx * 2 * ROW, 0,
                                         long_ctx - 1, C.FULL, long_ctx) for i in range(n_seq)])

    def go32b():
        batch = gpu.batch([qf, kf, vf, of, sinks32])
        batch.attention_decode_batched(0, 1, 2, 3, 4, items, H, G, D, SCALE, C.F32)
        done = batch.run()
        batch.drop()
        return done.gpu_time

    for _ in range(3):
        go32b()
    f32_batch = sorted(go32b() for _ in range(9))[4]
    f32_batch_bytes = n_seq * (long_ctx * 2 * ROW * 2 + 4 * QO + H * 4)
    for b in (qf, of, kf, vf, sinks32):
        b.free()
    nbytes = decode_bytes(ctx, C.FULL)
    g1, w1 = one[len(one) // 2]
    gb, wb = many[len(many) // 2]
    return {"workload": "C2 decode, 1 query, 4096 cached positions, full-causal", "bytes": nbytes,
            "f32_caches_single_launch_gpu_us": f32_us,
            "one_sequence_131072": {"gpu_us": far_s * 1e6, "bytes": far_bytes, "gbs": far_bytes / far_s / 1e9,
                                    "hbm_frac": far_bytes / far_s / 1e9 / HBM_PEAK_GBS},
            "f32_caches_16_sequences_32768": {"gpu_us": f32_batch * 1e6, "bytes": f32_batch_bytes,
                                              "gbs": f32_batch_bytes / f32_batch / 1e9,
                                              "hbm_frac": f32_batch_bytes / f32_batch / 1e9 / HBM_PEAK_GBS},
            "single_launch_gpu_us": g1 * 1e6, "single_launch_wall_us": w1 * 1e6,
            "single_launch_gbs": nbytes / g1 / 1e9 if g1 > 0 else None,
            "burst": burst, "burst_gpu_us_per_launch": gb / burst * 1e6,
            "burst_gbs": nbytes * burst / gb / 1e9,
            "note": "8 MB working set stays in the 256 MB Infinity Cache across launches: cache-fed, not HBM-fed"}


def ragged_case(gpu, steps, warmup, n_seq):
    """n_seq sequences with lengths U{128..8192} (seed 3); per sequence one full-causal layer and one
    128-window layer. Timed as a model runs it (a dispatch per layer: all sequences of the full-causal
    layer, then all of the window layer) and with every (sequence, layer) in one dispatch."""
    rng = np.random.default_rng(3)
    lens = rng.integers(128, 8193, size=n_seq)
    offs = np.concatenate([[0], np.cumsum(lens)[:-1]])
    total = int(lens.sum())
    q, out = gpu.buffer(2 * n_seq * QO), gpu.buffer(2 * n_seq * QO)
    k, v = gpu.buffer(total * ROW), gpu.buffer(total * ROW)
    sinks = gpu.upload(rng.standard_normal((2, H)).astype(np.float32))
    for i, b in enumerate((q, k, v)):
        fill(gpu, b, 20 + i)
    bufs = [q, k, v, out, sinks]
    per_layer, nbytes = [], 0
    for layer, window in enumerate((C.FULL, 128)):
        items = []
        for s in range(n_seq):
            i = layer * n_seq + s
            items.append(C.DecodeItem(i * QO, i * QO, int(offs[s]) * ROW, int(offs[s]) * ROW, layer * H * 4,
                                      int(lens[s]) - 1, window, int(lens[s])))
            nbytes += decode_bytes(int(lens[s]), window)
        per_layer.append(items)
    tables = [C.decode_items(items) for items in per_layer]
    together = [C.decode_items(per_layer[0] + per_layer[1])]

    def go(tbs):
        batch = gpu.batch(bufs)
        for tb in tbs:
            batch.attention_decode_batched(0, 1, 2, 3, 4, tb, H, G, D, SCALE, C.BF16)
        t0 = time.perf_counter()
        done = batch.run()
        wall = time.perf_counter() - t0
        batch.drop()
        return done.gpu_time, wall

    res = {}
    for name, tbs in (("dispatch_per_layer", tables), ("one_dispatch", together)):
        for _ in range(max(warmup, 5)):
            go(tbs)
        runs = sorted(go(tbs) for _ in range(max(steps, 20)))
        res[name] = runs[len(runs) // 2]
    for b in bufs:
        b.free()
    return nbytes, res


def run_ragged(gpu, steps, warmup, n_seq=32):
    """Configuration 3 (32 sequences: 261 MB, which the 256 MB last-level cache partly holds across
    launches) and the same draw with 128 sequences (1.1 GB: fed from HBM). The figure reported is the step as ONE
    dispatch: a table of every (sequence, layer) row, full-causal rows first and window rows last, live workgroups
    only, then the merge of the rows that were cut; the step as a model with a dispatch per layer issues it is
    beside it."""
    nbytes, res = ragged_case(gpu, steps, warmup, n_seq)
    g, w = res["one_dispatch"]
    g2, w2 = res["dispatch_per_layer"]
    big_bytes, big = ragged_case(gpu, steps, warmup, 4 * n_seq)
    bg, bw = big["one_dispatch"]
    bg2, bw2 = big["dispatch_per_layer"]
    return {"workload": "C3 batched decode: %d sequences, lengths U{128..8192} (seed 3), full + 128-window layer each, "
                        "every (sequence, layer) row in one dispatch" % n_seq,
            "bytes": nbytes, "gpu_us": g * 1e6, "wall_us": w * 1e6, "gbs": nbytes / g / 1e9, "hbm_frac": nbytes / g / 1e9 / HBM_PEAK_GBS,
            "tokens_per_s": n_seq / w,
            "one_dispatch_per_layer": {"gpu_us": g2 * 1e6, "wall_us": w2 * 1e6, "gbs": nbytes / g2 / 1e9,
                                       "hbm_frac": nbytes / g2 / 1e9 / HBM_PEAK_GBS},
            "hbm_fed_%d_sequences" % (4 * n_seq): {"bytes": big_bytes, "gpu_us": bg * 1e6, "wall_us": bw * 1e6,
                                                    "gbs": big_bytes / bg / 1e9, "hbm_frac": big_bytes / bg / 1e9 / HBM_PEAK_GBS,
                                                    "tokens_per_s": 4 * n_seq / bw,
                                                    "one_dispatch_per_layer": {"gpu_us": bg2 * 1e6, "hbm_frac": big_bytes / bg2 / 1e9 / HBM_PEAK_GBS}},
            "note": "the %d-sequence step is about 280 MB: close to the 256 MB Infinity Cache, partly cache-fed; "
                    "the %d-sequence one is not" % (n_seq, 4 * n_seq)}


def run_prefill(gpu, steps, warmup, t=8192):
    """Configuration 4: one prompt pass of 8192 positions, once full-causal and once with a
    128-token window. FLOPs = 4 * dim * heads * (unmasked query-key pairs)."""
    q, out = gpu.buffer(t * QO), gpu.buffer(t * QO)
    k, v = gpu.buffer(t * ROW), gpu.buffer(t * ROW)
    sinks = gpu.upload(np.random.default_rng(4).standard_normal(H).astype(np.float32))
    for i, b in enumerate((q, k, v)):
        fill(gpu, b, 30 + i)
    bufs = [q, k, v, out, sinks]
    sl = (C.Slice(0, 0, t * QO), C.Slice(1, 0, t * ROW), C.Slice(2, 0, t * ROW))
    res = {}
    for name, window in (("full", C.FULL), ("window128", 128)):
        shape = C.GroupedShape(t, 0, H, G, D, window, t, SCALE)
        w = t if window == C.FULL else window
        pairs = w * (w + 1) // 2 + (t - w) * w
        flops = 4 * D * H * pairs

        def go(n=1):
            batch = gpu.batch(bufs)
            for _ in range(n):
                batch.attention_grouped_tiled_with_sinks(sl, C.Slice(4, 0, H * 4), C.Slice(3, 0, t * QO), shape,
                                                         C.BF16)
            done = batch.run()
            batch.drop()
            return done.gpu_time / n

        for _ in range(max(warmup, 5)):
            go()
        # after idle the clocks take tens of milliseconds of continuous work to settle (the first launches of a
        # pass run 15-30 % slower than the hundredth): batches of 20 launches until the time per launch stops falling
        last = go(20)
        for _ in range(12):
            cur = go(20)
            if cur > 0.99 * last:
                break
            last = cur
        runs = sorted(go() for _ in range(max(steps, 20)))
        g = runs[len(runs) // 2]
        go(20)
        sustained = sorted(go(20) for _ in range(5))[2]  # 20 launches back to back: no gap before each kernel
        traffic = 2 * t * QO + 2 * t * ROW
        res[name] = {"pairs": pairs, "flops": flops, "gpu_ms": g * 1e3, "tflops": flops / g / 1e12,
                     "mfma_frac": flops / g / 1e12 / MFMA_BF16_PEAK_TFLOPS,
                     "back_to_back_ms": sustained * 1e3, "back_to_back_tflops": flops / sustained / 1e12,
                     "back_to_back_mfma_frac": flops / sustained / 1e12 / MFMA_BF16_PEAK_TFLOPS,
                     "qkvo_bytes": traffic, "hbm_frac": traffic / g / 1e9 / HBM_PEAK_GBS}
    # the same full-causal pass the way the reference makes it: 512 rows at a time (engine.rs:51), 16 calls in
    # one batch; too few query tiles per call to fill the device, so the library takes the kernel of a workgroup
    # per pair of heads (lng_prefill_bf16_d64_pair)
    chunk = 512
    pairs = t * (t + 1) // 2

    def chunked():
        batch = gpu.batch(bufs)
        for start in range(0, t, chunk):
            rows = (start + chunk + 31) // 32 * 32
            batch.attention_grouped_tiled_with_sinks(
                (C.Slice(0, start * QO, chunk * QO), C.Slice(1, 0, rows * ROW), C.Slice(2, 0, rows * ROW)),
                C.Slice(4, 0, H * 4), C.Slice(3, start * QO, chunk * QO), C.GroupedShape(chunk, start, H, G, D, C.FULL, t, SCALE),
                C.BF16)
        done = batch.run()
        batch.drop()
        return done.gpu_time

    for _ in range(3):
        chunked()
    runs = sorted(chunked() for _ in range(max(steps, 10)))
    g = runs[len(runs) // 2]
    res["full_in_chunks_of_512"] = {"calls": t // chunk, "gpu_ms": g * 1e3, "tflops": 4 * D * H * pairs / g / 1e12,
                                    "mfma_frac": 4 * D * H * pairs / g / 1e12 / MFMA_BF16_PEAK_TFLOPS}
    # The timed fills above are benign (scores of standard deviation 0.25: the pass that keeps the maximum fixed never
    # fails its range check). The same full-causal pass on scores of standard deviation 4 (q and k of standard deviation
    # 2), with the query tiles counted that had to be made again with the maximum tracked.
    for i, b in enumerate((q, k)):
        fill(gpu, b, 30 + i, scale=2.0)
    shape = C.GroupedShape(t, 0, H, G, D, C.FULL, t, SCALE)

    def go4(n=1):
        batch = gpu.batch(bufs)
        for _ in range(n):
            batch.attention_grouped_tiled_with_sinks(sl, C.Slice(4, 0, H * 4), C.Slice(3, 0, t * QO), shape, C.BF16)
        done = batch.run()
        batch.drop()
        return done.gpu_time / n

    go4(20)
    go4(20)
    runs = sorted(go4() for _ in range(max(steps, 20)))
    g = runs[len(runs) // 2]
    gpu.debug_set("LNG_COUNT_SECOND_PASSES", "1")
    gpu.debug_get("LNG_COUNT_SECOND_PASSES")
    go4()
    repeated = gpu.debug_get("LNG_COUNT_SECOND_PASSES")
    gpu.debug_set("LNG_COUNT_SECOND_PASSES", None)
    res["full_std4"] = {"score_std": 4.0, "gpu_ms": g * 1e3, "tflops": 4 * D * H * pairs / g / 1e12,
                        "mfma_frac": 4 * D * H * pairs / g / 1e12 / MFMA_BF16_PEAK_TFLOPS,
                        "query_tiles": (t // 64) * G, "query_tiles_made_again_with_the_maximum_tracked": repeated}
    for b in bufs:
        b.free()
    # the same pass on f32 operands (the reference's element type): lng_prefill_f32_d64, bound by the f32 matrix rate
    q, out = gpu.buffer(t * QO * 2), gpu.buffer(t * QO * 2)
    k, v = gpu.buffer(t * ROW * 2), gpu.buffer(t * ROW * 2)
    for i, b in enumerate((q, k, v)):
        batch = gpu.batch([b])
        batch.fill_synthetic(C.Slice(0, 0, b.len), C.F32, 30 + i, 0.5, 0)
        batch.run()
        batch.drop()
    shape = C.GroupedShape(t, 0, H, G, D, C.FULL, t, SCALE)
    sinks = gpu.upload(np.random.default_rng(4).standard_normal(H).astype(np.float32))

    def go32():
        batch = gpu.batch([q, k, v, out, sinks])
        batch.attention_grouped_tiled_with_sinks((C.Slice(0, 0, q.len), C.Slice(1, 0, k.len), C.Slice(2, 0, v.len)),
                                                 C.Slice(4, 0, H * 4), C.Slice(3, 0, out.len), shape, C.F32)
        done = batch.run()
        batch.drop()
        return done.gpu_time

    go32()
    runs = sorted(go32() for _ in range(5))
    g = runs[len(runs) // 2]
    res["full_f32"] = {"gpu_ms": g * 1e3, "tflops": 4 * D * H * pairs / g / 1e12,
                       "mfma_f32_frac": 4 * D * H * pairs / g / 1e12 / MFMA_F32_PEAK_TFLOPS}
    for b in (q, out, k, v, sinks):
        b.free()
    res["workload"] = "C4 causal prefill, 8192 positions, 64 q / 8 kv heads, head_dim 64, bf16"
    return res


def run_prefill_lengths(gpu, steps, warmup):
    """The full-causal prompt pass at four lengths, split into what a query tile costs however many key tiles it
    walks and what a key tile costs. The resident kernel runs one workgroup per compute unit; a workgroup's time is
    (query tiles it takes) * a + (key tiles it walks) * b, and the four lengths give a and b by least squares."""
    cus = 256
    rows = []
    for t in (6144, 8192, 10240, 12288):  # (K and V of a kv head stay under 3 MB: past the 4 MB of an XCD's L2 the key tiles get dearer)
        q, out = gpu.buffer(t * QO), gpu.buffer(t * QO)
        k, v = gpu.buffer(t * ROW), gpu.buffer(t * ROW)
        sinks = gpu.upload(np.random.default_rng(4).standard_normal(H).astype(np.float32))
        for i, b in enumerate((q, k, v)):
            fill(gpu, b, 30 + i)
        bufs = [q, k, v, out, sinks]
        sl = (C.Slice(0, 0, t * QO), C.Slice(1, 0, t * ROW), C.Slice(2, 0, t * ROW))
        shape = C.GroupedShape(t, 0, H, G, D, C.FULL, t, SCALE)

        def go(n=20):
            batch = gpu.batch(bufs)
            for _ in range(n):
                batch.attention_grouped_tiled_with_sinks(sl, C.Slice(4, 0, H * 4), C.Slice(3, 0, t * QO), shape, C.BF16)
            done = batch.run()
            batch.drop()
            return done.gpu_time / n

        last = go()
        for _ in range(12):
            cur = go()
            if cur > 0.99 * last:
                break
            last = cur
        sec = sorted(go() for _ in range(5))[2]
        n = t // 64
        rows.append({"positions": t, "back_to_back_ms": sec * 1e3, "query_tiles_per_workgroup": n * G / cus,
                     "key_tiles_per_workgroup": G * n * (n + 1) / 2 / cus,
                     "mfma_frac": 4 * D * H * (t * (t + 1) // 2) / sec / 1e12 / MFMA_BF16_PEAK_TFLOPS})
        for b in bufs:
            b.free()
    a_mat = np.array([[r["query_tiles_per_workgroup"], r["key_tiles_per_workgroup"]] for r in rows])
    y = np.array([r["back_to_back_ms"] * 1e3 for r in rows])
    (per_query_tile, per_key_tile), *_ = np.linalg.lstsq(a_mat, y, rcond=None)
    first = rows[1]
    return {"kernel": "lng_prefill_bf16_d64_stream", "workgroups": cus, "lengths": rows,
            "us_per_query_tile_beyond_its_key_tiles": float(per_query_tile), "us_per_key_tile": float(per_key_tile),
            "share_outside_the_key_tiles_at_8192": float(per_query_tile * first["query_tiles_per_workgroup"] /
                                                         (first["back_to_back_ms"] * 1e3)),
            "residual_us": [float(x) for x in (a_mat @ np.array([per_query_tile, per_key_tile]) - y)]}


def run_prefill_activity(gpu, steps, warmup, t=8192):
    """The full-causal prompt pass of configuration 4 on all-zero inputs and on random inputs of two
    magnitudes, one launch at a time and 50 launches back to back in one batch. Same instructions, same
    memory traffic: a difference in time is the clock following the switching activity of the data."""
    res = {}
    for label, scale in (("zeros", 0.0), ("random_0.5", 0.5), ("random_2.0", 2.0)):
        q, out = gpu.buffer(t * QO), gpu.buffer(t * QO)
        k, v = gpu.buffer(t * ROW), gpu.buffer(t * ROW)
        sinks = gpu.upload(np.zeros(H, np.float32))
        for i, b in enumerate((q, k, v)):
            fill(gpu, b, 30 + i, scale=scale)
        bufs = [q, k, v, out, sinks]
        sl = (C.Slice(0, 0, t * QO), C.Slice(1, 0, t * ROW), C.Slice(2, 0, t * ROW))
        shape = C.GroupedShape(t, 0, H, G, D, C.FULL, t, SCALE)

        def go(n):
            batch = gpu.batch(bufs)
            for _ in range(n):
                batch.attention_grouped_tiled_with_sinks(sl, C.Slice(4, 0, H * 4), C.Slice(3, 0, t * QO), shape, C.BF16)
            done = batch.run()
            batch.drop()
            return done.gpu_time / n

        for _ in range(warmup):
            go(1)
        single = sorted(go(1) for _ in range(max(steps, 5)))
        res[label] = {"single_ms": single[len(single) // 2] * 1e3, "back_to_back_ms": go(50) * 1e3}
        for b in bufs:
            b.free()
    res["workload"] = "C4 full-causal prefill, 8192 positions, inputs of different switching activity"
    return res


def run_q8(gpu, steps, warmup):
    """The Q8_0 projection of gpt-oss-20b's queries (4096 x 2880) for one position, for one decoding
    step of 16 sequences and for a prompt pass of 8192 positions; the first two are bound by reading the
    matrix once (rows * cols code bytes + 2 bytes per 32), the last by the matrix unit."""
    rows, cols = 4096, 2880
    rng = np.random.default_rng(12)
    codes = gpu.resident(rng.integers(-127, 128, rows * cols, dtype=np.int8))
    scales = gpu.resident((rng.random(rows * cols // 32, dtype=np.float32) * 0.01 + 0.001).astype(np.float16).view(np.uint16))
    out = {}
    for label, n, kind in (("one_position", 1, "gemv"), ("decode_16_sequences", 16, "gemm"), ("prompt_8192", 8192, "tiled")):
        x, y = gpu.buffer(n * cols * 4), gpu.buffer(n * rows * 4)
        b = gpu.batch([x])
        b.fill_synthetic(C.Slice(0, 0, x.len), C.F32, 77, 0.5, 0)
        b.run()
        b.drop()

        def go():
            batch = gpu.batch([x, y])
            m = (batch.attach(codes), batch.attach(scales))
            xs, ys = C.Slice(0, 0, x.len), C.Slice(1, 0, y.len)
            if kind == "gemv":
                batch.gemv_q8_0(m, xs, ys, rows, cols)
            elif kind == "gemm":
                batch.gemm_q8_0(m, xs, ys, rows, cols, n, (cols, rows))
            else:
                batch.gemm_q8_0_tiled(m, xs, ys, rows, cols, n, (cols, rows))
            done = batch.run()
            batch.drop()
            return done.gpu_time

        for _ in range(warmup):
            go()
        runs = sorted(go() for _ in range(max(steps, 5)))
        g = runs[len(runs) // 2]
        nbytes = rows * cols + rows * cols // 32 * 2 + n * cols * 4 + n * rows * 4
        flops = 2 * n * rows * cols
        out[label] = {"positions": n, "gpu_us": g * 1e6, "bytes": nbytes, "gbs": nbytes / g / 1e9,
                      "hbm_frac": nbytes / g / 1e9 / HBM_PEAK_GBS, "tflops": flops / g / 1e12}
        x.free()
        y.free()
    # the q, k and v projections of one decoding position (4096, 512 and 512 rows): three products as the reference
    # records them (gpu.rs:724-732), and as one dispatch
    kv_rows = 512
    k_codes = gpu.resident(rng.integers(-127, 128, kv_rows * cols, dtype=np.int8))
    k_scales = gpu.resident((rng.random(kv_rows * cols // 32, dtype=np.float32) * 0.01 + 0.001).astype(np.float16).view(np.uint16))
    x, y = gpu.buffer(cols * 4), gpu.buffer((rows + 2 * kv_rows) * 4)
    b = gpu.batch([x])
    b.fill_synthetic(C.Slice(0, 0, x.len), C.F32, 79, 0.5, 0)
    b.run()
    b.drop()
    for label, together in (("qkv_one_position_three_dispatches", False), ("qkv_one_position_one_dispatch", True)):
        def go3():
            batch = gpu.batch([x, y])
            mq, mk = (batch.attach(codes), batch.attach(scales)), (batch.attach(k_codes), batch.attach(k_scales))
            xs = C.Slice(0, 0, x.len)
            ys = [C.Slice(1, 0, rows * 4), C.Slice(1, rows * 4, kv_rows * 4), C.Slice(1, (rows + kv_rows) * 4, kv_rows * 4)]
            if together:
                batch.gemm_q8_0_many([(mq, ys[0], rows), (mk, ys[1], kv_rows), (mk, ys[2], kv_rows)], xs, cols, 1, cols)
            else:
                batch.gemv_q8_0(mq, xs, ys[0], rows, cols)
                batch.gemv_q8_0(mk, xs, ys[1], kv_rows, cols)
                batch.gemv_q8_0(mk, xs, ys[2], kv_rows, cols)
            done = batch.run()
            batch.drop()
            return done.gpu_time

        for _ in range(warmup):
            go3()
        runs = sorted(go3() for _ in range(max(steps, 9)))
        out[label] = {"gpu_us": runs[len(runs) // 2] * 1e6}
    x.free()
    y.free()
    # the same matrix on bf16 positions (what a bf16 attention leaves for the output projection): one operand
    # plane instead of two, no split of x
    for label, n in (("decode_16_sequences_bf16_positions", 16), ("prompt_8192_bf16_positions", 8192)):
        x, y = gpu.buffer(n * cols * 2), gpu.buffer(n * rows * 4)
        b = gpu.batch([x])
        b.fill_synthetic(C.Slice(0, 0, x.len), C.BF16, 78, 0.5, 0)
        b.run()
        b.drop()

        def go16():
            batch = gpu.batch([x, y])
            batch.gemm_q8_0_bf16((batch.attach(codes), batch.attach(scales)), C.Slice(0, 0, x.len), C.Slice(1, 0, y.len),
                                 rows, cols, n, (cols, rows))
            done = batch.run()
            batch.drop()
            return done.gpu_time

        for _ in range(warmup):
            go16()
        runs = sorted(go16() for _ in range(max(steps, 5)))
        g = runs[len(runs) // 2]
        out[label] = {"positions": n, "gpu_us": g * 1e6, "tflops": 2 * n * rows * cols / g / 1e12}
        x.free()
        y.free()
    codes.free()
    scales.free()
    out["workload"] = "Q8_0 product, 4096 x 2880 (gpt-oss-20b query projection), f32 positions unless named otherwise"
    return out


def run_config1(gpu, steps, warmup):
    """Configuration 1 (the reference's own CPU-runnable case): f32, 4 query heads over 1 kv head of 64,
    32 positions, full causal, through the plain operator (the general kernel)."""
    t, heads, kv = 32, 4, 1
    rng = np.random.default_rng(0)
    q = rng.standard_normal((t, heads, D)).astype(np.float32)
    k = rng.standard_normal((t, kv, D)).astype(np.float32)
    v = rng.standard_normal((t, kv, D)).astype(np.float32)
    sinks = rng.standard_normal(heads).astype(np.float32)
    bufs = [gpu.upload(q), gpu.upload(k), gpu.upload(v), gpu.buffer(q.nbytes), gpu.upload(sinks)]
    shape = C.GroupedShape(t, 0, heads, kv, D, C.FULL, t, SCALE)

    def go():
        batch = gpu.batch(bufs)
        batch.attention_grouped_with_sinks((C.Slice(0, 0, q.nbytes), C.Slice(1, 0, k.nbytes), C.Slice(2, 0, v.nbytes)),
                                           C.Slice(4, 0, heads * 4), C.Slice(3, 0, q.nbytes), shape, C.F32)
        done = batch.run()
        batch.drop()
        return done.gpu_time

    for _ in range(warmup):
        go()
    runs = sorted(go() for _ in range(max(steps, 20)))
    for b in bufs:
        b.free()
    return {"workload": "C1 fp32: 4 q heads / 1 kv head of 64, 32 positions, full causal", "gpu_us": runs[len(runs) // 2] * 1e6}


def cpu_extras():
    """The oracle (f32 port of gpt-oss/src/model.rs:434-464) timed on the host for configurations 1-4, on
    all cores (OpenMP over query rows and heads) and on one thread. Configuration 4 is timed on 64
    query rows spread over the pass and scaled by the ratio of query-key pairs (stated as extrapolated)."""
    from oracle import oracle
    cores = oracle_threads()
    rng = np.random.default_rng(21)

    def timed(fn):
        out = {}
        for label, threads in (("all", cores), ("one", 1)):
            t0 = time.perf_counter()
            fn(threads)
            out[label] = time.perf_counter() - t0
        return out

    res = {}
    # C1
    q = rng.standard_normal((32, 4, D)).astype(np.float32)
    k = rng.standard_normal((32, 1, D)).astype(np.float32)
    v = rng.standard_normal((32, 1, D)).astype(np.float32)
    s4 = rng.standard_normal(4).astype(np.float32)
    t1 = timed(lambda th: oracle.attention_f32(q, k, v, s4, 0, scale=SCALE, threads=th))
    res["c1"] = {"us": t1["all"] * 1e6, "us_1thread": t1["one"] * 1e6, "cores": cores, "kind": "port", "sample": "whole case"}
    # C2
    sinks = rng.standard_normal(H).astype(np.float32)
    q = bf16_widen(bf16_bits(rng.standard_normal((1, H, D), dtype=np.float32) * 0.5))
    k = bf16_widen(bf16_bits(rng.standard_normal((8192, G, D), dtype=np.float32) * 0.5))
    v = bf16_widen(bf16_bits(rng.standard_normal((8192, G, D), dtype=np.float32) * 0.5))
    t2 = timed(lambda th: oracle.attention_f32(q, k[:4096], v[:4096], sinks, 4095, scale=SCALE, threads=th))
    nb = decode_bytes(4096, C.FULL)
    res["c2"] = {"us": t2["all"] * 1e6, "gbs": nb / t2["all"] / 1e9, "us_1thread": t2["one"] * 1e6,
                 "gbs_1thread": nb / t2["one"] / 1e9, "cores": cores, "kind": "port", "sample": "whole case"}
    # C3: the same lengths as the GPU leg; every sequence reads a prefix of one 8192-position cache
    lens = np.random.default_rng(3).integers(128, 8193, size=32)
    nb = sum(decode_bytes(int(n), C.FULL) + decode_bytes(int(n), 128) for n in lens)

    def c3(th):
        for n in lens:
            n = int(n)
            oracle.attention_f32(q, k[:n], v[:n], sinks, n - 1, scale=SCALE, threads=th)
            oracle.attention_f32(q, k[:n], v[:n], sinks, n - 1, window=128, scale=SCALE, threads=th)
    t3 = timed(c3)
    res["c3"] = {"ms": t3["all"] * 1e3, "gbs": nb / t3["all"] / 1e9, "tokens_per_s": 32 / t3["all"],
                 "ms_1thread": t3["one"] * 1e3, "gbs_1thread": nb / t3["one"] / 1e9, "cores": cores, "kind": "port",
                 "sample": "whole case (32 sequences x 2 layers)"}
    # C4: 64 sampled query rows of the 8192-position pass
    t = 8192
    pos = np.linspace(63, t - 1, 64).astype(np.uint64)
    qs = bf16_widen(bf16_bits(rng.standard_normal((64, H, D), dtype=np.float32) * 0.5))
    res["c4"] = {}
    for name, window in (("full", C.FULL), ("window128", 128)):
        w = t if window == C.FULL else window
        pairs = w * (w + 1) // 2 + (t - w) * w
        sampled = int(sum(min(int(p) + 1, w) for p in pos))
        t4 = timed(lambda th: oracle.attention_rows_f32(qs, k, v, sinks, pos, window=window, scale=SCALE, threads=th))
        flops = 4 * D * H * pairs
        scale_up = pairs / sampled
        res["c4"][name] = {"extrapolated_s": t4["all"] * scale_up, "tflops": flops / (t4["all"] * scale_up) / 1e12,
                           "extrapolated_s_1thread": t4["one"] * scale_up,
                           "tflops_1thread": flops / (t4["one"] * scale_up) / 1e12, "cores": cores, "kind": "port",
                           "sample": "64 of 8192 query rows, evenly spaced; time scaled by %.1f (ratio of query-key pairs)" % scale_up}
    return res


def run_copy(gpu, steps, warmup, nbytes=1 << 30):
    """A plain copy of known size through lng_copy_rows: the yardstick that the FETCH_SIZE and
    WRITE_SIZE counters of a profile are scaled by (it reads nbytes and writes nbytes)."""
    src, dst = gpu.buffer(nbytes), gpu.buffer(nbytes)
    fill(gpu, src, 99)
    width = 1 << 16
    rows = nbytes // 4 // width

    def go():
        batch = gpu.batch([src, dst])
        batch.copy_rows((C.Slice(0, 0, nbytes), width), (C.Slice(1, 0, nbytes), width), rows, width, C.F32, C.F32)
        done = batch.run()
        batch.drop()
        return done.gpu_time

    for _ in range(warmup):
        go()
    runs = sorted(go() for _ in range(max(steps, 3)))
    src.free()
    dst.free()
    g = runs[len(runs) // 2]
    return {"workload": "copy of %d bytes (lng_copy_rows, f32)" % nbytes, "read_bytes": nbytes, "write_bytes": nbytes,
            "gpu_ms": g * 1e3, "gbs": 2 * nbytes / g / 1e9}


def run_read(gpu, steps, warmup, nbytes=4 << 30):
    """A plain streaming read of 4 GiB (lng_checksum: nothing but whole-line loads and an XOR): what the memory system
    of this box delivers to a kernel that only reads, the yardstick beside the decode kernels' rate."""
    src, dst = gpu.buffer(nbytes), gpu.buffer(16)
    fill(gpu, src, 98)

    def go():
        batch = gpu.batch([src, dst])
        batch.set_timing(True)
        batch.checksum(C.Slice(0, 0, nbytes), C.Slice(1, 0, 16))
        batch.run()
        t = batch.kernel_seconds("lng_checksum")[0]
        batch.drop()
        return t

    for _ in range(max(warmup, 2)):
        go()
    runs = sorted(go() for _ in range(max(steps, 7)))
    src.free()
    dst.free()
    g = runs[len(runs) // 2]
    return {"workload": "streaming read of %d bytes (lng_checksum)" % nbytes, "read_bytes": nbytes, "gpu_ms": g * 1e3,
            "gbs": nbytes / g / 1e9, "hbm_frac": nbytes / g / 1e9 / HBM_PEAK_GBS}


def run_block(gpu, steps, warmup, ctx=4096, layers=24):
    """One decoding token through the attention block of gpt-oss/src/gpu.rs:703-827 at gpt-oss-20b's sizes (hidden
    2880, 64 q / 8 kv heads of 64, Q8_0 projections), `layers` times in one batch over a bf16 cache of `ctx` tokens:
    as the reference records it (with prepare_attention for its seven pre-attention dispatches), with the q, k and v
    projections as one call, and with the RMS norm, the bias and the residual folded into the products as well.
    Launch-bound: microseconds per layer."""
    hidden, qw, kw = 2880, H * D, G * D
    rng = np.random.default_rng(21)

    def q8(rows, cols):
        return (gpu.resident(rng.integers(-127, 128, rows * cols, dtype=np.int8)),
                gpu.resident((rng.random(rows * cols // 32, dtype=np.float32) * 0.01 + 0.001).astype(np.float16).view(np.uint16)))

    wq, wk, wv, wo = q8(qw, hidden), q8(kw, hidden), q8(kw, hidden), q8(hidden, qw)
    consts = {name: gpu.resident(arr) for name, arr in (
        ("norm", np.ones(hidden, np.float32)), ("qb", np.zeros(qw, np.float32)), ("kb", np.zeros(kw, np.float32)),
        ("vb", np.zeros(kw, np.float32)), ("ob", np.zeros(hidden, np.float32)), ("sinks", np.zeros(H, np.float32)))}
    f32 = lambda n: gpu.buffer(n * 4)  # noqa: E731
    bufs = [f32(hidden), f32(hidden), f32(qw), f32(kw), f32(kw), f32(D), gpu.buffer(qw * 2), gpu.buffer(ctx * kw * 2),
            gpu.buffer(ctx * kw * 2), gpu.buffer(qw * 2), f32(hidden)]
    iH, iX, iQ, iK, iV, iT, iQR, iKC, iVC, iATT, iTMP = range(11)
    for i in (iH, iT):
        bufs[i].write(np.full(bufs[i].len // 4, 0.1, np.float32))
    for i in (iKC, iVC):
        fill(gpu, bufs[i], 50 + i)
    start = ctx - 1
    S = lambda b, n, es=4: C.Slice(b, 0, n * es)  # noqa: E731

    def go(mode):
        batch = gpu.batch(bufs)
        at = batch.attach
        mats = [((at(w[0]), at(w[1])), S(y, rows), rows) for w, y, rows in ((wq, iQ, qw), (wk, iK, kw), (wv, iV, kw))]
        for _ in range(layers):
            if mode == "folded":
                batch.gemm_q8_0_many_normed(mats, S(iH, hidden), (at(consts["norm"]), 1e-5), hidden, 1, hidden)
            else:
                batch.copy_rows((S(iH, hidden), hidden), (S(iX, hidden), hidden), 1, hidden)
                batch.rmsnorm_rows((S(iX, hidden), at(consts["norm"])), 1, (hidden, hidden), 1e-5)
                if mode == "one_qkv_call":
                    batch.gemm_q8_0_many(mats, S(iX, hidden), hidden, 1, hidden)
                else:
                    for m, y, rows in mats:
                        batch.gemv_q8_0(m, S(iX, hidden), y, rows, hidden)
            batch.prepare_attention(dict(q=iQ, k=iK, v=iV, table=iT, q_out=iQR, k_cache=iKC, v_cache=iVC),
                                    [C.PrepareItem(n=1, start=start, slots=ctx)], H, G, D, D, C.BF16, at(consts["qb"]),
                                    at(consts["kb"]), at(consts["vb"]))
            batch.attention_grouped_with_sinks((S(iQR, qw, 2), S(iKC, ctx * kw, 2), S(iVC, ctx * kw, 2)), at(consts["sinks"]),
                                               S(iATT, qw, 2), C.GroupedShape(1, start, H, G, D, C.FULL, ctx, SCALE), C.BF16)
            mo = (at(wo[0]), at(wo[1]))
            if mode == "folded":
                batch.gemm_q8_0_residual(mo, S(iATT, qw, 2), at(consts["ob"]), S(iH, hidden), hidden, qw, 1, (qw, hidden), C.BF16)
            else:
                batch.gemm_q8_0_bf16(mo, S(iATT, qw, 2), S(iTMP, hidden), hidden, qw, 1, (qw, hidden))
                batch.add_rows(S(iTMP, hidden), (at(consts["ob"]), 0), 1, hidden)
                batch.add_rows(S(iH, hidden), (S(iTMP, hidden), hidden), 1, hidden)
        n = batch.dispatches()
        done = batch.run()
        batch.drop()
        return done.gpu_time, n

    out = {"workload": "one decoding token through %d attention blocks (gpt-oss-20b sizes), bf16 cache of %d tokens" % (layers, ctx)}
    for mode in ("as_the_reference_records_it", "one_qkv_call", "folded"):
        for _ in range(warmup):
            go(mode)
        runs = sorted(go(mode) for _ in range(max(steps, 7)))
        t, n = runs[len(runs) // 2]
        out[mode] = {"dispatches_per_layer": n // layers, "gpu_us_per_layer": t * 1e6 / layers}
    for b in bufs:
        b.free()
    return out


def run_prepare(gpu, steps, warmup):
    """The step before attention (biases, rotation by halves, bf16 narrowing, ring append) at gpt-oss
    shapes: a prompt pass of 8192 rows into a flat cache, and one decoding step of 16 sequences (one
    dispatch each). Bytes: per row 80 heads x 64 f32 in, 64 (cos, sin) f32, 80 x 64 bf16 out; biases once."""
    qw, kw = H * D, G * D
    row_bytes = (qw + 2 * kw) * 4 + D * 4 + (qw + 2 * kw) * 2
    out = {}
    for label, seqs, n, slots in (("prompt_8192", 1, 8192, 8192), ("decode_16_sequences", 16, 1, 640)):
        rows = seqs * n
        bufs = [gpu.buffer(rows * qw * 4), gpu.buffer(rows * kw * 4), gpu.buffer(rows * kw * 4),
                gpu.buffer(rows * D * 4), gpu.buffer(rows * qw * 2), gpu.buffer(seqs * slots * kw * 2),
                gpu.buffer(seqs * slots * kw * 2), gpu.buffer((qw + 2 * kw) * 4)]
        for i in (0, 1, 2, 7):
            b = gpu.batch([bufs[i]])
            b.fill_synthetic(C.Slice(0, 0, bufs[i].len), C.F32, 40 + i, 0.5, 0)
            b.run()
            b.drop()
        inv = 150000.0 ** (-np.arange(D // 2, dtype=np.float64) / (D // 2))
        bufs[3].write(np.concatenate([C.rope_table(inv, 1.3465736, 5000 + 37 * s, n) for s in range(seqs)]))
        items = C.prepare_items([C.PrepareItem(q_offset=s * n * qw * 4, k_offset=s * n * kw * 4, v_offset=s * n * kw * 4,
                                               table_offset=s * n * D * 4, q_out_offset=s * n * qw * 2,
                                               k_cache_offset=s * slots * kw * 2, v_cache_offset=s * slots * kw * 2,
                                               n=n, start=5000 + 37 * s, slots=slots) for s in range(seqs)])
        names = dict(q=0, k=1, v=2, table=3, q_out=4, k_cache=5, v_cache=6)
        bias = [C.Slice(7, 0, qw * 4), C.Slice(7, qw * 4, kw * 4), C.Slice(7, (qw + kw) * 4, kw * 4)]

        def go():
            batch = gpu.batch(bufs)
            batch.prepare_attention(names, items, H, G, D, D, C.BF16, *bias)
            done = batch.run()
            batch.drop()
            return done.gpu_time

        for _ in range(warmup):
            go()
        runs = sorted(go() for _ in range(max(steps, 5)))
        g = runs[len(runs) // 2]
        nbytes = rows * row_bytes + (qw + 2 * kw) * 4
        out[label] = {"rows": rows, "bytes": nbytes, "gpu_us": g * 1e6, "gbs": nbytes / g / 1e9,
                      "hbm_frac": nbytes / g / 1e9 / HBM_PEAK_GBS}
        for b in bufs:
            b.free()
    out["kernel"] = "lng_prepare_v4"
    return out


def run_wide_heads(gpu, steps, warmup):
    """The operator's other caller in the reference (decider/src/gpu.rs:878-893): 32 heads over 16 kv heads of
    width 256, decoding. bf16 caches, one dispatch per layer: one sequence and sixteen at 32,768 cached positions
    (0.5 and 8.6 GB of cache rows per launch: HBM-fed), the kernels that walk the head in slices of 64 beside the
    kernel of one wavefront per (row, head) (LNG_WIDE_GENERIC=1)."""
    heads, kv_heads, dim, ctx = 32, 16, 256, 32768
    row, qo = kv_heads * dim * 2, heads * dim * 2
    scale = 1.0 / float(np.sqrt(np.float32(dim)))
    out = {"workload": "32 heads over 16 kv heads of width 256, bf16, 32768 cached positions, decode"}
    sinks = gpu.upload(np.random.default_rng(3).standard_normal(heads).astype(np.float32))
    for n_seq in (1, 16):
        q, o = gpu.buffer(n_seq * qo), gpu.buffer(n_seq * qo)
        k, v = gpu.buffer(n_seq * ctx * row), gpu.buffer(n_seq * ctx * row)
        for i, b in enumerate((q, k, v)):
            fill(gpu, b, 60 + i)
        items = C.decode_items([C.DecodeItem(i * qo, i * qo, i * ctx * row, i * ctx * row, 0, ctx - 1, C.FULL, ctx)
                                for i in range(n_seq)])

        def go():
            batch = gpu.batch([q, k, v, o, sinks])
            batch.attention_decode_batched(0, 1, 2, 3, 4, items, heads, kv_heads, dim, scale, C.BF16)
            done = batch.run()
            batch.drop()
            return done.gpu_time

        nbytes = n_seq * (2 * ctx * row + 2 * qo + heads * 4)
        res = {"bytes": nbytes}
        for name, env in (("sliced", None), ("one_wavefront_per_head", "1")):
            if env:
                gpu.debug_set("LNG_WIDE_GENERIC", env)
            try:
                for _ in range(max(2, warmup)):
                    go()
                n = max(steps, 9)
                t = sorted(go() for _ in range(n))[n // 2]
            finally:
                gpu.debug_set("LNG_WIDE_GENERIC", None)
            res[name] = {"gpu_us": t * 1e6, "gbs": nbytes / t / 1e9, "hbm_frac": nbytes / t / 1e9 / HBM_PEAK_GBS}
        out["%d_sequences" % n_seq] = res
        for b in (q, o, k, v):
            b.free()
    # the reference's own element type at the same shape: 16 sequences of 16,384 positions (8.6 GB of f32 cache rows)
    n_seq, ctx32 = 16, 16384
    row32, qo32 = kv_heads * dim * 4, heads * dim * 4
    q, o = gpu.buffer(n_seq * qo32), gpu.buffer(n_seq * qo32)
    k, v = gpu.buffer(n_seq * ctx32 * row32), gpu.buffer(n_seq * ctx32 * row32)
    for i, b in enumerate((q, k, v)):
        bb = gpu.batch([b])
        bb.fill_synthetic(C.Slice(0, 0, b.len), C.F32, 70 + i, 0.5, 0)
        bb.run()
        bb.drop()
    items = C.decode_items([C.DecodeItem(i * qo32, i * qo32, i * ctx32 * row32, i * ctx32 * row32, 0, ctx32 - 1, C.FULL, ctx32)
                            for i in range(n_seq)])

    def go32():
        batch = gpu.batch([q, k, v, o, sinks])
        batch.attention_decode_batched(0, 1, 2, 3, 4, items, heads, kv_heads, dim, scale, C.F32)
        done = batch.run()
        batch.drop()
        return done.gpu_time

    for _ in range(max(2, warmup)):
        go32()
    n = max(steps, 9)
    t = sorted(go32() for _ in range(n))[n // 2]
    nbytes = n_seq * (2 * ctx32 * row32 + 2 * qo32 + heads * 4)
    out["f32_16_sequences_16384"] = {"bytes": nbytes, "gpu_us": t * 1e6, "gbs": nbytes / t / 1e9, "hbm_frac": nbytes / t / 1e9 / HBM_PEAK_GBS}
    for b in (q, o, k, v):
        b.free()
    sinks.free()
    return out


def run_gemma(gpu, steps, warmup):
    """The reference's own timing harness (metal-compute/tests/attention_grouped.rs:281-358 `gemma_shapes_timing`):
    five attention shapes of its other model (32 heads over 16 kv heads of width 256 with a 1024-token window in a ring
    of 1536; 32 over 4 of width 512, full), the tiled operator from 32 positions on and the row-by-row one below, f32
    as the reference times them, scale 1, no sinks; bf16 beside. Median GPU time of one dispatch. `m4_pro_gpu_ms` is the
    figure docs/NPU_ACCELERATION.md:202-208 publishes for the Metal kernel on an M4 Pro (context, not a baseline on this
    hardware). FLOPs = 4 * dim * heads * (unmasked query-key pairs)."""
    full = C.FULL
    cases = [("sliding_512_pass_wrapped", (512, 2600, 32, 16, 256, 1024, 1536), 21.9),
             ("sliding_first_512", (512, 0, 32, 16, 256, 1024, 1536), 6.1),
             ("sliding_one_token_at_3000", (1, 3000, 32, 16, 256, 1024, 1536), 0.6),
             ("full_77_after_700", (77, 700, 32, 4, 512, full, 32768), 8.1),
             ("full_one_token_at_1500", (1, 1500, 32, 4, 512, full, 32768), 1.7)]
    out = {"workload": "attention_grouped.rs:286-306, five shapes, scale 1, no sinks; synthetic fill (centred sum of four uniforms, std 0.5)"}
    for name, (t, start, heads, kv_heads, dim, window, slots), m4 in cases:
        tiled = t >= 32
        end = start + t
        rows = (t + 31) // 32 * 32 if tiled else t
        kv_rows = min(slots, end) if not tiled else (slots if slots < end else (end + 31) // 32 * 32)
        pairs = sum(min(start + i + 1, window) for i in range(t))
        flops = 4 * dim * heads * pairs
        res = {"shape": [t, start, heads, kv_heads, dim, "full" if window == full else window, slots], "operator": "tiled" if tiled else "plain",
               "pairs": pairs, "flops": flops, "m4_pro_gpu_ms": m4}
        for label, dtype, es in (("f32", C.F32, 4), ("bf16", C.BF16, 2)):
            q, o = gpu.buffer(rows * heads * dim * es), gpu.buffer(rows * heads * dim * es)
            k, v = gpu.buffer(kv_rows * kv_heads * dim * es), gpu.buffer(kv_rows * kv_heads * dim * es)
            for i, b in enumerate((q, k, v)):
                batch = gpu.batch([b])
                batch.fill_synthetic(C.Slice(0, 0, b.len), dtype, 70 + i, 0.5, 0)
                batch.run()
                batch.drop()
            shape = C.GroupedShape(t, start, heads, kv_heads, dim, window, slots, 1.0)
            sl = (C.Slice(0, 0, q.len), C.Slice(1, 0, k.len), C.Slice(2, 0, v.len), C.Slice(3, 0, o.len))

            def go():
                batch = gpu.batch([q, k, v, o])
                (batch.attention_grouped_tiled if tiled else batch.attention_grouped)(*sl, shape, dtype)
                done = batch.run()
                batch.drop()
                return done.gpu_time

            for _ in range(max(warmup, 3)):
                go()
            n = max(steps, 15)
            g = sorted(go() for _ in range(n))[n // 2]
            nbytes = (2 * rows * heads * dim + 2 * min(kv_rows, min(end, window + t)) * kv_heads * dim) * es
            peak = MFMA_F32_PEAK_TFLOPS if dtype == C.F32 else MFMA_BF16_PEAK_TFLOPS
            res[label] = {"gpu_ms": g * 1e3, "tflops": flops / g / 1e12, "mfma_frac": flops / g / 1e12 / peak,
                          "bytes": nbytes, "hbm_frac": nbytes / g / 1e9 / HBM_PEAK_GBS}
            for b in (q, o, k, v):
                b.free()
        out[name] = res
    return out


def oracle_threads():
    """Threads the oracle is timed on: the cores this process may use (its affinity mask, and OMP_NUM_THREADS when
    the environment sets it: the GPU boxes grant a one-GPU job 16 of the host's cores), never more than the host has."""
    n = os.cpu_count() or 1
    try:
        n = min(n, len(os.sched_getaffinity(0)))
    except (AttributeError, OSError):
        pass
    env = os.environ.get("OMP_NUM_THREADS", "")
    if env.isdigit() and int(env) > 0:
        n = min(n, int(env))
    return n


def cpu_baseline(step_bytes_per_seq_pair, ctx=131072):
    """The oracle (port of the reference's CPU attention, f32 on widened bf16 inputs) on a
    bounded sample of the headline workload: one sequence, one full-causal and one 128-window
    layer at the full context. GB/s is counted on the same algorithmic bf16 bytes as the GPU."""
    from oracle import oracle
    rng = np.random.default_rng(9)
    q = bf16_widen(bf16_bits(rng.standard_normal((1, H, D), dtype=np.float32) * 0.5))
    k = bf16_widen(bf16_bits(rng.standard_normal((ctx, G, D), dtype=np.float32) * 0.5))
    v = bf16_widen(bf16_bits(rng.standard_normal((ctx, G, D), dtype=np.float32) * 0.5))
    sinks = rng.standard_normal(H).astype(np.float32)
    cores = oracle_threads()
    nbytes = decode_bytes(ctx, C.FULL) + decode_bytes(ctx, 128)
    out = {}
    for label, threads in (("all", cores), ("one", 1)):
        times = []
        for _ in range(3):  # about 7 s of CPU work in all; the median of three
            t0 = time.perf_counter()
            oracle.attention_f32(q, k, v, sinks, ctx - 1, window=C.FULL, scale=SCALE, threads=threads)
            oracle.attention_f32(q, k, v, sinks, ctx - 1, window=128, scale=SCALE, threads=threads)
            times.append(time.perf_counter() - t0)
        out[label] = sorted(times)[1]
    return {"value": nbytes / out["all"] / 1e9, "unit": "GB/s", "cores": cores, "host_cpu_count": os.cpu_count(), "kind": "port",
            "sample": "1 sequence x (1 full-causal + 1 window-128 layer) at context %d, %.0f MB of bf16 KV; "
                      "the 16 x 12 such pairs of a step scale linearly; median of 3 runs" % (ctx, nbytes / 1e6),
            "seconds": out["all"], "value_1thread": nbytes / out["one"] / 1e9, "seconds_1thread": out["one"],
            "note": "the reference walks heads on one thread (gpt-oss/src/model.rs:439); "
                    "value uses OpenMP over (query, head) on `cores` threads"}


def main():
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=10)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--ctx", type=int, default=131072, help="context of the decode stack")
    ap.add_argument("--batch", type=int, default=16)
    ap.add_argument("--kv-gap-gib", type=int, default=None, help="allocate all K caches, this many GiB unused, then "
                    "all V caches, instead of K and V layer by layer (placement experiment)")
    ap.add_argument("--no-extras", action="store_true", help="skip configurations 2, 3 and 4")
    ap.add_argument("--only", default="", help="comma list of c2,c3,c4,c4act,c4fit,copy,read,prep,q8,block,wide,gemma: run just these and print their results "
                    "(a development aid; no headline line)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline")
    ap.add_argument("--record-traffic", metavar="DIR", default="", help="no GPU work: turn the rocprofv3 counter runs under DIR "
                    "(see record_traffic) into profiles/decode_stack_c5_hbm_traffic.json")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (--gpus must be 1)", file=sys.stderr)
        sys.exit(2)
    if args.record_traffic:
        record_traffic(args.record_traffic, args.ctx, args.batch)
        return
    gpu = C.Gpu(0)
    log("device:", gpu.name())
    extra = {}
    if args.only:
        runs = {"c2": run_single_decode, "c3": run_ragged, "c4": run_prefill, "copy": run_copy, "prep": run_prepare, "block": run_block,
                "c4act": run_prefill_activity, "c4fit": run_prefill_lengths, "q8": run_q8, "wide": run_wide_heads, "gemma": run_gemma, "read": run_read}
        for name in args.only.split(","):
            print(json.dumps({name: runs[name](gpu, args.steps, args.warmup)}))
        gpu.close()
        return
    if not args.no_extras:
        extra["c2_single_decode"] = run_single_decode(gpu, args.steps, args.warmup)
        log("c2", extra["c2_single_decode"])
        extra["c3_ragged_batch"] = run_ragged(gpu, args.steps, args.warmup)
        log("c3", extra["c3_ragged_batch"])
        extra["c4_prefill"] = run_prefill(gpu, args.steps, args.warmup)
        extra["c4_prefill"]["full_by_length"] = run_prefill_lengths(gpu, args.steps, args.warmup)
        log("c4", extra["c4_prefill"])
        extra["pre_attention_step"] = run_prepare(gpu, args.steps, args.warmup)
        log("prep", extra["pre_attention_step"])
        extra["q8_0_projection"] = run_q8(gpu, args.steps, args.warmup)
        log("q8", extra["q8_0_projection"])
        extra["decode_block_one_token"] = run_block(gpu, args.steps, args.warmup)
        log("block", extra["decode_block_one_token"])
        extra["c1_fp32"] = run_config1(gpu, args.steps, args.warmup)
        extra["head_width_256"] = run_wide_heads(gpu, args.steps, args.warmup)
        log("wide", extra["head_width_256"])
        extra["streaming_read"] = run_read(gpu, args.steps, args.warmup)
        log("read", extra["streaming_read"])
        extra["reference_timing_shapes"] = run_gemma(gpu, args.steps, args.warmup)
        log("gemma", extra["reference_timing_shapes"])
    r = run_stack(gpu, args.steps, args.warmup, args.batch, args.ctx, kv_gap_gib=args.kv_gap_gib)
    log("c5", r)
    gpu.close()
    cpu = None if args.no_cpu else cpu_baseline(0, args.ctx)
    if not args.no_cpu and not args.no_extras:
        host = cpu_extras()
        extra["c1_fp32"]["cpu_baseline"] = host["c1"]
        extra["c2_single_decode"]["cpu_baseline"] = host["c2"]
        extra["c3_ragged_batch"]["cpu_baseline"] = host["c3"]
        for name in ("full", "window128"):
            extra["c4_prefill"][name]["cpu_baseline"] = host["c4"][name]
    extra["c5_stack"] = {k: r[k] for k in ("tokens_per_s", "gpu_s_per_step", "step_bytes", "kernel_launches_per_step", "outputs_checked")}
    line = {
        "metric": METRIC, "value": r["value_gbs"], "unit": "GB/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": r["wall_s_per_step"] * 1e3, "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": r["workload"], "heads": H, "kv_heads": G, "head_dim": D,
                   "hbm_frac_of_value": r["value_gbs"] / HBM_PEAK_GBS},
        "roofline": {"bound": "hbm", "kernel": r["kernel"], "achieved": r["kernel_gbs"], "peak": HBM_PEAK_GBS,
                     "unit": "GB/s", "frac": r["kernel_gbs"] / HBM_PEAK_GBS,
                     "traffic": stack_traffic_per_launch(args.ctx, args.batch),
                     "bytes_per_launch": r["kernel_bytes_per_launch"], "s_per_launch": r["kernel_s_per_launch"]},
        "cpu_baseline": cpu,
        "extra": extra,
    }
    print(json.dumps(line))


if __name__ == "__main__":
    main()
