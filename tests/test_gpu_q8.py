"""GPU parity of the Q8_0 products (Batch::gemv_q8_0 / gemm_q8_0 / gemm_q8_0_tiled) through the C
ABI: the reference's own test (metal-compute/tests/q8_0_and_gpt_oss_glue.rs:155-177: its matrices,
shapes and bound, largest error below 1e-5 of the largest |y| against float64), strides, refusals,
and the tiny-model golden with the device doing projections, pre-attention step and attention."""
import os

import numpy as np
import pytest

from loadngo_amd import compute as C
from oracle import oracle as orc
from oracle import tiny_model as tm
from tests.gpu_common import gpu  # noqa: F401
from tests.helpers import REF_Q8_CASES, q8_test_matrix, xorshift_values
from tests.test_gpu_tiny_model import FIXTURE, TOLERANCE, DeviceSession

pytestmark = pytest.mark.gpu


def q8_run(gpu, codes, bits, x, rows, cols, kind, y_stride=None):
    n, x_stride = x.shape
    y_stride = rows if y_stride is None else y_stride
    y_len = ((n - 1) * y_stride + rows) * 4
    bufs = [gpu.upload(codes), gpu.upload(bits), gpu.upload(x), gpu.buffer(y_len)]
    bufs[3].fill(0xFF)
    batch = gpu.batch(bufs)
    m = (C.Slice(0, 0, codes.nbytes), C.Slice(1, 0, bits.nbytes))
    xs, ys = C.Slice(2, 0, ((n - 1) * x_stride + cols) * 4), C.Slice(3, 0, y_len)
    try:
        if kind == "gemv":
            batch.gemv_q8_0(m, xs, ys, rows, cols)
        elif kind == "gemm":
            batch.gemm_q8_0(m, xs, ys, rows, cols, n, (x_stride, y_stride))
        else:
            batch.gemm_q8_0_tiled(m, xs, ys, rows, cols, n, (x_stride, y_stride))
        assert batch.dispatches() == 1
        done = batch.run()
        assert not isinstance(done.gpu_time, Exception), done.gpu_time
        raw = bufs[3].read(np.float32)
    finally:
        batch.drop()
        for b in bufs:
            b.free()
    out = np.full((n, y_stride), np.nan, np.float32)
    out.reshape(-1)[:raw.size] = raw
    return out


@pytest.mark.parametrize("rows,cols,n,kind", REF_Q8_CASES + [(4096, 2880, 16, "gemm"), (2880, 4096, 31, "gemm"),
                                                             (5120, 2880, 512, "tiled"), (64, 32, 32, "tiled")])
def test_products_match_the_float64_definition(gpu, rows, cols, n, kind):
    codes, bits, elements = q8_test_matrix(rows, cols, 7 + rows)
    x = xorshift_values(11, n * cols).reshape(n, cols)
    want = x.astype(np.float64) @ elements.T
    got = q8_run(gpu, codes, bits, x, rows, cols, kind)
    assert not np.isnan(got).any()
    error = np.abs(got - want).max() / np.abs(want).max()
    assert error < 1e-5, f"{rows} x {cols}, {n} positions, {kind}: relative error {error:e}"  # glue.rs:171
    # and against the f32 CPU form, whose own distance from float64 is of the same size
    cpu = orc.q8_mul(codes, bits, x, rows, cols)
    assert np.abs(got - cpu).max() / np.abs(want).max() < 2e-5


@pytest.mark.parametrize("rows,cols,n,kind", [(320, 96, 1120, "tiled"), (2112, 64, 1056, "tiled"), (576, 160, 4224, "tiled"),
                                              (256, 32, 1024, "tiled"), (300, 96, 1100, "gemm"), (2100, 64, 1030, "gemm")])
def test_product_with_eight_position_tiles_or_more(gpu, rows, cols, n, kind):
    """From eight tiles of 128 positions on, workgroup ids are mapped to tiles per XCD in blocks of 8 row
    tiles x 4 position tiles and the grid is rounded up to whole blocks: every tile must be computed exactly
    once (ragged tile counts in both directions, ids without a tile), nothing outside y written."""
    codes, bits, elements = q8_test_matrix(rows, cols, 40 + rows)
    x = xorshift_values(13, n * cols).reshape(n, cols)
    want = x.astype(np.float64) @ elements.T
    got = q8_run(gpu, codes, bits, x, rows, cols, kind, y_stride=rows + 4)
    assert not np.isnan(got[:, :rows]).any()
    assert np.abs(got[:, :rows] - want).max() / np.abs(want).max() < 1e-5
    assert np.isnan(got[:-1, rows:]).all()           # 0xFF fill: gaps of y untouched


@pytest.mark.parametrize("rows,cols,n", [(4096, 2880, 1), (512, 2880, 5), (37, 96, 13), (2880, 4096, 32), (2880, 4096, 31),
                                         (320, 96, 1120), (2100, 64, 1030), (64, 32, 32), (5120, 2880, 512)])
def test_product_of_bf16_positions(gpu, rows, cols, n):
    """gemm_q8_0_bf16 (no counterpart in the reference): positions given in bf16, as a bf16 attention leaves them
    for the output projection. Against the float64 product of the same bf16 values, the reference's bound for
    its f32 kernels (glue.rs:171); strided x and y, gaps of y untouched."""
    from tests.helpers import from_bf16_bits, to_bf16_bits
    codes, bits, elements = q8_test_matrix(rows, cols, 60 + rows)
    x_stride, y_stride = cols + 8, rows + 4
    xb = np.full((n, x_stride), 0x7FC0, np.uint16)            # NaN between the rows of x: never read
    xb[:, :cols] = to_bf16_bits(xorshift_values(19, n * cols).reshape(n, cols))
    want = from_bf16_bits(xb[:, :cols]).astype(np.float64) @ elements.T
    y_len = ((n - 1) * y_stride + rows) * 4
    bufs = [gpu.upload(codes), gpu.upload(bits), gpu.upload(xb), gpu.buffer(y_len)]
    bufs[3].fill(0xFF)
    batch = gpu.batch(bufs)
    try:
        batch.gemm_q8_0_bf16((C.Slice(0, 0, codes.nbytes), C.Slice(1, 0, bits.nbytes)),
                             C.Slice(2, 0, ((n - 1) * x_stride + cols) * 2), C.Slice(3, 0, y_len), rows, cols, n,
                             (x_stride, y_stride))
        done = batch.run()
        assert not isinstance(done.gpu_time, Exception), done.gpu_time
        raw = bufs[3].read(np.float32)
    finally:
        batch.drop()
        for b in bufs:
            b.free()
    got = np.full((n, y_stride), np.nan, np.float32)
    got.reshape(-1)[:raw.size] = raw
    assert not np.isnan(got[:, :rows]).any()
    assert np.abs(got[:, :rows] - want).max() / np.abs(want).max() < 1e-5
    assert np.isnan(got[:-1, rows:]).all()


def test_strided_positions_and_untouched_gaps(gpu):
    rows, cols, n = 80, 96, 21
    codes, bits, elements = q8_test_matrix(rows, cols, 3)
    x = np.full((n, cols + 8), np.nan, np.float32)   # the gap between rows of x is never read
    x[:, :cols] = xorshift_values(5, n * cols).reshape(n, cols)
    got = q8_run(gpu, codes, bits, x, rows, cols, "gemm", y_stride=rows + 12)
    want = x[:, :cols].astype(np.float64) @ elements.T
    assert np.abs(got[:, :rows] - want).max() / np.abs(want).max() < 1e-5
    assert np.isnan(got[:-1, rows:]).all()           # 0xFF fill: gaps of y untouched


@pytest.mark.parametrize("n", [1, 9])
def test_scales_at_an_offset_of_two_bytes(gpu, n):
    """The reference asks 2-byte alignment of the scales (apple.rs:1799-1811); the few-position kernel copies
    a workgroup's scales to LDS a dword at a time only when they start on a 4-byte boundary."""
    rows, cols = 96, 160
    codes, bits, elements = q8_test_matrix(rows, cols, 21)
    x = xorshift_values(17, n * cols).reshape(n, cols)
    padded = np.concatenate([np.array([0x7E00], np.uint16), bits])   # a NaN in front of the scales
    bufs = [gpu.upload(codes), gpu.upload(padded), gpu.upload(x), gpu.buffer(n * rows * 4)]
    batch = gpu.batch(bufs)
    m = (C.Slice(0, 0, codes.nbytes), C.Slice(1, 2, bits.nbytes))
    try:
        if n == 1:
            batch.gemv_q8_0(m, C.Slice(2, 0, x.nbytes), C.Slice(3, 0, rows * 4), rows, cols)
        else:
            batch.gemm_q8_0(m, C.Slice(2, 0, x.nbytes), C.Slice(3, 0, n * rows * 4), rows, cols, n, (cols, rows))
        done = batch.run()
        assert not isinstance(done.gpu_time, Exception), done.gpu_time
        got = bufs[3].read(np.float32).reshape(n, rows)
    finally:
        batch.drop()
        for b in bufs:
            b.free()
    want = x.astype(np.float64) @ elements.T
    assert np.abs(got - want).max() / np.abs(want).max() < 1e-5


def test_refusals_of_the_reference(gpu):
    """q8_0_and_gpt_oss_glue.rs:180-210 and the checks of apple.rs:889-894, 995-999, 1799-1806, 1868-1872."""
    bufs = [gpu.buffer(1 << 16) for _ in range(4)]
    res = gpu.resident(np.zeros(1 << 14, np.float32))
    batch = gpu.batch(bufs)
    s = lambda b, n: C.Slice(b, 0, n)
    with pytest.raises(C.Dispatch):   # rows of 40 are not whole blocks
        batch.gemv_q8_0((s(0, 160), s(1, 10)), s(2, 160), s(3, 16), 4, 40)
    with pytest.raises(C.Dispatch):   # 31 positions in the tiled product
        batch.gemm_q8_0_tiled((s(0, 2048), s(1, 128)), s(2, 31 * 128), s(3, 31 * 256), 64, 32, 31, (32, 64))
    with pytest.raises(C.Dispatch):   # 48 rows in the tiled product
        batch.gemm_q8_0_tiled((s(0, 48 * 32), s(1, 96)), s(2, 32 * 128), s(3, 32 * 48 * 4), 48, 32, 32, (32, 48))
    good = ((s(0, 64 * 64), s(1, 64 * 2 * 2)), s(2, 5 * 64 * 4), s(3, 5 * 64 * 4), 64, 64, 5, (64, 64))
    bad = [
        (good[0], good[1], good[2], 0, 64, 5, (64, 64)),                        # no rows
        (good[0], good[1], good[2], 64, 64, 0, (64, 64)),                       # no positions
        (good[0], s(2, 5 * 64 * 4), good[2], 64, 64, 5, (60, 64)),              # x rows closer than cols
        (good[0], s(2, (4 * 66 + 64) * 4), good[2], 64, 64, 5, (66, 64)),       # x stride not a multiple of 4
        (good[0], good[1], good[2], 64, 64, 5, (64, 63)),                       # y rows closer than rows
        ((C.Slice(0, 8, 64 * 64), good[0][1]), good[1], good[2], 64, 64, 5, (64, 64)),   # codes off 16 bytes
        ((good[0][0], s(1, 100)), good[1], good[2], 64, 64, 5, (64, 64)),       # scales of the wrong length
        (good[0], C.Slice(2, 4, 5 * 64 * 4), good[2], 64, 64, 5, (64, 64)),     # x off 16 bytes
        (good[0], good[1], s(0, 5 * 64 * 4), 64, 64, 5, (64, 64)),              # y over the codes
    ]
    for case in bad:
        with pytest.raises(C.Dispatch):
            batch.gemm_q8_0(*case)
    with pytest.raises(C.Dispatch):   # output in resident memory
        att = batch.attach(res)
        batch.gemm_q8_0(good[0], good[1], C.Slice(att.buffer, 0, 5 * 64 * 4), 64, 64, 5, (64, 64))
    with pytest.raises(C.Dispatch):   # bf16 positions: rows of x must stay on 16-byte boundaries (stride % 8)
        batch.gemm_q8_0_bf16(good[0], s(2, (4 * 68 + 64) * 2), good[2], 64, 64, 5, (68, 64))
    with pytest.raises(C.Dispatch):   # bf16 positions: x of the f32 length
        batch.gemm_q8_0_bf16(good[0], good[1], good[2], 64, 64, 5, (64, 64))
    assert batch.dispatches() == 0
    batch.gemm_q8_0(*good)
    assert batch.dispatches() == 1
    batch.gemm_q8_0_bf16(good[0], s(2, 5 * 64 * 2), good[2], 64, 64, 5, (64, 64))
    assert batch.dispatches() == 2
    batch.drop()
    for b in bufs:
        b.free()
    res.free()


def test_split_blocks_host_helper_matches_the_oracle():
    raw = np.random.default_rng(0).integers(0, 256, 34 * 50, dtype=np.uint8)
    codes, scales = C.split_q8_0_blocks(raw.tobytes())
    want_codes, want_scales = orc.q8_split_blocks(raw)
    assert np.array_equal(codes, want_codes) and np.array_equal(scales, want_scales)


@pytest.mark.parametrize("chunk", [1, 40])
def test_tiny_model_golden_with_device_projections(gpu, chunk):
    """Projections (Q8_0), pre-attention step and attention on the device; transformers' logits within 2e-3."""
    model = tm.TinyModel(os.path.join(FIXTURE, "model.gguf"))
    ids, want = tm.load_fixture(FIXTURE)
    held = {}
    for name, (raw, rows, cols) in model.q8_raw.items():
        codes, scales = C.split_q8_0_blocks(raw)
        held[name] = (gpu.resident(codes), gpu.resident(scales), rows, cols)

    def project(name, x):
        codes, scales, rows, cols = held[name]
        n = x.shape[0]
        xb, yb = gpu.upload(x), gpu.buffer(n * rows * 4)
        batch = gpu.batch([xb, yb])
        m = (batch.attach(codes), batch.attach(scales))
        if n == 1:
            batch.gemv_q8_0(m, C.Slice(0, 0, x.nbytes), C.Slice(1, 0, n * rows * 4), rows, cols)
        else:
            batch.gemm_q8_0(m, C.Slice(0, 0, x.nbytes), C.Slice(1, 0, n * rows * 4), rows, cols, n, (cols, rows))
        batch.run()
        batch.drop()
        y = yb.read(np.float32).reshape(n, rows)
        xb.free()
        yb.free()
        return y

    s = DeviceSession(gpu, model, chunk, C.F32, False)
    try:
        got = model.forward(ids, s.prepare, s.attention, chunk=chunk, project=project)
    finally:
        s.close()
        for codes, scales, _, _ in held.values():
            codes.free()
            scales.free()
    assert np.abs(got - want).max() < TOLERANCE


@pytest.mark.parametrize("n", [1, 5, 16, 17, 31, 40])
def test_several_matrices_in_one_dispatch_give_the_separate_products(gpu, n):
    """The q, k and v projections of a layer (gpu.rs:724-732 records three products) as one call: bit for bit
    the three separate gemm_q8_0 products, in one dispatch below 32 positions (three from 32 on); rows that are
    not a multiple of 16, a fourth matrix, and the refusals."""
    cols = 2880
    shapes = [(4096, 21), (512, 22), (37, 23), (528, 24)]
    mats = [q8_test_matrix(rows, cols, seed)[:2] for rows, seed in shapes]
    x = xorshift_values(31 + n, n * cols).reshape(n, cols)
    bufs = [gpu.upload(x)]
    for codes, bits in mats:
        bufs += [gpu.upload(codes), gpu.upload(bits)]
    y_lens = [n * rows * 4 for rows, _ in shapes]
    bufs += [gpu.buffer(2 * sum(y_lens))]                   # all outputs, once per way of computing them
    bufs[-1].fill(0xFF)
    batch = gpu.batch(bufs)
    xs = C.Slice(0, 0, x.nbytes)
    many, offset = [], 0
    for i, ((rows, _), (codes, bits)) in enumerate(zip(shapes, mats)):
        m = (C.Slice(1 + 2 * i, 0, codes.nbytes), C.Slice(2 + 2 * i, 0, bits.nbytes))
        many.append((m, C.Slice(9, offset, y_lens[i]), rows))
        batch.gemm_q8_0(m, xs, C.Slice(9, sum(y_lens) + offset, y_lens[i]), rows, cols, n, (cols, rows))
        offset += y_lens[i]
    before = batch.dispatches()
    batch.gemm_q8_0_many(many, xs, cols, n, cols)
    assert batch.dispatches() - before == (1 if n < 32 else 4)
    # refusals: nothing is recorded
    with pytest.raises(C.Dispatch):
        batch.gemm_q8_0_many(many + many[:1], xs, cols, n, cols)                       # five matrices
    with pytest.raises(C.Dispatch):
        batch.gemm_q8_0_many([], xs, cols, n, cols)
    with pytest.raises(C.Dispatch):
        batch.gemm_q8_0_many([many[0], (many[1][0], many[0][1], many[0][2])], xs, cols, n, cols)   # same output twice
    with pytest.raises(C.Dispatch):
        batch.gemm_q8_0_many([many[0], (many[1][0], many[1][1], 513)], xs, cols, n, cols)          # rows do not fit the slices
    with pytest.raises(C.Dispatch):
        batch.gemm_q8_0_many([(many[0][0], C.Slice(1, 0, y_lens[0]), 4096)], xs, cols, n, cols)     # output over a matrix
    assert batch.dispatches() - before == (1 if n < 32 else 4)
    batch.run()
    raw = bufs[-1].read(np.float32)
    batch.drop()
    for b in bufs:
        b.free()
    together, apart = raw[:raw.size // 2], raw[raw.size // 2:]
    assert not np.isnan(together).any() and np.array_equal(together, apart)


@pytest.mark.parametrize("n,cols", [(1, 2880), (5, 2880), (16, 2880), (31, 2880), (1, 12288), (3, 12288), (2, 32)])
def test_products_of_rms_normalised_positions(gpu, n, cols):
    """gemm_q8_0_many_normed against the reference's sequence (gpu.rs:712-732): copy the hidden rows, normalise the
    copy in place, three products. Within 1e-5 of the largest |y| (the sums of squares are added in another
    order); the hidden rows themselves are not touched; refusals."""
    eps = 1e-5
    shapes = [(4096, 41), (512, 42), (512, 43)] if cols == 2880 else [(80, 41), (64, 42), (37, 43)]
    mats = [q8_test_matrix(rows, cols, seed)[:2] for rows, seed in shapes]
    h = (xorshift_values(51 + n, n * cols) * 3).reshape(n, cols)
    w = 1 + 0.2 * xorshift_values(52, cols)
    bufs = [gpu.upload(h), gpu.buffer(h.nbytes), gpu.upload(w)]
    for codes, bits in mats:
        bufs += [gpu.upload(codes), gpu.upload(bits)]
    y_lens = [n * rows * 4 for rows, _ in shapes]
    bufs += [gpu.buffer(2 * sum(y_lens))]
    batch = gpu.batch(bufs)
    hs, xs, ws = C.Slice(0, 0, h.nbytes), C.Slice(1, 0, h.nbytes), C.Slice(2, 0, w.nbytes)
    batch.copy_rows((hs, cols), (xs, cols), n, cols)
    batch.rmsnorm_rows((xs, ws), n, (cols, cols), eps)
    many, offset = [], 0
    for i, ((rows, _), (codes, bits)) in enumerate(zip(shapes, mats)):
        m = (C.Slice(3 + 2 * i, 0, codes.nbytes), C.Slice(4 + 2 * i, 0, bits.nbytes))
        many.append((m, C.Slice(9, offset, y_lens[i]), rows))
        batch.gemm_q8_0(m, xs, C.Slice(9, sum(y_lens) + offset, y_lens[i]), rows, cols, n, (cols, rows))
        offset += y_lens[i]
    before = batch.dispatches()
    batch.gemm_q8_0_many_normed(many, hs, (ws, eps), cols, n, cols)
    assert batch.dispatches() == before + 1
    with pytest.raises(C.Dispatch):
        batch.gemm_q8_0_many_normed(many, hs, (C.Slice(2, 4, w.nbytes - 4), eps), cols, n, cols)    # weights too short
    with pytest.raises(C.Dispatch):
        batch.gemm_q8_0_many_normed([(many[0][0], C.Slice(2, 0, w.nbytes), 1)], hs, (ws, eps), cols, n, cols)
    assert batch.dispatches() == before + 1
    batch.run()
    raw = bufs[-1].read(np.float32)
    assert np.array_equal(bufs[0].read(np.float32).reshape(n, cols), h)
    batch.drop()
    for b in bufs:
        b.free()
    together, apart = raw[:raw.size // 2], raw[raw.size // 2:]
    assert not np.isnan(together).any()
    assert np.abs(together - apart).max() <= 1e-5 * np.abs(apart).max()


def test_the_normalised_product_is_for_decoding(gpu):
    cols = 64
    codes, bits, _ = q8_test_matrix(64, cols, 3)
    bufs = [gpu.buffer(32 * cols * 4), gpu.upload(np.ones(cols, np.float32)), gpu.upload(codes), gpu.upload(bits),
            gpu.buffer(32 * 64 * 4)]
    batch = gpu.batch(bufs)
    m = [((C.Slice(2, 0, codes.nbytes), C.Slice(3, 0, bits.nbytes)), C.Slice(4, 0, 32 * 64 * 4), 64)]
    with pytest.raises(C.Dispatch, match="fewer than 32"):
        batch.gemm_q8_0_many_normed(m, C.Slice(0, 0, 32 * cols * 4), (C.Slice(1, 0, cols * 4), 1e-5), cols, 32, cols)
    with pytest.raises(C.Dispatch, match="fewer than 32"):
        batch.gemm_q8_0_residual(m[0][0], C.Slice(0, 0, 32 * cols * 4), None, C.Slice(4, 0, 32 * 64 * 4), 64, cols, 32, (cols, 64))
    assert batch.dispatches() == 0
    batch.drop()
    for b in bufs:
        b.free()


@pytest.mark.parametrize("n,bf16", [(1, False), (7, False), (31, False), (1, True), (16, True)])
def test_output_projection_with_bias_and_residual_folded_in(gpu, n, bf16):
    """gemm_q8_0_residual against the reference's three dispatches (gpu.rs:807-827: the product, add_rows of the
    bias, add_rows into the hidden state): the same bits, for f32 and bf16 positions, hidden rows wider than the
    product, with and without a bias."""
    from tests.helpers import to_bf16_bits
    rows, cols, h_stride = 2880, 4096, 2912
    codes, bits, _ = q8_test_matrix(rows, cols, 61)
    x = xorshift_values(62 + n, n * cols).reshape(n, cols)
    xin = to_bf16_bits(x) if bf16 else x
    h = xorshift_values(63, n * h_stride).reshape(n, h_stride)
    bias = xorshift_values(64, rows)
    for with_bias in (True, False):
        bufs = [gpu.upload(codes), gpu.upload(bits), gpu.upload(xin), gpu.upload(h), gpu.upload(h), gpu.upload(bias),
                gpu.buffer(n * rows * 4)]
        batch = gpu.batch(bufs)
        m = (C.Slice(0, 0, codes.nbytes), C.Slice(1, 0, bits.nbytes))
        xs = C.Slice(2, 0, xin.nbytes)
        h_len = ((n - 1) * h_stride + rows) * 4
        if bf16:
            batch.gemm_q8_0_bf16(m, xs, C.Slice(6, 0, n * rows * 4), rows, cols, n, (cols, rows))
        else:
            batch.gemm_q8_0(m, xs, C.Slice(6, 0, n * rows * 4), rows, cols, n, (cols, rows))
        if with_bias:
            batch.add_rows(C.Slice(6, 0, n * rows * 4), (C.Slice(5, 0, rows * 4), 0), n, rows)
        for p in range(n):  # add_rows writes dense rows: one call per row of the wider hidden state
            batch.add_rows(C.Slice(3, p * h_stride * 4, rows * 4), (C.Slice(6, p * rows * 4, rows * 4), rows), 1, rows)
        before = batch.dispatches()
        batch.gemm_q8_0_residual(m, xs, C.Slice(5, 0, rows * 4) if with_bias else None, C.Slice(4, 0, h_len), rows, cols, n,
                                 (cols, h_stride), C.BF16 if bf16 else C.F32)
        assert batch.dispatches() == before + 1
        batch.run()
        apart, together = bufs[3].read(np.float32), bufs[4].read(np.float32)
        batch.drop()
        for b in bufs:
            b.free()
        assert not np.isnan(together).any() and np.array_equal(together, apart)
        assert not np.array_equal(together.reshape(n, h_stride)[:, :rows], h[:, :rows])
        assert np.array_equal(together.reshape(n, h_stride)[:, rows:], h[:, rows:])
