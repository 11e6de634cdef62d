// The entry points that have no counterpart in the reference, through include/lng_compute.hpp, each
// against the sequence of reference operators it stands for:
//   * attention_decode_batched == one attention_grouped_with_sinks (t = 1) per sequence (gpt-oss/src/gpu.rs:794-805);
//   * prepare_attention == add_rows x 3, rotate_halves x 2 and copy_rows into the ring (gpu.rs:733-759), bit for bit in f32;
//   * gemm_q8_0_bf16 == gemm_q8_0 on positions that are exact in bf16; gemm_q8_0_many == one gemm_q8_0 per matrix;
//   * checksum == the XOR of the words on the host; debug_set / debug_get.
//
// Prints one line per test and exits with the number of failures.
#include <cmath>
#include <cstdio>
#include <cstring>
#include <string>
#include <vector>

#include "lng_compute.hpp"
#include "test_support.hpp"

using lng::Batch;
using lng::Buffer;
using lng::Completed;
using lng::Gpu;
using lng::GroupedShape;
using lng::Slice;
using support::expect;
using support::f32s;
using support::upload;
using support::upload_bytes;
using support::values;

namespace {

void batched_decode_is_one_plain_call_per_sequence(const Gpu &gpu) {
    const size_t heads = 64, kv_heads = 8, dim = 64, n_seq = 5;
    const size_t lengths[n_seq] = {1, 130, 700, 4097, 2500};       // positions cached, the query is the last one
    const size_t windows[n_seq] = {lng::FULL, 128, lng::FULL, lng::FULL, 128};
    const size_t q_row = heads * dim, kv_row = kv_heads * dim;
    size_t total = 0, at[n_seq];
    for (size_t i = 0; i < n_seq; ++i) {
        at[i] = total;
        total += lengths[i];
    }
    const std::vector<float> q = values(31, n_seq * q_row), k = values(32, total * kv_row), v = values(33, total * kv_row);
    std::vector<float> sinks = values(34, heads);
    for (float &x : sinks) x *= 3.0f;

    std::vector<Buffer> buffers;
    buffers.push_back(upload(gpu, q));
    buffers.push_back(upload(gpu, k));
    buffers.push_back(upload(gpu, v));
    buffers.push_back(gpu.buffer(n_seq * q_row * 4));
    buffers.push_back(upload(gpu, sinks));
    buffers.push_back(gpu.buffer(n_seq * q_row * 4)); // for the plain calls
    Batch batch = gpu.batch(std::move(buffers));
    std::vector<lng::DecodeItem> items;
    for (size_t i = 0; i < n_seq; ++i) {
        lng::DecodeItem it{};
        it.q_offset = it.out_offset = i * q_row * 4;
        it.k_offset = it.v_offset = at[i] * kv_row * 4;
        it.sinks_offset = 0;
        it.start = lengths[i] - 1;
        it.window = windows[i] == lng::FULL ? LNG_WINDOW_FULL : windows[i];
        it.slots = lengths[i];
        items.push_back(it);
    }
    batch.attention_decode_batched(0, 1, 2, 3, 4, items, heads, kv_heads, dim, 0.125f);
    for (size_t i = 0; i < n_seq; ++i) {
        GroupedShape s;
        s.t = 1, s.start = lengths[i] - 1, s.heads = heads, s.kv_heads = kv_heads, s.dim = dim, s.window = windows[i];
        s.slots = lengths[i], s.scale = 0.125f;
        batch.attention_grouped_with_sinks({Slice(0, i * q_row * 4, q_row * 4), Slice(1, at[i] * kv_row * 4, lengths[i] * kv_row * 4),
                                            Slice(2, at[i] * kv_row * 4, lengths[i] * kv_row * 4)},
                                           Slice(4, 0, heads * 4), Slice(5, i * q_row * 4, q_row * 4), s);
    }
    expect(batch.dispatches() == 1 + n_seq, "one dispatch for the batch, one per plain call");
    Completed done = std::move(batch).run();
    done.gpu_time();
    const std::vector<float> together = done.buffers[3].to_f32(), one_by_one = done.buffers[5].to_f32();
    float worst = 0.0f;
    for (size_t i = 0; i < together.size(); ++i) worst = std::max(worst, std::fabs(together[i] - one_by_one[i]));
    expect(worst <= 1e-5f, "batched decode against plain calls: max difference " + std::to_string(worst));
    std::printf("done batched_decode_is_one_plain_call_per_sequence\n");
}

void prepare_attention_is_the_reference_sequence_of_dispatches(const Gpu &gpu) {
    // one prompt chunk of n rows starting at `start`, into rings of `slots` rows (it wraps)
    const size_t heads = 8, kv_heads = 2, dim = 64, n = 40, start = 100, slots = 64;
    const size_t qw = heads * dim, kw = kv_heads * dim, half = dim / 2;
    const std::vector<float> q = values(41, n * qw), k = values(42, n * kw), v = values(43, n * kw);
    const std::vector<float> qb = values(44, qw), kb = values(45, kw), vb = values(46, kw);
    std::vector<float> angles;
    for (size_t r = 0; r < n; ++r) {
        for (size_t i = 0; i < half; ++i) {
            const double angle = (double)(start + r) * std::pow(10000.0, -(double)i / (double)half);
            angles.push_back((float)std::cos(angle));
            angles.push_back((float)std::sin(angle));
        }
    }
    const std::vector<float> table = angles;
    std::vector<Buffer> buffers;
    for (const auto *x : {&q, &k, &v, &table, &qb, &kb, &vb}) buffers.push_back(upload(gpu, *x)); // 0..6
    buffers.push_back(gpu.buffer(n * qw * 4));     // 7: prepared queries
    buffers.push_back(gpu.buffer(slots * kw * 4)); // 8: k ring
    buffers.push_back(gpu.buffer(slots * kw * 4)); // 9: v ring
    buffers.push_back(upload(gpu, q));             // 10..12: the same inputs for the reference's sequence (it works in place)
    buffers.push_back(upload(gpu, k));
    buffers.push_back(upload(gpu, v));
    buffers.push_back(gpu.buffer(slots * kw * 4)); // 13, 14: its rings
    buffers.push_back(gpu.buffer(slots * kw * 4));
    for (size_t b : {8u, 9u, 13u, 14u}) {
        std::vector<float> zeros(slots * kw, 0.0f);
        buffers[b].copy_from_f32(zeros);
    }
    Batch batch = gpu.batch(std::move(buffers));
    const Slice sqb = f32s(4, qw), skb = f32s(5, kw), svb = f32s(6, kw);
    lng_prepare_buffers pb{};
    pb.q = 0, pb.k = 1, pb.v = 2, pb.table = 3, pb.q_out = 7, pb.k_cache = 8, pb.v_cache = 9;
    const lng_slice cq = sqb.c(), ck = skb.c(), cv = svb.c();
    pb.q_bias = &cq, pb.k_bias = &ck, pb.v_bias = &cv;
    lng::PrepareItem item{};
    item.n = n, item.start = start, item.slots = slots;
    batch.prepare_attention(pb, {item}, heads, kv_heads, dim, dim);
    // gpu.rs:733-759: biases, rotations, then the new rows into the ring in one or two runs
    batch.add_rows(f32s(10, n * qw), {sqb, 0}, n, qw);
    batch.add_rows(f32s(11, n * kw), {skb, 0}, n, kw);
    batch.add_rows(f32s(12, n * kw), {svb, 0}, n, kw);
    batch.rotate_halves(f32s(10, n * qw), f32s(3, table.size()), n, {heads, dim});
    batch.rotate_halves(f32s(11, n * kw), f32s(3, table.size()), n, {kv_heads, dim});
    const size_t first_row = start % slots, run = std::min(n, slots - first_row);
    for (size_t which = 0; which < 2; ++which) {
        const size_t src = 11 + which, dst = 13 + which;
        batch.copy_rows({Slice(src, 0, run * kw * 4), kw}, {Slice(dst, first_row * kw * 4, run * kw * 4), kw}, run, kw);
        if (run < n) batch.copy_rows({Slice(src, run * kw * 4, (n - run) * kw * 4), kw}, {Slice(dst, 0, (n - run) * kw * 4), kw}, n - run, kw);
    }
    Completed done = std::move(batch).run();
    done.gpu_time();
    auto same = [&](size_t a, size_t b) {
        const std::vector<float> x = done.buffers[a].to_f32(), y = done.buffers[b].to_f32();
        return x.size() == y.size() && std::memcmp(x.data(), y.data(), x.size() * 4) == 0;
    };
    expect(same(7, 10), "prepared queries are bit for bit those of add_rows + rotate_halves");
    expect(same(8, 13), "the k ring is bit for bit the one copy_rows fills");
    expect(same(9, 14), "the v ring is bit for bit the one copy_rows fills");
    std::printf("done prepare_attention_is_the_reference_sequence_of_dispatches\n");
}

void q8_product_of_bf16_positions_is_the_f32_product(const Gpu &gpu) {
    const size_t rows = 320, cols = 2880;
    std::vector<uint8_t> codes;
    for (float x : values(51, rows * cols)) codes.push_back((uint8_t)(int8_t)(x * 127.9f));
    std::vector<uint8_t> scales;
    for (size_t i = 0; i < rows * cols / 32; ++i) {
        const uint16_t bits = (uint16_t)(0x2000 + 0x0400 * (i % 7)); // binary16 powers of two, 2^-7 .. 2^-1
        scales.push_back((uint8_t)(bits & 0xff));
        scales.push_back((uint8_t)(bits >> 8));
    }
    for (size_t n : {(size_t)1, (size_t)13, (size_t)160}) {
        std::vector<float> x = values(52 + n, n * cols);
        std::vector<uint16_t> xb(x.size());
        for (size_t i = 0; i < x.size(); ++i) { // keep what bf16 holds exactly
            uint32_t bits;
            std::memcpy(&bits, &x[i], 4);
            bits &= 0xffff0000u;
            std::memcpy(&x[i], &bits, 4);
            xb[i] = (uint16_t)(bits >> 16);
        }
        std::vector<Buffer> buffers;
        buffers.push_back(upload_bytes(gpu, codes));
        buffers.push_back(upload_bytes(gpu, scales));
        buffers.push_back(upload(gpu, x));
        Buffer narrow = gpu.buffer(xb.size() * 2);
        narrow.write(0, xb.data(), xb.size() * 2);
        buffers.push_back(std::move(narrow));
        buffers.push_back(gpu.buffer(n * rows * 4));
        buffers.push_back(gpu.buffer(n * rows * 4));
        buffers.push_back(gpu.buffer(n * rows * 4)); // 6: the two halves
        Batch batch = gpu.batch(std::move(buffers));
        const std::pair<Slice, Slice> matrix{Slice(0, 0, codes.size()), Slice(1, 0, scales.size())};
        batch.gemm_q8_0(matrix, f32s(2, x.size()), f32s(4, n * rows), {rows, cols}, n, {cols, rows});
        batch.gemm_q8_0_bf16(matrix, Slice(3, 0, xb.size() * 2), f32s(5, n * rows), {rows, cols}, n, {cols, rows});
        // the same matrix as two matrices of 160 rows each through the several-matrices form: the same bits
        const size_t h = rows / 2;
        batch.gemm_q8_0_many({{{Slice(0, 0, h * cols), Slice(1, 0, h * cols / 16)}, Slice(6, 0, n * h * 4), h},
                              {{Slice(0, h * cols, h * cols), Slice(1, h * cols / 16, h * cols / 16)}, Slice(6, n * h * 4, n * h * 4), h}},
                             f32s(2, x.size()), cols, n, cols);
        Completed done = std::move(batch).run();
        done.gpu_time();
        const std::vector<float> wide = done.buffers[4].to_f32(), narrow_y = done.buffers[5].to_f32(), halves = done.buffers[6].to_f32();
        bool same_bits = true;
        for (size_t p = 0; p < n; ++p) {
            for (size_t r = 0; r < rows; ++r) {
                const float split = r < h ? halves[p * h + r] : halves[n * h + p * h + (r - h)];
                same_bits = same_bits && std::memcmp(&split, &wide[p * rows + r], 4) == 0;
            }
        }
        expect(same_bits, std::to_string(n) + " positions: two half matrices in one call give the bits of the whole product");
        double worst = 0.0, largest = 0.0;
        for (size_t i = 0; i < wide.size(); ++i) {
            largest = std::max(largest, (double)std::fabs(wide[i]));
            worst = std::max(worst, (double)std::fabs(wide[i] - narrow_y[i]));
        }
        expect(worst <= 1e-5 * largest, std::to_string(n) + " positions: bf16 against f32 positions, relative " + std::to_string(worst / largest));
    }
    std::printf("done q8_product_of_bf16_positions_is_the_f32_product\n");
}

void decoding_products_fold_their_neighbours_in(const Gpu &gpu) {
    const size_t rows = 96, cols = 2880, n = 3;
    std::vector<uint8_t> codes;
    for (float x : values(71, rows * cols)) codes.push_back((uint8_t)(int8_t)(x * 127.9f));
    std::vector<uint8_t> scales;
    for (size_t i = 0; i < rows * cols / 32; ++i) {
        scales.push_back(0x00);
        scales.push_back((uint8_t)(0x20 + 4 * (i % 5))); // binary16 2^-7, 2^-6, ...
    }
    const std::vector<float> h = values(72, n * cols), w = values(73, cols), bias = values(74, rows), hidden = values(75, n * rows);
    std::vector<Buffer> buffers;
    buffers.push_back(upload_bytes(gpu, codes));   // 0
    buffers.push_back(upload_bytes(gpu, scales));  // 1
    buffers.push_back(upload(gpu, h));             // 2: positions
    buffers.push_back(upload(gpu, h));             // 3: their copy, normalised in place
    buffers.push_back(upload(gpu, w));             // 4
    buffers.push_back(gpu.buffer(n * rows * 4));   // 5: product of the normalised copy
    buffers.push_back(gpu.buffer(n * rows * 4));   // 6: the same in one dispatch
    buffers.push_back(upload(gpu, bias));          // 7
    buffers.push_back(upload(gpu, hidden));        // 8: hidden rows, three dispatches
    buffers.push_back(upload(gpu, hidden));        // 9: hidden rows, one dispatch
    Batch batch = gpu.batch(std::move(buffers));
    const std::pair<Slice, Slice> matrix{Slice(0, 0, codes.size()), Slice(1, 0, scales.size())};
    batch.rmsnorm_rows({f32s(3, n * cols), f32s(4, cols)}, n, {cols, cols}, 1e-5f);
    batch.gemm_q8_0(matrix, f32s(3, n * cols), f32s(5, n * rows), {rows, cols}, n, {cols, rows});
    batch.gemm_q8_0_many_normed({{matrix, f32s(6, n * rows), rows}}, f32s(2, n * cols), {f32s(4, cols), 1e-5f}, cols, n, cols);
    // the output-projection pattern on the product in buffer 5: bias, then into the hidden rows
    batch.add_rows(f32s(5, n * rows), {f32s(7, rows), 0}, n, rows);
    batch.add_rows(f32s(8, n * rows), {f32s(5, n * rows), rows}, n, rows);
    const Slice bias_slice = f32s(7, rows);
    batch.gemm_q8_0_residual(matrix, f32s(3, n * cols), &bias_slice, f32s(9, n * rows), {rows, cols}, n, {cols, rows});
    Completed done = std::move(batch).run();
    done.gpu_time();
    const std::vector<float> apart = done.buffers[5].to_f32(), together = done.buffers[6].to_f32();
    // buffer 5 holds product + bias by now: take the bias off on the host for the comparison of the products
    double worst = 0.0, largest = 0.0;
    for (size_t p = 0; p < n; ++p) {
        for (size_t r = 0; r < rows; ++r) {
            const double product = (double)apart[p * rows + r] - (double)bias[r];
            largest = std::max(largest, std::fabs(product));
            worst = std::max(worst, std::fabs(product - (double)together[p * rows + r]));
        }
    }
    expect(worst <= 2e-5 * largest, "the normalised product in one dispatch: relative " + std::to_string(worst / largest));
    const std::vector<float> three = done.buffers[8].to_f32(), one = done.buffers[9].to_f32();
    expect(std::memcmp(three.data(), one.data(), three.size() * 4) == 0, "bias and residual folded in give the bits of the three dispatches");
    expect(done.buffers[2].to_f32() == h, "the positions of the normalised product are left alone");
    std::printf("done decoding_products_fold_their_neighbours_in\n");
}

void checksum_is_the_xor_of_the_words_and_switches_pick_kernels(const Gpu &gpu) {
    const size_t n = 3 * 65536 + 4; // floats: a whole number of 16-byte words, several workgroups and a ragged end
    const std::vector<float> data = values(41, n);
    uint32_t want[4] = {0, 0, 0, 0};
    for (size_t i = 0; i < n; ++i) {
        uint32_t bits;
        std::memcpy(&bits, &data[i], 4);
        want[i & 3] ^= bits;
    }
    std::vector<Buffer> buffers;
    buffers.push_back(upload(gpu, data));
    buffers.push_back(gpu.buffer(32));
    Batch batch = gpu.batch(std::move(buffers));
    batch.checksum(f32s(0, n), Slice(1, 0, 16));
    gpu.debug_set("LNG_CHECKSUM_WGS", "7"); // another number of workgroups, the same sum
    batch.checksum(f32s(0, n), Slice(1, 16, 16));
    gpu.debug_set("LNG_CHECKSUM_WGS", nullptr);
    Completed done = std::move(batch).run();
    done.gpu_time();
    const std::vector<float> got = done.buffers[1].to_f32();
    expect(std::memcmp(got.data(), want, 16) == 0 && std::memcmp(got.data() + 4, want, 16) == 0, "checksum: the XOR of every 16-byte word");
    bool refused = false;
    try {
        gpu.debug_set("LNG_NO_SUCH_SWITCH", "1");
    } catch (const lng::Error &) {
        refused = true;
    }
    expect(refused, "an unknown switch is refused");
    expect(gpu.debug_get("LNG_COUNT_SECOND_PASSES") == 0, "no long causal pass has been made again");
    std::printf("done checksum_is_the_xor_of_the_words_and_switches_pick_kernels\n");
}

} // namespace

int main() {
    try {
        Gpu gpu;
        batched_decode_is_one_plain_call_per_sequence(gpu);
        prepare_attention_is_the_reference_sequence_of_dispatches(gpu);
        q8_product_of_bf16_positions_is_the_f32_product(gpu);
        decoding_products_fold_their_neighbours_in(gpu);
        checksum_is_the_xor_of_the_words_and_switches_pick_kernels(gpu);
    } catch (const lng::Error &e) {
        std::printf("FAILED with %s\n", e.what());
        return 100;
    }
    std::printf("%d failures\n", support::failures);
    return support::failures;
}
