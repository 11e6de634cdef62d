// The reference's tests of the operators either side of attention, written against
// include/lng_compute.hpp: the Q8_0 products and their refusals, the bias add and the rotations
// (metal-compute/tests/q8_0_and_gpt_oss_glue.rs), the strided RMS norm and row copy
// (metal-compute/tests/glue.rs:240-297). Same shapes, generator, float64 definitions and bounds.
// The parts of those tests that exercise operators outside the attention block (the gated
// activation, the sigmoid gate, expert routing) are not restated.
//
// Prints one line per test and exits with the number of failures.
#include <cmath>
#include <cstdio>
#include <string>
#include <vector>

#include "lng_compute.hpp"
#include "test_support.hpp"

using lng::Batch;
using lng::Buffer;
using lng::Completed;
using lng::Gpu;
using lng::Slice;
using support::expect;
using support::f32s;
using support::upload;
using support::upload_bytes;
using support::values;

namespace {

struct Q8Matrix {
    std::vector<uint8_t> codes, scale_bytes;
    std::vector<double> elements;
};

// q8_0_and_gpt_oss_glue.rs:52-82: codes, exact binary16 scales of either sign, and every element's value
Q8Matrix q8_matrix(size_t rows, size_t cols, uint64_t seed) {
    static const std::pair<uint16_t, double> SCALES[6] = {{0x3800, 0.5},  {0x2000, 0.0078125},    {0xB600, -0.375},
                                                          {0x3C00, 1.0},  {0x1400, 0.0009765625}, {0x4100, 2.5}};
    Q8Matrix m;
    for (float v : values(seed, rows * cols)) m.codes.push_back((uint8_t)(int8_t)(v * 127.9f));
    std::vector<double> scale_values;
    const std::vector<float> picks = values(seed + 1, rows * cols / 32);
    for (size_t i = 0; i < picks.size(); ++i) {
        const auto &s = SCALES[((size_t)((picks[i] + 1.0f) * 3.0f) + i) % 6];
        m.scale_bytes.push_back((uint8_t)(s.first & 0xff));
        m.scale_bytes.push_back((uint8_t)(s.first >> 8));
        scale_values.push_back(s.second);
    }
    for (size_t i = 0; i < m.codes.size(); ++i) m.elements.push_back((double)(int8_t)m.codes[i] * scale_values[i / 32]);
    return m;
}

enum class Kind { Gemv, Gemm, Tiled };

// q8_0_and_gpt_oss_glue.rs:91-137: largest error of y = W x over n positions, relative to the largest |y|
double q8_error(const Gpu &gpu, size_t rows, size_t cols, size_t n, Kind kind) {
    const Q8Matrix m = q8_matrix(rows, cols, 7 + rows);
    const std::vector<float> x = values(11, n * cols);
    std::vector<Buffer> buffers;
    buffers.push_back(upload_bytes(gpu, m.codes));
    buffers.push_back(upload_bytes(gpu, m.scale_bytes));
    buffers.push_back(upload(gpu, x));
    buffers.push_back(gpu.buffer(n * rows * 4));
    Batch batch = gpu.batch(std::move(buffers), lng::Dispatch::Serial);
    const std::pair<Slice, Slice> matrix{Slice(0, 0, m.codes.size()), Slice(1, 0, m.scale_bytes.size())};
    const Slice xs(2, 0, x.size() * 4), ys(3, 0, n * rows * 4);
    if (kind == Kind::Gemv) batch.gemv_q8_0(matrix, xs, ys, rows, cols);
    if (kind == Kind::Gemm) batch.gemm_q8_0(matrix, xs, ys, {rows, cols}, n, {cols, rows});
    if (kind == Kind::Tiled) batch.gemm_q8_0_tiled(matrix, xs, ys, {rows, cols}, n, {cols, rows});
    Completed done = std::move(batch).run();
    done.gpu_time();
    const std::vector<float> got = done.buffers[3].to_f32();
    double worst = 0.0, largest = 0.0;
#pragma omp parallel for collapse(2) reduction(max : worst, largest)
    for (size_t p = 0; p < n; ++p) {
        for (size_t r = 0; r < rows; ++r) {
            double want = 0.0;
            for (size_t c = 0; c < cols; ++c) want += m.elements[r * cols + c] * (double)x[p * cols + c];
            largest = std::max(largest, std::fabs(want));
            worst = std::max(worst, std::fabs((double)got[p * rows + r] - want));
        }
    }
    return worst / largest;
}

// q8_0_and_gpt_oss_glue.rs:139-160
void q8_0_products_match_the_float64_definition(const Gpu &gpu) {
    struct {
        size_t rows, cols, n;
        Kind kind;
    } cases[] = {{4096, 2880, 1, Kind::Gemv}, {512, 2880, 1, Kind::Gemv}, {37, 96, 1, Kind::Gemv}, {512, 2880, 5, Kind::Gemm},
                 {37, 96, 13, Kind::Gemm},    {2880, 4096, 32, Kind::Tiled}, {512, 2880, 96, Kind::Tiled}};
    for (const auto &c : cases) {
        const double error = q8_error(gpu, c.rows, c.cols, c.n, c.kind);
        char text[160];
        std::snprintf(text, sizeof text, "%zu x %zu, %zu positions, kind %d: relative error %.3e", c.rows, c.cols, c.n, (int)c.kind, error);
        expect(error < 1e-5, text);
    }
    std::printf("done q8_0_products_match_the_float64_definition\n");
}

template <class F> bool refused(F &&record) {
    try {
        record();
    } catch (const lng::Error &e) {
        return e.kind == lng::Error::Kind::Dispatch;
    }
    return false;
}

// q8_0_and_gpt_oss_glue.rs:162-188
void q8_0_rejects_partial_blocks(const Gpu &gpu) {
    std::vector<Buffer> buffers;
    for (int i = 0; i < 4; ++i) buffers.push_back(gpu.buffer(1 << 16));
    Batch batch = gpu.batch(std::move(buffers));
    auto s = [](size_t b, size_t len) { return Slice(b, 0, len); };
    expect(refused([&] { batch.gemv_q8_0({s(0, 4 * 40), s(1, 4 * 40 / 16)}, s(2, 160), s(3, 16), 4, 40); }), "40 columns are not whole blocks");
    expect(refused([&] { batch.gemm_q8_0_tiled({s(0, 64 * 32), s(1, 128)}, s(2, 31 * 128), s(3, 31 * 256), {64, 32}, 31, {32, 64}); }),
           "31 positions are not a whole tile");
    expect(batch.dispatches() == 0, "refused products were recorded");
    std::printf("done q8_0_rejects_partial_blocks\n");
}

void check_rotation(const std::vector<float> &rotated, const std::vector<float> &x, const std::vector<float> &table, size_t rows,
                    size_t heads, size_t dim, size_t rotary, const char *what) {
    const size_t half = rotary / 2;
    bool close = true, untouched = true;
    for (size_t r = 0; r < rows; ++r) {
        for (size_t hd = 0; hd < heads; ++hd) {
            const size_t base = (r * heads + hd) * dim;
            for (size_t i = 0; i < half; ++i) {
                const double c = table[(r * half + i) * 2], s = table[(r * half + i) * 2 + 1];
                const double a = x[base + i], b = x[base + i + half];
                close = close && std::fabs((double)rotated[base + i] - (a * c - b * s)) < 1e-6 &&
                        std::fabs((double)rotated[base + i + half] - (b * c + a * s)) < 1e-6;
            }
            for (size_t i = rotary; i < dim; ++i) untouched = untouched && rotated[base + i] == x[base + i];
        }
    }
    expect(close, std::string(what) + ": rotated pairs within 1e-6");
    expect(untouched, std::string(what) + ": dimensions past the rotary part are untouched");
}

// q8_0_and_gpt_oss_glue.rs:190-258 (the rotation and the bias add)
void glue_adds_and_rotates_as_defined(const Gpu &gpu) {
    const size_t rows = 3, heads = 4, dim = 64, width = 96;
    const std::vector<float> x = values(1, rows * heads * dim), bias = values(2, width), h = values(3, rows * width);
    std::vector<float> table;
    for (size_t i = 0; i < rows * dim / 2; ++i) {
        const double angle = (double)i * 0.37;
        table.push_back((float)std::cos(angle) * 1.3f);
        table.push_back((float)std::sin(angle) * 1.3f);
    }
    std::vector<Buffer> buffers;
    buffers.push_back(upload(gpu, x));
    buffers.push_back(upload(gpu, table));
    buffers.push_back(upload(gpu, h));
    buffers.push_back(upload(gpu, bias));
    Batch batch = gpu.batch(std::move(buffers));
    batch.rotate_halves(f32s(0, x.size()), f32s(1, table.size()), rows, {heads, dim});
    batch.add_rows(f32s(2, h.size()), {f32s(3, width), 0}, rows, width);
    Completed done = std::move(batch).run();
    done.gpu_time();
    check_rotation(done.buffers[0].to_f32(), x, table, rows, heads, dim, dim, "rotate_halves");
    const std::vector<float> added = done.buffers[2].to_f32();
    bool exact = true;
    for (size_t i = 0; i < rows * width; ++i) exact = exact && added[i] == h[i] + bias[i % width];
    expect(exact, "add_rows of one bias row is the f32 sum");
    std::printf("done glue_adds_and_rotates_as_defined\n");
}

// q8_0_and_gpt_oss_glue.rs:486-540 (the rotation)
void partial_rotation_is_as_defined(const Gpu &gpu) {
    const size_t rows = 5, heads = 3, dim = 256, rotary = 64;
    const std::vector<float> x = values(11, rows * heads * dim);
    std::vector<float> table;
    for (size_t i = 0; i < rows * rotary / 2; ++i) {
        const double angle = (double)i * 0.53;
        table.push_back((float)std::cos(angle));
        table.push_back((float)std::sin(angle));
    }
    std::vector<Buffer> buffers;
    buffers.push_back(upload(gpu, x));
    buffers.push_back(upload(gpu, table));
    Batch batch = gpu.batch(std::move(buffers));
    for (size_t bad : {(size_t)63, (size_t)258}) { // odd and too-wide rotary parts are refused
        expect(refused([&] { batch.rotate_halves_partial(f32s(0, x.size()), f32s(1, table.size()), rows, {heads, dim, bad}); }),
               "a rotary part of " + std::to_string(bad) + " is refused");
    }
    batch.rotate_halves_partial(f32s(0, x.size()), f32s(1, table.size()), rows, {heads, dim, rotary});
    Completed done = std::move(batch).run();
    done.gpu_time();
    check_rotation(done.buffers[0].to_f32(), x, table, rows, heads, dim, rotary, "rotate_halves_partial");
    std::printf("done partial_rotation_is_as_defined\n");
}

// glue.rs:240-297
void strided_rmsnorm_and_row_copy_touch_only_their_columns(const Gpu &gpu) {
    const size_t rows = 9, d = 12, stride = 20; // rows of 20 floats: normalize the first 12, copy columns 12..20 elsewhere
    const std::vector<float> v = values(20, rows * stride), w = values(21, d);
    std::vector<Buffer> buffers;
    buffers.push_back(upload(gpu, v));
    buffers.push_back(upload(gpu, w));
    buffers.push_back(gpu.buffer(rows * 16 * 4));
    Batch batch = gpu.batch(std::move(buffers), lng::Dispatch::Concurrent);
    // copy first (reads columns the norm does not write), then normalize
    batch.copy_rows({Slice(0, d * 4, ((rows - 1) * stride + 8) * 4), stride}, {Slice(2, 0, ((rows - 1) * 16 + 8) * 4), 16}, rows, 8);
    batch.rmsnorm_rows({Slice(0, 0, ((rows - 1) * stride + d) * 4), f32s(1, d)}, rows, {d, stride}, 1e-5f);
    Completed done = std::move(batch).run();
    done.gpu_time();
    std::vector<float> want = v;
    for (size_t r = 0; r < rows; ++r) {
        double ss = 0.0;
        for (size_t i = 0; i < d; ++i) ss += (double)v[r * stride + i] * (double)v[r * stride + i];
        const float inv = (float)(1.0 / std::sqrt(ss / (double)d + 1e-5));
        for (size_t i = 0; i < d; ++i) want[r * stride + i] = w[i] * v[r * stride + i] * inv;
    }
    const std::vector<float> got = done.buffers[0].to_f32();
    float worst = 0.0f;
    for (size_t i = 0; i < v.size(); ++i) worst = std::max(worst, std::fabs(got[i] - want[i]));
    expect(worst <= 2e-6f, "rmsnorm_rows: max error " + std::to_string(worst));
    const std::vector<float> copied = done.buffers[2].to_f32();
    bool same = true;
    for (size_t r = 0; r < rows; ++r) {
        for (size_t i = 0; i < 8; ++i) same = same && copied[r * 16 + i] == v[r * stride + d + i];
    }
    expect(same, "copy_rows moved columns 12..20 of every row");
    std::printf("done strided_rmsnorm_and_row_copy_touch_only_their_columns\n");
}

} // namespace

int main() {
    try {
        Gpu gpu;
        q8_0_products_match_the_float64_definition(gpu);
        q8_0_rejects_partial_blocks(gpu);
        glue_adds_and_rotates_as_defined(gpu);
        partial_rotation_is_as_defined(gpu);
        strided_rmsnorm_and_row_copy_touch_only_their_columns(gpu);
    } catch (const lng::Error &e) {
        std::printf("FAILED with %s\n", e.what());
        return 100;
    }
    std::printf("%d failures\n", support::failures);
    return support::failures;
}
