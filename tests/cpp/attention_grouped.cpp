// The reference's operator tests (metal-compute/tests/attention_grouped.rs), written against
// include/lng_compute.hpp: the same shapes, the same generator, the same float64 definition and
// the same bounds (2e-5 row by row, 1e-4 tiled and with sinks), plus what the C++ layer adds to
// them: ownership of buffers, residents, errors as exceptions, a bf16 pass.
//
// Prints one line per test and exits with the number of failures.
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <limits>
#include <mutex>
#include <string>
#include <thread>
#include <vector>

#include "lng_compute.hpp"
#include "test_support.hpp"

using lng::Batch;
using lng::Buffer;
using lng::Completed;
using lng::Gpu;
using lng::GroupedShape;
using lng::Slice;

namespace {

using support::expect;
using support::upload;
using support::values;

size_t up32(size_t n) { return (n + 31) / 32 * 32; }

// attention_grouped.rs:44-64: the newest rows in a ring of `slots`; rows the row-by-row kernel must never read are NaN
std::vector<float> ring(const std::vector<float> &all, const GroupedShape &s, bool tiled) {
    const size_t row = s.kv_heads * s.dim, end = s.start + s.t;
    const size_t rows = !tiled ? std::min(s.slots, end) : (s.slots < end ? s.slots : up32(end));
    std::vector<float> out(rows * row, tiled ? 0.0f : std::numeric_limits<float>::quiet_NaN());
    for (size_t p = end > s.slots ? end - s.slots : 0; p < end; ++p) {
        const size_t slot = p % s.slots;
        std::copy(all.begin() + p * row, all.begin() + (p + 1) * row, out.begin() + slot * row);
    }
    return out;
}

// attention_grouped.rs:66-105: the definition, in float64
std::vector<float> reference(const std::vector<float> &q, const std::vector<float> &k, const std::vector<float> &v,
                             const GroupedShape &s, const std::vector<float> *sinks) {
    const size_t row = s.kv_heads * s.dim, group = s.heads / s.kv_heads;
    std::vector<float> out(s.t * s.heads * s.dim, 0.0f);
#pragma omp parallel for collapse(2) schedule(dynamic)
    for (size_t i = 0; i < s.t; ++i) {
        for (size_t h = 0; h < s.heads; ++h) {
            const size_t last = s.start + i;
            const size_t first = s.window == lng::FULL || last + 1 < s.window ? 0 : last + 1 - s.window;
            const size_t g = h / group;
            const float *qt = &q[(i * s.heads + h) * s.dim];
            std::vector<double> scores(last + 1 - first);
            const double sink = sinks ? (double)(*sinks)[h] : -INFINITY;
            double m = sink;
            for (size_t p = first; p <= last; ++p) {
                double dot = 0.0;
                for (size_t d = 0; d < s.dim; ++d) dot += (double)qt[d] * (double)k[p * row + g * s.dim + d];
                scores[p - first] = dot * (double)s.scale;
                m = std::max(m, scores[p - first]);
            }
            double z = std::exp(sink - m);
            for (double x : scores) z += std::exp(x - m);
            for (size_t d = 0; d < s.dim; ++d) {
                double acc = 0.0;
                for (size_t p = first; p <= last; ++p) acc += std::exp(scores[p - first] - m) / z * (double)v[p * row + g * s.dim + d];
                out[(i * s.heads + h) * s.dim + d] = (float)acc;
            }
        }
    }
    return out;
}

// attention_grouped.rs:107-160
float max_error(const Gpu &gpu, const GroupedShape &s, float sharp, bool tiled, const std::vector<float> *sinks) {
    const size_t end = s.start + s.t, rows = tiled ? up32(s.t) : s.t;
    std::vector<float> q = values(1, s.t * s.heads * s.dim);
    for (float &x : q) x *= sharp;
    const std::vector<float> want_q = q;
    q.resize(rows * s.heads * s.dim, 0.0f);
    const std::vector<float> k = values(2, end * s.kv_heads * s.dim), v = values(3, end * s.kv_heads * s.dim);
    const std::vector<float> kr = ring(k, s, tiled), vr = ring(v, s, tiled);
    const size_t out_len = rows * s.heads * s.dim * 4;
    std::vector<Buffer> buffers;
    buffers.push_back(upload(gpu, q));
    buffers.push_back(upload(gpu, kr));
    buffers.push_back(upload(gpu, vr));
    buffers.push_back(gpu.buffer(out_len));
    buffers.push_back(upload(gpu, sinks ? *sinks : std::vector<float>{0.0f}));
    Batch batch = gpu.batch(std::move(buffers), lng::Dispatch::Serial);
    const Slice qs(0, 0, q.size() * 4), ks(1, 0, kr.size() * 4), vs(2, 0, vr.size() * 4), os(3, 0, out_len);
    const Slice sink_slice(4, 0, s.heads * 4);
    if (tiled && !sinks) batch.attention_grouped_tiled(qs, ks, vs, os, s);
    if (!tiled && !sinks) batch.attention_grouped(qs, ks, vs, os, s);
    if (tiled && sinks) batch.attention_grouped_tiled_with_sinks({qs, ks, vs}, sink_slice, os, s);
    if (!tiled && sinks) batch.attention_grouped_with_sinks({qs, ks, vs}, sink_slice, os, s);
    Completed done = std::move(batch).run();
    done.gpu_time();
    const std::vector<float> want = reference(want_q, k, v, s, sinks);
    const std::vector<float> got = done.buffers[3].to_f32();
    float worst = 0.0f;
    for (size_t i = 0; i < want.size(); ++i) {
        const float e = std::fabs(got[i] - want[i]);
        worst = std::isnan(e) ? INFINITY : std::max(worst, e);
    }
    return worst;
}

GroupedShape shape(size_t t, size_t start, size_t heads, size_t kv_heads, size_t dim, size_t window, size_t slots) {
    GroupedShape s;
    s.t = t, s.start = start, s.heads = heads, s.kv_heads = kv_heads, s.dim = dim, s.window = window, s.slots = slots;
    s.scale = 1.0f;
    return s;
}

std::string text(const GroupedShape &s) {
    char b[200];
    std::snprintf(b, sizeof b, "t %zu start %zu heads %zu/%zu dim %zu window %zu slots %zu", s.t, s.start, s.heads, s.kv_heads,
                  s.dim, s.window == lng::FULL ? (size_t)0 : s.window, s.slots);
    return b;
}

struct Case {
    GroupedShape s;
    float sharp;
};

// attention_grouped.rs:181-205
void matches_the_float64_definition(const Gpu &gpu) {
    const size_t full = lng::FULL;
    const Case cases[] = {
        {shape(1, 0, 32, 4, 512, full, 1), 1.0f},          {shape(1, 700, 32, 4, 512, full, 701), 0.05f},
        {shape(37, 300, 32, 4, 512, full, 337), 0.05f},    {shape(1, 3000, 32, 16, 256, 1024, 1536), 0.08f},
        {shape(200, 1400, 32, 16, 256, 1024, 1536), 0.08f}, {shape(512, 0, 32, 16, 256, 1024, 1536), 0.08f},
        {shape(5, 97, 4, 1, 64, 7, 12), 3.0f},             {shape(3, 2, 8, 2, 32, 16, 40), 1.0f},
    };
    for (const Case &c : cases) {
        const float error = max_error(gpu, c.s, c.sharp, false, nullptr);
        expect(error < 2e-5f, text(c.s) + ": max error " + std::to_string(error));
    }
    std::printf("done matches_the_float64_definition\n");
}

// attention_grouped.rs:207-229
void tiled_matches_the_float64_definition(const Gpu &gpu) {
    const size_t full = lng::FULL;
    const Case cases[] = {
        {shape(512, 0, 32, 4, 512, full, 512), 0.05f},       {shape(77, 700, 32, 4, 512, full, 4096), 0.05f},
        {shape(33, 5, 32, 4, 512, full, 40), 0.05f},         {shape(512, 2600, 32, 16, 256, 1024, 1536), 0.08f},
        {shape(200, 1400, 32, 16, 256, 1024, 1536), 0.08f},  {shape(512, 0, 32, 16, 256, 1024, 1536), 0.08f},
        {shape(40, 97, 4, 1, 64, 7, 64), 3.0f},
    };
    for (const Case &c : cases) {
        const float error = max_error(gpu, c.s, c.sharp, true, nullptr);
        expect(error < 1e-4f, "tiled " + text(c.s) + ": max error " + std::to_string(error));
    }
    std::printf("done tiled_matches_the_float64_definition\n");
}

// attention_grouped.rs:231-258
void sinks_take_probability_without_value_on_gpt_oss_shapes(const Gpu &gpu) {
    const size_t full = lng::FULL;
    std::vector<float> sinks = values(4, 64);
    for (float &x : sinks) x *= 3.0f;
    auto gpt_oss = [](size_t t, size_t start, size_t window, size_t slots) {
        GroupedShape s = shape(t, start, 64, 8, 64, window, slots);
        s.scale = 0.125f;
        return s;
    };
    const std::pair<GroupedShape, bool> cases[] = {
        {gpt_oss(1, 0, 128, 640), false},     {gpt_oss(1, 3000, 128, 640), false}, {gpt_oss(9, 700, 128, 640), false},
        {gpt_oss(512, 0, 128, 640), true},    {gpt_oss(512, 2600, 128, 640), true}, {gpt_oss(1, 4095, full, 4096), false},
        {gpt_oss(300, 200, full, 4096), true},
    };
    for (const auto &c : cases) {
        const float error = max_error(gpu, c.first, 1.0f, c.second, &sinks);
        expect(error < 1e-4f, std::string(c.second ? "tiled " : "") + "sinks " + text(c.first) + ": max error " + std::to_string(error));
    }
    std::printf("done sinks_take_probability_without_value_on_gpt_oss_shapes\n");
}

// attention_grouped.rs:260-281
void rejects_shapes_it_cannot_run(const Gpu &gpu) {
    const GroupedShape cases[] = {
        shape(1, 0, 6, 4, 64, 8, 8),    // heads not a multiple of KV heads
        shape(1, 0, 4, 4, 48, 8, 8),    // dim not a multiple of 32
        shape(1, 0, 4, 4, 544, 8, 8),   // dim over 512
        shape(4, 100, 4, 4, 64, 8, 10), // ring smaller than window + t
        shape(0, 0, 4, 4, 64, 8, 8),    // nothing to do
    };
    for (const GroupedShape &s : cases) {
        std::vector<Buffer> buffers;
        for (int i = 0; i < 4; ++i) buffers.push_back(gpu.buffer(1 << 20));
        Batch batch = gpu.batch(std::move(buffers));
        auto slice = [](size_t b) { return Slice(b, 0, 1 << 20); };
        bool refused = false;
        try {
            batch.attention_grouped(slice(0), slice(1), slice(2), slice(3), s);
        } catch (const lng::Error &e) {
            refused = e.kind == lng::Error::Kind::Dispatch && std::string(e.what()).rfind("invalid dispatch: ", 0) == 0;
        }
        expect(refused, "not refused: " + text(s));
        expect(batch.dispatches() == 0, "a refused dispatch was recorded");
    }
    std::printf("done rejects_shapes_it_cannot_run\n");
}

// What the C++ layer adds: buffers move into the batch and come back in Completed; a callback runs once, off
// the calling thread; a resident is attached after the batch's own buffers and stays alive until the batch is
// done; a batch dropped uncommitted runs nothing; a bf16 pass agrees with the f32 one to bf16 accuracy.
void ownership_residents_and_bf16(const Gpu &gpu) {
    GroupedShape s = shape(64, 0, 64, 8, 64, lng::FULL, 64);
    s.scale = 0.125f;
    const size_t n_q = s.t * s.heads * s.dim, n_kv = s.t * s.kv_heads * s.dim;
    const std::vector<float> q = values(11, n_q), k = values(12, n_kv), v = values(13, n_kv);
    std::vector<float> sink_values = values(14, 64);
    auto sinks = gpu.resident(sink_values.data(), sink_values.size() * 4);
    std::vector<float> f32_out;
    {
        std::vector<Buffer> buffers;
        buffers.push_back(upload(gpu, q));
        buffers.push_back(upload(gpu, k));
        buffers.push_back(upload(gpu, v));
        buffers.push_back(gpu.buffer(n_q * 4));
        Batch batch = gpu.batch(std::move(buffers));
        const Slice sink_slice = batch.attach(sinks);
        expect(sink_slice == Slice(4, 0, 256), "the resident is buffer 4 of the batch");
        expect(batch.attach(sinks) == sink_slice, "a resident attached twice is named once");
        batch.attention_grouped_tiled_with_sinks({Slice(0, 0, n_q * 4), Slice(1, 0, n_kv * 4), Slice(2, 0, n_kv * 4)}, sink_slice,
                                                 Slice(3, 0, n_q * 4), s);
        expect(batch.dispatches() == 1, "one dispatch recorded");
        std::mutex mu;
        std::promise<Completed> slot;
        auto filled = slot.get_future();
        const auto caller = std::this_thread::get_id();
        bool other_thread = false;
        std::move(batch).commit([&](Completed done) {
            other_thread = std::this_thread::get_id() != caller;
            slot.set_value(std::move(done));
        });
        sinks.reset(); // the batch keeps the resident alive
        Completed done = filled.get();
        expect(other_thread, "on_done runs on the completion thread");
        expect(done.buffers.size() == 4 && !done.error && done.gpu_time().count() > 0.0, "the buffers come back with a GPU time");
        f32_out = done.buffers[3].to_f32();
        const std::vector<float> want = reference(q, k, v, s, &sink_values);
        float worst = 0.0f;
        for (size_t i = 0; i < want.size(); ++i) worst = std::max(worst, std::fabs(f32_out[i] - want[i]));
        expect(worst < 1e-4f, "resident sinks: max error " + std::to_string(worst));
        // the same buffers go into the next batch; dropped uncommitted, it leaves them untouched and frees them
        Batch again = gpu.batch(std::move(done.buffers));
        again.attention_grouped_tiled(Slice(0, 0, n_q * 4), Slice(1, 0, n_kv * 4), Slice(2, 0, n_kv * 4), Slice(3, 0, n_q * 4), s);
    }
    // bf16 in and out: narrow on the host (truncation is enough for a comparison at bf16 accuracy)
    auto narrow = [](const std::vector<float> &x) {
        std::vector<uint16_t> y(x.size());
        for (size_t i = 0; i < x.size(); ++i) {
            uint32_t bits;
            std::memcpy(&bits, &x[i], 4);
            y[i] = (uint16_t)((bits + 0x7fffu + ((bits >> 16) & 1u)) >> 16);
        }
        return y;
    };
    const auto qb = narrow(q), kb = narrow(k), vb = narrow(v);
    std::vector<Buffer> buffers;
    for (const auto *src : {&qb, &kb, &vb}) {
        Buffer b = gpu.buffer(src->size() * 2);
        b.write(0, src->data(), src->size() * 2);
        buffers.push_back(std::move(b));
    }
    buffers.push_back(gpu.buffer(n_q * 2));
    buffers.push_back(upload(gpu, sink_values));
    Batch batch = gpu.batch(std::move(buffers));
    batch.attention_grouped_tiled_with_sinks({Slice(0, 0, n_q * 2), Slice(1, 0, n_kv * 2), Slice(2, 0, n_kv * 2)}, Slice(4, 0, 256),
                                             Slice(3, 0, n_q * 2), s, lng::DType::BF16);
    Completed done = std::move(batch).run();
    std::vector<uint16_t> out(n_q);
    done.buffers[3].read(0, out.data(), n_q * 2);
    float worst = 0.0f;
    for (size_t i = 0; i < n_q; ++i) {
        const uint32_t bits = (uint32_t)out[i] << 16;
        float x;
        std::memcpy(&x, &bits, 4);
        worst = std::max(worst, std::fabs(x - f32_out[i]));
    }
    expect(worst < 2e-2f, "bf16 against f32: max difference " + std::to_string(worst));
    std::printf("done ownership_residents_and_bf16\n");
}

} // namespace

int main() {
    try {
        Gpu gpu;
        std::printf("device %s\n", gpu.name().c_str());
        matches_the_float64_definition(gpu);
        tiled_matches_the_float64_definition(gpu);
        sinks_take_probability_without_value_on_gpt_oss_shapes(gpu);
        rejects_shapes_it_cannot_run(gpu);
        ownership_residents_and_bf16(gpu);
    } catch (const lng::Error &e) {
        std::printf("FAILED with %s\n", e.what());
        return 100;
    }
    std::printf("%d failures\n", support::failures);
    return support::failures;
}
