// lng_compute.hpp: the host side above the C ABI (lng_hip.h), in C++17, header only.
//
// It mirrors the slice of loadngo's metal-compute crate that the gpt-oss attention block uses,
// with the reference's names, argument order and error behaviour, so that code written against
//   metal-compute/src/apple.rs   Gpu (105), Buffer (391), Resident (465), Slice (507), Completed (536),
//                                Batch (541), GroupedShape (598), Dispatch (67)
//   metal-compute/src/lib.rs     Error (41-53)
// reads the same here. Differences that the hardware forces:
//   * buffers are device memory, not CPU-shared: Buffer::as_f32() of the reference becomes the
//     explicit copies Buffer::to_f32() / Buffer::copy_from_f32() (and read / write for bytes);
//   * Result<T, Error> becomes a thrown lng::Error; Completed::gpu_time keeps its two arms
//     (a duration, or the error of the batch);
//   * Batch::commit(proactor, on_done) posts on_done to the caller's proactor in the reference;
//     here on_done runs on the library's completion thread and the caller re-posts it where it
//     wants it (Batch::run() is the blocking form the reference's tests build from the two);
//   * every attention method takes the element type of q, k, v and out as a trailing argument
//     (f32 as in the reference by default, or bf16 in and out with f32 accumulation).
#ifndef LNG_COMPUTE_HPP
#define LNG_COMPUTE_HPP

#include <chrono>
#include <cstdint>
#include <cstring>
#include <functional>
#include <future>
#include <memory>
#include <optional>
#include <stdexcept>
#include <string>
#include <tuple>
#include <utility>
#include <vector>

#include "lng_hip.h"

namespace lng {

// GroupedShape::window for "every earlier position" (usize::MAX in the reference).
constexpr std::size_t FULL = SIZE_MAX;

// lib.rs:41-53, same variants and the same texts (with "HIP" where they say "Metal").
class Error : public std::runtime_error {
  public:
    enum class Kind { NoDevice, Compile, Alloc, Dispatch, Gpu };
    Error(Kind kind, const std::string &detail) : std::runtime_error(text(kind, detail)), kind(kind), detail(detail) {}
    Kind kind;
    std::string detail;

    static Error from_status(int status, const char *message) {
        const std::string m = message ? message : "";
        switch (status) {
        case LNG_ERR_NO_DEVICE: return Error(Kind::NoDevice, m);
        case LNG_ERR_COMPILE: return Error(Kind::Compile, m);
        case LNG_ERR_ALLOC: return Error(Kind::Alloc, m);
        case LNG_ERR_DISPATCH: return Error(Kind::Dispatch, m);
        default: return Error(Kind::Gpu, m);
        }
    }

  private:
    static std::string text(Kind kind, const std::string &detail) {
        switch (kind) {
        case Kind::NoDevice: return "no HIP device";
        case Kind::Compile: return "HIP kernel compilation failed: " + detail;
        case Kind::Alloc: return detail; // "could not allocate a N-byte buffer"
        case Kind::Dispatch: return "invalid dispatch: " + detail;
        default: return "GPU command buffer failed: " + detail;
        }
    }
};

namespace detail {
inline void check(int status) {
    if (status != LNG_OK) throw Error::from_status(status, lng_hip_last_error());
}
} // namespace detail

enum class DType : int { F32 = LNG_F32, BF16 = LNG_BF16 };

// apple.rs:67. Dispatches of a batch run in order on the device either way.
enum class Dispatch { Serial, Concurrent };

// apple.rs:507-521: bytes offset..offset+len of the batch's buffer number `buffer`: its own
// buffers first, then the residents it attached, in order.
struct Slice {
    std::size_t buffer = 0, offset = 0, len = 0;
    constexpr Slice() = default;
    constexpr Slice(std::size_t buffer, std::size_t offset, std::size_t len) : buffer(buffer), offset(offset), len(len) {}
    lng_slice c() const { return lng_slice{buffer, offset, len}; }
    bool operator==(const Slice &o) const { return buffer == o.buffer && offset == o.offset && len == o.len; }
};

// apple.rs:598-614.
struct GroupedShape {
    std::size_t t = 0, start = 0, heads = 0, kv_heads = 0, dim = 0, window = FULL, slots = 0;
    float scale = 1.0f;
    lng_grouped_shape c() const {
        return lng_grouped_shape{t, start, heads, kv_heads, dim, window == FULL ? LNG_WINDOW_FULL : (uint64_t)window, slots, scale};
    }
};

class Gpu;
class Batch;

// apple.rs:391 Buffer: memory a batch takes by value and hands back when it has finished.
class Buffer {
  public:
    Buffer() = default;
    Buffer(Buffer &&o) noexcept : h_(o.h_) { o.h_ = nullptr; }
    Buffer &operator=(Buffer &&o) noexcept {
        if (this != &o) {
            reset();
            h_ = o.h_;
            o.h_ = nullptr;
        }
        return *this;
    }
    Buffer(const Buffer &) = delete;
    Buffer &operator=(const Buffer &) = delete;
    ~Buffer() { reset(); }

    std::size_t len() const { return lng_hip_buffer_len(h_); }
    bool is_empty() const { return len() == 0; }
    void write(std::size_t offset, const void *src, std::size_t n) { detail::check(lng_hip_upload(h_, offset, src, n)); }
    void read(std::size_t offset, void *dst, std::size_t n) const { detail::check(lng_hip_download(h_, offset, dst, n)); }
    // as_f32() / as_f32_mut() of the reference, as copies
    std::vector<float> to_f32() const {
        std::vector<float> v(len() / 4);
        if (!v.empty()) read(0, v.data(), v.size() * 4);
        return v;
    }
    void copy_from_f32(const std::vector<float> &v, std::size_t first = 0) {
        if (!v.empty()) write(first * 4, v.data(), v.size() * 4);
    }
    void *device_ptr() const { return lng_hip_buffer_device_ptr(h_); }

  private:
    friend class Gpu;
    friend class Batch;
    explicit Buffer(lng_buffer *h) : h_(h) {}
    void reset() {
        if (h_) lng_hip_buffer_free(h_);
        h_ = nullptr;
    }
    lng_buffer *h_ = nullptr;
};

// apple.rs:465 Resident: immutable bytes (weights) that any number of batches may attach.
class Resident {
  public:
    Resident(const Resident &) = delete;
    Resident &operator=(const Resident &) = delete;
    ~Resident() {
        if (h_) lng_hip_buffer_free(h_);
    }
    std::size_t len() const { return lng_hip_buffer_len(h_); }
    bool is_empty() const { return len() == 0; }

  private:
    friend class Gpu;
    friend class Batch;
    explicit Resident(lng_buffer *h) : h_(h) {}
    lng_buffer *h_ = nullptr;
};

// apple.rs:536-539: what a finished batch hands back: its buffers, and how long the GPU spent on
// it or why it failed.
struct Completed {
    std::vector<Buffer> buffers;
    std::chrono::duration<double> seconds{0.0};
    std::optional<Error> error;
    // Result<Duration, Error>::unwrap()
    std::chrono::duration<double> gpu_time() const {
        if (error) throw *error;
        return seconds;
    }
};

// One decoding query of Batch::attention_decode_batched.
using DecodeItem = lng_decode_item;
// One sequence of Batch::prepare_attention.
using PrepareItem = lng_prepare_item;

// apple.rs:541 Batch: one batch being recorded. Dropped without commit it runs nothing and its
// buffers are freed with it (apple.rs:553-561).
class Batch {
  public:
    Batch(Batch &&o) noexcept : h_(o.h_), buffers_(std::move(o.buffers_)), residents_(std::move(o.residents_)) { o.h_ = nullptr; }
    Batch &operator=(Batch &&) = delete;
    Batch(const Batch &) = delete;
    Batch &operator=(const Batch &) = delete;
    ~Batch() {
        if (h_) lng_hip_batch_drop(h_); // before the buffers go: the batch owns them until then
    }

    std::size_t dispatches() const { return lng_hip_batch_dispatches(h_); }

    // apple.rs:835
    Slice attach(const std::shared_ptr<Resident> &resident) {
        lng_slice whole{};
        detail::check(lng_hip_batch_attach(h_, resident->h_, &whole));
        bool held = false;
        for (const auto &r : residents_) held = held || r == resident;
        if (!held) residents_.push_back(resident);
        return Slice(whole.buffer, whole.offset, whole.len);
    }

    // apple.rs:1199
    void attention_grouped(Slice q, Slice k, Slice v, Slice out, const GroupedShape &shape, DType dtype = DType::F32) {
        const lng_grouped_shape s = shape.c();
        detail::check(lng_hip_attention_grouped(h_, q.c(), k.c(), v.c(), out.c(), nullptr, &s, (int)dtype));
    }
    // apple.rs:1213
    void attention_grouped_with_sinks(std::tuple<Slice, Slice, Slice> qkv, Slice sinks, Slice out, const GroupedShape &shape,
                                      DType dtype = DType::F32) {
        const lng_grouped_shape s = shape.c();
        const lng_slice sk = sinks.c();
        detail::check(lng_hip_attention_grouped(h_, std::get<0>(qkv).c(), std::get<1>(qkv).c(), std::get<2>(qkv).c(), out.c(), &sk,
                                                &s, (int)dtype));
    }
    // apple.rs:1311
    void attention_grouped_tiled(Slice q, Slice k, Slice v, Slice out, const GroupedShape &shape, DType dtype = DType::F32) {
        const lng_grouped_shape s = shape.c();
        detail::check(lng_hip_attention_grouped_tiled(h_, q.c(), k.c(), v.c(), out.c(), nullptr, &s, (int)dtype));
    }
    // apple.rs:1324
    void attention_grouped_tiled_with_sinks(std::tuple<Slice, Slice, Slice> qkv, Slice sinks, Slice out,
                                            const GroupedShape &shape, DType dtype = DType::F32) {
        const lng_grouped_shape s = shape.c();
        const lng_slice sk = sinks.c();
        detail::check(lng_hip_attention_grouped_tiled(h_, std::get<0>(qkv).c(), std::get<1>(qkv).c(), std::get<2>(qkv).c(),
                                                      out.c(), &sk, &s, (int)dtype));
    }
    // apple.rs:1762 copy_rows((src, src_stride), (dst, dst_stride), rows, width); strides and width in elements.
    void copy_rows(std::pair<Slice, std::size_t> src, std::pair<Slice, std::size_t> dst, std::size_t rows, std::size_t width,
                   DType src_dtype = DType::F32, DType dst_dtype = DType::F32) {
        detail::check(lng_hip_copy_rows(h_, src.first.c(), src.second, (int)src_dtype, dst.first.c(), dst.second, (int)dst_dtype,
                                        rows, width));
    }
    // apple.rs:1733 rmsnorm_rows((v, w), rows, (d, stride), eps)
    void rmsnorm_rows(std::pair<Slice, Slice> v_w, std::size_t rows, std::pair<std::size_t, std::size_t> d_stride, float eps) {
        detail::check(lng_hip_rmsnorm_rows(h_, v_w.first.c(), v_w.second.c(), rows, d_stride.first, d_stride.second, eps));
    }
    // apple.rs:1886 add_rows(dst, (src, src_stride), rows, width)
    void add_rows(Slice dst, std::pair<Slice, std::size_t> src, std::size_t rows, std::size_t width) {
        detail::check(lng_hip_add_rows(h_, dst.c(), src.first.c(), src.second, rows, width));
    }
    // apple.rs:1916 rotate_halves(x, table, rows, (heads, dim))
    void rotate_halves(Slice x, Slice table, std::size_t rows, std::pair<std::size_t, std::size_t> heads_dim) {
        detail::check(lng_hip_rotate_halves(h_, x.c(), table.c(), rows, heads_dim.first, heads_dim.second, heads_dim.second));
    }
    // apple.rs:1929 rotate_halves_partial(x, table, rows, (heads, dim, rotary))
    void rotate_halves_partial(Slice x, Slice table, std::size_t rows, std::tuple<std::size_t, std::size_t, std::size_t> shape) {
        detail::check(lng_hip_rotate_halves(h_, x.c(), table.c(), rows, std::get<0>(shape), std::get<1>(shape), std::get<2>(shape)));
    }
    // apple.rs:1812 gemv_q8_0((codes, scales), x, y, rows, cols)
    void gemv_q8_0(std::pair<Slice, Slice> matrix, Slice x, Slice y, std::size_t rows, std::size_t cols) {
        detail::check(lng_hip_gemv_q8_0(h_, matrix.first.c(), matrix.second.c(), x.c(), y.c(), rows, cols));
    }
    // apple.rs:1833 gemm_q8_0((codes, scales), x, y, (rows, cols), n, (x_stride, y_stride))
    void gemm_q8_0(std::pair<Slice, Slice> matrix, Slice x, Slice y, std::pair<std::size_t, std::size_t> rows_cols, std::size_t n,
                   std::pair<std::size_t, std::size_t> strides) {
        detail::check(lng_hip_gemm_q8_0(h_, matrix.first.c(), matrix.second.c(), x.c(), y.c(), rows_cols.first, rows_cols.second, n,
                                        strides.first, strides.second));
    }
    // apple.rs:1857
    void gemm_q8_0_tiled(std::pair<Slice, Slice> matrix, Slice x, Slice y, std::pair<std::size_t, std::size_t> rows_cols,
                         std::size_t n, std::pair<std::size_t, std::size_t> strides) {
        detail::check(lng_hip_gemm_q8_0_tiled(h_, matrix.first.c(), matrix.second.c(), x.c(), y.c(), rows_cols.first,
                                              rows_cols.second, n, strides.first, strides.second));
    }
    // No counterpart in the reference: the same product on bf16 positions (the output of a bf16 attention).
    void gemm_q8_0_bf16(std::pair<Slice, Slice> matrix, Slice x, Slice y, std::pair<std::size_t, std::size_t> rows_cols,
                        std::size_t n, std::pair<std::size_t, std::size_t> strides) {
        detail::check(lng_hip_gemm_q8_0_bf16(h_, matrix.first.c(), matrix.second.c(), x.c(), y.c(), rows_cols.first,
                                             rows_cols.second, n, strides.first, strides.second));
    }
    // No counterpart in the reference (three gemv/gemm calls per layer, gpu.rs:724-732): up to four matrices
    // times the same positions, each y dense [n][rows]; one dispatch below 32 positions.
    struct Q8Matrix {
        std::pair<Slice, Slice> matrix; // (codes, scales)
        Slice y;
        std::size_t rows;
    };
    void gemm_q8_0_many(const std::vector<Q8Matrix> &matrices, Slice x, std::size_t cols, std::size_t n, std::size_t x_stride) {
        std::vector<lng_q8_matrix> raw;
        for (const Q8Matrix &m : matrices) raw.push_back(lng_q8_matrix{m.matrix.first.c(), m.matrix.second.c(), m.y.c(), m.rows});
        detail::check(lng_hip_gemm_q8_0_many(h_, raw.data(), raw.size(), x.c(), cols, n, x_stride));
    }
    // gemm_q8_0_many of RMS-normalised positions (x itself is left alone): copy_rows + rmsnorm_rows + the products
    // of gpu.rs:712-732 in one dispatch; fewer than 32 positions.
    void gemm_q8_0_many_normed(const std::vector<Q8Matrix> &matrices, Slice x, std::pair<Slice, float> norm, std::size_t cols,
                               std::size_t n, std::size_t x_stride) {
        std::vector<lng_q8_matrix> raw;
        for (const Q8Matrix &m : matrices) raw.push_back(lng_q8_matrix{m.matrix.first.c(), m.matrix.second.c(), m.y.c(), m.rows});
        detail::check(lng_hip_gemm_q8_0_many_normed(h_, raw.data(), raw.size(), x.c(), norm.first.c(), norm.second, cols, n, x_stride));
    }
    // h += W x + bias: the product, add_rows of the bias and add_rows into the hidden state (gpu.rs:807-827) in one
    // dispatch and with their bits; fewer than 32 positions; strides = (x_stride, h_stride).
    void gemm_q8_0_residual(std::pair<Slice, Slice> matrix, Slice x, const Slice *bias, Slice h, std::pair<std::size_t, std::size_t> rows_cols,
                            std::size_t n, std::pair<std::size_t, std::size_t> strides, DType x_dtype = DType::F32) {
        lng_slice b{};
        if (bias) b = bias->c();
        detail::check(lng_hip_gemm_q8_0_residual(h_, matrix.first.c(), matrix.second.c(), x.c(), (int)x_dtype, bias ? &b : nullptr, h.c(),
                                                 rows_cols.first, rows_cols.second, n, strides.first, strides.second));
    }
    // No counterpart in the reference: one decoding query per item, many sequences in one dispatch.
    void attention_decode_batched(std::size_t q_buffer, std::size_t k_buffer, std::size_t v_buffer, std::size_t out_buffer,
                                  std::size_t sinks_buffer, const std::vector<DecodeItem> &items, std::size_t heads,
                                  std::size_t kv_heads, std::size_t dim, float scale, DType dtype = DType::F32) {
        detail::check(lng_hip_attention_decode_batched(h_, q_buffer, k_buffer, v_buffer, out_buffer, sinks_buffer, items.data(),
                                                       items.size(), heads, kv_heads, dim, scale, (int)dtype));
    }
    // No counterpart in the reference: biases, rotation, narrowing and cache append (gpu.rs:733-759) in one dispatch.
    void prepare_attention(const lng_prepare_buffers &buffers, const std::vector<PrepareItem> &items, std::size_t heads,
                           std::size_t kv_heads, std::size_t dim, std::size_t rotary, DType out_dtype = DType::F32) {
        detail::check(lng_hip_prepare_attention(h_, &buffers, items.data(), items.size(), heads, kv_heads, dim, rotary,
                                                (int)out_dtype));
    }
    // No counterpart in the reference: the XOR of every 16-byte word of `src`, written to the 16 bytes of `dst` (a plain
    // streaming read: a yardstick for the memory system and a cheap check of what a large cache holds).
    void checksum(Slice src, Slice dst) { detail::check(lng_hip_checksum(h_, src.c(), dst.c())); }
    // apple.rs:2194
    void barrier() { detail::check(lng_hip_batch_barrier(h_)); }

    // apple.rs:2202 commit(proactor, on_done): sends the batch to the GPU; nothing blocks. When it has
    // finished, on_done runs with the batch's buffers, on the library's completion thread (the reference
    // posts it to the caller's proactor: do that inside on_done). Consumes the batch.
    template <class F> void commit(F &&on_done) && {
        auto *pending = new Pending{std::move(buffers_), std::move(residents_), std::function<void(Completed)>(std::forward<F>(on_done)), h_};
        h_ = nullptr;
        // A failed submission has already run on_done with the error, as a failed command buffer does in the reference.
        (void)lng_hip_batch_commit(pending->handle, &Batch::trampoline, pending);
    }
    // The blocking form the reference's tests build from commit and a proactor loop.
    Completed run() && {
        std::promise<Completed> slot;
        std::future<Completed> filled = slot.get_future();
        std::move(*this).commit([&slot](Completed done) { slot.set_value(std::move(done)); });
        return filled.get();
    }

  private:
    friend class Gpu;
    struct Pending {
        std::vector<Buffer> buffers;
        std::vector<std::shared_ptr<Resident>> residents; // stay referenced until the GPU is done with them
        std::function<void(Completed)> on_done;
        lng_batch *handle;
    };
    static void trampoline(const lng_completed *done, void *user) {
        std::unique_ptr<Pending> pending(static_cast<Pending *>(user));
        Completed completed;
        completed.buffers = std::move(pending->buffers);
        completed.seconds = std::chrono::duration<double>(done->gpu_seconds);
        if (done->status != LNG_OK) completed.error = Error::from_status(done->status, done->message);
        pending->residents.clear();
        lng_hip_batch_drop(pending->handle); // from inside on_done: freed when this function returns
        pending->on_done(std::move(completed));
    }
    Batch(lng_batch *h, std::vector<Buffer> buffers) : h_(h), buffers_(std::move(buffers)) {}
    lng_batch *h_ = nullptr;
    std::vector<Buffer> buffers_;
    std::vector<std::shared_ptr<Resident>> residents_;
};

// apple.rs:73 Gpu.
class Gpu {
  public:
    // apple.rs:105 Gpu::new()
    explicit Gpu(int device = 0) { detail::check(lng_hip_open(device, &h_)); }
    Gpu(const Gpu &) = delete;
    Gpu &operator=(const Gpu &) = delete;
    ~Gpu() { lng_hip_close(h_); }

    // apple.rs:235
    std::string name() const {
        char text[128] = {0};
        detail::check(lng_hip_device_name(h_, text, sizeof text));
        return text;
    }
    // apple.rs:255
    Buffer buffer(std::size_t len) const {
        lng_buffer *b = nullptr;
        detail::check(lng_hip_buffer(h_, len, &b));
        return Buffer(b);
    }
    // apple.rs:297
    std::shared_ptr<Resident> resident(const void *bytes, std::size_t len) const {
        lng_buffer *b = nullptr;
        detail::check(lng_hip_resident(h_, bytes, len, &b));
        return std::shared_ptr<Resident>(new Resident(b));
    }
    // apple.rs:302
    std::shared_ptr<Resident> resident_words(const std::vector<uint16_t> &words) const {
        return resident(words.data(), words.size() * 2);
    }
    // Development switches and counters (no counterpart in the reference, not part of the interface: see lng_hip.h).
    // `value` nullptr puts the switch's default back.
    void debug_set(const char *name, const char *value) const { detail::check(lng_hip_debug_set(h_, name, value)); }
    uint64_t debug_get(const char *name) const {
        uint64_t value = 0;
        detail::check(lng_hip_debug_get(h_, name, &value));
        return value;
    }
    // apple.rs:365 Gpu::batch(buffers, dispatch): the batch owns `buffers` until it completes or is dropped.
    Batch batch(std::vector<Buffer> buffers, Dispatch = Dispatch::Serial) const {
        std::vector<lng_buffer *> raw;
        raw.reserve(buffers.size());
        for (const Buffer &b : buffers) raw.push_back(b.h_);
        lng_batch *h = nullptr;
        detail::check(lng_hip_batch(h_, raw.data(), raw.size(), &h));
        return Batch(h, std::move(buffers));
    }

  private:
    lng_gpu *h_ = nullptr;
};

} // namespace lng

#endif // LNG_COMPUTE_HPP
