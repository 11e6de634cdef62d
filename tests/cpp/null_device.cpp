// The host library on the null device (loadngo_amd/csrc/null_device), under AddressSanitizer and
// UndefinedBehaviorSanitizer: what lng_hip.cpp decides before anything reaches a GPU.
//
//  - refusals: the reference's own rejected shapes (metal-compute/tests/attention_grouped.rs:262-279), slices of the
//    wrong length, outside their buffer or off their element size (apple.rs:860-887), outputs in resident memory or
//    over an input (apple.rs:889-906), buffers that belong to a batch in flight, and the refusals of copy_rows,
//    prepare_attention and the Q8_0 products; a refused call records nothing.
//  - the development switches (environment at open, lng_hip_debug_set afterwards) and lng_hip_checksum: refusals and
//    what is recorded.
//  - ownership: batches hand their buffers back; close with buffers alive; the last buffer freed on one thread while
//    the handle is closed on another.
//  - allocation failures while recording: reported, nothing recorded, nothing leaked.
//  - a fuzz of the decode planner: random tables of rows through lng_hip_attention_decode_batched and random
//    row-by-row calls; for every recorded dispatch the grid is the sum of the rows' live workgroups, every
//    (row, kv head, chunk) is taken by exactly one workgroup (the kernel's own search restated below), every chunk
//    has positions, the partials and arrival counters it names lie inside the scratch that was allocated, and the
//    merge that must follow does.
//
// Usage: null_device [fuzz dispatches, default 100000]. Exit status 0 = everything held.
#include <hip/hip_runtime_api.h> // the null device's

#include <algorithm>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <random>
#include <string>
#include <thread>
#include <vector>

#include "../../include/lng_hip.h"
#include "../../loadngo_amd/csrc/lng_kernel_args.h"

static int g_failures = 0;
#define CHECK(cond)                                                                      \
    do {                                                                                 \
        if (!(cond)) {                                                                   \
            fprintf(stderr, "%s:%d: CHECK failed: %s (last error: %s)\n", __FILE__, __LINE__, #cond, lng_hip_last_error()); \
            if (++g_failures > 20) exit(1);                                              \
        }                                                                                \
    } while (0)

static bool refused(int rc, const char *needle) {
    if (rc != LNG_ERR_DISPATCH) return false;
    return strstr(lng_hip_last_error(), needle) != nullptr;
}

static lng_grouped_shape shape(uint64_t t, uint64_t start, uint64_t heads, uint64_t kv_heads, uint64_t dim, uint64_t window,
                               uint64_t slots, float scale = 1.0f) {
    return lng_grouped_shape{t, start, heads, kv_heads, dim, window, slots, scale};
}

struct Fixture {
    lng_gpu *gpu = nullptr;
    std::vector<lng_buffer *> bufs;
    lng_batch *batch = nullptr;
    Fixture(size_t n, size_t bytes) {
        CHECK(lng_hip_open(0, &gpu) == LNG_OK);
        for (size_t i = 0; i < n; ++i) {
            lng_buffer *b = nullptr;
            CHECK(lng_hip_buffer(gpu, bytes, &b) == LNG_OK);
            bufs.push_back(b);
        }
        CHECK(lng_hip_batch(gpu, bufs.data(), bufs.size(), &batch) == LNG_OK);
    }
    void rebatch() {
        lng_hip_batch_drop(batch);
        CHECK(lng_hip_batch(gpu, bufs.data(), bufs.size(), &batch) == LNG_OK);
    }
    ~Fixture() {
        if (batch) lng_hip_batch_drop(batch);
        for (lng_buffer *b : bufs) CHECK(lng_hip_buffer_free(b) == LNG_OK);
        lng_hip_close(gpu);
    }
};

static void refusals() {
    const uint64_t MB = 1u << 20;
    Fixture f(5, MB);
    lng_batch *b = f.batch;
    auto whole = [&](uint64_t i) { return lng_slice{i, 0, MB}; };
    // attention_grouped.rs:262-279
    const lng_grouped_shape rejected[] = {shape(1, 0, 6, 4, 64, 8, 8), shape(1, 0, 4, 4, 48, 8, 8), shape(1, 0, 4, 4, 544, 8, 8),
                                          shape(4, 100, 4, 4, 64, 8, 10), shape(0, 0, 4, 4, 64, 8, 8)};
    for (const lng_grouped_shape &s : rejected) {
        CHECK(refused(lng_hip_attention_grouped(b, whole(0), whole(1), whole(2), whole(3), nullptr, &s, LNG_F32), "unsupported"));
        CHECK(lng_hip_check_grouped(&s, 0) == LNG_ERR_DISPATCH);
    }
    // tiled: the ring must be a multiple of 32 rows (apple.rs:1356-1385)
    {
        const lng_grouped_shape s = shape(40, 97, 4, 1, 64, 7, 50);
        CHECK(lng_hip_check_grouped(&s, 1) == LNG_ERR_DISPATCH);
        const lng_grouped_shape ok = shape(40, 97, 4, 1, 64, 7, 64);
        CHECK(lng_hip_check_grouped(&ok, 1) == LNG_OK);
    }
    // counts past u32
    {
        const lng_grouped_shape s = shape(1, 1ull << 33, 4, 4, 64, 8, 8);
        CHECK(lng_hip_check_grouped(&s, 0) == LNG_ERR_DISPATCH);
    }
    CHECK(lng_hip_batch_dispatches(b) == 0 && lng_null_launch_count() == 0);

    // a good call, then every way its slices can be wrong (apple.rs:860-906)
    const lng_grouped_shape s = shape(2, 5, 8, 2, 64, LNG_WINDOW_FULL, 16);
    const uint64_t qn = 2 * 8 * 64 * 4, kn = 7 * 2 * 64 * 4;
    const lng_slice q{0, 0, qn}, k{1, 0, kn}, v{2, 0, kn}, o{3, 0, qn}, sk{4, 0, 8 * 4};
    CHECK(lng_hip_attention_grouped(b, q, k, v, o, &sk, &s, LNG_F32) == LNG_OK);
    CHECK(lng_hip_batch_dispatches(b) == 1);
    lng_slice bad = q;
    bad.len -= 4;
    CHECK(refused(lng_hip_attention_grouped(b, bad, k, v, o, &sk, &s, LNG_F32), "the shape needs"));
    bad = k;
    bad.offset = MB - kn + 4;
    CHECK(refused(lng_hip_attention_grouped(b, q, bad, v, o, &sk, &s, LNG_F32), "outside"));
    bad = v;
    bad.offset = 2;
    CHECK(refused(lng_hip_attention_grouped(b, q, k, bad, o, &sk, &s, LNG_F32), "not a multiple"));
    bad = o;
    bad.buffer = 9;
    CHECK(refused(lng_hip_attention_grouped(b, q, k, v, bad, &sk, &s, LNG_F32), "no buffer"));
    bad = lng_slice{0, qn / 2, qn}; // output over the query
    CHECK(refused(lng_hip_attention_grouped(b, q, k, v, bad, &sk, &s, LNG_F32), "overlaps"));
    bad = sk;
    bad.len = 4;
    CHECK(refused(lng_hip_attention_grouped(b, q, k, v, o, &bad, &s, LNG_F32), "the shape needs"));
    CHECK(refused(lng_hip_attention_grouped(b, q, k, v, o, &sk, &s, 7), "unknown element type"));
    CHECK(refused(lng_hip_attention_grouped(b, q, k, v, o, &sk, nullptr, LNG_F32), "no shape"));
    CHECK(lng_hip_batch_dispatches(b) == 1);

    // resident memory is never an output (apple.rs:896-900)
    std::vector<char> bytes(qn, 1);
    lng_buffer *res = nullptr;
    CHECK(lng_hip_resident(f.gpu, bytes.data(), bytes.size(), &res) == LNG_OK);
    lng_slice rs{};
    CHECK(lng_hip_batch_attach(b, res, &rs) == LNG_OK && rs.buffer == 5 && rs.len == qn);
    CHECK(refused(lng_hip_attention_grouped(b, q, k, v, rs, &sk, &s, LNG_F32), "read-only resident"));
    CHECK(lng_hip_attention_grouped(b, rs, k, v, o, &sk, &s, LNG_F32) == LNG_OK); // ... but an input
    CHECK(refused(lng_hip_batch_attach(b, f.bufs[0], &rs), "not a resident"));
    CHECK(refused(lng_hip_upload(res, 0, bytes.data(), 4), "read-only"));
    CHECK(refused(lng_hip_buffer_free(res), "belongs to a batch"));

    // copy_rows (apple.rs:1769-1781)
    CHECK(refused(lng_hip_copy_rows(b, whole(0), 64, LNG_F32, whole(1), 64, LNG_F32, 0, 64), "unsupported copy"));
    CHECK(refused(lng_hip_copy_rows(b, whole(0), 32, LNG_F32, whole(1), 64, LNG_F32, 4, 64), "unsupported copy"));
    CHECK(refused(lng_hip_copy_rows(b, lng_slice{0, 0, 4 * 64 * 4}, 64, LNG_F32, lng_slice{0, 64, 4 * 64 * 4}, 64, LNG_F32, 4, 64), "overlaps"));
    CHECK(lng_hip_copy_rows(b, lng_slice{0, 0, (3 * 80 + 64) * 4}, 80, LNG_F32, lng_slice{1, 0, (3 * 64 + 64) * 2}, 64, LNG_BF16, 4, 64) == LNG_OK);
    // rmsnorm / add_rows / rotate_halves (apple.rs:1740-1744, 1893-1897, 1936-1940)
    CHECK(refused(lng_hip_rmsnorm_rows(b, whole(0), lng_slice{1, 0, 64 * 4}, 4, 64, 32, 1e-5f), "unsupported rows"));
    CHECK(refused(lng_hip_add_rows(b, whole(0), whole(1), 8, 4, 64), "unsupported add"));
    CHECK(refused(lng_hip_rotate_halves(b, whole(0), whole(1), 4, 8, 64, 65), "unsupported"));
    // Q8_0 products: columns in whole blocks, codes and x on 16-byte boundaries
    CHECK(lng_hip_gemv_q8_0(b, lng_slice{0, 0, 64 * 96}, lng_slice{1, 0, 64 * 3 * 2}, lng_slice{2, 0, 96 * 4}, lng_slice{3, 0, 64 * 4}, 64, 96) == LNG_OK);
    CHECK(lng_hip_gemv_q8_0(b, lng_slice{0, 0, 64 * 90}, lng_slice{1, 0, 64 * 3 * 2}, lng_slice{2, 0, 90 * 4}, lng_slice{3, 0, 64 * 4}, 64, 90) == LNG_ERR_DISPATCH);
    CHECK(lng_hip_gemv_q8_0(b, lng_slice{0, 4, 64 * 96}, lng_slice{1, 0, 64 * 3 * 2}, lng_slice{2, 0, 96 * 4}, lng_slice{3, 0, 64 * 4}, 64, 96) == LNG_ERR_DISPATCH);
    CHECK(lng_hip_gemm_q8_0_tiled(b, lng_slice{0, 0, 64 * 96}, lng_slice{1, 0, 64 * 3 * 2}, lng_slice{2, 0, 33 * 96 * 4}, lng_slice{3, 0, 33 * 64 * 4}, 64, 96, 33, 96, 64) == LNG_ERR_DISPATCH);
    // the fused pre-attention step: two new rows on one cache row, outputs over one another
    {
        lng_prepare_buffers pb{0, 1, 2, 4, 3, 3, 3, nullptr, nullptr, nullptr};
        lng_prepare_item it{};
        it.n = 4, it.start = 0, it.slots = 2;
        CHECK(refused(lng_hip_prepare_attention(b, &pb, &it, 1, 8, 2, 64, 64, LNG_BF16), "unsupported preparation"));
        it.slots = 8; // q_out, k and v caches all at offset 0 of buffer 3
        CHECK(refused(lng_hip_prepare_attention(b, &pb, &it, 1, 8, 2, 64, 64, LNG_BF16), "overlap"));
    }
    // decode items: outputs of two items over one another
    {
        lng_decode_item items[2] = {};
        for (lng_decode_item &it : items) it = lng_decode_item{0, 0, 0, 0, LNG_NO_SINKS, 3, LNG_WINDOW_FULL, 4};
        items[1].q_offset = 8 * 64 * 2;
        CHECK(refused(lng_hip_attention_decode_batched(b, 0, 1, 2, 3, 4, items, 2, 8, 2, 64, 0.125f, LNG_BF16), "overlap"));
        items[1].out_offset = 8 * 64 * 2;
        CHECK(lng_hip_attention_decode_batched(b, 0, 1, 2, 3, 4, items, 2, 8, 2, 64, 0.125f, LNG_BF16) == LNG_OK);
        items[1].start = 9; // a row the cache cannot hold
        CHECK(lng_hip_attention_decode_batched(b, 0, 1, 2, 3, 4, items, 2, 8, 2, 64, 0.125f, LNG_BF16) == LNG_ERR_DISPATCH);
    }

    // ownership: while the batch is alive its buffers are its own (apple.rs:365-389)
    char word[4] = {0};
    CHECK(refused(lng_hip_upload(f.bufs[0], 0, word, 4), "belongs to a batch"));
    CHECK(refused(lng_hip_download(f.bufs[0], 0, word, 4), "belongs to a batch"));
    CHECK(refused(lng_hip_buffer_free(f.bufs[0]), "belongs to a batch"));
    lng_batch *second = nullptr;
    CHECK(refused(lng_hip_batch(f.gpu, f.bufs.data(), 1, &second), "belongs to a batch") && second == nullptr);
    lng_buffer *twice[2] = {res, res};
    CHECK(lng_hip_batch(f.gpu, twice, 2, &second) == LNG_ERR_DISPATCH); // a resident is attached, not owned
    const size_t recorded = lng_hip_batch_dispatches(b);
    CHECK(lng_null_launch_count() == 0); // nothing runs before commit (apple.rs:553-561)
    double seconds = -1.0;
    CHECK(refused(lng_hip_batch_wait(b, &seconds), "not committed"));
    CHECK(lng_hip_batch_commit(b, nullptr, nullptr) == LNG_OK);
    CHECK(lng_null_launch_count() >= recorded);
    CHECK(refused(lng_hip_attention_grouped(b, q, k, v, o, &sk, &s, LNG_F32), "already committed"));
    CHECK(lng_hip_batch_wait(b, &seconds) == LNG_OK && seconds >= 0.0);
    CHECK(lng_hip_upload(f.bufs[0], 0, word, 4) == LNG_OK); // the buffers are the caller's again
    CHECK(lng_hip_upload(f.bufs[0], MB - 2, word, 4) == LNG_ERR_DISPATCH);
    f.rebatch();
    CHECK(lng_hip_buffer_free(res) == LNG_OK);
    lng_null_clear();
}

// The development switches (read from the environment once, at open; afterwards only lng_hip_debug_set) and the
// streaming read: refusals, and what the planner records under a switch.
static void switches_and_checksum() {
    const size_t MB = 1 << 20;
    setenv("LNG_PREFILL_SPLITS", "3", 1); // read at open ...
    Fixture f(5, MB);
    unsetenv("LNG_PREFILL_SPLITS"); // ... and never again
    lng_batch *b = f.batch;
    lng_null_clear();
    auto prefill_splits = [&]() { // a prompt pass of 64 rows over 1,024 cached positions: one query tile per kv head
        const lng_grouped_shape s = shape(64, 960, 8, 2, 64, LNG_WINDOW_FULL, 1024, 0.125f);
        const lng_slice q{0, 0, 64 * 8 * 64 * 2}, k{1, 0, 1024 * 2 * 64 * 2}, v{2, 0, 1024 * 2 * 64 * 2}, o{3, 0, 64 * 8 * 64 * 2};
        CHECK(lng_hip_attention_grouped_tiled(f.batch, q, k, v, o, nullptr, &s, LNG_BF16) == LNG_OK);
        CHECK(lng_hip_batch_commit(f.batch, nullptr, nullptr) == LNG_OK);
        CHECK(lng_hip_batch_wait(f.batch, nullptr) == LNG_OK);
        const char *name = nullptr;
        const void *args = nullptr;
        size_t args_size = 0;
        unsigned grid[3], block[3];
        CHECK(lng_null_launch_count() >= 1 && lng_null_launch(0, &name, grid, block, &args, &args_size) == 0);
        lng_k_prefill p{};
        CHECK(args_size == sizeof p);
        memcpy(&p, args, sizeof p);
        // (the kernel of a workgroup per pair of heads never splits: its grid has the pairs instead)
        const bool pairs = !strcmp(name, "lng_prefill_bf16_d64_pair");
        CHECK(grid[0] == p.q_tiles * p.kv_heads * (pairs ? (p.heads / p.kv_heads + 1) / 2 : p.splits));
        CHECK(!pairs || p.splits == 1);
        CHECK(p.splits == 1 || lng_null_launch_count() == 2);
        lng_null_clear();
        f.rebatch();
        return p.splits;
    };
    CHECK(prefill_splits() == 3); // the environment's value at open
    CHECK(lng_hip_debug_set(f.gpu, "LNG_PREFILL_SPLITS", "5") == LNG_OK);
    CHECK(prefill_splits() == 5);
    CHECK(lng_hip_debug_set(f.gpu, "LNG_PREFILL_SPLITS", nullptr) == LNG_OK);
    const uint32_t planned = prefill_splits(); // the planner's own: one workgroup per compute unit, four key tiles each at least
    CHECK(planned >= 1 && planned <= 4);
    // a prompt fed 512 rows at a time (64 heads over 8): 64 (query tile, kv head) pairs on 256 units go to the kernel of a
    // workgroup per pair of heads while a call walks few enough keys, and to split keys plus a merge beyond that
    {
        Fixture big(5, 40 * MB);
        auto chunk_call = [&](uint64_t start, const char *want_kernel, unsigned want_grid, size_t want_launches) {
            const lng_grouped_shape s = shape(512, start, 64, 8, 64, LNG_WINDOW_FULL, start + 512, 0.125f);
            const lng_slice q{0, 0, 512 * 64 * 64 * 2}, k{1, 0, (start + 512) * 8 * 64 * 2}, v{2, 0, (start + 512) * 8 * 64 * 2}, o{3, 0, 512 * 64 * 64 * 2};
            lng_null_clear();
            CHECK(lng_hip_attention_grouped_tiled(big.batch, q, k, v, o, nullptr, &s, LNG_BF16) == LNG_OK);
            CHECK(lng_hip_batch_commit(big.batch, nullptr, nullptr) == LNG_OK);
            CHECK(lng_hip_batch_wait(big.batch, nullptr) == LNG_OK);
            const char *name = nullptr;
            const void *args = nullptr;
            size_t args_size = 0;
            unsigned grid[3], block[3];
            CHECK(lng_null_launch_count() == want_launches && lng_null_launch(0, &name, grid, block, &args, &args_size) == 0);
            CHECK(!strcmp(name, want_kernel) && grid[0] == want_grid && block[0] == 512);
            big.rebatch();
        };
        const unsigned cus = 256; // the null device's
        chunk_call(3584, "lng_prefill_bf16_d64_pair", 8 * 8 * 4, 1);
        chunk_call(0, "lng_prefill_bf16_d64_pair", 8 * 8 * 4, 1);
        chunk_call(15872, "lng_prefill_bf16_d64", cus, 2);
        CHECK(lng_hip_debug_set(big.gpu, "LNG_PREFILL_PAIR", "0") == LNG_OK);
        chunk_call(3584, "lng_prefill_bf16_d64", cus, 2);
        CHECK(lng_hip_debug_set(big.gpu, "LNG_PREFILL_PAIR", "1") == LNG_OK);
        chunk_call(15872, "lng_prefill_bf16_d64_pair", 8 * 8 * 4, 1);
        CHECK(lng_hip_debug_set(big.gpu, "LNG_PREFILL_PAIR", nullptr) == LNG_OK);
        lng_null_clear();
    }
    CHECK(refused(lng_hip_debug_set(f.gpu, "LNG_NO_SUCH_SWITCH", "1"), "no development switch"));
    CHECK(refused(lng_hip_debug_set(f.gpu, nullptr, "1"), "no name"));
    CHECK(lng_hip_debug_set(nullptr, "LNG_PREFILL_SPLITS", "1") != LNG_OK);
    uint64_t n = 99;
    CHECK(lng_hip_debug_get(f.gpu, "LNG_COUNT_SECOND_PASSES", &n) == LNG_OK && n == 0);
    CHECK(refused(lng_hip_debug_get(f.gpu, "LNG_PREFILL_SPLITS", &n), "no development counter"));
    CHECK(lng_hip_debug_get(f.gpu, "LNG_COUNT_SECOND_PASSES", nullptr) != LNG_OK);

    // the streaming read: whole 16-byte words on a 16-byte boundary, 16 bytes out, not over its input
    b = f.batch;
    CHECK(refused(lng_hip_checksum(b, lng_slice{0, 0, 100}, lng_slice{1, 0, 16}), "16-byte words"));
    CHECK(refused(lng_hip_checksum(b, lng_slice{0, 0, 0}, lng_slice{1, 0, 16}), "16-byte words"));
    CHECK(refused(lng_hip_checksum(b, lng_slice{0, 8, 160}, lng_slice{1, 0, 16}), "not a multiple"));
    CHECK(refused(lng_hip_checksum(b, lng_slice{0, 0, 160}, lng_slice{1, 0, 32}), "the shape needs"));
    CHECK(refused(lng_hip_checksum(b, lng_slice{0, 0, 160}, lng_slice{1, 4, 16}), "not a multiple"));
    CHECK(refused(lng_hip_checksum(b, lng_slice{0, 0, 160}, lng_slice{0, 32, 16}), "overlaps"));
    CHECK(refused(lng_hip_checksum(b, lng_slice{0, MB - 16, 32}, lng_slice{1, 0, 16}), "outside"));
    CHECK(lng_hip_batch_dispatches(b) == 0);
    CHECK(lng_hip_checksum(b, lng_slice{0, 0, 160}, lng_slice{1, 0, 16}) == LNG_OK);       // ten words: one workgroup
    CHECK(lng_hip_checksum(b, lng_slice{0, 0, MB}, lng_slice{1, 16, 16}) == LNG_OK);        // 65,536 words: 256 workgroups
    CHECK(lng_hip_debug_set(f.gpu, "LNG_CHECKSUM_WGS", "1") == LNG_OK);
    CHECK(lng_hip_checksum(b, lng_slice{2, 0, MB}, lng_slice{1, 32, 16}) == LNG_OK);
    CHECK(lng_hip_batch_dispatches(b) == 3);
    CHECK(lng_hip_batch_commit(b, nullptr, nullptr) == LNG_OK);
    CHECK(lng_hip_batch_wait(b, nullptr) == LNG_OK);
    CHECK(lng_null_launch_count() == 6);
    for (size_t i = 0; i < 6; i += 2) {
        const char *name = nullptr, *fold = nullptr;
        const void *args = nullptr;
        size_t args_size = 0;
        unsigned grid[3], fgrid[3];
        CHECK(lng_null_launch(i, &name, grid, nullptr, &args, &args_size) == 0 && std::string(name) == "lng_checksum");
        CHECK(lng_null_launch(i + 1, &fold, fgrid, nullptr, nullptr, nullptr) == 0 && std::string(fold) == "lng_checksum_fold" && fgrid[0] == 1);
        lng_k_checksum a{};
        CHECK(args_size == sizeof a);
        memcpy(&a, args, sizeof a);
        CHECK(grid[0] == a.n_parts && a.n_parts >= 1 && a.n_parts <= (a.n16 + 255) / 256);
        CHECK(a.n16 == (i == 0 ? 10u : MB / 16));
        CHECK(lng_null_bytes_from(a.parts) >= (size_t)a.n_parts * 16); // a 16-byte word per workgroup, in the library's scratch
        CHECK(lng_null_bytes_from(a.src) >= a.n16 * 16 && lng_null_bytes_from(a.dst) >= 16);
        if (i == 0) CHECK(a.n_parts == 1);
        if (i == 4) { // one workgroup per compute unit instead of two
            lng_k_checksum two{};
            const void *args2 = nullptr;
            CHECK(lng_null_launch(2, nullptr, nullptr, nullptr, &args2, nullptr) == 0);
            memcpy(&two, args2, sizeof two);
            CHECK(two.n_parts == 256 ? a.n_parts <= 256 : a.n_parts * 2 == two.n_parts);
        }
    }
    lng_null_clear();
    f.rebatch();
}

static void on_done_count(const lng_completed *done, void *user) {
    if (done->status == LNG_OK) ++*(int *)user;
}

static void lifetimes() {
    // a committed batch with a callback, dropped from another thread than the completion thread
    {
        Fixture f(4, 1 << 16);
        const lng_grouped_shape s = shape(1, 3, 8, 2, 64, LNG_WINDOW_FULL, 8, 0.125f);
        const lng_slice q{0, 0, 8 * 64 * 2}, k{1, 0, 4 * 2 * 64 * 2}, v{2, 0, 4 * 2 * 64 * 2}, o{3, 0, 8 * 64 * 2};
        int done = 0;
        CHECK(lng_hip_attention_grouped(f.batch, q, k, v, o, nullptr, &s, LNG_BF16) == LNG_OK);
        CHECK(lng_hip_batch_commit(f.batch, on_done_count, &done) == LNG_OK);
        CHECK(lng_hip_batch_wait(f.batch, nullptr) == LNG_OK);
        CHECK(done == 1);
        f.rebatch();
    }
    // buffers outlive a closed device, whichever thread lets go last (the handle is one reference among them)
    for (int round = 0; round < 200; ++round) {
        lng_gpu *gpu = nullptr;
        CHECK(lng_hip_open(0, &gpu) == LNG_OK);
        lng_buffer *a = nullptr, *b = nullptr;
        CHECK(lng_hip_buffer(gpu, 256, &a) == LNG_OK && lng_hip_buffer(gpu, 256, &b) == LNG_OK);
        CHECK(lng_hip_buffer_free(a) == LNG_OK);
        std::thread closer([&] { lng_hip_close(gpu); });
        std::thread freer([&] { CHECK(lng_hip_buffer_free(b) == LNG_OK); });
        closer.join();
        freer.join();
    }
    CHECK(lng_null_live_allocations() == 0);
    lng_null_clear();
}

static void allocation_failures() {
    lng_gpu *gpu = nullptr;
    CHECK(lng_hip_open(0, &gpu) == LNG_OK);
    lng_buffer *buf = nullptr;
    lng_null_fail_malloc_after(1);
    CHECK(lng_hip_buffer(gpu, 1024, &buf) == LNG_ERR_ALLOC && buf == nullptr);
    CHECK(lng_hip_buffer(gpu, 0, &buf) == LNG_ERR_ALLOC); // Alloc(0), apple.rs:256-258
    // a decode that needs split-K scratch: the scratch allocation fails, the call is refused and records nothing
    const uint64_t ctx = 40000, row = 8 * 64 * 2;
    std::vector<lng_buffer *> bufs(4);
    const size_t sizes[4] = {64 * 64 * 2, ctx * row, ctx * row, 64 * 64 * 2};
    for (int i = 0; i < 4; ++i) CHECK(lng_hip_buffer(gpu, sizes[i], &bufs[i]) == LNG_OK);
    lng_batch *batch = nullptr;
    CHECK(lng_hip_batch(gpu, bufs.data(), 4, &batch) == LNG_OK);
    const lng_grouped_shape s = shape(1, ctx - 1, 64, 8, 64, LNG_WINDOW_FULL, ctx, 0.125f);
    const lng_slice q{0, 0, 64 * 64 * 2}, k{1, 0, ctx * row}, v{2, 0, ctx * row}, o{3, 0, 64 * 64 * 2};
    // the counters, the partial outputs, the (max, sum) pairs: each allocation fails once (what was allocated before
    // a failure stays with the device, so the second and third failures are the second allocation of their call)
    for (size_t nth : {1, 2, 2}) {
        lng_null_fail_malloc_after(nth);
        CHECK(lng_hip_attention_grouped(batch, q, k, v, o, nullptr, &s, LNG_BF16) == LNG_ERR_ALLOC);
        CHECK(lng_hip_batch_dispatches(batch) == 0);
        lng_null_fail_malloc_after(0);
    }
    CHECK(lng_hip_attention_grouped(batch, q, k, v, o, nullptr, &s, LNG_BF16) == LNG_OK);
    CHECK(lng_hip_batch_dispatches(batch) == 1);
    lng_hip_batch_drop(batch);
    for (lng_buffer *b : bufs) CHECK(lng_hip_buffer_free(b) == LNG_OK);
    lng_hip_close(gpu);
    CHECK(lng_null_live_allocations() == 0);
    lng_null_clear();
}

// ---- the planner fuzz -------------------------------------------------------------------------------------

static uint64_t visible_from_tile(const lng_k_row &r) { // the run a row's chunks cover: from the 32-aligned window start
    const uint64_t last = r.start;
    const uint64_t first = (r.window != LNG_WINDOW_FULL && last + 1 > r.window) ? last + 1 - r.window : 0;
    return last + 1 - (first & ~(uint64_t)31);
}

// The kernels' own search (work_of in lng_kernels.hip) on the host: the row of workgroup w in cum[0..n_rows].
static uint32_t row_of_workgroup(const uint32_t *cum, uint32_t n_rows, uint32_t w) {
    uint32_t lo = 0, n = n_rows;
    while (n > 64u) {
        const uint32_t stride = (n + 63u) / 64u;
        uint32_t cnt = 0;
        for (uint32_t lane = 0; lane < 64; ++lane) cnt += lane * stride < n && cum[lo + lane * stride] <= w;
        const uint32_t step = (cnt - 1u) * stride;
        n = n - step < stride ? n - step : stride;
        lo += step;
    }
    uint32_t cnt = 0;
    for (uint32_t lane = 0; lane < 64; ++lane) cnt += lane < n && cum[lo + lane] <= w;
    return lo + cnt - 1u;
}

struct FuzzStats {
    size_t dispatches = 0, split = 0, fused = 0, tables = 0, generic = 0, wide = 0, prefill = 0;
};

// Checks the launches recorded for ONE dispatch whose rows are `rows` (one per query row).
static void check_rows_dispatch(const std::vector<lng_k_row> &rows, uint32_t heads, uint32_t kv_heads, uint32_t dim, FuzzStats &st) {
    const size_t n_launches = lng_null_launch_count();
    CHECK(n_launches >= 1 && n_launches <= 2);
    const char *name = nullptr;
    unsigned grid[3], block[3];
    const void *args = nullptr;
    size_t args_size = 0;
    CHECK(lng_null_launch(0, &name, grid, block, &args, &args_size) == 0);
    const std::string kernel = name;
    if (kernel.rfind("lng_prefill_", 0) == 0) { // several rows over a long cache: the prompt-pass kernels
        CHECK(args_size == sizeof(lng_k_prefill));
        lng_k_prefill p;
        memcpy(&p, args, sizeof p);
        CHECK(p.splits >= 1 && p.splits <= 64 && p.t == rows.size());
        if (p.splits > 1) {
            const uint64_t slots = p.t * p.heads * p.splits;
            CHECK(lng_null_bytes_from(p.partial_o) >= slots * p.dim * 4);
            CHECK(lng_null_bytes_from(p.partial_ml) >= slots * 2 * 4);
            CHECK(n_launches == 2);
        } else {
            CHECK(n_launches == 1);
        }
        st.prefill += 1;
        return;
    }
    CHECK(args_size == sizeof(lng_k_attn));
    lng_k_attn a;
    memcpy(&a, args, sizeof a);
    CHECK(a.n_rows == rows.size() && a.heads == heads && a.kv_heads == kv_heads && a.dim == dim);
    CHECK(block[0] == 256 && grid[1] == 1 && grid[2] == 1);
    const uint32_t group = heads / kv_heads;
    if (kernel.rfind("lng_attn_generic", 0) == 0) {
        CHECK(grid[0] == rows.size() * heads && n_launches == 1);
        st.generic += 1;
        return;
    }
    if (kernel.find("_w") != std::string::npos) st.wide += 1;
    CHECK(a.chunk >= 128 && a.chunk % 128 == 0 && a.n_chunks >= 1 && a.n_chunks <= LNG_MAX_CHUNKS);
    uint64_t longest = 0, live = 0;
    for (const lng_k_row &r : rows) {
        longest = std::max(longest, visible_from_tile(r));
        live += (visible_from_tile(r) + a.chunk - 1) / a.chunk * kv_heads;
    }
    CHECK((longest + a.chunk - 1) / a.chunk == a.n_chunks); // the partials keep n_chunks slots per (row, kv head)
    const uint64_t pairs = rows.size() * (uint64_t)kv_heads;
    std::vector<uint8_t> taken(pairs * a.n_chunks, 0);
    if (a.work) {
        st.tables += 1;
        CHECK(a.n_chunks > 1 && grid[0] == live);
        CHECK(lng_null_bytes_from(a.work) >= (rows.size() + 1) * 4);
        const uint32_t *cum = a.work; // the null device's device memory is host memory: the table as the kernel reads it
        CHECK(cum[0] == 0 && cum[rows.size()] == grid[0]);
        for (size_t r = 0; r < rows.size(); ++r) {
            CHECK(cum[r + 1] - cum[r] == (visible_from_tile(rows[r]) + a.chunk - 1) / a.chunk * kv_heads);
        }
        for (uint32_t w = 0; w < grid[0]; ++w) {
            const uint32_t row = row_of_workgroup(cum, (uint32_t)rows.size(), w);
            CHECK(row < rows.size() && cum[row] <= w && w < cum[row + 1]);
            const uint32_t chunks = (cum[row + 1] - cum[row]) / kv_heads, local = w - cum[row];
            const uint64_t pair = (uint64_t)row * kv_heads + local / chunks, chunk = local % chunks;
            CHECK(pair < pairs && chunk < a.n_chunks && !taken[pair * a.n_chunks + chunk]);
            taken[pair * a.n_chunks + chunk] = 1;
        }
    } else {
        CHECK(grid[0] == pairs * a.n_chunks);
        for (uint32_t w = 0; w < grid[0]; ++w) taken[w] = 1; // pair w / n_chunks, chunk w % n_chunks
    }
    // every chunk a row has was taken once, and has positions: chunk c of a row's n takes its groups of 128 positions
    // c, c + n, ...: the first of them must start inside the row's run
    for (size_t r = 0; r < rows.size(); ++r) {
        const uint64_t run = visible_from_tile(rows[r]), chunks = (run + a.chunk - 1) / a.chunk;
        for (uint32_t g = 0; g < kv_heads; ++g) {
            for (uint64_t c = 0; c < a.n_chunks; ++c) {
                const bool has = c < chunks;
                if (has) CHECK(taken[(r * kv_heads + g) * a.n_chunks + c] && c * 128 < run);
                if (!has && a.work) CHECK(!taken[(r * kv_heads + g) * a.n_chunks + c]);
            }
        }
    }
    if (a.n_chunks > 1) {
        st.split += 1;
        const uint64_t slots = pairs * a.n_chunks * group;
        CHECK(lng_null_bytes_from(a.partial_o) >= slots * dim * 4);
        CHECK(lng_null_bytes_from(a.partial_ml) >= slots * 2 * 4);
        if (a.fused) {
            st.fused += 1;
            CHECK(lng_null_bytes_from(a.tickets) >= pairs * 4 && n_launches == 1);
            for (uint64_t i = 0; i < pairs; ++i) CHECK(a.tickets[i] == 0); // zero whenever no dispatch is running
        } else {
            CHECK(n_launches == 2);
            const char *merge = nullptr;
            unsigned mgrid[3];
            CHECK(lng_null_launch(1, &merge, mgrid, nullptr, nullptr, nullptr) == 0);
            const std::string m = merge;
            CHECK(m == "lng_decode_merge" || m == "lng_decode_merge_few");
            CHECK(mgrid[0] == (m == "lng_decode_merge" ? pairs * group : pairs * ((group + 3) / 4)));
            if (m == "lng_decode_merge_few") CHECK(a.n_chunks <= 32);
        }
    } else {
        CHECK(n_launches == 1 && !a.fused);
    }
}

static void planner_fuzz(size_t dispatches) {
    std::mt19937_64 rng(20251125);
    auto below = [&](uint64_t n) { return (uint64_t)(rng() % n); };
    lng_gpu *gpu = nullptr;
    CHECK(lng_hip_open(0, &gpu) == LNG_OK);
    // one big cache for every row (inputs may share; outputs may not)
    const uint64_t max_rows = 70000;
    const size_t kv_bytes = max_rows * 2 * 64 * 4, qo_bytes = (size_t)300 * 160 * 512 * 4; // the most rows x heads x width x 4 drawn below
    std::vector<lng_buffer *> bufs(5);
    const size_t sizes[5] = {qo_bytes, kv_bytes, kv_bytes, qo_bytes, 4096};
    for (int i = 0; i < 5; ++i) CHECK(lng_hip_buffer(gpu, sizes[i], &bufs[i]) == LNG_OK);
    FuzzStats st;
    const uint32_t dims[] = {64, 64, 64, 64, 128, 256, 512, 96, 32};
    for (size_t it = 0; it < dispatches; ++it) {
        lng_batch *batch = nullptr;
        CHECK(lng_hip_batch(gpu, bufs.data(), bufs.size(), &batch) == LNG_OK);
        const uint32_t dim = dims[below(9)];
        const uint32_t kv_heads = 1u << below(dim >= 256 ? 2 : 4); // 1..8
        const uint32_t group = (uint32_t)(1 + below(below(8) == 0 ? 20 : 8));
        const uint32_t heads = kv_heads * group;
        const int dtype = below(4) == 0 ? LNG_F32 : LNG_BF16;
        const uint64_t es = dtype == LNG_F32 ? 4 : 2, row_bytes = (uint64_t)kv_heads * dim * es, qrow = (uint64_t)heads * dim * es;
        const uint64_t most = std::min<uint64_t>(max_rows, kv_bytes / row_bytes);
        // lengths: mostly short, sometimes long, sometimes all alike
        auto length = [&]() -> uint64_t {
            switch (below(6)) {
            case 0: return 1 + below(160);
            case 1: return 1 + below(most);
            case 2: return 128 * (1 + below(64));
            default: return 1 + below(9000);
            }
        };
        std::vector<lng_k_row> rows;
        int rc;
        if (below(3) == 0) { // the row-by-row operator: t consecutive rows of one cache
            const uint64_t t = 1 + below(below(4) == 0 ? 40 : 4);
            const uint64_t end = std::min<uint64_t>(most, std::max<uint64_t>(length(), t));
            const uint64_t start = end - t;
            uint64_t window = below(3) == 0 ? 1 + below(3000) : LNG_WINDOW_FULL;
            uint64_t slots = end;
            if (window != LNG_WINDOW_FULL && below(2) == 0) slots = std::min<uint64_t>(end, window + t + below(64)); // a ring
            const lng_grouped_shape s = shape(t, start, heads, kv_heads, dim, window, slots, 0.125f);
            const uint64_t kv_rows = std::min(slots, end);
            const uint64_t off = below(4) == 0 ? es * (1 + below(3)) : 0; // sometimes off a 16-byte boundary
            const lng_slice q{0, off, t * qrow}, k{1, 0, kv_rows * row_bytes}, v{2, 0, kv_rows * row_bytes}, o{3, 0, t * qrow}, sk{4, 0, heads * 4ull};
            rc = lng_hip_attention_grouped(batch, q, k, v, o, below(2) ? &sk : nullptr, &s, dtype);
            if (dim % 32 != 0) {
                CHECK(rc == LNG_ERR_DISPATCH);
            } else {
                CHECK(rc == LNG_OK);
            }
            for (uint64_t i = 0; i < t; ++i) rows.push_back(lng_k_row{0, 0, 0, 0, 0, start + i, window, slots});
        } else { // a table of sequences
            const size_t n = 1 + below(below(5) == 0 ? 300 : 40);
            std::vector<lng_decode_item> items(n);
            const bool alike = below(5) == 0;
            const uint64_t same = length();
            for (size_t i = 0; i < n; ++i) {
                const uint64_t len = std::min<uint64_t>(most, alike ? same : length());
                const uint64_t window = below(4) == 0 ? 1 + below(2000) : LNG_WINDOW_FULL;
                uint64_t slots = len;
                if (window != LNG_WINDOW_FULL && below(2) == 0) slots = std::min<uint64_t>(len, window + 1 + below(32));
                items[i] = lng_decode_item{i * qrow, i * qrow, 0, 0, below(2) ? 0 : LNG_NO_SINKS, len - 1, window, slots};
                rows.push_back(items[i]);
            }
            rc = lng_hip_attention_decode_batched(batch, 0, 1, 2, 3, 4, items.data(), n, heads, kv_heads, dim, 0.125f, dtype);
            if (dim % 32 != 0) {
                CHECK(rc == LNG_ERR_DISPATCH);
            } else {
                CHECK(rc == LNG_OK);
            }
        }
        if (rc == LNG_OK) {
            CHECK(lng_hip_batch_commit(batch, nullptr, nullptr) == LNG_OK);
            CHECK(lng_hip_batch_wait(batch, nullptr) == LNG_OK);
            check_rows_dispatch(rows, heads, kv_heads, dim, st);
            st.dispatches += 1;
        }
        lng_hip_batch_drop(batch);
        lng_null_clear();
        if (g_failures) {
            fprintf(stderr, "fuzz dispatch %zu: %zu rows, %u heads over %u of width %u, dtype %d\n", it, rows.size(), heads, kv_heads, dim, dtype);
            break;
        }
    }
    for (lng_buffer *b : bufs) CHECK(lng_hip_buffer_free(b) == LNG_OK);
    lng_hip_close(gpu);
    CHECK(lng_null_live_allocations() == 0);
    printf("planner fuzz: %zu dispatches checked (%zu split, %zu merged in the kernel, %zu with a table of live workgroups, %zu on the "
           "generic kernel, %zu at widths 128-512, %zu on a prompt-pass kernel)\n",
           st.dispatches, st.split, st.fused, st.tables, st.generic, st.wide, st.prefill);
    CHECK(st.split > st.dispatches / 20 && st.fused > 0 && st.tables > 0 && st.generic > 0 && st.wide > 0 && st.prefill > 0);
}

int main(int argc, char **argv) {
    const size_t dispatches = argc > 1 ? (size_t)strtoull(argv[1], nullptr, 10) : 100000;
    refusals();
    switches_and_checksum();
    lifetimes();
    allocation_failures();
    planner_fuzz(dispatches);
    if (g_failures) {
        fprintf(stderr, "%d checks failed\n", g_failures);
        return 1;
    }
    printf("null device: all checks held\n");
    return 0;
}
