// Host side of liblng_hip.so: the C ABI declared in include/lng_hip.h.
//
// Plain HIP driver-style calls only (hipMalloc, hipModuleLoadData, hipModuleLaunchKernel,
// events): the gfx950 code object built from lng_kernels.hip is embedded in this library.
// A batch records dispatches on the host and submits them in order on one stream at
// commit, so an uncommitted batch runs nothing (metal-compute/src/apple.rs:553-561) and a
// refused dispatch leaves nothing behind (apple.rs:1243-1256 run before any encoding).
#include <hip/hip_runtime_api.h>

#include <algorithm>
#include <atomic>
#include <condition_variable>
#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <deque>
#include <mutex>
#include <string>
#include <thread>
#include <vector>

#include "lng_kernel_args.h"
#include "lng_static.h"

#ifdef LNG_NULL_DEVICE
// The host-only build (csrc/null_device): launches are recorded, not run, and there is no code object to embed.
extern "C" const char lng_hsaco_begin[1] = {0};
#else
// The code object, placed in .rodata by the assembler (path given by the build).
#ifndef LNG_HSACO_PATH
#error "LNG_HSACO_PATH must name the gfx950 code object to embed"
#endif
__asm__(".section .rodata\n"
        ".balign 4096\n"
        ".global lng_hsaco_begin\n"
        "lng_hsaco_begin:\n"
        ".incbin \"" LNG_HSACO_PATH "\"\n"
        ".global lng_hsaco_end\n"
        "lng_hsaco_end:\n"
        ".byte 0\n"
        ".previous\n");
extern "C" const char lng_hsaco_begin[];
extern "C" const char lng_hsaco_end[];
#endif

namespace {

thread_local std::string g_error;

int fail(int code, const char *fmt, ...) {
    char text[512];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(text, sizeof text, fmt, ap);
    va_end(ap);
    g_error = text;
    return code;
}

const char *hip_text(hipError_t e) { return hipGetErrorString(e); }

size_t elem_size(int dtype) { return dtype == LNG_BF16 ? 2 : 4; }

// Development switches (not part of the interface): read from the environment once, at lng_hip_open, and changed
// afterwards only through lng_hip_debug_set. Nothing on the record path reads the environment.
struct Knobs {
    bool wide_generic = false;     // LNG_WIDE_GENERIC: head widths 128-512 row by row on the kernel of one workgroup per (row, head)
    bool f32_generic = false;      // LNG_F32_GENERIC: f32 operands on the generic kernel only
    bool plain_row_by_row = false; // LNG_PLAIN_ROW_BY_ROW: the row-by-row operator never takes a prompt-pass kernel
    bool decode_o3 = false;        // LNG_DECODE_O3: never the four-wavefront build of the decode kernel
    bool merge_wide = false;       // LNG_MERGE_WIDE: always the merge of one workgroup per query head
    bool q8_w16 = false;           // LNG_Q8_W16: the one-position Q8_0 kernel always as 16-wavefront workgroups
    bool wide_row_by_row = false;  // LNG_WIDE_ROW_BY_ROW: prompt passes of head widths 128-512 row by row on the decode kernels
    int prefill_stream = -1;       // LNG_PREFILL_STREAM: 0 never the resident prompt-pass kernel, 1 whenever it can run, -1 planner
    int prefill_pair = -1;         // LNG_PREFILL_PAIR: 0 never the head-pair prompt-pass kernel, 1 whenever it can run, -1 planner
    int prefill_upfront = -1;      // LNG_PREFILL_UPFRONT: 0 narrow windows on the tile-by-tile kernel
    int table_in_place = 8192;     // LNG_TABLE_IN_PLACE: row tables of this many bytes or more are read from pinned host memory; 0 never
    int prefill_splits = 0;        // LNG_PREFILL_SPLITS: workgroups per (query tile, kv head) of a split prompt pass; 0 planner
    int checksum_wgs = 0;          // LNG_CHECKSUM_WGS: workgroups per compute unit of the streaming read; 0 default (2)
    bool count_second_passes = false; // LNG_COUNT_SECOND_PASSES: long causal passes count the query tiles they repeat
    long decode_wgs = 0;           // LNG_DECODE_WGS: workgroups a decode dispatch aims for; 0 default
    long fuse_wgs = -1;            // LNG_FUSE_WGS: largest grid that merges inside the decode kernel; -1 default
};

struct Table { // row tables of batched dispatches: a pinned-host block and its device twin, or (in_place) a pinned-host block the kernels read
    char *host = nullptr;
    char *dev = nullptr; // == host when in_place
    size_t cap = 0;
    size_t used = 0;
    bool in_place = false;
};

struct Cmd {
    hipFunction_t fn = nullptr;
    const char *name = "";
    unsigned grid[3] = {1, 1, 1};
    unsigned block = 256;
    std::vector<char> args;
};

} // namespace

struct lng_buffer {
    lng_gpu *gpu = nullptr;
    void *ptr = nullptr;
    size_t len = 0;
    bool resident = false;
    std::atomic<int> holds{0}; // batches owning (buffer) or having attached (resident) it
};

struct lng_gpu {
    int device = 0;
    hipStream_t stream = nullptr;
    hipModule_t module = nullptr;
    // kernels of the embedded code object
    hipFunction_t generic_f32 = nullptr, generic_bf16 = nullptr;
    hipFunction_t decode_bf16_d64 = nullptr, decode_bf16_d64_o4 = nullptr, decode_f32_d64 = nullptr, decode_merge = nullptr, decode_merge_few = nullptr;
    hipFunction_t decode_bf16_wide[3] = {}, decode_f32_wide[3] = {}; // head widths 128, 256, 512
    hipFunction_t prefill_bf16_d64 = nullptr, prefill_bf16_d64_h1 = nullptr, prefill_bf16_d64_h1w = nullptr, prefill_bf16_d64_stream = nullptr, prefill_bf16_d64_pair = nullptr, prefill_f32_d64 = nullptr, prefill_f32_d64_w4 = nullptr, prefill_merge = nullptr;
    hipFunction_t prefill_bf16_wide[3] = {}, prefill_f32_wide[3] = {}; // head widths 128, 256, 512
    hipFunction_t checksum = nullptr, checksum_fold = nullptr;
    hipFunction_t copy_rows = nullptr, fill_synthetic = nullptr, add_rows = nullptr, rotate_halves = nullptr, rmsnorm_rows = nullptr, rmsnorm_row_wg = nullptr;
    hipFunction_t prepare_v4 = nullptr, prepare_v1 = nullptr;
    hipFunction_t q8_split_x = nullptr, q8_stream = nullptr, q8_stream_one = nullptr, q8_stream_one_w8 = nullptr, q8_stream_bf16 = nullptr, q8_tiled = nullptr,
                  q8_tiled_bf16 = nullptr;
    std::string name;
    unsigned cus = 256;

    std::mutex mu;
    std::mutex submit_mu; // one batch at a time puts its kernels on the stream: they share the scratch buffers
    std::vector<Table> free_tables;
    float *scratch_o = nullptr;  // split-K partial outputs, grown on demand
    float *scratch_ml = nullptr; // split-K partial (max, sum)
    uint32_t *tickets = nullptr; // split-K arrival counters, zero whenever no dispatch is running
    size_t scratch_o_len = 0, scratch_ml_len = 0, tickets_len = 0;
    char *scratch_x = nullptr;   // bf16 planes of the positions of a Q8_0 product
    size_t scratch_x_len = 0;
    std::vector<void *> retired; // outgrown scratch, freed at close (dispatches may name it)
    std::vector<hipEvent_t> spare_events; // events of finished batches, used again (under mu): creating a pair costs microseconds per batch
    std::atomic<long> live_buffers{1}; // the open handle, and the buffers, residents and batches that still name this gpu
    unsigned decode_wgs = 4096; // workgroups a decode dispatch aims for
    uint64_t fuse_wgs = 1024;   // decode dispatches of up to this many workgroups merge their chunks in the kernel
    Knobs knobs;                // development switches, see lng_hip_debug_set
    char *static_scratch = nullptr; // this device's copy of the fixed scratch array (LNG_STATIC_SCRATCH_BYTES)
    uint32_t *second_passes = nullptr; // device counter of repeated query tiles (LNG_COUNT_SECOND_PASSES), else NULL

    // completion thread (only for batches committed with a callback)
    std::thread worker;
    std::mutex qmu;
    std::condition_variable qcv;
    std::deque<lng_batch *> queue;
    bool stopping = false;
};

struct lng_batch {
    lng_gpu *gpu = nullptr;
    std::vector<lng_buffer *> buffers;
    std::vector<lng_buffer *> residents;
    std::vector<Cmd> cmds;
    std::vector<Table> tables;
    size_t dispatches = 0;
    enum State { Recording, Committed, Done } state = Recording;
    hipEvent_t ev0 = nullptr, ev1 = nullptr;
    bool timing = false;
    std::vector<hipEvent_t> marks; // timing: one event after every command
    std::vector<double> cmd_seconds;
    lng_on_done on_done = nullptr;
    void *user = nullptr;
    int status = LNG_OK;
    double seconds = 0.0;
    std::string message;
    std::mutex mu;
    std::condition_variable cv;
    bool released = false;
    bool drop_when_done = false; // lng_hip_batch_drop was called from inside on_done
};

namespace {

struct Operand { // a checked slice resolved to its buffer
    lng_buffer *buf;
    uint64_t index;
    uint64_t offset;
    uint64_t len;
};

lng_buffer *buffer_at(lng_batch *b, uint64_t index) {
    if (index < b->buffers.size()) return b->buffers[index];
    index -= b->buffers.size();
    if (index < b->residents.size()) return b->residents[index];
    return nullptr;
}

// apple.rs:860-887 Batch::check
int check_slice(lng_batch *b, const char *what, const lng_slice &s, uint64_t len, uint64_t align,
                Operand *out) {
    lng_buffer *buf = buffer_at(b, s.buffer);
    if (!buf) {
        return fail(LNG_ERR_DISPATCH, "%s: no buffer %llu (batch has %zu)", what,
                    (unsigned long long)s.buffer, b->buffers.size() + b->residents.size());
    }
    if (s.len != len) {
        return fail(LNG_ERR_DISPATCH, "%s: %llu bytes, the shape needs %llu", what,
                    (unsigned long long)s.len, (unsigned long long)len);
    }
    if (s.offset > buf->len || s.len > buf->len - s.offset) {
        return fail(LNG_ERR_DISPATCH, "%s: bytes %llu..%llu outside a %zu-byte buffer", what,
                    (unsigned long long)s.offset, (unsigned long long)(s.offset + s.len), buf->len);
    }
    if (s.offset % align != 0) {
        return fail(LNG_ERR_DISPATCH, "%s: offset %llu is not a multiple of %llu", what,
                    (unsigned long long)s.offset, (unsigned long long)align);
    }
    *out = Operand{buf, s.buffer, s.offset, s.len};
    return LNG_OK;
}

bool overlaps(const Operand &a, const Operand &b) {
    return a.index == b.index && a.offset < b.offset + b.len && b.offset < a.offset + a.len;
}

// apple.rs:889-906 Batch::check_output
int check_output(lng_batch *b, const Operand &y, std::initializer_list<const Operand *> inputs) {
    if (y.index >= b->buffers.size()) {
        return fail(LNG_ERR_DISPATCH, "output is in read-only resident memory");
    }
    for (const Operand *in : inputs) {
        if (overlaps(y, *in)) return fail(LNG_ERR_DISPATCH, "output overlaps an input");
    }
    return LNG_OK;
}

std::string shape_text(const lng_grouped_shape &s) {
    char text[256];
    snprintf(text, sizeof text,
             "GroupedShape { t: %llu, start: %llu, heads: %llu, kv_heads: %llu, dim: %llu, window: %llu, "
             "slots: %llu, scale: %g }",
             (unsigned long long)s.t, (unsigned long long)s.start, (unsigned long long)s.heads,
             (unsigned long long)s.kv_heads, (unsigned long long)s.dim, (unsigned long long)s.window,
             (unsigned long long)s.slots, (double)s.scale);
    return text;
}

bool fits_u32(uint64_t n) { return n <= 0xffffffffull; }

// apple.rs:1243-1272 (plain) and 1356-1385 (tiled)
int check_shape(const lng_grouped_shape &s, bool tiled) {
    const uint64_t end = s.start + s.t;
    const uint64_t need = s.window > UINT64_MAX - s.t ? UINT64_MAX : s.window + s.t;
    const bool ring = s.slots < end;
    bool bad = s.t == 0 || s.kv_heads == 0 || (s.kv_heads && s.heads % s.kv_heads != 0) || s.dim == 0 ||
               s.dim > 512 || s.window == 0 || s.slots == 0 || end < s.start;
    if (!tiled) {
        bad = bad || s.dim % 32 != 0 || (ring && s.slots < need);
    } else {
        bad = bad || s.dim % 16 != 0 || (ring && (s.slots % 32 != 0 || s.slots < need));
    }
    if (bad) {
        return fail(LNG_ERR_DISPATCH, "unsupported %sgrouped attention shape %s", tiled ? "tiled " : "",
                    shape_text(s).c_str());
    }
    const uint64_t window = std::min(s.window, end);
    const uint64_t groups = tiled ? (s.t + 31) / 32 * s.heads : s.t * s.heads;
    for (uint64_t n : {s.t, s.start, s.heads, s.kv_heads, s.dim, window, s.slots, groups}) {
        if (!fits_u32(n)) return fail(LNG_ERR_DISPATCH, "%llu does not fit in u32", (unsigned long long)n);
    }
    if (s.heads == 0) return fail(LNG_ERR_DISPATCH, "unsupported grouped attention shape %s", shape_text(s).c_str());
    return LNG_OK;
}

// One development switch by its environment name; value NULL puts the default back. Returns false for an unknown name.
const char *const knob_names[] = {"LNG_WIDE_GENERIC", "LNG_F32_GENERIC", "LNG_PLAIN_ROW_BY_ROW", "LNG_DECODE_O3", "LNG_MERGE_WIDE",
                                  "LNG_Q8_W16", "LNG_WIDE_ROW_BY_ROW", "LNG_PREFILL_STREAM", "LNG_PREFILL_PAIR", "LNG_PREFILL_UPFRONT",
                                  "LNG_PREFILL_SPLITS", "LNG_DECODE_WGS", "LNG_FUSE_WGS", "LNG_COUNT_SECOND_PASSES", "LNG_CHECKSUM_WGS", "LNG_TABLE_IN_PLACE"};
bool set_knob(lng_gpu *g, const char *name, const char *value) {
    Knobs &k = g->knobs;
    const Knobs defaults;
    const long n = value ? atol(value) : 0;
    auto flag = [&](bool &field) { field = value != nullptr; return true; }; // present, whatever it holds: on
    auto choice = [&](int &field, int dflt) { field = value ? (int)n : dflt; return true; };
    if (!strcmp(name, "LNG_WIDE_GENERIC")) return flag(k.wide_generic);
    if (!strcmp(name, "LNG_F32_GENERIC")) return flag(k.f32_generic);
    if (!strcmp(name, "LNG_PLAIN_ROW_BY_ROW")) return flag(k.plain_row_by_row);
    if (!strcmp(name, "LNG_DECODE_O3")) return flag(k.decode_o3);
    if (!strcmp(name, "LNG_MERGE_WIDE")) return flag(k.merge_wide);
    if (!strcmp(name, "LNG_Q8_W16")) return flag(k.q8_w16);
    if (!strcmp(name, "LNG_WIDE_ROW_BY_ROW")) return flag(k.wide_row_by_row);
    if (!strcmp(name, "LNG_COUNT_SECOND_PASSES")) return flag(k.count_second_passes);
    if (!strcmp(name, "LNG_PREFILL_STREAM")) return choice(k.prefill_stream, defaults.prefill_stream);
    if (!strcmp(name, "LNG_PREFILL_PAIR")) return choice(k.prefill_pair, defaults.prefill_pair);
    if (!strcmp(name, "LNG_PREFILL_UPFRONT")) return choice(k.prefill_upfront, defaults.prefill_upfront);
    if (!strcmp(name, "LNG_CHECKSUM_WGS")) return choice(k.checksum_wgs, defaults.checksum_wgs);
    if (!strcmp(name, "LNG_TABLE_IN_PLACE")) {
        k.table_in_place = value ? (int)std::max(0l, std::min(n, 1l << 30)) : defaults.table_in_place;
        return true;
    }
    if (!strcmp(name, "LNG_PREFILL_SPLITS")) {
        k.prefill_splits = value ? (int)std::max(1l, std::min(n, 64l)) : 0;
        return true;
    }
    if (!strcmp(name, "LNG_DECODE_WGS")) {
        g->decode_wgs = value && n >= 1 && n <= (1 << 20) ? (unsigned)n : 4096u;
        return true;
    }
    if (!strcmp(name, "LNG_FUSE_WGS")) {
        g->fuse_wgs = value && n >= 0 ? (uint64_t)n : 4ull * g->cus;
        return true;
    }
    return false;
}

int need_recording(lng_batch *b) {
    if (!b) return fail(LNG_ERR_DISPATCH, "no batch");
    if (b->state != lng_batch::Recording) return fail(LNG_ERR_DISPATCH, "the batch was already committed");
    return LNG_OK;
}

template <typename A> void set_args(Cmd &c, const A &a) {
    c.args.resize(sizeof(A));
    memcpy(c.args.data(), &a, sizeof(A));
}

// Device scratch for split-K partials, shared by every dispatch of the gpu: dispatches run
// in order on one stream, so the next one starts after the previous combine has read it.
// The three pointers are handed out as they were under the lock: a batch recorded on another thread may grow and
// swap them right after (the outgrown ones stay allocated until close, so a dispatch recorded with them is safe).
struct Scratch {
    float *o = nullptr;
    float *ml = nullptr;
    uint32_t *tickets = nullptr;
};
int reserve_scratch(lng_gpu *g, size_t o_floats, size_t ml_floats, size_t n_tickets, Scratch *out) {
    std::lock_guard<std::mutex> lock(g->mu);
    if (n_tickets > g->tickets_len) {
        void *p = nullptr;
        const size_t want = std::max(n_tickets, g->tickets_len * 2);
        if (hipMalloc(&p, want * sizeof(uint32_t)) != hipSuccess) return fail(LNG_ERR_ALLOC, "could not allocate a %zu-byte scratch buffer", want * sizeof(uint32_t));
        // Zeroed on the dispatch stream: later dispatches are ordered after it, earlier ones keep
        // the retired counters they were recorded with.
        if (hipMemsetAsync(p, 0, want * sizeof(uint32_t), g->stream) != hipSuccess) {
            hipFree(p);
            return fail(LNG_ERR_GPU, "could not clear the scratch counters");
        }
        if (g->tickets) g->retired.push_back(g->tickets);
        g->tickets = (uint32_t *)p;
        g->tickets_len = want;
    }
    if (o_floats > g->scratch_o_len) {
        void *p = nullptr;
        const size_t want = std::max(o_floats, g->scratch_o_len * 2);
        if (hipMalloc(&p, want * sizeof(float)) != hipSuccess) return fail(LNG_ERR_ALLOC, "could not allocate a %zu-byte scratch buffer", want * sizeof(float));
        if (g->scratch_o) g->retired.push_back(g->scratch_o);
        g->scratch_o = (float *)p;
        g->scratch_o_len = want;
    }
    if (ml_floats > g->scratch_ml_len) {
        void *p = nullptr;
        const size_t want = std::max(ml_floats, g->scratch_ml_len * 2);
        if (hipMalloc(&p, want * sizeof(float)) != hipSuccess) return fail(LNG_ERR_ALLOC, "could not allocate a %zu-byte scratch buffer", want * sizeof(float));
        if (g->scratch_ml) g->retired.push_back(g->scratch_ml);
        g->scratch_ml = (float *)p;
        g->scratch_ml_len = want;
    }
    out->o = g->scratch_o;
    out->ml = g->scratch_ml;
    out->tickets = g->tickets;
    return LNG_OK;
}

// Space for a row table: pinned host memory now, its device twin filled at commit.
// A table of up to a few kilobytes is copied to the device ahead of the batch's kernels (one copy per block of
// tables: about 3 us and a dependency); a larger one stays in pinned host memory and the kernels read it there - the
// copy of a 17 KB table took 10 us of a 217 us dispatch of 128 sequences, and a workgroup reads only its own row and
// a few running counts (LNG_TABLE_IN_PLACE: the size in bytes from which tables stay; 0 never).
// `decides`: the size that says where the table goes, when it is not the table's own (the running counts of a row
// table go where the rows went).
int reserve_table(lng_batch *b, size_t bytes, char **host, char **dev, size_t decides = 0) {
    lng_gpu *g = b->gpu;
    const bool in_place = g->knobs.table_in_place > 0 && (decides ? decides : bytes) >= (size_t)g->knobs.table_in_place;
    Table *block = nullptr;
    for (size_t i = b->tables.size(); i-- > 0;) { // the newest block of the kind that has room
        Table &t = b->tables[i];
        if (t.in_place == in_place) {
            if (t.cap - t.used >= bytes) block = &t;
            break;
        }
    }
    if (!block) {
        Table t;
        {
            std::lock_guard<std::mutex> lock(g->mu);
            for (size_t i = 0; i < g->free_tables.size(); ++i) {
                if (g->free_tables[i].cap >= bytes && g->free_tables[i].in_place == in_place) {
                    t = g->free_tables[i];
                    g->free_tables.erase(g->free_tables.begin() + i);
                    break;
                }
            }
        }
        if (!t.host) {
            t.cap = std::max<size_t>(bytes, 64 * 1024);
            t.in_place = in_place;
            if (hipHostMalloc((void **)&t.host, t.cap, hipHostMallocDefault) != hipSuccess) return fail(LNG_ERR_ALLOC, "could not allocate a %zu-byte pinned table", t.cap);
            if (in_place) {
                t.dev = t.host; // (pinned host memory has the same address on the device)
            } else if (hipMalloc((void **)&t.dev, t.cap) != hipSuccess) {
                hipHostFree(t.host);
                return fail(LNG_ERR_ALLOC, "could not allocate a %zu-byte device table", t.cap);
            }
        }
        t.used = 0;
        b->tables.push_back(t);
        block = &b->tables.back();
    }
    Table &t = *block;
    *host = t.host + t.used;
    *dev = t.dev + t.used;
    t.used += (bytes + 255) / 256 * 256;
    if (t.used > t.cap) t.used = t.cap;
    return LNG_OK;
}

void release(lng_batch *b) { // buffers and tables go back; idempotent
    if (b->released) return;
    b->released = true;
    for (lng_buffer *buf : b->buffers) buf->holds.fetch_sub(1);
    for (lng_buffer *buf : b->residents) buf->holds.fetch_sub(1);
    std::lock_guard<std::mutex> lock(b->gpu->mu);
    for (Table &t : b->tables) b->gpu->free_tables.push_back(t);
    b->tables.clear();
}

// Events are pooled per gpu: a batch takes two (more when it is timed dispatch by dispatch) and gives them back.
// (Creating and destroying a pair per batch cost 1.5 us of a 5 us commit, and more with the completion thread
// destroying while the caller creates: a one-dispatch batch with a callback 25 -> 19 us from record to completion.
// Polling for the batch's end instead of sleeping until it was measured and gains nothing: what separates the 7 us
// the GPU takes from the 12 us the wait lasts is the dispatch's way to the GPU, not the wake-up.)
hipError_t take_event(lng_gpu *g, hipEvent_t *ev) {
    {
        std::lock_guard<std::mutex> lock(g->mu);
        if (!g->spare_events.empty()) {
            *ev = g->spare_events.back();
            g->spare_events.pop_back();
            return hipSuccess;
        }
    }
    return hipEventCreate(ev);
}
void give_event(lng_gpu *g, hipEvent_t ev) {
    if (!ev) return;
    {
        std::lock_guard<std::mutex> lock(g->mu);
        if (g->spare_events.size() < 64) {
            g->spare_events.push_back(ev);
            return;
        }
    }
    hipEventDestroy(ev);
}

// Waits for the GPU, fills status/seconds, hands the buffers back. Called once per batch.
void finish(lng_batch *b) {
    hipSetDevice(b->gpu->device);
    hipError_t e = hipEventSynchronize(b->ev1);
    if (e == hipSuccess) {
        float ms = 0.0f;
        e = hipEventElapsedTime(&ms, b->ev0, b->ev1);
        if (e == hipSuccess) b->seconds = std::max(0.0, (double)ms * 1e-3);
        b->cmd_seconds.assign(b->marks.size(), 0.0);
        for (size_t i = 0; e == hipSuccess && i < b->marks.size(); ++i) {
            e = hipEventElapsedTime(&ms, i ? b->marks[i - 1] : b->ev0, b->marks[i]);
            if (e == hipSuccess) b->cmd_seconds[i] = std::max(0.0, (double)ms * 1e-3);
        }
    }
    if (e != hipSuccess) {
        b->status = LNG_ERR_GPU;
        b->message = hip_text(e);
    }
    release(b);
}

void object_gone(lng_gpu *g);

void destroy(lng_batch *b) {
    lng_gpu *g = b->gpu;
    give_event(g, b->ev0);
    give_event(g, b->ev1);
    for (hipEvent_t mark : b->marks) give_event(g, mark);
    delete b;
    object_gone(g);
}

void worker_loop(lng_gpu *g) {
    for (;;) {
        lng_batch *b = nullptr;
        {
            std::unique_lock<std::mutex> lock(g->qmu);
            g->qcv.wait(lock, [&] { return g->stopping || !g->queue.empty(); });
            if (g->queue.empty()) return;
            b = g->queue.front();
            g->queue.pop_front();
        }
        finish(b);
        if (b->on_done) {
            lng_completed done{b->status, b->seconds, b->message.c_str()};
            b->on_done(&done, b->user);
        }
        bool drop = false;
        {
            // Notified under the lock: a waiter may delete the batch as soon as it sees Done, and
            // it cannot see it before this thread has let go of the batch for good.
            std::lock_guard<std::mutex> lock(b->mu);
            b->state = lng_batch::Done;
            drop = b->drop_when_done;
            b->cv.notify_all();
        }
        if (drop) destroy(b); // the callback dropped its own batch: nobody else holds the handle
    }
}

// Rows of one dispatch, and how to split them over workgroups.
struct DecodePlan {
    uint32_t chunk = 128;
    uint32_t n_chunks = 1;
};

uint64_t visible_from_tile(const lng_k_row &r) { // positions from the tile-aligned window start
    const uint64_t last = r.start;
    const uint64_t first = (r.window != LNG_WINDOW_FULL && last + 1 > r.window) ? last + 1 - r.window : 0;
    return last + 1 - (first & ~(uint64_t)31);
}

DecodePlan plan_decode(lng_gpu *g, const lng_k_row *rows, size_t n, uint64_t t_uniform, uint32_t kv_heads, unsigned wgs_per_cu,
                       unsigned width = 1 /* head width in units of 64: bytes per position grow with it */) {
    // rows == the table, or one row standing for t_uniform consecutive queries of one cache
    uint64_t total = 0, longest = 0;
    if (t_uniform) {
        for (uint64_t i = 0; i < t_uniform; ++i) {
            lng_k_row r = rows[0];
            r.start += i;
            const uint64_t v = visible_from_tile(r);
            total += v;
            longest = std::max(longest, v);
        }
    } else {
        for (size_t i = 0; i < n; ++i) {
            const uint64_t v = visible_from_tile(rows[i]);
            total += v;
            longest = std::max(longest, v);
        }
    }
    DecodePlan p;
    const uint64_t per_wg = (total * kv_heads + g->decode_wgs - 1) / g->decode_wgs;
    uint64_t chunk = (per_wg + 127) / 128 * 128;
    chunk = std::max<uint64_t>(chunk, 128);
    // The merge of a row walks its chunks one after another: no more than 32 chunks per row (16 up to 8,192
    // positions when the dispatch has one or two sequences: with many rows the merges run side by side and
    // larger chunks only unbalance the workgroups), unless so few rows are in the dispatch that this would leave compute units without
    // a workgroup (bf16; two workgroups for the f32 kernel, which has twice the bytes per position and a merge
    // of its own dispatch anyway) and the chunks would stay at 512 positions or more (all measured on one
    // sequence: 4,096 keys 13.9 -> 12.3 us, 131,072 keys 76 -> 50 us); never more than LNG_MAX_CHUNKS (the merge
    // keeps one weight per chunk in LDS).
    const uint64_t pairs = (t_uniform ? t_uniform : (uint64_t)n) * kv_heads;
    const uint64_t fill = std::min<uint64_t>((wgs_per_cu * g->cus + pairs - 1) / pairs, longest / std::max(128u, 512u / width));
    const uint64_t most = std::min<uint64_t>(LNG_MAX_CHUNKS, std::max<uint64_t>(longest <= 8192 && pairs <= 16 ? 16 : 32, fill));
    chunk = std::max<uint64_t>(chunk, ((longest + most - 1) / most + 127) / 128 * 128);
    chunk = std::max<uint64_t>(chunk, ((longest + LNG_MAX_CHUNKS - 1) / LNG_MAX_CHUNKS + 127) / 128 * 128);
    // Short runs (a 128-token window seen from its 32-aligned start is up to 159 positions) stay whole: two
    // chunks would mean partials, arrival counters and a merge for five tiles of work.
    if (longest <= 512) chunk = std::max<uint64_t>(chunk, (longest + 127) / 128 * 128);
    p.chunk = (uint32_t)chunk;
    p.n_chunks = (uint32_t)((longest + chunk - 1) / chunk);
    return p;
}

// What a set of single-query rows (decode, and short passes row by row) runs as.
struct RowsPlan {
    enum Kind { Generic, Bf16, F32 } kind = Generic;
    int wide = -1;               // -1: head width 64; 0, 1, 2: the kernels for widths 128, 256, 512
    DecodePlan chunks;
    bool fused = false;          // split-K merged inside the decode kernel (tickets) instead of by lng_decode_merge
    size_t partial_slots = 0;    // (row, kv head, chunk, query head of the group) slots of split-K partials; 0: none
    size_t pairs = 0;            // rows x kv heads
};

RowsPlan plan_rows(lng_gpu *g, const lng_k_attn &a, const lng_k_row *host_rows, size_t n_rows, uint64_t t_uniform,
                   bool aligned16) {
    RowsPlan p;
    const uint32_t group = a.heads / a.kv_heads;
    // Head widths the matrix kernels serve: 64 (gpt-oss), and 128, 256, 512 in slices of 64. Anything else, groups of
    // more than 16 query heads and operands off 16-byte boundaries go to the kernel of one wavefront per (row, head).
    const int wide = a.dim == 128 ? 0 : a.dim == 256 ? 1 : a.dim == 512 ? 2 : -1;
    const bool dim_ok = a.dim == 64 || (wide >= 0 && !g->knobs.wide_generic);
    const bool fast = a.dtype == LNG_BF16 && dim_ok && group <= 16 && aligned16;
    // f32 (the reference's own element type) at the gpt-oss head width: the same chunks and partials on the f32 matrix instruction
    // (that kernel counts positions in 32 bits and steps by up to 256 chunks x 128 positions past the last one)
    uint64_t latest = t_uniform ? host_rows[0].start + t_uniform - 1 : 0;
    for (size_t i = 0; !t_uniform && i < n_rows; ++i) latest = std::max(latest, host_rows[i].start);
    const bool fast_f32 = a.dtype == LNG_F32 && dim_ok && group <= 16 && aligned16 && latest < 0xffff0000ull &&
                          a.scale > 0.0f && a.scale <= 3.0e38f && !g->knobs.f32_generic;
    p.pairs = n_rows * (size_t)a.kv_heads;
    if (!fast && !fast_f32) return p;
    p.kind = fast ? RowsPlan::Bf16 : RowsPlan::F32;
    p.wide = wide;
    p.chunks = plan_decode(g, host_rows, n_rows, t_uniform, a.kv_heads, fast ? 1u : 2u, a.dim / 64);
    if (p.chunks.n_chunks > 1) {
        p.partial_slots = p.pairs * (size_t)p.chunks.n_chunks * group;
        // Small grids merge inside the kernel; large ones with a second dispatch (the f32 and wide-head kernels always).
        p.fused = fast && wide < 0 && (uint64_t)p.chunks.n_chunks * p.pairs <= g->fuse_wgs;
    }
    return p;
}

// The (at most two) launches of a planned set of rows; no heap, so that the entry point that allocates
// nothing can share it.
struct RowsLaunches {
    int n = 0;
    struct One {
        hipFunction_t fn;
        const char *name;
        unsigned grid;
        lng_k_attn args;
    } l[2];
};

// `a` already names its scratch. With a table of rows of unequal length the decode kernel launches its live
// workgroups only and finds each one's row in a table of running counts (`work_host` / `work_dev`, room for
// n_rows + 1 counts of 4 bytes; NULL: a rectangle of n_chunks workgroups per pair, those past a row's end
// returning at once).
int rows_launches(lng_gpu *g, lng_k_attn a, const RowsPlan &p, const lng_k_row *host_rows, size_t n_rows,
                  uint32_t *work_host, const uint32_t *work_dev, RowsLaunches *out) {
    const uint32_t group = a.heads / a.kv_heads;
    out->n = 0;
    if (p.kind == RowsPlan::Generic) {
        if (n_rows * (uint64_t)a.heads > 0x7fffffffull) return fail(LNG_ERR_DISPATCH, "%zu rows of %u heads are more workgroups than one dispatch holds", n_rows, a.heads);
        out->l[out->n++] = {a.dtype == LNG_BF16 ? g->generic_bf16 : g->generic_f32,
                            a.dtype == LNG_BF16 ? "lng_attn_generic_bf16" : "lng_attn_generic_f32",
                            (unsigned)(n_rows * a.heads), a};
        return LNG_OK;
    }
    a.chunk = p.chunks.chunk;
    a.n_chunks = p.chunks.n_chunks;
    a.fused = p.fused ? 1u : 0u;
    uint64_t wgs = (uint64_t)p.pairs * a.n_chunks;
    if (wgs > 0x7fffffffull || (uint64_t)p.pairs * group > 0x7fffffffull) {
        return fail(LNG_ERR_DISPATCH, "%zu rows of %u kv heads in %u chunks are more workgroups than one dispatch holds", n_rows, a.kv_heads, a.n_chunks);
    }
    a.work = nullptr;
    if (work_host && a.n_chunks > 1) {
        uint64_t n = 0;
        for (size_t r = 0; r < n_rows; ++r) {
            work_host[r] = (uint32_t)n;
            n += (visible_from_tile(host_rows[r]) + a.chunk - 1) / a.chunk * a.kv_heads;
        }
        work_host[n_rows] = (uint32_t)n;
        a.work = work_dev;
        wgs = n;
    }
    static const char *const wide_bf16[3] = {"lng_decode_bf16_w128", "lng_decode_bf16_w256", "lng_decode_bf16_w512"};
    static const char *const wide_f32[3] = {"lng_decode_f32_w128", "lng_decode_f32_w256", "lng_decode_f32_w512"};
    if (p.wide >= 0) {
        out->l[out->n++] = {p.kind == RowsPlan::Bf16 ? g->decode_bf16_wide[p.wide] : g->decode_f32_wide[p.wide],
                            p.kind == RowsPlan::Bf16 ? wide_bf16[p.wide] : wide_f32[p.wide], (unsigned)wgs, a};
    } else {
        // (many workgroups of short chunks - a table of sequences: the build of the bf16 kernel with four wavefronts per SIMD)
        const bool o4 = p.kind == RowsPlan::Bf16 && a.chunk < 2048u && wgs > 3ull * g->cus && !g->knobs.decode_o3;
        out->l[out->n++] = {p.kind == RowsPlan::Bf16 ? (o4 ? g->decode_bf16_d64_o4 : g->decode_bf16_d64) : g->decode_f32_d64,
                            p.kind == RowsPlan::Bf16 ? (o4 ? "lng_decode_bf16_d64_o4" : "lng_decode_bf16_d64") : "lng_decode_f32_d64", (unsigned)wgs, a};
    }
    if (a.n_chunks > 1 && !a.fused) {
        if (a.n_chunks <= 32 && !g->knobs.merge_wide) { // a wavefront per (row, kv head, query head), four to a workgroup (LNG_MERGE_FEW)
            out->l[out->n++] = {g->decode_merge_few, "lng_decode_merge_few", (unsigned)(p.pairs * ((group + 3) / 4)), a};
        } else {                                            // a workgroup per (row, kv head, query head)
            out->l[out->n++] = {g->decode_merge, "lng_decode_merge", (unsigned)(p.pairs * group), a};
        }
    }
    return LNG_OK;
}

// Records the kernels for a set of single-query rows (decode, and short passes row by row).
int record_rows(lng_batch *b, lng_k_attn a, const lng_k_row *host_rows, size_t n_rows, uint64_t t_uniform,
                bool aligned16) {
    lng_gpu *g = b->gpu;
    const RowsPlan p = plan_rows(g, a, host_rows, n_rows, t_uniform, aligned16);
    if (p.partial_slots) {
        Scratch sc;
        if (int rc = reserve_scratch(g, p.partial_slots * a.dim, p.partial_slots * 2, p.pairs, &sc)) return rc;
        a.partial_o = sc.o;
        a.partial_ml = sc.ml;
        a.tickets = sc.tickets;
    }
    // Rows of unequal length (a table of sequences): room for the running counts of live workgroups.
    char *work_host = nullptr, *work_dev = nullptr;
    if (!t_uniform && p.chunks.n_chunks > 1 && p.kind != RowsPlan::Generic) {
        uint64_t live = 0;
        for (size_t r = 0; r < n_rows; ++r) live += (visible_from_tile(host_rows[r]) + p.chunks.chunk - 1) / p.chunks.chunk;
        if (live < (uint64_t)n_rows * p.chunks.n_chunks && live * a.kv_heads <= 0x7fffffffull) {
            if (int rc = reserve_table(b, (n_rows + 1) * 4, &work_host, &work_dev, n_rows * sizeof(lng_k_row))) return rc;
        }
    }
    RowsLaunches launches;
    if (int rc = rows_launches(g, a, p, host_rows, n_rows, (uint32_t *)work_host, (const uint32_t *)work_dev, &launches)) return rc;
    for (int i = 0; i < launches.n; ++i) {
        Cmd c;
        c.fn = launches.l[i].fn;
        c.name = launches.l[i].name;
        c.grid[0] = launches.l[i].grid;
        c.block = 256;
        set_args(c, launches.l[i].args);
        b->cmds.push_back(std::move(c));
    }
    return LNG_OK;
}

int attention(lng_batch *b, lng_slice q, lng_slice k, lng_slice v, lng_slice out, const lng_slice *sinks,
              const lng_grouped_shape *shape, int dtype, bool tiled) {
    if (int rc = need_recording(b)) return rc;
    if (!shape) return fail(LNG_ERR_DISPATCH, "no shape");
    if (dtype != LNG_F32 && dtype != LNG_BF16) return fail(LNG_ERR_DISPATCH, "unknown element type %d", dtype);
    const lng_grouped_shape &s = *shape;
    if (int rc = check_shape(s, tiled)) return rc;
    const uint64_t es = elem_size(dtype);
    const uint64_t end = s.start + s.t;
    uint64_t q_rows, kv_rows;
    if (!tiled) {
        q_rows = s.t; // apple.rs:1273-1277
        kv_rows = std::min(s.slots, end);
    } else {
        q_rows = (s.t + 31) / 32 * 32; // apple.rs:1386-1395
        kv_rows = s.slots < end ? s.slots : (end + 31) / 32 * 32;
    }
    // (slots and rows x heads fit in u32; a row of all heads below 2^32 bytes keeps the byte counts inside 64 bits)
    if (!fits_u32(s.heads * s.dim * es)) return fail(LNG_ERR_DISPATCH, "rows of %llu bytes do not fit in u32", (unsigned long long)(s.heads * s.dim * es));
    Operand oq, ok, ov, oo, os{};
    if (int rc = check_slice(b, "q", q, q_rows * s.heads * s.dim * es, es, &oq)) return rc;
    if (int rc = check_slice(b, "k", k, kv_rows * s.kv_heads * s.dim * es, es, &ok)) return rc;
    if (int rc = check_slice(b, "v", v, kv_rows * s.kv_heads * s.dim * es, es, &ov)) return rc;
    if (int rc = check_slice(b, "out", out, q_rows * s.heads * s.dim * es, es, &oo)) return rc;
    if (int rc = check_output(b, oo, {&oq, &ok, &ov})) return rc;
    if (sinks) {
        if (int rc = check_slice(b, "sinks", *sinks, s.heads * 4, 4, &os)) return rc;
    }
    lng_gpu *g = b->gpu;
    const bool aligned16 = ((q.offset | k.offset | v.offset | out.offset) & 15u) == 0;

    // The row-by-row operator with several rows over a long run of keys (the tail of a prompt, a few
    // tokens at once late in a context) reads the cache once per row in the decode kernel; the prompt-pass
    // kernel reads it once per call and gives the same rows (it touches no row outside
    // [first visible position, last position], which is all the row-by-row operator promises to be there).
    // Measured break-even on 64/8 heads: rows x visible keys of about 32 K at 2,048 keys (16 rows), 16 K from 4,096 keys on.
    const uint64_t seen = std::min<uint64_t>(end, s.window > UINT64_MAX - s.t ? UINT64_MAX : s.window + s.t);
    const bool several_rows = !tiled && s.t >= 4 && seen >= 1024 && (s.t * seen >= 32768 || (seen >= 4096 && s.t * seen >= 16384)) &&
                              !b->gpu->knobs.plain_row_by_row;
    // (the matrix kernels take the maximum of the raw products and scale it afterwards: scale > 0; any other
    // scale goes to the kernels that scale first)
    const bool scale_positive = s.scale > 0.0f && s.scale <= 3.0e38f;
    // (the prompt-pass kernels compare distances between positions as signed 32-bit numbers)
    if ((tiled || several_rows) && s.dim == 64 && s.heads / s.kv_heads <= 8 && aligned16 && scale_positive && end <= 0x7fffffffull &&
        (dtype == LNG_BF16 || !g->knobs.f32_generic)) {
        const bool f32 = dtype == LNG_F32;
        lng_k_prefill p{};
        p.dtype = (uint32_t)dtype;
        p.q = (const char *)oq.buf->ptr + q.offset;
        p.k = (const char *)ok.buf->ptr + k.offset;
        p.v = (const char *)ov.buf->ptr + v.offset;
        p.out = (char *)oo.buf->ptr + out.offset;
        p.sinks = sinks ? (const float *)((const char *)os.buf->ptr + sinks->offset) : nullptr;
        p.t = s.t;
        p.start = s.start;
        p.window = s.window >= end ? LNG_WINDOW_FULL : s.window; // a window over everything is no window
        p.slots = s.slots;
        p.heads = (uint32_t)s.heads;
        p.kv_heads = (uint32_t)s.kv_heads;
        p.dim = (uint32_t)s.dim;
        // Two heads per wavefront (64 query rows per workgroup) for long causal runs; one head
        // per wavefront (32 rows, two workgroups per compute unit) when each query sees few keys
        // and the pass is bound by latency, not by the matrix pipe.
        // (the f32 kernel has one form: 32 rows, one head per wavefront; it is bound by the f32 matrix rate)
        // Up to 32 rows (the tail of a prompt, a few tokens at once) would leave half of a 64-row tile empty: the
        // 32-row form again (measured 10-30 % faster there; from 64 rows on the two-head form wins at long contexts).
        const bool few_rows = s.t <= 32;
        const bool narrow = !f32 && ((p.window != LNG_WINDOW_FULL && p.window <= 1024) || few_rows);
        const unsigned rows_per_wg = narrow || f32 ? 32 : 64;
        p.q_tiles = (uint32_t)((s.t + rows_per_wg - 1) / rows_per_wg);
        p.scale = s.scale;
        p.second_passes = g->knobs.count_second_passes ? g->second_passes : nullptr;
        // Few query tiles over many keys (a chunk of a long prompt, a handful of rows late in a long
        // context) would leave most compute units idle with one workgroup per (query tile, kv head):
        // the keys of a tile are then split between several workgroups and lng_prefill_merge combines
        // them, as the decode path does. Splits for one workgroup per compute unit (what is resident at a
        // time; measured best: the merge grows with the splits), each keeping at least four key tiles.
        p.splits = 1;
        const uint64_t visible = p.window == LNG_WINDOW_FULL ? end : std::min<uint64_t>(end, p.window + rows_per_wg);
        const uint64_t key_tiles = (visible + 63) / 64;
        const uint64_t plain_wgs = (uint64_t)p.q_tiles * s.kv_heads;
        // LNG_PREFILL_STREAM: 0 never takes the kernel of workgroups that walk several query tiles, 1 takes it for
        // every full-causal pass it can run (tests: small shapes), otherwise only when every compute unit has a tile.
        const bool stream_can = !f32 && !narrow && p.window == LNG_WINDOW_FULL && s.slots >= end && g->knobs.prefill_stream != 0;
        const bool stream = stream_can && (plain_wgs >= g->cus || g->knobs.prefill_stream == 1);
        // Between the two - 64-row tiles, but fewer (query tile, kv head) pairs than compute units (a prompt fed 512 rows
        // at a time) - a workgroup per (query tile, kv head, PAIR of heads) that deals the keys out among its own
        // wavefronts: four times the workgroups and nothing to merge afterwards
        // (LNG_PREFILL_PAIR: 0 never, 1 whenever it can run).
        const uint64_t head_pairs = (s.heads / s.kv_heads + 1) / 2;
        const bool pair_can = !f32 && !narrow && !stream && g->knobs.prefill_pair != 0 && g->knobs.prefill_splits == 0;
        bool pair = pair_can && g->knobs.prefill_pair == 1;
        if (pair_can && g->knobs.prefill_pair < 0 && plain_wgs < g->cus && head_pairs > 1) {
            // Which is faster depends on how many keys a call walks: a head-pair workgroup walks all keys of its query
            // tile, a split workgroup only its share. Fitted to single calls of 192-1,920 rows after 0-4,096 positions
            // and to the 16 calls of 512 rows of an 8,192-position prompt (64/8 heads, to within 3 us): head pairs take
            // 3 us + per round of workgroups on the device's units (9 us + 1.9 us per 256 keys that a row sees on
            // average); the other kernel 10 us + 1.6 us per 64 keys of the longest run, or, with the keys split, 25 us
            // (the merge dispatch included) + 1.6 us per 64 keys of a split's share.
            // 8,192 positions in calls of 512 rows: 855 -> 686 us; 16,384 in calls of 512: 2,543 -> 2,364 us (head pairs
            // up to about 12,000 keys); 4,096 in calls of 256: 506 -> 407 us; 2,048 in calls of 128: 384 -> 277 us; one
            // call of 1,024 rows: 40.8 -> 28.7 us; calls of 256 rows beyond about 3,300 keys and one call of 1,920 rows
            // stay with the other kernel.
            const double seen_avg = (double)visible - (p.window == LNG_WINDOW_FULL ? 0.5 * (double)std::min<uint64_t>(s.t, visible) : 0.0);
            const uint64_t rounds = (plain_wgs * head_pairs + g->cus - 1) / g->cus;
            const double pair_us = 3.0 + (double)rounds * (9.0 + (1.9 / 256.0) * seen_avg);
            const uint64_t would_split = std::max<uint64_t>(1, std::min<uint64_t>(std::min<uint64_t>(g->cus / plain_wgs, key_tiles / 4), 64));
            const bool splits = would_split > 1 && key_tiles >= 12;
            const double split_us = splits ? 25.0 + (1.6 / 64.0) * (double)visible / (double)would_split : 10.0 + (1.6 / 64.0) * (double)visible;
            pair = pair_us < split_us;
        }
        if (!stream && !pair && (!narrow || few_rows) && plain_wgs < g->cus && s.t * s.kv_heads <= 65535) {
            uint64_t want = g->cus / plain_wgs;
            want = std::min<uint64_t>(want, key_tiles / 4);
            want = std::min<uint64_t>(want, 64);
            // (under a dozen key tiles the partial rows and the merge cost what two splits save: the first 512 rows of a
            // prompt 24.5 us unsplit, 30.8 us in two)
            if (key_tiles < 12) want = 1;
            if (g->knobs.prefill_splits > 0) want = std::min<uint64_t>(g->knobs.prefill_splits, 64);
            if (want > 1) p.splits = (uint32_t)want;
        }
        if (p.splits > 1) {
            const size_t slots = (size_t)s.t * s.heads * p.splits;
            Scratch sc;
            if (int rc = reserve_scratch(g, slots * 64, slots * 2, 0, &sc)) return rc;
            p.partial_o = sc.o;
            p.partial_ml = sc.ml;
        }
        // The long full-causal pass with every compute unit busy anyway: one workgroup per compute unit that stays
        // there and walks several query tiles (balanced by construction, no per-workgroup start-up between them).
        Cmd c;
        c.grid[0] = p.q_tiles * (unsigned)s.kv_heads * p.splits; // kv head fastest: one XCD's L2 per kv head
        c.block = 512;
        if (stream) {
            const uint64_t per_head = std::min<uint64_t>(p.q_tiles, std::max<uint64_t>(1, g->cus / s.kv_heads));
            c.grid[0] = (unsigned)(per_head * s.kv_heads);
        }
        if (pair) c.grid[0] = (unsigned)(plain_wgs * head_pairs);
        // f32: two workgroups per compute unit only when there are four rounds of them or more (see the kernels)
        const bool f32_two = f32 && c.grid[0] >= 4u * g->cus;
        // Windows of up to 160 positions: the 32 query rows of a workgroup see at most four tiles of 64 keys, and the
        // one-head kernel asks for all of them at its start, straight into LDS (LNG_PREFILL_UPFRONT=0: never).
        const bool upfront = narrow && p.window != LNG_WINDOW_FULL && p.window <= 160 && p.splits == 1 && g->knobs.prefill_upfront != 0;
        c.fn = f32 ? (f32_two ? g->prefill_f32_d64_w4 : g->prefill_f32_d64) : upfront ? g->prefill_bf16_d64_h1w : narrow ? g->prefill_bf16_d64_h1 : stream ? g->prefill_bf16_d64_stream : pair ? g->prefill_bf16_d64_pair : g->prefill_bf16_d64;
        c.name = f32 ? (f32_two ? "lng_prefill_f32_d64_w4" : "lng_prefill_f32_d64") : upfront ? "lng_prefill_bf16_d64_h1w" : narrow ? "lng_prefill_bf16_d64_h1" : stream ? "lng_prefill_bf16_d64_stream" : pair ? "lng_prefill_bf16_d64_pair" : "lng_prefill_bf16_d64";
        set_args(c, p);
        b->cmds.push_back(std::move(c));
        if (p.splits > 1) {
            Cmd m;
            m.fn = g->prefill_merge;
            m.name = "lng_prefill_merge";
            if (p.splits <= 8) {
                m.grid[0] = (unsigned)((s.t * s.heads + 15) / 16); // a thread per (row, head, four dims)
            } else {
                m.grid[1] = (unsigned)(s.t * s.kv_heads);          // a workgroup per (row, kv head)
            }
            m.block = 256;
            set_args(m, p);
            b->cmds.push_back(std::move(m));
        }
        b->dispatches += 1;
        return LNG_OK;
    }

    // Head widths 128, 256 and 512: the prompt-pass kernels that walk the head in slices of 64 dimensions, groups of
    // up to 16 query heads. A workgroup of four wavefronts takes 1, 2 or 4 heads of one kv head (as many as the
    // group has, up to four) and 4, 2 or 1 blocks of 32 query rows.
    const int wide = s.dim == 128 ? 0 : s.dim == 256 ? 1 : s.dim == 512 ? 2 : -1;
    if ((tiled || several_rows) && wide >= 0 && s.heads / s.kv_heads <= 16 && aligned16 && scale_positive && end <= 0x7fffffffull &&
        !g->knobs.wide_row_by_row && !g->knobs.wide_generic && (dtype == LNG_BF16 || !g->knobs.f32_generic)) {
        const bool f32 = dtype == LNG_F32;
        const uint64_t group = s.heads / s.kv_heads;
        const uint64_t hw = group >= 3 ? 4 : group, bm = 32 * (4 / hw), head_blocks = (group + hw - 1) / hw;
        lng_k_prefill p{};
        p.dtype = (uint32_t)dtype;
        p.q = (const char *)oq.buf->ptr + q.offset;
        p.k = (const char *)ok.buf->ptr + k.offset;
        p.v = (const char *)ov.buf->ptr + v.offset;
        p.out = (char *)oo.buf->ptr + out.offset;
        p.sinks = sinks ? (const float *)((const char *)os.buf->ptr + sinks->offset) : nullptr;
        p.t = s.t;
        p.start = s.start;
        p.window = s.window >= end ? LNG_WINDOW_FULL : s.window;
        p.slots = s.slots;
        p.heads = (uint32_t)s.heads;
        p.kv_heads = (uint32_t)s.kv_heads;
        p.dim = (uint32_t)s.dim;
        p.q_tiles = (uint32_t)((s.t + bm - 1) / bm);
        p.scale = s.scale;
        // Fewer workgroups than compute units: the key tiles of a query tile are split between up to eight
        // workgroups, merged by lng_prefill_merge; each keeps two tiles or more in bf16, where a tile is short
        // against what a workgroup pays to start and to write its partial rows, and one or more in f32, where a
        // tile is sixteen times the matrix work (77 rows of width 512 over 777 keys: 141 us in six splits, 112 in eight).
        p.splits = 1;
        const uint64_t visible = p.window == LNG_WINDOW_FULL ? end : std::min<uint64_t>(end, p.window + bm);
        const uint64_t key_tiles = (visible + 63) / 64;
        const uint64_t plain_wgs = (uint64_t)p.q_tiles * head_blocks * s.kv_heads;
        if (plain_wgs < g->cus) {
            uint64_t want = std::min<uint64_t>(std::min<uint64_t>(g->cus / plain_wgs, f32 ? key_tiles : key_tiles / 2), 8);
            if (g->knobs.prefill_splits > 0) want = std::min<uint64_t>(g->knobs.prefill_splits, 8);
            if (want > 1) p.splits = (uint32_t)want;
        }
        if ((uint64_t)plain_wgs * p.splits > 0x7fffffffull) return fail(LNG_ERR_DISPATCH, "%llu rows of %llu heads are more workgroups than one dispatch holds", (unsigned long long)s.t, (unsigned long long)s.heads);
        if (p.splits > 1) {
            const size_t slots = (size_t)s.t * s.heads * p.splits;
            Scratch sc;
            if (int rc = reserve_scratch(g, slots * s.dim, slots * 2, 0, &sc)) return rc;
            p.partial_o = sc.o;
            p.partial_ml = sc.ml;
        }
        static const char *const names_bf16[3] = {"lng_prefill_bf16_w128", "lng_prefill_bf16_w256", "lng_prefill_bf16_w512"};
        static const char *const names_f32[3] = {"lng_prefill_f32_w128", "lng_prefill_f32_w256", "lng_prefill_f32_w512"};
        Cmd c;
        c.grid[0] = (unsigned)(plain_wgs * p.splits); // kv head fastest: one XCD's L2 per kv head
        c.block = 256;
        c.fn = f32 ? g->prefill_f32_wide[wide] : g->prefill_bf16_wide[wide];
        c.name = f32 ? names_f32[wide] : names_bf16[wide];
        set_args(c, p);
        b->cmds.push_back(std::move(c));
        if (p.splits > 1) {
            Cmd m;
            m.fn = g->prefill_merge;
            m.name = "lng_prefill_merge";
            const uint64_t pairs_per_wg = 1024 / s.dim; // a thread per (row, head, four dims)
            m.grid[0] = (unsigned)((s.t * s.heads + pairs_per_wg - 1) / pairs_per_wg);
            m.block = 256;
            set_args(m, p);
            b->cmds.push_back(std::move(m));
        }
        b->dispatches += 1;
        return LNG_OK;
    }

    lng_k_attn a{};
    a.q = (const char *)oq.buf->ptr;
    a.k = (const char *)ok.buf->ptr;
    a.v = (const char *)ov.buf->ptr;
    a.out = (char *)oo.buf->ptr;
    a.sinks = sinks ? (const char *)os.buf->ptr : nullptr;
    a.rows = nullptr;
    a.first.q_offset = q.offset;
    a.first.out_offset = out.offset;
    a.first.k_offset = k.offset;
    a.first.v_offset = v.offset;
    a.first.sinks_offset = sinks ? sinks->offset : LNG_NO_SINKS;
    a.first.start = s.start;
    a.first.window = s.window;
    a.first.slots = s.slots;
    a.n_rows = (uint32_t)s.t;
    a.heads = (uint32_t)s.heads;
    a.kv_heads = (uint32_t)s.kv_heads;
    a.dim = (uint32_t)s.dim;
    a.chunk = 128;
    a.n_chunks = 1;
    a.dtype = (uint32_t)dtype;
    a.scale = s.scale;
    if (int rc = record_rows(b, a, &a.first, s.t, s.t, aligned16)) return rc;
    b->dispatches += 1;
    return LNG_OK;
}

} // namespace

// ================================== C ABI =====================================================

extern "C" const char *lng_hip_last_error(void) { return g_error.c_str(); }

extern "C" int lng_hip_open(int device, lng_gpu **out) {
    if (!out) return fail(LNG_ERR_DISPATCH, "no place for the gpu handle");
    *out = nullptr;
    int count = 0;
    if (hipInit(0) != hipSuccess || hipGetDeviceCount(&count) != hipSuccess || count <= 0) {
        (void)hipGetLastError();
        return fail(LNG_ERR_NO_DEVICE, "no HIP device");
    }
    if (device < 0 || device >= count) return fail(LNG_ERR_NO_DEVICE, "no HIP device %d (%d present)", device, count);
    if (hipSetDevice(device) != hipSuccess) return fail(LNG_ERR_NO_DEVICE, "cannot select HIP device %d", device);
    lng_gpu *g = new lng_gpu;
    g->device = device;
    hipDeviceProp_t prop;
    if (hipGetDeviceProperties(&prop, device) == hipSuccess) {
        g->name = prop.gcnArchName;
        g->cus = (unsigned)prop.multiProcessorCount;
    }
    // LNG_HSACO names a code object file to load instead of the embedded one (kernel development).
    hipError_t e;
    if (const char *path = getenv("LNG_HSACO")) {
        e = hipModuleLoad(&g->module, path);
    } else {
        e = hipModuleLoadData(&g->module, lng_hsaco_begin);
    }
    if (e != hipSuccess) {
        const int rc = fail(LNG_ERR_COMPILE, "the gfx950 code object does not load on %s: %s", g->name.c_str(), hip_text(e));
        delete g;
        return rc;
    }
    struct { const char *name; hipFunction_t *fn; bool required; } wanted[] = {
        {"lng_attn_generic_f32", &g->generic_f32, true},
        {"lng_attn_generic_bf16", &g->generic_bf16, true},
        {"lng_decode_bf16_d64", &g->decode_bf16_d64, true},
        {"lng_decode_bf16_d64_o4", &g->decode_bf16_d64_o4, true},
        {"lng_decode_merge", &g->decode_merge, true},
        {"lng_decode_merge_few", &g->decode_merge_few, true},
        {"lng_decode_f32_d64", &g->decode_f32_d64, true},
        {"lng_decode_bf16_w128", &g->decode_bf16_wide[0], true},
        {"lng_decode_bf16_w256", &g->decode_bf16_wide[1], true},
        {"lng_decode_bf16_w512", &g->decode_bf16_wide[2], true},
        {"lng_decode_f32_w128", &g->decode_f32_wide[0], true},
        {"lng_decode_f32_w256", &g->decode_f32_wide[1], true},
        {"lng_decode_f32_w512", &g->decode_f32_wide[2], true},
        {"lng_prefill_bf16_d64", &g->prefill_bf16_d64, true},
        {"lng_prefill_bf16_d64_h1", &g->prefill_bf16_d64_h1, true},
        {"lng_prefill_bf16_d64_h1w", &g->prefill_bf16_d64_h1w, true},
        {"lng_prefill_bf16_d64_stream", &g->prefill_bf16_d64_stream, true},
        {"lng_prefill_bf16_d64_pair", &g->prefill_bf16_d64_pair, true},
        {"lng_prefill_f32_d64", &g->prefill_f32_d64, true},
        {"lng_prefill_f32_d64_w4", &g->prefill_f32_d64_w4, true},
        {"lng_prefill_merge", &g->prefill_merge, true},
        {"lng_prefill_bf16_w128", &g->prefill_bf16_wide[0], true},
        {"lng_prefill_bf16_w256", &g->prefill_bf16_wide[1], true},
        {"lng_prefill_bf16_w512", &g->prefill_bf16_wide[2], true},
        {"lng_prefill_f32_w128", &g->prefill_f32_wide[0], true},
        {"lng_prefill_f32_w256", &g->prefill_f32_wide[1], true},
        {"lng_prefill_f32_w512", &g->prefill_f32_wide[2], true},
        {"lng_copy_rows", &g->copy_rows, true},
        {"lng_fill_synthetic", &g->fill_synthetic, true},
        {"lng_checksum", &g->checksum, true},
        {"lng_checksum_fold", &g->checksum_fold, true},
        {"lng_add_rows", &g->add_rows, true},
        {"lng_rotate_halves", &g->rotate_halves, true},
        {"lng_prepare_v4", &g->prepare_v4, true},
        {"lng_prepare_v1", &g->prepare_v1, true},
        {"lng_q8_split_x", &g->q8_split_x, true},
        {"lng_q8_stream", &g->q8_stream, true},
        {"lng_q8_stream_one", &g->q8_stream_one, true},
        {"lng_q8_stream_one_w8", &g->q8_stream_one_w8, true},
        {"lng_q8_tiled", &g->q8_tiled, true},
        {"lng_q8_tiled_bf16", &g->q8_tiled_bf16, true},
        {"lng_q8_stream_bf16", &g->q8_stream_bf16, true},
        {"lng_rmsnorm_rows", &g->rmsnorm_rows, true},
        {"lng_rmsnorm_row_wg", &g->rmsnorm_row_wg, true},
    };
    for (auto &w : wanted) {
        e = hipModuleGetFunction(w.fn, g->module, w.name);
        if (e != hipSuccess && w.required) {
            const int rc = fail(LNG_ERR_COMPILE, "kernel %s missing: %s", w.name, hip_text(e));
            hipModuleUnload(g->module);
            delete g;
            return rc;
        }
    }
    if (hipStreamCreateWithFlags(&g->stream, hipStreamNonBlocking) != hipSuccess) {
        hipModuleUnload(g->module);
        delete g;
        return fail(LNG_ERR_NO_DEVICE, "cannot create a stream");
    }
    // this device's copy of the fixed scratch array (for lng_hip_attention_grouped_static)
    if (const int rc = lng_static_scratch_setup(device)) {
        const int code = fail(LNG_ERR_COMPILE, "the fixed scratch array is not there on device %d: %s", device, hip_text((hipError_t)rc));
        hipStreamDestroy(g->stream);
        hipModuleUnload(g->module);
        delete g;
        return code;
    }
    g->static_scratch = (char *)lng_static_scratch(device);
    if (hipMalloc((void **)&g->second_passes, sizeof(uint32_t)) != hipSuccess || hipMemset(g->second_passes, 0, sizeof(uint32_t)) != hipSuccess) {
        const int code = fail(LNG_ERR_ALLOC, "could not allocate a 4-byte counter");
        if (g->second_passes) hipFree(g->second_passes);
        hipStreamDestroy(g->stream);
        hipModuleUnload(g->module);
        delete g;
        return code;
    }
    g->fuse_wgs = 4ull * g->cus;
    // the development switches, read once here
    for (const char *name : knob_names) {
        if (const char *value = getenv(name)) set_knob(g, name, value);
    }
    *out = g;
    return LNG_OK;
}

extern "C" int lng_hip_debug_set(lng_gpu *g, const char *name, const char *value) {
    if (!g || !name) return fail(LNG_ERR_DISPATCH, "no gpu or no name");
    std::lock_guard<std::mutex> lock(g->mu);
    if (!set_knob(g, name, value)) return fail(LNG_ERR_DISPATCH, "no development switch called %s", name);
    return LNG_OK;
}

namespace {
void destroy_gpu(lng_gpu *g) {
    hipSetDevice(g->device);
    for (Table &t : g->free_tables) {
        hipHostFree(t.host);
        if (!t.in_place) hipFree(t.dev);
    }
    for (void *p : g->retired) hipFree(p);
    for (hipEvent_t ev : g->spare_events) hipEventDestroy(ev);
    if (g->scratch_o) hipFree(g->scratch_o);
    if (g->scratch_ml) hipFree(g->scratch_ml);
    if (g->tickets) hipFree(g->tickets);
    if (g->scratch_x) hipFree(g->scratch_x);
    if (g->second_passes) hipFree(g->second_passes);
    hipStreamDestroy(g->stream);
    hipModuleUnload(g->module);
    delete g;
}

// A buffer, a batch or the open handle of `g` went away: whoever takes the count to zero takes the gpu with it.
// Nothing of `g` is read after the decrement, so the last two holders may let go on different threads.
void object_gone(lng_gpu *g) {
    if (g->live_buffers.fetch_sub(1, std::memory_order_acq_rel) == 1) destroy_gpu(g);
}
} // namespace

extern "C" int lng_hip_debug_get(lng_gpu *g, const char *name, uint64_t *value) {
    if (!g || !name || !value) return fail(LNG_ERR_DISPATCH, "no gpu, no name or no place for the value");
    if (strcmp(name, "LNG_COUNT_SECOND_PASSES") != 0) return fail(LNG_ERR_DISPATCH, "no development counter called %s", name);
    // waits for everything submitted so far, reads the counter and puts it back to zero
    hipSetDevice(g->device);
    uint32_t n = 0;
    hipError_t e = hipStreamSynchronize(g->stream);
    if (e == hipSuccess) e = hipMemcpy(&n, g->second_passes, sizeof n, hipMemcpyDeviceToHost);
    if (e == hipSuccess) e = hipMemset(g->second_passes, 0, sizeof n);
    if (e != hipSuccess) return fail(LNG_ERR_GPU, "could not read the counter: %s", hip_text(e));
    *value = n;
    return LNG_OK;
}

extern "C" void lng_hip_close(lng_gpu *g) {
    if (!g) return;
    hipSetDevice(g->device);
    if (g->worker.joinable()) {
        {
            std::lock_guard<std::mutex> lock(g->qmu);
            g->stopping = true;
        }
        g->qcv.notify_all();
        g->worker.join();
    }
    hipStreamSynchronize(g->stream);
    // Buffers, residents and batches keep the gpu alive, as the reference's own do (they borrow or share it): with
    // some still around, the handle stays valid for freeing and dropping them and goes with the last of them.
    object_gone(g); // the handle's own reference, held since lng_hip_open
}

extern "C" int lng_hip_device_name(lng_gpu *g, char *name, size_t cap) {
    if (!g || !name || cap == 0) return fail(LNG_ERR_DISPATCH, "no gpu or no room for the name");
    snprintf(name, cap, "%s", g->name.c_str());
    return LNG_OK;
}

extern "C" int lng_hip_buffer(lng_gpu *g, size_t len, lng_buffer **out) {
    if (!g || !out) return fail(LNG_ERR_DISPATCH, "no gpu");
    *out = nullptr;
    if (len == 0) return fail(LNG_ERR_ALLOC, "could not allocate a 0-byte buffer");
    hipSetDevice(g->device);
    void *p = nullptr;
    if (hipMalloc(&p, len) != hipSuccess) {
        (void)hipGetLastError();
        return fail(LNG_ERR_ALLOC, "could not allocate a %zu-byte buffer", len);
    }
    lng_buffer *b = new lng_buffer;
    b->gpu = g;
    b->ptr = p;
    b->len = len;
    g->live_buffers.fetch_add(1);
    *out = b;
    return LNG_OK;
}

extern "C" int lng_hip_resident(lng_gpu *g, const void *bytes, size_t len, lng_buffer **out) {
    if (!bytes && len) return fail(LNG_ERR_DISPATCH, "no bytes");
    if (int rc = lng_hip_buffer(g, len, out)) return rc;
    if (hipMemcpy((*out)->ptr, bytes, len, hipMemcpyHostToDevice) != hipSuccess) {
        lng_hip_buffer_free(*out);
        *out = nullptr;
        return fail(LNG_ERR_GPU, "could not fill a %zu-byte resident", len);
    }
    (*out)->resident = true;
    return LNG_OK;
}

extern "C" int lng_hip_buffer_free(lng_buffer *b) {
    if (!b) return LNG_OK;
    if (b->holds.load() != 0) return fail(LNG_ERR_DISPATCH, "the buffer belongs to a batch that has not finished");
    hipSetDevice(b->gpu->device);
    hipFree(b->ptr);
    lng_gpu *g = b->gpu;
    delete b;
    object_gone(g);
    return LNG_OK;
}

extern "C" size_t lng_hip_buffer_len(const lng_buffer *b) { return b ? b->len : 0; }

extern "C" void *lng_hip_buffer_device_ptr(lng_buffer *b) { return b ? b->ptr : nullptr; }

static int host_access(lng_buffer *b, size_t offset, size_t len, bool write) {
    if (!b) return fail(LNG_ERR_DISPATCH, "no buffer");
    if (write && b->resident) return fail(LNG_ERR_DISPATCH, "resident memory is read-only");
    if (!b->resident && b->holds.load() != 0) return fail(LNG_ERR_DISPATCH, "the buffer belongs to a batch that has not finished");
    if (offset > b->len || len > b->len - offset) return fail(LNG_ERR_DISPATCH, "bytes %zu..%zu outside a %zu-byte buffer", offset, offset + len, b->len);
    hipSetDevice(b->gpu->device);
    return LNG_OK;
}

extern "C" int lng_hip_upload(lng_buffer *b, size_t offset, const void *src, size_t len) {
    if (int rc = host_access(b, offset, len, true)) return rc;
    if (len == 0) return LNG_OK;
    const hipError_t e = hipMemcpy((char *)b->ptr + offset, src, len, hipMemcpyHostToDevice);
    return e == hipSuccess ? LNG_OK : fail(LNG_ERR_GPU, "upload failed: %s", hip_text(e));
}

extern "C" int lng_hip_download(lng_buffer *b, size_t offset, void *dst, size_t len) {
    if (int rc = host_access(b, offset, len, false)) return rc;
    if (len == 0) return LNG_OK;
    const hipError_t e = hipMemcpy(dst, (const char *)b->ptr + offset, len, hipMemcpyDeviceToHost);
    return e == hipSuccess ? LNG_OK : fail(LNG_ERR_GPU, "download failed: %s", hip_text(e));
}

extern "C" int lng_hip_fill(lng_buffer *b, size_t offset, int byte, size_t len) {
    if (int rc = host_access(b, offset, len, true)) return rc;
    if (len == 0) return LNG_OK;
    hipError_t e = hipMemset((char *)b->ptr + offset, byte, len);
    if (e == hipSuccess) e = hipDeviceSynchronize();
    return e == hipSuccess ? LNG_OK : fail(LNG_ERR_GPU, "fill failed: %s", hip_text(e));
}

extern "C" int lng_hip_batch(lng_gpu *g, lng_buffer *const *buffers, size_t n, lng_batch **out) {
    if (!g || !out || (n && !buffers)) return fail(LNG_ERR_DISPATCH, "no gpu or no buffers");
    *out = nullptr;
    for (size_t i = 0; i < n; ++i) {
        if (!buffers[i] || buffers[i]->gpu != g) return fail(LNG_ERR_DISPATCH, "buffer %zu is not of this gpu", i);
        if (buffers[i]->resident) return fail(LNG_ERR_DISPATCH, "buffer %zu is resident memory: attach it instead", i);
        for (size_t j = 0; j < i; ++j) {
            if (buffers[j] == buffers[i]) return fail(LNG_ERR_DISPATCH, "buffer %zu is given twice", i);
        }
    }
    // take ownership of all or none
    size_t taken = 0;
    for (; taken < n; ++taken) {
        int expected = 0;
        if (!buffers[taken]->holds.compare_exchange_strong(expected, 1)) break;
    }
    if (taken < n) {
        for (size_t i = 0; i < taken; ++i) buffers[i]->holds.store(0);
        return fail(LNG_ERR_DISPATCH, "buffer %zu belongs to a batch that has not finished", taken);
    }
    lng_batch *b = new lng_batch;
    b->gpu = g;
    b->buffers.assign(buffers, buffers + n);
    g->live_buffers.fetch_add(1);
    *out = b;
    return LNG_OK;
}

extern "C" int lng_hip_batch_attach(lng_batch *b, lng_buffer *resident, lng_slice *whole) {
    if (int rc = need_recording(b)) return rc;
    if (!resident || !whole) return fail(LNG_ERR_DISPATCH, "no resident");
    if (!resident->resident || resident->gpu != b->gpu) return fail(LNG_ERR_DISPATCH, "not a resident of this gpu");
    size_t index = 0;
    for (; index < b->residents.size(); ++index) {
        if (b->residents[index] == resident) break;
    }
    if (index == b->residents.size()) {
        resident->holds.fetch_add(1);
        b->residents.push_back(resident);
    }
    *whole = lng_slice{b->buffers.size() + index, 0, resident->len};
    return LNG_OK;
}

extern "C" size_t lng_hip_batch_dispatches(const lng_batch *b) { return b ? b->dispatches : 0; }

extern "C" int lng_hip_batch_barrier(lng_batch *b) { return need_recording(b); }

extern "C" int lng_hip_batch_commit(lng_batch *b, lng_on_done on_done, void *user) {
    if (int rc = need_recording(b)) return rc;
    lng_gpu *g = b->gpu;
    hipSetDevice(g->device);
    hipError_t e = take_event(g, &b->ev0);
    if (e == hipSuccess) e = take_event(g, &b->ev1);
    // The dispatches of one batch stay together on the stream: split-K partials, arrival counters and
    // the planes of a Q8_0 product live in scratch that the next dispatch of any batch reuses.
    std::unique_lock<std::mutex> submitting(g->submit_mu);
    if (e == hipSuccess) e = hipEventRecord(b->ev0, g->stream);
    // the row tables of every batched dispatch, one copy per table block, ahead of the kernels
    for (size_t i = 0; e == hipSuccess && i < b->tables.size(); ++i) {
        const Table &t = b->tables[i];
        if (t.used && !t.in_place) e = hipMemcpyAsync(t.dev, t.host, t.used, hipMemcpyHostToDevice, g->stream);
    }
    for (size_t i = 0; e == hipSuccess && i < b->cmds.size(); ++i) {
        Cmd &c = b->cmds[i];
        size_t size = c.args.size();
        void *config[] = {HIP_LAUNCH_PARAM_BUFFER_POINTER, c.args.data(), HIP_LAUNCH_PARAM_BUFFER_SIZE, &size,
                          HIP_LAUNCH_PARAM_END};
        e = hipModuleLaunchKernel(c.fn, c.grid[0], c.grid[1], c.grid[2], c.block, 1, 1, 0, g->stream, nullptr, config);
        if (e == hipSuccess && b->timing) {
            hipEvent_t mark = nullptr;
            e = take_event(g, &mark);
            if (e == hipSuccess) {
                b->marks.push_back(mark);
                e = hipEventRecord(mark, g->stream);
            }
        }
    }
    if (e == hipSuccess) e = hipEventRecord(b->ev1, g->stream);
    submitting.unlock();
    b->on_done = on_done;
    b->user = user;
    b->state = lng_batch::Committed;
    if (e != hipSuccess) {
        // What was submitted before the failure still runs; wait for it, then report.
        hipStreamSynchronize(g->stream);
        b->status = LNG_ERR_GPU;
        b->message = hip_text(e);
        release(b);
        b->state = lng_batch::Done;
        const std::string message = b->message; // on_done may drop the batch
        if (on_done) {
            lng_completed done{LNG_ERR_GPU, 0.0, message.c_str()};
            on_done(&done, user);
        }
        return fail(LNG_ERR_GPU, "submission failed: %s", message.c_str());
    }
    if (on_done) {
        std::lock_guard<std::mutex> lock(g->qmu);
        if (!g->worker.joinable()) g->worker = std::thread(worker_loop, g);
        g->queue.push_back(b);
        g->qcv.notify_one();
    }
    return LNG_OK;
}

extern "C" int lng_hip_batch_wait(lng_batch *b, double *gpu_seconds) {
    if (!b) return fail(LNG_ERR_DISPATCH, "no batch");
    if (b->state == lng_batch::Recording) return fail(LNG_ERR_DISPATCH, "the batch was not committed");
    if (b->on_done) { // the completion thread finishes it
        std::unique_lock<std::mutex> lock(b->mu);
        b->cv.wait(lock, [&] { return b->state == lng_batch::Done; });
    } else if (b->state != lng_batch::Done) {
        finish(b);
        b->state = lng_batch::Done;
    }
    if (gpu_seconds) *gpu_seconds = b->seconds;
    if (b->status != LNG_OK) return fail(b->status, "the batch failed on the GPU: %s", b->message.c_str());
    return LNG_OK;
}

extern "C" void lng_hip_batch_drop(lng_batch *b) {
    if (!b) return;
    if (b->state == lng_batch::Committed && b->on_done) {
        bool on_completion_thread;
        {
            std::lock_guard<std::mutex> lock(b->gpu->qmu); // commit starts the thread under this lock
            on_completion_thread = b->gpu->worker.get_id() == std::this_thread::get_id();
        }
        if (on_completion_thread) { // inside its own on_done: freed when the callback returns
            b->drop_when_done = true;
            return;
        }
    }
    if (b->state == lng_batch::Recording) {
        release(b);
    } else {
        lng_hip_batch_wait(b, nullptr);
    }
    destroy(b);
}

extern "C" int lng_hip_batch_set_timing(lng_batch *b, int enabled) {
    if (int rc = need_recording(b)) return rc;
    b->timing = enabled != 0;
    return LNG_OK;
}

extern "C" int lng_hip_batch_kernel_seconds(lng_batch *b, const char *kernel, double *seconds, size_t *launches) {
    if (!b || !kernel) return fail(LNG_ERR_DISPATCH, "no batch or no kernel name");
    if (b->state != lng_batch::Done) return fail(LNG_ERR_DISPATCH, "the batch has not finished");
    if (!b->timing) return fail(LNG_ERR_DISPATCH, "the batch was not committed with timing on");
    double total = 0.0;
    size_t n = 0;
    for (size_t i = 0; i < b->cmds.size() && i < b->cmd_seconds.size(); ++i) {
        if (strcmp(b->cmds[i].name, kernel) == 0) {
            total += b->cmd_seconds[i];
            n += 1;
        }
    }
    if (seconds) *seconds = total;
    if (launches) *launches = n;
    return LNG_OK;
}

extern "C" int lng_hip_check_grouped(const lng_grouped_shape *shape, int tiled) {
    if (!shape) return fail(LNG_ERR_DISPATCH, "no shape");
    return check_shape(*shape, tiled != 0);
}

extern "C" int lng_hip_attention_grouped(lng_batch *b, lng_slice q, lng_slice k, lng_slice v, lng_slice out,
                                         const lng_slice *sinks, const lng_grouped_shape *shape, int dtype) {
    return attention(b, q, k, v, out, sinks, shape, dtype, false);
}

extern "C" int lng_hip_attention_grouped_tiled(lng_batch *b, lng_slice q, lng_slice k, lng_slice v, lng_slice out,
                                               const lng_slice *sinks, const lng_grouped_shape *shape, int dtype) {
    return attention(b, q, k, v, out, sinks, shape, dtype, true);
}

// The plain operator on raw device pointers, launched at once on the caller's stream, with its split-K
// partials in the fixed scratch array: no hipMalloc, no hipFree, no pinned tables, no host heap.
extern "C" int lng_hip_attention_grouped_static(lng_gpu *g, void *stream, const void *q, const void *k, const void *v,
                                                void *out, const float *sinks, const lng_grouped_shape *shape,
                                                int dtype) {
    if (!g) return fail(LNG_ERR_DISPATCH, "no gpu");
    if (!shape) return fail(LNG_ERR_DISPATCH, "no shape");
    if (dtype != LNG_F32 && dtype != LNG_BF16) return fail(LNG_ERR_DISPATCH, "unknown element type %d", dtype);
    if (!q || !k || !v || !out) return fail(LNG_ERR_DISPATCH, "q, k, v and out must be device addresses");
    const lng_grouped_shape &s = *shape;
    if (int rc = check_shape(s, false)) return rc;
    const uint64_t width = std::max<uint64_t>(1, (s.dim + 63) / 64); // partial outputs take `dim` floats per slot
    if (s.t * s.heads * width > LNG_STATIC_MAX_ROW_HEADS) {
        return fail(LNG_ERR_DISPATCH, "%llu rows of %llu heads of width %llu: the fixed scratch array is sized for rows x heads x ceil(dim / 64) <= %u",
                    (unsigned long long)s.t, (unsigned long long)s.heads, (unsigned long long)s.dim, (unsigned)LNG_STATIC_MAX_ROW_HEADS);
    }
    const uint64_t es = elem_size(dtype);
    if (!fits_u32(s.heads * s.dim * es)) return fail(LNG_ERR_DISPATCH, "rows of %llu bytes do not fit in u32", (unsigned long long)(s.heads * s.dim * es));
    const uint64_t end = s.start + s.t;
    const uint64_t q_bytes = s.t * s.heads * s.dim * es, kv_bytes = std::min(s.slots, end) * s.kv_heads * s.dim * es;
    const uintptr_t pq = (uintptr_t)q, pk = (uintptr_t)k, pv = (uintptr_t)v, po = (uintptr_t)out;
    if ((pq | pk | pv | po) % es != 0 || (uintptr_t)sinks % 4 != 0) return fail(LNG_ERR_DISPATCH, "an operand is not aligned to its element size");
    // apple.rs:896-906: the output may not overlap an input
    auto apart = [&](uintptr_t x, uint64_t n) { return po + q_bytes <= x || x + n <= po; };
    if (!apart(pq, q_bytes) || !apart(pk, kv_bytes) || !apart(pv, kv_bytes) || (sinks && !apart((uintptr_t)sinks, s.heads * 4))) {
        return fail(LNG_ERR_DISPATCH, "output overlaps an input");
    }
    lng_k_attn a{};
    a.q = (const char *)q;
    a.k = (const char *)k;
    a.v = (const char *)v;
    a.out = (char *)out;
    a.sinks = (const char *)sinks;
    a.rows = nullptr;
    a.first.sinks_offset = sinks ? 0 : LNG_NO_SINKS;
    a.first.start = s.start;
    a.first.window = s.window;
    a.first.slots = s.slots;
    a.n_rows = (uint32_t)s.t;
    a.heads = (uint32_t)s.heads;
    a.kv_heads = (uint32_t)s.kv_heads;
    a.dim = (uint32_t)s.dim;
    a.chunk = 128;
    a.n_chunks = 1;
    a.dtype = (uint32_t)dtype;
    a.scale = s.scale;
    const bool aligned16 = ((pq | pk | pv | po) & 15u) == 0;
    RowsPlan p = plan_rows(g, a, &a.first, s.t, s.t, aligned16);
    p.fused = false; // lng_decode_merge as the second launch: no arrival counters, nothing that must start at zero
    if (p.partial_slots * (s.dim / 64) > LNG_STATIC_MAX_SLOTS) { // only a planner told to make more workgroups than usual gets here
        return fail(LNG_ERR_DISPATCH,
                    "%llu rows of %llu heads in %u chunks need %zu slots of split-K scratch; the fixed array holds %u (%zu bytes)",
                    (unsigned long long)s.t, (unsigned long long)s.heads, p.chunks.n_chunks, p.partial_slots * (size_t)(s.dim / 64),
                    (unsigned)LNG_STATIC_MAX_SLOTS, (size_t)LNG_STATIC_SCRATCH_BYTES);
    }
    if (p.partial_slots) {
        if (!g->static_scratch) return fail(LNG_ERR_COMPILE, "the fixed scratch array was not set up");
        a.partial_o = (float *)g->static_scratch;
        a.partial_ml = (float *)(g->static_scratch + LNG_STATIC_O_BYTES);
        a.tickets = nullptr;
    }
    RowsLaunches launches;
    if (int rc = rows_launches(g, a, p, &a.first, s.t, nullptr, nullptr, &launches)) return rc;
    // The calling thread's current device is the caller's business (it made `stream` on one): it is put back.
    int before = g->device;
    if (hipGetDevice(&before) != hipSuccess) before = g->device;
    if (before != g->device && hipSetDevice(g->device) != hipSuccess) return fail(LNG_ERR_NO_DEVICE, "cannot select HIP device %d", g->device);
    int rc = LNG_OK;
    for (int i = 0; i < launches.n && rc == LNG_OK; ++i) {
        size_t size = sizeof(lng_k_attn);
        void *config[] = {HIP_LAUNCH_PARAM_BUFFER_POINTER, &launches.l[i].args, HIP_LAUNCH_PARAM_BUFFER_SIZE, &size,
                          HIP_LAUNCH_PARAM_END};
        const hipError_t e = hipModuleLaunchKernel(launches.l[i].fn, launches.l[i].grid, 1, 1, 256, 1, 1, 0, (hipStream_t)stream, nullptr, config);
        if (e != hipSuccess) rc = fail(LNG_ERR_GPU, "%s did not launch: %s", launches.l[i].name, hip_text(e));
    }
    if (before != g->device) hipSetDevice(before);
    return rc;
}

extern "C" int lng_hip_copy_rows(lng_batch *b, lng_slice src, uint64_t src_stride, int src_dtype, lng_slice dst,
                                 uint64_t dst_stride, int dst_dtype, uint64_t rows, uint64_t width) {
    if (int rc = need_recording(b)) return rc;
    for (int d : {src_dtype, dst_dtype}) {
        if (d != LNG_F32 && d != LNG_BF16) return fail(LNG_ERR_DISPATCH, "unknown element type %d", d);
    }
    // apple.rs:1769-1781
    if (rows == 0 || width == 0 || src_stride < width || dst_stride < width) {
        return fail(LNG_ERR_DISPATCH, "unsupported copy: %llu x %llu, strides %llu and %llu", (unsigned long long)rows,
                    (unsigned long long)width, (unsigned long long)src_stride, (unsigned long long)dst_stride);
    }
    for (uint64_t n : {rows, width, src_stride, dst_stride}) {
        if (!fits_u32(n)) return fail(LNG_ERR_DISPATCH, "%llu does not fit in u32", (unsigned long long)n);
    }
    if (!fits_u32(rows * std::max(src_stride, dst_stride))) {
        return fail(LNG_ERR_DISPATCH, "%llu does not fit in u32", (unsigned long long)(rows * std::max(src_stride, dst_stride)));
    }
    const uint64_t ss = elem_size(src_dtype), ds = elem_size(dst_dtype);
    Operand os, od;
    if (int rc = check_slice(b, "src", src, ((rows - 1) * src_stride + width) * ss, ss, &os)) return rc;
    if (int rc = check_slice(b, "dst", dst, ((rows - 1) * dst_stride + width) * ds, ds, &od)) return rc;
    if (int rc = check_output(b, od, {&os})) return rc;
    lng_k_copy a{};
    a.src = (const char *)os.buf->ptr + src.offset;
    a.dst = (char *)od.buf->ptr + dst.offset;
    a.rows = rows;
    a.width = width;
    a.src_stride = src_stride;
    a.dst_stride = dst_stride;
    a.src_dtype = (uint32_t)src_dtype;
    a.dst_dtype = (uint32_t)dst_dtype;
    Cmd c;
    c.fn = b->gpu->copy_rows;
    c.name = "lng_copy_rows";
    c.grid[0] = (unsigned)((rows * width + 255) / 256);
    c.block = 256;
    set_args(c, a);
    b->cmds.push_back(std::move(c));
    b->dispatches += 1;
    return LNG_OK;
}

extern "C" int lng_hip_attention_decode_batched(lng_batch *b, uint64_t q_buffer, uint64_t k_buffer, uint64_t v_buffer,
                                                uint64_t out_buffer, uint64_t sinks_buffer, const lng_decode_item *items,
                                                size_t n_items, uint64_t heads, uint64_t kv_heads, uint64_t dim,
                                                float scale, int dtype) {
    if (int rc = need_recording(b)) return rc;
    if (dtype != LNG_F32 && dtype != LNG_BF16) return fail(LNG_ERR_DISPATCH, "unknown element type %d", dtype);
    if (!items || n_items == 0) return fail(LNG_ERR_DISPATCH, "no items");
    if (!fits_u32(n_items) || !fits_u32(n_items * heads)) return fail(LNG_ERR_DISPATCH, "%zu items do not fit in u32", n_items);
    lng_buffer *bq = buffer_at(b, q_buffer), *bk = buffer_at(b, k_buffer), *bv = buffer_at(b, v_buffer),
               *bo = buffer_at(b, out_buffer);
    if (!bq || !bk || !bv || !bo) return fail(LNG_ERR_DISPATCH, "no such buffer (batch has %zu)", b->buffers.size() + b->residents.size());
    if (out_buffer >= b->buffers.size()) return fail(LNG_ERR_DISPATCH, "output is in read-only resident memory");
    const uint64_t es = elem_size(dtype);
    if (!fits_u32(heads) || !fits_u32(heads * dim * es)) return fail(LNG_ERR_DISPATCH, "rows of %llu x %llu elements do not fit in u32", (unsigned long long)heads, (unsigned long long)dim);
    bool any_sinks = false, aligned16 = true;
    for (size_t i = 0; i < n_items; ++i) {
        const lng_decode_item &it = items[i];
        // every item is the reference's plain dispatch with t = 1
        lng_grouped_shape s{1, it.start, heads, kv_heads, dim, it.window, it.slots, scale};
        if (int rc = check_shape(s, false)) return fail(rc, "item %zu: %s", i, std::string(g_error).c_str());
        const uint64_t rows = std::min(it.slots, it.start + 1);
        const lng_slice sq{q_buffer, it.q_offset, heads * dim * es}, sk{k_buffer, it.k_offset, rows * kv_heads * dim * es},
            sv{v_buffer, it.v_offset, rows * kv_heads * dim * es}, so{out_buffer, it.out_offset, heads * dim * es};
        Operand oq, ok, ov, oo;
        if (int rc = check_slice(b, "q", sq, sq.len, es, &oq)) return fail(rc, "item %zu: %s", i, std::string(g_error).c_str());
        if (int rc = check_slice(b, "k", sk, sk.len, es, &ok)) return fail(rc, "item %zu: %s", i, std::string(g_error).c_str());
        if (int rc = check_slice(b, "v", sv, sv.len, es, &ov)) return fail(rc, "item %zu: %s", i, std::string(g_error).c_str());
        if (int rc = check_slice(b, "out", so, so.len, es, &oo)) return fail(rc, "item %zu: %s", i, std::string(g_error).c_str());
        if (int rc = check_output(b, oo, {&oq, &ok, &ov})) return fail(rc, "item %zu: %s", i, std::string(g_error).c_str());
        if (it.sinks_offset != LNG_NO_SINKS) {
            Operand os;
            const lng_slice ss{sinks_buffer, it.sinks_offset, heads * 4};
            if (int rc = check_slice(b, "sinks", ss, ss.len, 4, &os)) return fail(rc, "item %zu: %s", i, std::string(g_error).c_str());
            any_sinks = true;
        }
        aligned16 = aligned16 && ((it.q_offset | it.k_offset | it.v_offset | it.out_offset) & 15u) == 0;
    }
    // outputs of different items must not overlap each other
    {
        std::vector<std::pair<uint64_t, uint64_t>> spans(n_items);
        for (size_t i = 0; i < n_items; ++i) spans[i] = {items[i].out_offset, items[i].out_offset + heads * dim * es};
        std::sort(spans.begin(), spans.end());
        for (size_t i = 1; i < n_items; ++i) {
            if (spans[i].first < spans[i - 1].second) return fail(LNG_ERR_DISPATCH, "outputs of two items overlap");
        }
    }
    char *host = nullptr, *dev = nullptr;
    if (int rc = reserve_table(b, n_items * sizeof(lng_k_row), &host, &dev)) return rc;
    memcpy(host, items, n_items * sizeof(lng_k_row));
    lng_k_attn a{};
    a.q = (const char *)bq->ptr;
    a.k = (const char *)bk->ptr;
    a.v = (const char *)bv->ptr;
    a.out = (char *)bo->ptr;
    a.sinks = any_sinks ? (const char *)buffer_at(b, sinks_buffer)->ptr : nullptr;
    a.rows = (const lng_k_row *)dev;
    a.n_rows = (uint32_t)n_items;
    a.heads = (uint32_t)heads;
    a.kv_heads = (uint32_t)kv_heads;
    a.dim = (uint32_t)dim;
    a.chunk = 128;
    a.n_chunks = 1;
    a.dtype = (uint32_t)dtype;
    a.scale = scale;
    if (int rc = record_rows(b, a, (const lng_k_row *)host, n_items, 0, aligned16)) return rc;
    b->dispatches += 1;
    return LNG_OK;
}

extern "C" int lng_hip_rmsnorm_rows(lng_batch *b, lng_slice v, lng_slice w, uint64_t rows, uint64_t d, uint64_t stride,
                                    float eps) {
    if (int rc = need_recording(b)) return rc;
    // apple.rs:1740-1744
    if (rows == 0 || d == 0 || stride < d) {
        return fail(LNG_ERR_DISPATCH, "unsupported rows: %llu x %llu, stride %llu", (unsigned long long)rows,
                    (unsigned long long)d, (unsigned long long)stride);
    }
    for (uint64_t n : {rows, d, stride}) {
        if (!fits_u32(n)) return fail(LNG_ERR_DISPATCH, "%llu does not fit in u32", (unsigned long long)n);
    }
    if (!fits_u32(rows * stride)) return fail(LNG_ERR_DISPATCH, "%llu does not fit in u32", (unsigned long long)(rows * stride));
    Operand ov, ow;
    if (int rc = check_slice(b, "v", v, ((rows - 1) * stride + d) * 4, 4, &ov)) return rc;
    if (int rc = check_slice(b, "w", w, d * 4, 4, &ow)) return rc;
    if (int rc = check_output(b, ov, {&ow})) return rc;
    lng_k_rmsnorm a{};
    a.v = (float *)((char *)ov.buf->ptr + v.offset);
    a.w = (const float *)((const char *)ow.buf->ptr + w.offset);
    a.rows = (uint32_t)rows;
    a.d = (uint32_t)d;
    a.stride = (uint32_t)stride;
    a.eps = eps;
    Cmd c;
    const bool wide = d > 256 && d <= 4096; // a workgroup per row, elements held in registers; else a wavefront per row
    c.fn = wide ? b->gpu->rmsnorm_row_wg : b->gpu->rmsnorm_rows;
    c.name = wide ? "lng_rmsnorm_row_wg" : "lng_rmsnorm_rows";
    c.grid[0] = wide ? (unsigned)rows : (unsigned)((rows + 3) / 4);
    c.block = 256;
    set_args(c, a);
    b->cmds.push_back(std::move(c));
    b->dispatches += 1;
    return LNG_OK;
}

extern "C" int lng_hip_add_rows(lng_batch *b, lng_slice dst, lng_slice src, uint64_t src_stride, uint64_t rows,
                                uint64_t width) {
    if (int rc = need_recording(b)) return rc;
    // apple.rs:1893-1897
    if (rows == 0 || width == 0 || (src_stride != 0 && src_stride < width)) {
        return fail(LNG_ERR_DISPATCH, "unsupported add: %llu x %llu, source stride %llu", (unsigned long long)rows,
                    (unsigned long long)width, (unsigned long long)src_stride);
    }
    for (uint64_t n : {rows, width, src_stride}) {
        if (!fits_u32(n)) return fail(LNG_ERR_DISPATCH, "%llu does not fit in u32", (unsigned long long)n);
    }
    if (!fits_u32(rows * width)) return fail(LNG_ERR_DISPATCH, "%llu does not fit in u32", (unsigned long long)(rows * width));
    Operand od, os;
    if (int rc = check_slice(b, "dst", dst, rows * width * 4, 4, &od)) return rc;
    if (int rc = check_slice(b, "src", src, ((rows - 1) * src_stride + width) * 4, 4, &os)) return rc;
    if (int rc = check_output(b, od, {&os})) return rc;
    lng_k_add a{};
    a.dst = (float *)((char *)od.buf->ptr + dst.offset);
    a.src = (const float *)((const char *)os.buf->ptr + src.offset);
    a.rows = rows;
    a.width = width;
    a.src_stride = src_stride;
    Cmd c;
    c.fn = b->gpu->add_rows;
    c.name = "lng_add_rows";
    c.grid[0] = (unsigned)((rows * width + 255) / 256);
    c.block = 256;
    set_args(c, a);
    b->cmds.push_back(std::move(c));
    b->dispatches += 1;
    return LNG_OK;
}

extern "C" int lng_hip_rotate_halves(lng_batch *b, lng_slice x, lng_slice table, uint64_t rows, uint64_t heads,
                                     uint64_t dim, uint64_t rotary) {
    if (int rc = need_recording(b)) return rc;
    // apple.rs:1936-1940
    if (rows == 0 || heads == 0 || rotary == 0 || rotary > dim || rotary % 2 != 0) {
        return fail(LNG_ERR_DISPATCH, "unsupported rotation: %llu rows of %llu x %llu, %llu rotated",
                    (unsigned long long)rows, (unsigned long long)heads, (unsigned long long)dim,
                    (unsigned long long)rotary);
    }
    for (uint64_t n : {rows, heads, dim, rotary}) {
        if (!fits_u32(n)) return fail(LNG_ERR_DISPATCH, "%llu does not fit in u32", (unsigned long long)n);
    }
    if (!fits_u32(rows * heads) || !fits_u32(rows * heads * dim)) {
        return fail(LNG_ERR_DISPATCH, "%llu rows of %llu x %llu do not fit in u32", (unsigned long long)rows,
                    (unsigned long long)heads, (unsigned long long)dim);
    }
    Operand ox, ot;
    if (int rc = check_slice(b, "x", x, rows * heads * dim * 4, 4, &ox)) return rc;
    if (int rc = check_slice(b, "table", table, rows * rotary * 4, 8, &ot)) return rc;
    if (int rc = check_output(b, ox, {&ot})) return rc;
    lng_k_rotate a{};
    a.x = (float *)((char *)ox.buf->ptr + x.offset);
    a.table = (const float *)((const char *)ot.buf->ptr + table.offset);
    a.rows = rows;
    a.heads = (uint32_t)heads;
    a.dim = (uint32_t)dim;
    a.rotary = (uint32_t)rotary;
    Cmd c;
    c.fn = b->gpu->rotate_halves;
    c.name = "lng_rotate_halves";
    c.grid[0] = (unsigned)((rows * heads * (rotary / 2) + 255) / 256);
    c.block = 256;
    set_args(c, a);
    b->cmds.push_back(std::move(c));
    b->dispatches += 1;
    return LNG_OK;
}

namespace {
struct Span {
    uint64_t buffer, lo, hi;
    bool operator<(const Span &o) const { return buffer != o.buffer ? buffer < o.buffer : lo < o.lo; }
};
// True when two spans of one buffer share a byte (sorts `spans`).
bool any_overlap(std::vector<Span> &spans) {
    std::sort(spans.begin(), spans.end());
    for (size_t i = 1; i < spans.size(); ++i) {
        if (spans[i].buffer == spans[i - 1].buffer && spans[i].lo < spans[i - 1].hi) return true;
    }
    return false;
}
} // namespace

extern "C" int lng_hip_prepare_attention(lng_batch *b, const lng_prepare_buffers *pb, const lng_prepare_item *items,
                                         size_t n_items, uint64_t heads, uint64_t kv_heads, uint64_t dim,
                                         uint64_t rotary, int out_dtype) {
    if (int rc = need_recording(b)) return rc;
    if (out_dtype != LNG_F32 && out_dtype != LNG_BF16) return fail(LNG_ERR_DISPATCH, "unknown element type %d", out_dtype);
    if (!pb || !items || n_items == 0) return fail(LNG_ERR_DISPATCH, "no items");
    if (n_items > 65535) return fail(LNG_ERR_DISPATCH, "%zu items are more than one dispatch takes (65535)", n_items);
    if (heads == 0 || kv_heads == 0 || dim == 0 || rotary == 0 || rotary > dim || rotary % 2 != 0) {
        return fail(LNG_ERR_DISPATCH, "unsupported preparation: %llu + %llu heads of %llu, %llu rotated",
                    (unsigned long long)heads, (unsigned long long)kv_heads, (unsigned long long)dim,
                    (unsigned long long)rotary);
    }
    for (uint64_t n : {heads, kv_heads, dim, (uint64_t)n_items}) {
        if (!fits_u32(n)) return fail(LNG_ERR_DISPATCH, "%llu does not fit in u32", (unsigned long long)n);
    }
    if (!fits_u32((heads + 2 * kv_heads) * dim)) return fail(LNG_ERR_DISPATCH, "rows of %llu elements do not fit in u32", (unsigned long long)((heads + 2 * kv_heads) * dim));
    const uint64_t es = elem_size(out_dtype), qw = heads * dim, kw = kv_heads * dim, half = rotary / 2;
    for (uint64_t out : {pb->q_out, pb->k_cache, pb->v_cache}) {
        if (!buffer_at(b, out)) return fail(LNG_ERR_DISPATCH, "no buffer %llu (batch has %zu)", (unsigned long long)out, b->buffers.size() + b->residents.size());
        if (out >= b->buffers.size()) return fail(LNG_ERR_DISPATCH, "output is in read-only resident memory");
    }
    Operand oqb{}, okb{}, ovb{};
    if (pb->q_bias) if (int rc = check_slice(b, "q_bias", *pb->q_bias, qw * 4, 4, &oqb)) return rc;
    if (pb->k_bias) if (int rc = check_slice(b, "k_bias", *pb->k_bias, kw * 4, 4, &okb)) return rc;
    if (pb->v_bias) if (int rc = check_slice(b, "v_bias", *pb->v_bias, kw * 4, 4, &ovb)) return rc;
    std::vector<Span> outs, ins;
    uint64_t most = 0;
    uint64_t align = 0;
    for (const Operand *o : {&oqb, &okb, &ovb}) {
        if (o->buf) {
            ins.push_back(Span{o->index, o->offset, o->offset + o->len});
            align |= o->offset;
        }
    }
    for (size_t i = 0; i < n_items; ++i) {
        const lng_prepare_item &it = items[i];
        if (it.n == 0 || it.slots == 0 || it.n > it.slots || it.start + it.n < it.start) {
            return fail(LNG_ERR_DISPATCH, "item %zu: unsupported preparation of %llu rows from %llu into %llu slots", i,
                        (unsigned long long)it.n, (unsigned long long)it.start, (unsigned long long)it.slots);
        }
        if (!fits_u32(it.n) || !fits_u32(it.slots)) return fail(LNG_ERR_DISPATCH, "item %zu: %llu does not fit in u32", i, (unsigned long long)std::max(it.n, it.slots));
        struct { const char *what; uint64_t buffer, offset, len, align; bool out; } parts[] = {
            {"q", pb->q, it.q_offset, it.n * qw * 4, 4, false},
            {"k", pb->k, it.k_offset, it.n * kw * 4, 4, false},
            {"v", pb->v, it.v_offset, it.n * kw * 4, 4, false},
            {"table", pb->table, it.table_offset, it.n * rotary * 4, 8, false},
            {"q_out", pb->q_out, it.q_out_offset, it.n * qw * es, es, true},
            {"k_cache", pb->k_cache, it.k_cache_offset, it.slots * kw * es, es, true},
            {"v_cache", pb->v_cache, it.v_cache_offset, it.slots * kw * es, es, true},
        };
        for (const auto &p : parts) {
            Operand o;
            const lng_slice sl{p.buffer, p.offset, p.len};
            if (int rc = check_slice(b, p.what, sl, p.len, p.align, &o)) return fail(rc, "item %zu: %s", i, std::string(g_error).c_str());
            (p.out ? outs : ins).push_back(Span{p.buffer, p.offset, p.offset + p.len});
            align |= p.offset;
        }
        most = std::max(most, it.n);
    }
    // An output may share bytes neither with another output nor with an input.
    if (any_overlap(outs)) return fail(LNG_ERR_DISPATCH, "outputs of the preparation overlap");
    {
        std::sort(ins.begin(), ins.end());
        for (const Span &o : outs) {
            // inputs are sorted by (buffer, lo) but may overlap one another: scan this buffer's run
            auto at = std::lower_bound(ins.begin(), ins.end(), Span{o.buffer, 0, 0});
            for (; at != ins.end() && at->buffer == o.buffer && at->lo < o.hi; ++at) {
                if (at->hi > o.lo) return fail(LNG_ERR_DISPATCH, "output overlaps an input");
            }
        }
    }
    const bool vec4 = half % 4 == 0 && (dim - rotary) % 4 == 0 && (align & 15u) == 0;
    const uint64_t w = vec4 ? 4 : 1;
    const uint64_t units = (heads + kv_heads) * (half / w + (dim - rotary) / w) + kw / w;
    if (!fits_u32(most * units + 256)) return fail(LNG_ERR_DISPATCH, "%llu rows do not fit in one dispatch", (unsigned long long)most);
    lng_k_prepare a{};
    a.q = (const char *)buffer_at(b, pb->q)->ptr;
    a.k = (const char *)buffer_at(b, pb->k)->ptr;
    a.v = (const char *)buffer_at(b, pb->v)->ptr;
    a.q_bias = oqb.buf ? (const float *)((const char *)oqb.buf->ptr + oqb.offset) : nullptr;
    a.k_bias = okb.buf ? (const float *)((const char *)okb.buf->ptr + okb.offset) : nullptr;
    a.v_bias = ovb.buf ? (const float *)((const char *)ovb.buf->ptr + ovb.offset) : nullptr;
    a.table = (const char *)buffer_at(b, pb->table)->ptr;
    a.q_out = (char *)buffer_at(b, pb->q_out)->ptr;
    a.k_cache = (char *)buffer_at(b, pb->k_cache)->ptr;
    a.v_cache = (char *)buffer_at(b, pb->v_cache)->ptr;
    if (n_items == 1) {
        a.items = nullptr;
        a.first = items[0];
    } else {
        char *host = nullptr, *dev = nullptr;
        if (int rc = reserve_table(b, n_items * sizeof(lng_prepare_item), &host, &dev)) return rc;
        memcpy(host, items, n_items * sizeof(lng_prepare_item));
        a.items = (const lng_prepare_item *)dev;
    }
    a.n_items = (uint32_t)n_items;
    a.heads = (uint32_t)heads;
    a.kv_heads = (uint32_t)kv_heads;
    a.dim = (uint32_t)dim;
    a.rotary = (uint32_t)rotary;
    a.out_dtype = (uint32_t)out_dtype;
    a.units_per_row = (uint32_t)units;
    a.vec = (uint32_t)w;
    Cmd c;
    c.fn = vec4 ? b->gpu->prepare_v4 : b->gpu->prepare_v1;
    c.name = vec4 ? "lng_prepare_v4" : "lng_prepare_v1";
    c.grid[0] = (unsigned)((most * units + 255) / 256);
    c.grid[1] = (unsigned)n_items;
    c.block = 256;
    set_args(c, a);
    b->cmds.push_back(std::move(c));
    b->dispatches += 1;
    return LNG_OK;
}

namespace {

// Device scratch for the two bf16 planes of x, shared by every Q8_0 product of the gpu (they run
// in order on one stream, each split immediately before its product).
int reserve_x(lng_gpu *g, size_t bytes, char **out) {
    std::lock_guard<std::mutex> lock(g->mu);
    if (bytes > g->scratch_x_len) {
        void *p = nullptr;
        const size_t want = std::max(bytes, g->scratch_x_len * 2);
        if (hipMalloc(&p, want) != hipSuccess) return fail(LNG_ERR_ALLOC, "could not allocate a %zu-byte scratch buffer", want);
        if (g->scratch_x) g->retired.push_back(g->scratch_x);
        g->scratch_x = (char *)p;
        g->scratch_x_len = want;
    }
    *out = g->scratch_x;
    return LNG_OK;
}

// The Q8_0 products share their checks (apple.rs:1792-1883) and their kernels.
// x_bf16: the positions are bf16 (exact as one operand plane: no split, one matrix instruction per block).
struct Q8Checked {
    lng_k_q8 a{};
    Operand codes{}, scales{}, x{}, y{};
};

int q8_check(lng_batch *b, const lng_slice &codes, const lng_slice &scales, const lng_slice &x, const lng_slice &y,
             uint64_t rows, uint64_t cols, uint64_t n, uint64_t x_stride, uint64_t y_stride, bool gemm, bool tiled,
             bool x_bf16, Q8Checked *out) {
    if (int rc = need_recording(b)) return rc;
    if (tiled && (rows % 64 != 0 || cols % 32 != 0 || n % 32 != 0)) { // apple.rs:1868-1872
        return fail(LNG_ERR_DISPATCH, "tiled Q8_0 product needs rows %% 64, cols %% 32 and n %% 32 == 0: %llu x %llu, n %llu",
                    (unsigned long long)rows, (unsigned long long)cols, (unsigned long long)n);
    }
    if (rows == 0 || cols == 0 || !fits_u32(rows) || !fits_u32(cols)) { // apple.rs:889-894
        return fail(LNG_ERR_DISPATCH, "unsupported shape %llux%llu", (unsigned long long)rows, (unsigned long long)cols);
    }
    if (gemm && (n == 0 || x_stride < cols || y_stride < rows || x_stride % (x_bf16 ? 8 : 4) != 0)) { // apple.rs:995-999 (16-byte rows)
        return fail(LNG_ERR_DISPATCH, "%llu positions of %llux%llu with strides %llu/%llu", (unsigned long long)n,
                    (unsigned long long)rows, (unsigned long long)cols, (unsigned long long)x_stride,
                    (unsigned long long)y_stride);
    }
    for (uint64_t v : {n, x_stride, y_stride}) {
        if (!fits_u32(v)) return fail(LNG_ERR_DISPATCH, "too large");
    }
    if (cols % 32 != 0) return fail(LNG_ERR_DISPATCH, "Q8_0 rows of %llu are not whole blocks", (unsigned long long)cols); // apple.rs:1799-1803
    Q8Checked &q = *out;
    if (int rc = check_slice(b, "codes", codes, rows * cols, 16, &q.codes)) return rc;
    if (int rc = check_slice(b, "scales", scales, rows * cols / 32 * 2, 2, &q.scales)) return rc;
    if (int rc = check_slice(b, "x", x, ((n - 1) * x_stride + cols) * (x_bf16 ? 2 : 4), 16, &q.x)) return rc;
    if (int rc = check_slice(b, "y", y, ((n - 1) * y_stride + rows) * 4, 4, &q.y)) return rc;
    if (int rc = check_output(b, q.y, {&q.codes, &q.scales, &q.x})) return rc;
    lng_k_q8 &a = q.a;
    a.codes = (const int8_t *)((const char *)q.codes.buf->ptr + codes.offset);
    a.scales = (const uint16_t *)((const char *)q.scales.buf->ptr + scales.offset);
    a.x = (const float *)((const char *)q.x.buf->ptr + x.offset);
    a.y = (float *)((char *)q.y.buf->ptr + y.offset);
    a.rows = (uint32_t)rows;
    a.cols = (uint32_t)cols;
    a.n = (uint32_t)n;
    a.x_stride = (uint32_t)x_stride;
    a.y_stride = (uint32_t)y_stride;
    if (x_bf16) {
        a.x_hi = (const uint16_t *)a.x;
        a.x = nullptr;
        a.plane_stride = (uint32_t)x_stride;
    }
    return LNG_OK;
}

// Few positions (n < 32): bound by reading the matrix, one pass over it per 16 positions, x split in registers.
// `a` may name further matrices of the same dispatch (a.more); row_tiles counts the tiles of all of them.
void q8_record_stream(lng_batch *b, const lng_k_q8 &a, uint64_t row_tiles, bool x_bf16) {
    const bool one = a.n == 1 && a.cols <= 12288 && !x_bf16; // x of a single position is held in LDS (Q8S_X1 floats)
    // more row tiles than compute units (several matrices): 8-wavefront workgroups, two per unit, one round
    const bool w8 = one && row_tiles > b->gpu->cus && !b->gpu->knobs.q8_w16;
    Cmd c;
    c.fn = x_bf16 ? b->gpu->q8_stream_bf16 : w8 ? b->gpu->q8_stream_one_w8 : one ? b->gpu->q8_stream_one : b->gpu->q8_stream;
    c.name = x_bf16 ? "lng_q8_stream_bf16" : w8 ? "lng_q8_stream_one_w8" : one ? "lng_q8_stream_one" : "lng_q8_stream";
    c.grid[0] = (unsigned)row_tiles;
    c.grid[1] = (unsigned)((a.n + 15) / 16);
    c.block = w8 ? 512 : 1024;
    set_args(c, a);
    b->cmds.push_back(std::move(c));
    b->dispatches += 1;
}

// Many positions: bound by the matrix unit.
int q8_record_tiled(lng_batch *b, lng_k_q8 a, bool x_bf16) {
    const uint64_t n = a.n, cols = a.cols, rows = a.rows;
    const uint64_t n_pad = (n + 127) / 128 * 128;
    if (n_pad / 128 > 65535) return fail(LNG_ERR_DISPATCH, "too large");
    // one-dimensional grid; the kernel maps ids to tiles (XCD-aware from eight position tiles on,
    // rounded up to blocks of 8 row tiles x 4 position tiles per XCD)
    const uint64_t row_tiles = (rows + 255) / 256, pos_tiles = n_pad / 128;
    uint64_t ids = row_tiles * pos_tiles;
    if (pos_tiles >= 8) {
        const uint64_t per_xcd = (pos_tiles + 7) / 8;
        ids = 8 * ((per_xcd + 3) / 4) * ((row_tiles + 7) / 8) * 32;
    }
    if (ids > 0x7fffffffull) return fail(LNG_ERR_DISPATCH, "too large");
    Cmd c1;
    c1.grid[0] = (unsigned)ids;
    c1.block = 512;
    if (x_bf16) {
        c1.fn = b->gpu->q8_tiled_bf16;
        c1.name = "lng_q8_tiled_bf16";
    } else {
        if (!fits_u32(n_pad * cols)) return fail(LNG_ERR_DISPATCH, "too large");
        char *planes = nullptr;
        if (int rc = reserve_x(b->gpu, 2 * n_pad * cols * 2, &planes)) return rc;
        lng_k_q8_split sp{};
        sp.x = a.x;
        sp.hi = (uint16_t *)planes;
        sp.lo = (uint16_t *)(planes + n_pad * cols * 2);
        sp.n = (uint32_t)n;
        sp.n_pad = (uint32_t)n_pad;
        sp.cols = (uint32_t)cols;
        sp.x_stride = a.x_stride;
        Cmd c0;
        c0.fn = b->gpu->q8_split_x;
        c0.name = "lng_q8_split_x";
        c0.grid[0] = (unsigned)((n_pad * (cols / 4) + 255) / 256);
        c0.block = 256;
        set_args(c0, sp);
        b->cmds.push_back(std::move(c0));
        a.x_hi = sp.hi;
        a.x_lo = sp.lo;
        a.plane_stride = (uint32_t)cols;
        c1.fn = b->gpu->q8_tiled;
        c1.name = "lng_q8_tiled";
    }
    set_args(c1, a);
    b->cmds.push_back(std::move(c1));
    b->dispatches += 1;
    return LNG_OK;
}

int q8_product(lng_batch *b, const lng_slice &codes, const lng_slice &scales, const lng_slice &x, const lng_slice &y,
               uint64_t rows, uint64_t cols, uint64_t n, uint64_t x_stride, uint64_t y_stride, bool gemm, bool tiled,
               bool x_bf16 = false) {
    Q8Checked q;
    if (int rc = q8_check(b, codes, scales, x, y, rows, cols, n, x_stride, y_stride, gemm, tiled, x_bf16, &q)) return rc;
    if (n < 32) {
        q8_record_stream(b, q.a, (rows + 15) / 16, x_bf16);
        return LNG_OK;
    }
    return q8_record_tiled(b, q.a, x_bf16);
}

} // namespace

extern "C" int lng_hip_gemv_q8_0(lng_batch *b, lng_slice codes, lng_slice scales, lng_slice x, lng_slice y,
                                 uint64_t rows, uint64_t cols) {
    return q8_product(b, codes, scales, x, y, rows, cols, 1, cols, rows, false, false);
}

extern "C" int lng_hip_gemm_q8_0(lng_batch *b, lng_slice codes, lng_slice scales, lng_slice x, lng_slice y,
                                 uint64_t rows, uint64_t cols, uint64_t n, uint64_t x_stride, uint64_t y_stride) {
    return q8_product(b, codes, scales, x, y, rows, cols, n, x_stride, y_stride, true, false);
}

extern "C" int lng_hip_gemm_q8_0_tiled(lng_batch *b, lng_slice codes, lng_slice scales, lng_slice x, lng_slice y,
                                       uint64_t rows, uint64_t cols, uint64_t n, uint64_t x_stride,
                                       uint64_t y_stride) {
    return q8_product(b, codes, scales, x, y, rows, cols, n, x_stride, y_stride, true, true);
}

extern "C" int lng_hip_gemm_q8_0_bf16(lng_batch *b, lng_slice codes, lng_slice scales, lng_slice x, lng_slice y,
                                      uint64_t rows, uint64_t cols, uint64_t n, uint64_t x_stride, uint64_t y_stride) {
    return q8_product(b, codes, scales, x, y, rows, cols, n, x_stride, y_stride, true, false, true);
}

namespace {
int q8_many(lng_batch *b, const lng_q8_matrix *matrices, size_t n_matrices, lng_slice x, const lng_slice *norm_w, float eps,
            uint64_t cols, uint64_t n, uint64_t x_stride);
}

extern "C" int lng_hip_gemm_q8_0_many(lng_batch *b, const lng_q8_matrix *matrices, size_t n_matrices, lng_slice x,
                                      uint64_t cols, uint64_t n, uint64_t x_stride) {
    return q8_many(b, matrices, n_matrices, x, nullptr, 0.0f, cols, n, x_stride);
}

extern "C" int lng_hip_gemm_q8_0_many_normed(lng_batch *b, const lng_q8_matrix *matrices, size_t n_matrices, lng_slice x,
                                             lng_slice norm_w, float eps, uint64_t cols, uint64_t n, uint64_t x_stride) {
    return q8_many(b, matrices, n_matrices, x, &norm_w, eps, cols, n, x_stride);
}

extern "C" int lng_hip_gemm_q8_0_residual(lng_batch *b, lng_slice codes, lng_slice scales, lng_slice x, int x_dtype,
                                          const lng_slice *bias, lng_slice h, uint64_t rows, uint64_t cols, uint64_t n,
                                          uint64_t x_stride, uint64_t h_stride) {
    if (x_dtype != LNG_F32 && x_dtype != LNG_BF16) return fail(LNG_ERR_DISPATCH, "unknown element type %d", x_dtype);
    Q8Checked q;
    if (int rc = q8_check(b, codes, scales, x, h, rows, cols, n, x_stride, h_stride, true, false, x_dtype == LNG_BF16, &q)) return rc;
    if (n >= 32) {
        return fail(LNG_ERR_DISPATCH, "%llu positions: the product with bias and residual folded in is for fewer than 32 "
                    "(use gemm_q8_0[_tiled] and add_rows)", (unsigned long long)n);
    }
    if (bias) {
        Operand ob;
        if (int rc = check_slice(b, "bias", *bias, rows * 4, 4, &ob)) return rc;
        if (overlaps(q.y, ob)) return fail(LNG_ERR_DISPATCH, "output overlaps an input");
        q.a.bias = (const float *)((const char *)ob.buf->ptr + bias->offset);
    }
    q.a.accumulate = 1;
    q8_record_stream(b, q.a, (rows + 15) / 16, x_dtype == LNG_BF16);
    return LNG_OK;
}

namespace {
int q8_many(lng_batch *b, const lng_q8_matrix *matrices, size_t n_matrices, lng_slice x, const lng_slice *norm_w, float eps,
            uint64_t cols, uint64_t n, uint64_t x_stride) {
    if (int rc = need_recording(b)) return rc;
    if (!matrices || n_matrices == 0 || n_matrices > 1 + LNG_Q8_MORE) {
        return fail(LNG_ERR_DISPATCH, "%zu matrices: one dispatch takes 1 to %d", n_matrices, 1 + LNG_Q8_MORE);
    }
    Q8Checked q[1 + LNG_Q8_MORE];
    for (size_t i = 0; i < n_matrices; ++i) {
        const lng_q8_matrix &m = matrices[i];
        if (int rc = q8_check(b, m.codes, m.scales, x, m.y, m.rows, cols, n, x_stride, m.rows, true, false, false, &q[i])) {
            return fail(rc, "matrix %zu: %s", i, std::string(g_error).c_str());
        }
    }
    for (size_t i = 0; i < n_matrices; ++i) { // no product's output may share bytes with another's output or inputs
        for (size_t j = 0; j < n_matrices; ++j) {
            if (i == j) continue;
            if (overlaps(q[i].y, q[j].y)) return fail(LNG_ERR_DISPATCH, "outputs of matrices %zu and %zu overlap", i, j);
            if (overlaps(q[i].y, q[j].codes) || overlaps(q[i].y, q[j].scales)) return fail(LNG_ERR_DISPATCH, "output overlaps an input");
        }
    }
    Operand onw{};
    if (norm_w) {
        if (n >= 32 || cols > 12288) {
            return fail(LNG_ERR_DISPATCH, "%llu positions of %llu columns: the product with the RMS norm folded in is for fewer "
                        "than 32 positions of up to 12288 columns (use rmsnorm_rows and gemm_q8_0[_tiled])",
                        (unsigned long long)n, (unsigned long long)cols);
        }
        if (int rc = check_slice(b, "norm_w", *norm_w, cols * 4, 16, &onw)) return rc;
        for (size_t i = 0; i < n_matrices; ++i) {
            if (overlaps(q[i].y, onw)) return fail(LNG_ERR_DISPATCH, "output overlaps an input");
        }
    }
    if (n >= 32) { // the matrix unit is the bound there, not the launches: one product after the other
        const size_t cmds = b->cmds.size(), dispatches = b->dispatches;
        for (size_t i = 0; i < n_matrices; ++i) {
            if (int rc = q8_record_tiled(b, q[i].a, false)) {
                b->cmds.resize(cmds); // a refused dispatch leaves nothing behind
                b->dispatches = dispatches;
                return rc;
            }
        }
        return LNG_OK;
    }
    lng_k_q8 a = q[0].a;
    uint64_t tiles = (a.rows + 15) / 16;
    a.n_more = (uint32_t)(n_matrices - 1);
    for (size_t i = 1; i < n_matrices; ++i) {
        auto &m = a.more[i - 1];
        m.codes = q[i].a.codes;
        m.scales = q[i].a.scales;
        m.y = q[i].a.y;
        m.rows = q[i].a.rows;
        m.y_stride = q[i].a.y_stride;
        m.first_tile = (uint32_t)tiles;
        tiles += (q[i].a.rows + 15) / 16;
    }
    if (!fits_u32(tiles) || tiles > 0x7fffffffull) return fail(LNG_ERR_DISPATCH, "too large");
    if (norm_w) {
        a.norm_w = (const float *)((const char *)onw.buf->ptr + norm_w->offset);
        a.eps = eps;
    }
    q8_record_stream(b, a, tiles, false);
    return LNG_OK;
}
} // namespace

extern "C" int lng_hip_checksum(lng_batch *b, lng_slice src, lng_slice dst) {
    if (int rc = need_recording(b)) return rc;
    if (src.len == 0 || src.len % 16 != 0) return fail(LNG_ERR_DISPATCH, "src: %llu bytes is not a whole number of 16-byte words", (unsigned long long)src.len);
    Operand os, od;
    if (int rc = check_slice(b, "src", src, src.len, 16, &os)) return rc;
    if (int rc = check_slice(b, "dst", dst, 16, 16, &od)) return rc;
    if (int rc = check_output(b, od, {&os})) return rc;
    lng_gpu *g = b->gpu;
    lng_k_checksum a{};
    a.src = (const char *)os.buf->ptr + src.offset;
    a.dst = (uint32_t *)((char *)od.buf->ptr + dst.offset);
    a.n16 = src.len / 16;
    a.n_parts = (uint32_t)std::min<uint64_t>((a.n16 + 255) / 256, (uint64_t)(g->knobs.checksum_wgs > 0 ? g->knobs.checksum_wgs : 2) * g->cus);
    // (two workgroups per compute unit that stay and sweep the buffer together, 2 MiB a turn: measured the fastest
    // way to read, 6.3 TB/s against 5.5-6.0 with 4-128 per unit)
    Scratch sc; // one 16-byte word per workgroup, in the scratch every dispatch of the gpu shares
    if (int rc = reserve_scratch(g, (size_t)a.n_parts * 4, 0, 0, &sc)) return rc;
    a.parts = (uint32_t *)sc.o;
    Cmd c;
    c.fn = g->checksum;
    c.name = "lng_checksum";
    c.grid[0] = a.n_parts;
    c.block = 256;
    set_args(c, a);
    b->cmds.push_back(std::move(c));
    Cmd f;
    f.fn = g->checksum_fold;
    f.name = "lng_checksum_fold";
    f.grid[0] = 1;
    f.block = 256;
    set_args(f, a);
    b->cmds.push_back(std::move(f));
    b->dispatches += 1;
    return LNG_OK;
}

extern "C" int lng_hip_fill_synthetic(lng_batch *b, lng_slice dst, int dtype, uint64_t seed, float scale,
                                      uint64_t period) {
    if (int rc = need_recording(b)) return rc;
    if (dtype != LNG_F32 && dtype != LNG_BF16) return fail(LNG_ERR_DISPATCH, "unknown element type %d", dtype);
    const uint64_t es = elem_size(dtype);
    if (dst.len == 0 || dst.len % es != 0) return fail(LNG_ERR_DISPATCH, "dst: %llu bytes is not a whole number of elements", (unsigned long long)dst.len);
    Operand od;
    if (int rc = check_slice(b, "dst", dst, dst.len, es, &od)) return rc;
    if (od.index >= b->buffers.size()) return fail(LNG_ERR_DISPATCH, "output is in read-only resident memory");
    lng_k_fill a{};
    a.dst = (char *)od.buf->ptr + dst.offset;
    a.n = dst.len / es;
    a.seed = seed;
    a.period = period;
    a.factor = scale / LNG_SYNTH_STD;
    a.dtype = (uint32_t)dtype;
    Cmd c;
    c.fn = b->gpu->fill_synthetic;
    c.name = "lng_fill_synthetic";
    c.grid[0] = (unsigned)std::min<uint64_t>((a.n + 255) / 256, 256u * 64u);
    c.block = 256;
    set_args(c, a);
    b->cmds.push_back(std::move(c));
    b->dispatches += 1;
    return LNG_OK;
}
