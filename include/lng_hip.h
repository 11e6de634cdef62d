/*
 * lng_hip.h — C ABI of the MI355X (gfx950) grouped-attention operator library.
 *
 * One shared library, liblng_hip.so, replaces the part of loadngo's `metal-compute` crate
 * that the gpt-oss attention path uses. Every entry point names the reference interface it
 * stands in for (paths relative to the reference repository). Plain pointers and sizes
 * only; errors are negative codes plus a thread-local message.
 *
 * Differences from the Metal original that a binding must know:
 *  - Device memory is not CPU-visible: Buffer::as_f32()/as_bytes_mut() become
 *    lng_hip_download()/lng_hip_upload().
 *  - Every attention entry point takes an element type (f32 as in the reference, or bf16
 *    in/out with f32 accumulation). Sinks are always f32.
 *  - Counts are 64-bit throughout (the reference narrows to u32 and refuses what does not
 *    fit; the same refusals are kept so behaviour is identical).
 */
#ifndef LNG_HIP_H
#define LNG_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* GroupedShape.window = usize::MAX: a query sees every earlier position. */
#define LNG_WINDOW_FULL UINT64_MAX
/* lng_decode_item.sinks_offset when the item has no sinks. */
#define LNG_NO_SINKS UINT64_MAX

/* metal-compute/src/lib.rs:41-53 — enum Error {NoDevice, Compile, Alloc, Dispatch, Gpu}. */
typedef enum lng_status {
    LNG_OK = 0,
    LNG_ERR_NO_DEVICE = -1, /* Error::NoDevice */
    LNG_ERR_COMPILE = -2,   /* Error::Compile(String): code object missing or a kernel not found */
    LNG_ERR_ALLOC = -3,     /* Error::Alloc(usize) */
    LNG_ERR_DISPATCH = -4,  /* Error::Dispatch(String): refused before anything is recorded */
    LNG_ERR_GPU = -5        /* Error::Gpu(String): the submitted work failed */
} lng_status;

typedef enum lng_dtype {
    LNG_F32 = 0, /* the reference's only element type */
    LNG_BF16 = 1 /* weights/src/dtype.rs:95-116 convention: high half of an f32, RNE narrowing */
} lng_dtype;

typedef struct lng_gpu lng_gpu;       /* apple.rs:105   struct Gpu */
typedef struct lng_buffer lng_buffer; /* apple.rs:391   struct Buffer, and apple.rs:465 Resident */
typedef struct lng_batch lng_batch;   /* apple.rs:541   struct Batch */

/* apple.rs:507-521 — Slice {buffer, offset, len}: bytes offset..offset+len of the batch's
 * buffer number `buffer`: its own buffers first, then the residents it attached, in order. */
typedef struct lng_slice {
    uint64_t buffer;
    uint64_t offset;
    uint64_t len;
} lng_slice;

/* apple.rs:598-614 — GroupedShape. `window` counts the query itself; position s of the
 * cache is in row s % slots. */
typedef struct lng_grouped_shape {
    uint64_t t;        /* new positions (queries) */
    uint64_t start;    /* absolute position of the first of them */
    uint64_t heads;    /* query heads */
    uint64_t kv_heads; /* key/value heads; heads is a multiple of it */
    uint64_t dim;      /* width of every head: multiple of 32 (16 for tiled), at most 512 */
    uint64_t window;   /* positions each query sees, itself included; LNG_WINDOW_FULL for all */
    uint64_t slots;    /* rows in the key and value buffers */
    float scale;
} lng_grouped_shape;

/* apple.rs:536-539 — Completed {buffers, gpu_time}: handed to the completion callback.
 * `status` is LNG_OK or LNG_ERR_GPU (then `message` says why); the buffers the batch owned
 * are the caller's again when the callback runs. */
typedef struct lng_completed {
    int status;
    double gpu_seconds;
    const char *message; /* valid during the callback only */
} lng_completed;

typedef void (*lng_on_done)(const lng_completed *done, void *user);

/* The message of the calling thread's most recent failed call ("" if none). */
const char *lng_hip_last_error(void);

/* ---- device --------------------------------------------------------------------------- */

/* apple.rs:105 Gpu::new — opens HIP device `device`, loads the gfx950 code object embedded
 * in the library and resolves every kernel. LNG_ERR_NO_DEVICE / LNG_ERR_COMPILE. */
int lng_hip_open(int device, lng_gpu **gpu);
/* Drop of Gpu. Waits for submitted batches. Buffers, residents and batches that are still alive keep working
 * for lng_hip_buffer_free / lng_hip_batch_drop (the reference's buffers share their device the same way); the
 * device's resources go when the last of them has gone. Recording or committing after close is an error of
 * the caller. */
void lng_hip_close(lng_gpu *gpu);
/* Device name (e.g. "gfx950..."), copied into `name` (NUL-terminated, truncated to `cap`). */
int lng_hip_device_name(lng_gpu *gpu, char *name, size_t cap);
/* Development switches. No counterpart in the reference and NOT part of the interface: they pick between kernels
 * that compute the same thing (tests compare them; experiments time them) and may change or go at any time. Each
 * has the name of an environment variable, which is read ONCE, at lng_hip_open; afterwards only this call changes
 * it (`value` NULL puts the default back). Nothing on the record path reads the environment. Calls recorded after
 * the change see it; it is the caller's business not to change switches while other threads record.
 *   LNG_DECODE_WGS n         workgroups a decode dispatch aims for (default 4096)
 *   LNG_FUSE_WGS n           largest decode grid that merges its chunks inside the kernel (default 4 x compute units)
 *   LNG_DECODE_O3            never the four-wavefront build of the decode kernel
 *   LNG_MERGE_WIDE           always the chunk merge of one workgroup per query head
 *   LNG_WIDE_GENERIC         head widths 128-512 row by row on the kernel of one workgroup per (row, head)
 *   LNG_F32_GENERIC          f32 operands on that kernel only
 *   LNG_PLAIN_ROW_BY_ROW     the row-by-row operator never takes a prompt-pass kernel
 *   LNG_WIDE_ROW_BY_ROW      prompt passes of head widths 128-512 row by row on the decode kernels
 *   LNG_PREFILL_STREAM 0|1   never / whenever possible the prompt-pass kernel whose workgroups walk several query tiles
 *   LNG_PREFILL_PAIR 0|1     never / whenever possible the prompt-pass kernel of one workgroup per (query tile, kv head, pair of heads)
 *   LNG_PREFILL_UPFRONT 0    narrow windows on the tile-by-tile kernel
 *   LNG_PREFILL_SPLITS n     workgroups per (query tile, kv head) of a prompt pass with fewer workgroups than compute units
 *   LNG_Q8_W16               the one-position Q8_0 kernel always as 16-wavefront workgroups
 *   LNG_CHECKSUM_WGS n       workgroups per compute unit of lng_hip_checksum's streaming read (default 2)
 *   LNG_TABLE_IN_PLACE n     row tables of n bytes or more stay in pinned host memory, where the kernels read them,
 *                            instead of being copied to the device ahead of the batch (default 8192; 0: always copied)
 *   LNG_COUNT_SECOND_PASSES  long causal prompt passes count the query tiles whose fixed-maximum pass failed its range
 *                            check and was made again with the maximum tracked (read with lng_hip_debug_get)
 * Read at lng_hip_open only: LNG_HSACO (a code object file to load instead of the embedded one). */
int lng_hip_debug_set(lng_gpu *gpu, const char *name, const char *value);
/* Development counters, no more part of the interface than the switches: waits for everything submitted so far,
 * hands out the counter called `name` (LNG_COUNT_SECOND_PASSES) and puts it back to zero. */
int lng_hip_debug_get(lng_gpu *gpu, const char *name, uint64_t *value);

/* ---- memory --------------------------------------------------------------------------- */

/* apple.rs:255 Gpu::buffer(len) — device memory, contents unspecified. len == 0 is
 * LNG_ERR_ALLOC ("Alloc(0)", apple.rs:256-258). */
int lng_hip_buffer(lng_gpu *gpu, size_t len, lng_buffer **buffer);
/* apple.rs:297 Gpu::resident(bytes) — read-only memory filled once; may be attached to any
 * number of batches at once and is never an output (apple.rs:896-900). */
int lng_hip_resident(lng_gpu *gpu, const void *bytes, size_t len, lng_buffer **resident);
/* Drop of Buffer / Arc<Resident>. LNG_ERR_DISPATCH while a batch owns or has attached it. */
int lng_hip_buffer_free(lng_buffer *buffer);
size_t lng_hip_buffer_len(const lng_buffer *buffer);
/* Raw device address, for callers that share the memory with other HIP code. */
void *lng_hip_buffer_device_ptr(lng_buffer *buffer);
/* Buffer::as_bytes_mut()[offset..offset+len].copy_from_slice(src) (apple.rs:409-416).
 * Refused while a batch owns the buffer and for residents. Blocking. */
int lng_hip_upload(lng_buffer *buffer, size_t offset, const void *src, size_t len);
/* Buffer::as_bytes()[offset..offset+len] (apple.rs:401-407). Refused while owned. Blocking. */
int lng_hip_download(lng_buffer *buffer, size_t offset, void *dst, size_t len);
/* Fills bytes [offset, offset+len) with `byte`. Refused while owned. Blocking. */
int lng_hip_fill(lng_buffer *buffer, size_t offset, int byte, size_t len);

/* ---- batches -------------------------------------------------------------------------- */

/* apple.rs:365 Gpu::batch(buffers, dispatch) — starts recording a batch that owns `buffers` until it completes
 * or is dropped; dispatches name them by position. Both of the reference's modes (apple.rs:67-70
 * Dispatch::Serial / Dispatch::Concurrent, the latter ordered by explicit barrier() calls) record the same
 * thing here: dispatches run in the order recorded, which is a valid execution of either mode, so there is
 * no mode argument and lng_hip_batch_barrier has nothing to add. */
int lng_hip_batch(lng_gpu *gpu, lng_buffer *const *buffers, size_t n_buffers, lng_batch **batch);
/* apple.rs:835 Batch::attach(&resident) -> Slice covering the whole resident. */
int lng_hip_batch_attach(lng_batch *batch, lng_buffer *resident, lng_slice *whole);
/* apple.rs:829 Batch::dispatches(). */
size_t lng_hip_batch_dispatches(const lng_batch *batch);
/* apple.rs:2194 Batch::barrier(). Dispatches of a batch already run in order here. */
int lng_hip_batch_barrier(lng_batch *batch);
/* apple.rs:2202 Batch::commit(proactor, on_done) — submits without blocking. `on_done` runs
 * once on a library thread when the GPU has finished (the Rust shim re-posts it to the
 * caller's proactor, as apple.rs:2231-2232 does); it may be NULL. The batch handle stays
 * valid for lng_hip_batch_wait / lng_hip_batch_drop. lng_hip_batch_wait may not be called from
 * inside `on_done` (it waits for the thread that is running it); lng_hip_batch_drop may: the
 * handle is then freed when the callback returns, which is how a binding whose commit consumes
 * the batch (apple.rs:2202 takes `self`) lets go of it. Batches may be recorded on
 * different threads at once; their submissions are serialised, and the dispatches of one batch
 * run back to back on the device. */
int lng_hip_batch_commit(lng_batch *batch, lng_on_done on_done, void *user);
/* Blocks until a committed batch has finished; gpu_seconds (may be NULL) receives the time
 * between its first and last dispatch on the device (Completed.gpu_time, apple.rs:2219-2221). */
int lng_hip_batch_wait(lng_batch *batch, double *gpu_seconds);
/* Per-kernel GPU time, the finer-grained form of the phase accounting in
 * gpt-oss/src/gpu.rs:247-317 (Profile / PhaseTime). With timing on (set before commit) an
 * event is recorded after every kernel of the batch; after the batch has finished,
 * lng_hip_batch_kernel_seconds sums the time and counts the launches of the kernel named
 * `kernel` (e.g. "lng_decode_bf16_d64"). */
int lng_hip_batch_set_timing(lng_batch *batch, int enabled);
int lng_hip_batch_kernel_seconds(lng_batch *batch, const char *kernel, double *seconds, size_t *launches);
/* Drop of Batch: an uncommitted batch runs nothing (apple.rs:553-561); a committed one is
 * waited for. Its buffers are the caller's again. */
void lng_hip_batch_drop(lng_batch *batch);

/* ---- the attention operator ------------------------------------------------------------ */

/* Shape rules alone, with no device: LNG_OK or LNG_ERR_DISPATCH, exactly the refusals of
 * apple.rs:1243-1272 (tiled == 0) and apple.rs:1356-1385 (tiled != 0). */
int lng_hip_check_grouped(const lng_grouped_shape *shape, int tiled);

/* apple.rs:1199 Batch::attention_grouped and apple.rs:1213 attention_grouped_with_sinks
 * (`sinks` NULL for the former). q, out: [t][heads][dim]; k, v: [rows][kv_heads][dim] with
 * rows = min(slots, start + t); sinks: [heads] f32. Slice lengths must be exactly what the
 * shape implies (apple.rs:868-873), inside their buffers (874-879), offsets aligned to the
 * element size; the output must not be resident memory nor overlap an input (896-906). */
int lng_hip_attention_grouped(lng_batch *batch, lng_slice q, lng_slice k, lng_slice v, lng_slice out,
                              const lng_slice *sinks, const lng_grouped_shape *shape, int dtype);

/* apple.rs:1311 Batch::attention_grouped_tiled and apple.rs:1324 ..._tiled_with_sinks: the
 * prompt-pass form. q and out hold t rounded up to 32 rows; k and v hold `slots` rows when
 * positions wrap (slots < start + t; then slots % 32 == 0) and start + t rounded up to 32
 * otherwise. Padded rows are never read here (the reference multiplies them by zero). */
int lng_hip_attention_grouped_tiled(lng_batch *batch, lng_slice q, lng_slice k, lng_slice v,
                                    lng_slice out, const lng_slice *sinks,
                                    const lng_grouped_shape *shape, int dtype);

/* No counterpart in the reference: lng_hip_attention_grouped for callers that cannot allocate - code
 * under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc. It takes raw device
 * addresses instead of slices of a batch, launches at once on the caller's stream `stream` (a hipStream_t;
 * NULL is the default stream) and returns without waiting; it calls no hipMalloc, hipFree or pinned
 * allocation and keeps nothing on the host heap. q, out: [t][heads][dim]; k, v: [min(slots, start + t)]
 * [kv_heads][dim]; sinks: [heads] f32 or NULL; every row is computed as the plain operator computes it
 * (same shape rules and refusals; operands aligned to their element size; the output may not overlap an
 * input). The caller vouches for the sizes behind the addresses, and for `stream` being a stream of the device
 * `gpu` was opened on; the calling thread's current device is the same after the call as before it. Up to 32
 * rows per call run row by row on the decode kernels (the cache is read once per row).
 *
 * Split-K partials go to a fixed array of LNG_STATIC_SCRATCH_SLOTS x 264 bytes (16.5 MiB) that every GPU the
 * library is opened on holds until the process ends. The limit: t x heads x ceil(dim / 64) <=
 * LNG_STATIC_MAX_ROW_HEADS (32 rows of 64 heads of width 64; 16 rows of 32 heads of width 256); more is
 * refused with LNG_ERR_DISPATCH (the partials of such a call fit: a row is cut into at most 32 chunks once
 * a call has 128 (row, kv head) pairs or more; a plan that would not fit is refused the same way). Every call on one GPU
 * shares that array: calls that may overlap in time on one GPU (different streams with no ordering between
 * them) race on it. Nothing in it has to start at zero: a call overwrites every slot it later reads. */
#define LNG_STATIC_SCRATCH_SLOTS 65536u
#define LNG_STATIC_MAX_ROW_HEADS 2048u
int lng_hip_attention_grouped_static(lng_gpu *gpu, void *stream, const void *q, const void *k, const void *v,
                                     void *out, const float *sinks, const lng_grouped_shape *shape, int dtype);

/* apple.rs:1762 Batch::copy_rows((src, src_stride), (dst, dst_stride), rows, width): how
 * gpt-oss/src/gpu.rs:744-759 writes new K and V rows into a cache. Strides and width count
 * elements. src_dtype != dst_dtype converts (f32 -> bf16 rounds to nearest even): the new
 * rows of an f32 projection go straight into a bf16 cache. */
int lng_hip_copy_rows(lng_batch *batch, lng_slice src, uint64_t src_stride, int src_dtype,
                      lng_slice dst, uint64_t dst_stride, int dst_dtype, uint64_t rows,
                      uint64_t width);

/* One decoding query per item, many sequences and layers in one dispatch. No counterpart
 * in the reference, which records one attention_grouped_with_sinks per sequence and layer
 * (gpt-oss/src/gpu.rs:794-805); each item computes exactly what that call computes with
 * t = 1. Offsets are bytes into the named buffers of the batch. */
typedef struct lng_decode_item {
    uint64_t q_offset;     /* [heads][dim] */
    uint64_t out_offset;   /* [heads][dim] */
    uint64_t k_offset;     /* [min(slots, start+1)][kv_heads][dim] */
    uint64_t v_offset;
    uint64_t sinks_offset; /* [heads] f32, or LNG_NO_SINKS */
    uint64_t start;        /* absolute position of the query */
    uint64_t window;       /* LNG_WINDOW_FULL for all */
    uint64_t slots;
} lng_decode_item;

int lng_hip_attention_decode_batched(lng_batch *batch, uint64_t q_buffer, uint64_t k_buffer,
                                     uint64_t v_buffer, uint64_t out_buffer, uint64_t sinks_buffer,
                                     const lng_decode_item *items, size_t n_items, uint64_t heads,
                                     uint64_t kv_heads, uint64_t dim, float scale, int dtype);

/* ---- The step before attention (gpt-oss/src/gpu.rs:733-759) -------------------------------- */

/* apple.rs:1731-1758 Batch::rmsnorm_rows((v, w), rows, (d, stride), eps), f32, in place over the
 * first d floats of `rows` rows `stride` floats apart: v = w * v / sqrt(mean(v^2) + eps), w of d
 * floats (gpt-oss/src/model.rs:274-280). Refused: rows == 0, d == 0, stride < d. */
int lng_hip_rmsnorm_rows(lng_batch *batch, lng_slice v, lng_slice w, uint64_t rows, uint64_t d,
                         uint64_t stride, float eps);

/* apple.rs:1886-1911 Batch::add_rows(dst, (src, src_stride), rows, width), f32:
 * dst[r][i] += src[r * src_stride + i]; src_stride == 0 adds one row (a bias) to every row.
 * Refused like the reference: rows == 0, width == 0, 0 < src_stride < width. */
int lng_hip_add_rows(lng_batch *batch, lng_slice dst, lng_slice src, uint64_t src_stride,
                     uint64_t rows, uint64_t width);

/* apple.rs:1916-1955 Batch::rotate_halves / rotate_halves_partial(x, table, rows, (heads, dim,
 * rotary)), f32, in place: x is [rows][heads][dim]; table holds per row rotary / 2 pairs
 * (cos, sin); element i of the first half of a head's first `rotary` dimensions turns with
 * element i of their second half: (a, b) -> (a cos - b sin, b cos + a sin), every product
 * rounded on its own. Refused: rows, heads or rotary == 0, rotary > dim, rotary odd. */
int lng_hip_rotate_halves(lng_batch *batch, lng_slice x, lng_slice table, uint64_t rows,
                          uint64_t heads, uint64_t dim, uint64_t rotary);

/* The whole step in one dispatch. No counterpart in the reference, which records three
 * add_rows, two rotate_halves and two to four copy_rows per layer (gpu.rs:733-759); this
 * computes exactly what those compute, in the same f32 operations, and narrows the results
 * to `out_dtype` as it stores them.
 *
 * An item is one sequence: its `n` new positions start, start + 1, ... Its projections q
 * [n][heads*dim], k and v [n][kv_heads*dim] are f32; the prepared queries go to q_out
 * [n][heads*dim]; the prepared k and v rows of position p go to row p % slots of caches
 * [slots][kv_heads*dim]. One item with n rows is a prompt pass; many items with n = 1 are one
 * decoding step of many sequences. Offsets are bytes into the buffers named by
 * lng_prepare_buffers. Refused: n == 0, n > slots (two new rows would land on one cache row),
 * outputs that overlap an input or one another, outputs in resident memory. */
typedef struct lng_prepare_item {
    uint64_t q_offset, k_offset, v_offset; /* f32 projections of the item's n rows */
    uint64_t table_offset;                 /* [n][rotary/2] (cos, sin) f32 pairs */
    uint64_t q_out_offset;                 /* [n][heads*dim] of out_dtype */
    uint64_t k_cache_offset;               /* row 0 of [slots][kv_heads*dim] of out_dtype */
    uint64_t v_cache_offset;
    uint64_t n;
    uint64_t start;
    uint64_t slots;
} lng_prepare_item;

typedef struct lng_prepare_buffers {
    uint64_t q, k, v;          /* indices (as in lng_slice.buffer) of the projection buffers */
    uint64_t table;
    uint64_t q_out;
    uint64_t k_cache, v_cache;
    const lng_slice *q_bias;   /* [heads*dim] f32, or NULL */
    const lng_slice *k_bias;   /* [kv_heads*dim] f32, or NULL */
    const lng_slice *v_bias;
} lng_prepare_buffers;

int lng_hip_prepare_attention(lng_batch *batch, const lng_prepare_buffers *buffers,
                              const lng_prepare_item *items, size_t n_items, uint64_t heads,
                              uint64_t kv_heads, uint64_t dim, uint64_t rotary, int out_dtype);

/* ---- Q8_0 products: the projections either side of attention (gpt-oss/src/gpu.rs:99-138) ----
 * `codes` holds each row's signed bytes in order (rows * cols), `scales` one little-endian
 * binary16 per 32 of them (weights/src/q8_0.rs:17-31 split_blocks makes both from ggml blocks);
 * element c of row r is scales[(r * cols + c) / 32] * codes[r * cols + c]. x and y are f32.
 * Refused like the reference: rows or cols == 0 or past u32, cols % 32 != 0, codes or x off a
 * 16-byte boundary, slices of the wrong length, y overlapping an input or in resident memory. */

/* apple.rs:1812-1830 Batch::gemv_q8_0((codes, scales), x, y, rows, cols): y = W x. */
int lng_hip_gemv_q8_0(lng_batch *batch, lng_slice codes, lng_slice scales, lng_slice x, lng_slice y,
                      uint64_t rows, uint64_t cols);

/* apple.rs:1833-1854 Batch::gemm_q8_0(..., n, (x_stride, y_stride)): y[p] = W x[p] for n
 * positions; x holds n rows of cols floats x_stride floats apart (a multiple of 4, >= cols), y n
 * rows of `rows` floats y_stride apart (apple.rs:987-1013 gemm_args). */
int lng_hip_gemm_q8_0(lng_batch *batch, lng_slice codes, lng_slice scales, lng_slice x, lng_slice y,
                      uint64_t rows, uint64_t cols, uint64_t n, uint64_t x_stride, uint64_t y_stride);

/* apple.rs:1857-1883 Batch::gemm_q8_0_tiled: the same product for prompt passes; also needs
 * rows % 64 == 0 and n % 32 == 0 (the caller pads the positions). */
int lng_hip_gemm_q8_0_tiled(lng_batch *batch, lng_slice codes, lng_slice scales, lng_slice x,
                            lng_slice y, uint64_t rows, uint64_t cols, uint64_t n, uint64_t x_stride,
                            uint64_t y_stride);

/* No counterpart in the reference (its attention output is f32): the same product for positions
 * that are bf16 already - the output of a bf16 attention, feeding the output projection
 * (gpt-oss/src/gpu.rs:807-817) without a widening pass. x holds n rows of cols bf16 values x_stride
 * values apart (a multiple of 8, >= cols), on a 16-byte boundary; y is f32 as above. Any n >= 1 and
 * any rows. A bf16 value is exact as a matrix operand, so this takes half the matrix instructions
 * of the f32 form and no split of x. */
int lng_hip_gemm_q8_0_bf16(lng_batch *batch, lng_slice codes, lng_slice scales, lng_slice x, lng_slice y,
                           uint64_t rows, uint64_t cols, uint64_t n, uint64_t x_stride, uint64_t y_stride);

/* No counterpart in the reference, which records one product per matrix (the q, k and v projections of a
 * layer are three gemv/gemm calls, gpt-oss/src/gpu.rs:724-732): up to four Q8_0 matrices of the same number of
 * columns multiplied by the same positions. Matrix i gives y_i[p] = W_i x[p], y_i dense ([n][rows_i] f32);
 * each product is exactly lng_hip_gemm_q8_0(codes_i, scales_i, x, y_i, rows_i, cols, n, x_stride, rows_i), with
 * its refusals, plus: outputs may not overlap one another or any matrix. Below 32 positions (decoding), where
 * a product is bound by launches and by reading its matrix once, all of them run as one dispatch. */
typedef struct lng_q8_matrix {
    lng_slice codes;
    lng_slice scales;
    lng_slice y;
    uint64_t rows;
} lng_q8_matrix;
int lng_hip_gemm_q8_0_many(lng_batch *batch, const lng_q8_matrix *matrices, size_t n_matrices, lng_slice x,
                           uint64_t cols, uint64_t n, uint64_t x_stride);

/* The same with the RMS norm of the positions folded in (no counterpart in the reference, which copies the
 * hidden state, normalises the copy in place and then multiplies: gpu.rs:712-732): y_i[p] = W_i x'[p] with
 * x'[p][c] = (x[p][c] / sqrt(mean_c(x[p]^2) + eps)) * norm_w[c], the arithmetic of lng_hip_rmsnorm_rows; x is
 * left as it is. norm_w holds cols f32 on a 16-byte boundary. For decoding only: fewer than 32 positions of up
 * to 12288 columns (refused otherwise: prompt passes are bound by the matrix unit and take the separate calls). */
int lng_hip_gemm_q8_0_many_normed(lng_batch *batch, const lng_q8_matrix *matrices, size_t n_matrices, lng_slice x,
                                  lng_slice norm_w, float eps, uint64_t cols, uint64_t n, uint64_t x_stride);

/* The output projection with its bias and the residual add folded in (no counterpart in the reference, which
 * records the product, add_rows of the bias and add_rows into the hidden state: gpu.rs:807-827):
 * h[p] = h[p] + ((W x[p]) + bias), every sum rounded as those three dispatches round it, so the result is theirs
 * bit for bit. x is f32 or bf16 (x_dtype; strides as in lng_hip_gemm_q8_0 / _bf16), bias rows f32 or NULL, h f32
 * with h_stride >= rows. For decoding only: fewer than 32 positions (refused otherwise). */
int lng_hip_gemm_q8_0_residual(lng_batch *batch, lng_slice codes, lng_slice scales, lng_slice x, int x_dtype,
                               const lng_slice *bias, lng_slice h, uint64_t rows, uint64_t cols, uint64_t n,
                               uint64_t x_stride, uint64_t h_stride);

/* Deterministic synthetic data written on the device (benchmarks and full-size tests):
 * element i of the slice gets g((seed, i mod period)) * scale, g a fixed integer hash mapped
 * to a centred sum of four uniforms (variance 1); period == 0 means no repetition. The
 * same integers are documented in the library source so a host can reproduce any element. */
int lng_hip_fill_synthetic(lng_batch *batch, lng_slice dst, int dtype, uint64_t seed, float scale,
                           uint64_t period);

/* No counterpart in the reference (benchmarks and tests): the XOR of every 16-byte word of `src` (a whole number of
 * them, on a 16-byte boundary), written to the 16 bytes of `dst`. A kernel that only reads, whole 128-byte lines per
 * wavefront instruction: what the memory system delivers to a plain streaming read, beside the decode kernels; and a
 * cheap way for a host to tell whether a 96 GiB cache holds what it should. */
int lng_hip_checksum(lng_batch *batch, lng_slice src, lng_slice dst);

#ifdef __cplusplus
}
#endif
#endif /* LNG_HIP_H */
