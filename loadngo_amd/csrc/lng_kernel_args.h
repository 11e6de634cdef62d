/*
 * Kernel argument blocks shared by the host library (lng_hip.cpp) and the gfx950 kernels
 * (lng_kernels.hip). Each kernel takes exactly one of these structs by value; the host
 * passes it as the raw kernarg buffer of hipModuleLaunchKernel.
 */
#ifndef LNG_KERNEL_ARGS_H
#define LNG_KERNEL_ARGS_H

#include <stdint.h>

#include "../../include/lng_hip.h"

/* One query row and the cache it attends over: the device-side form of lng_decode_item,
 * byte offsets relative to the base pointers in lng_k_attn. */
typedef lng_decode_item lng_k_row;

typedef struct lng_k_attn {
    const char *q;            /* base of the query buffer */
    const char *k;            /* base of the key cache buffer */
    const char *v;            /* base of the value cache buffer */
    char *out;                /* base of the output buffer */
    const char *sinks;        /* base of the sinks buffer (f32), unused when a row has none */
    const lng_k_row *rows;    /* device table of n_rows rows, or NULL: derive row i from `first` */
    float *partial_o;         /* split-K scratch: [row][kv_head][chunk][group][dim] f32 */
    float *partial_ml;        /* split-K scratch: [row][kv_head][chunk][group][2] f32 (max, sum) */
    uint32_t *tickets;        /* split-K scratch: [row][kv_head] arrival counters, zero between dispatches */
    const uint32_t *work;     /* device table cum[n_rows + 1]: cum[r] = decode workgroups of rows before r (each row has
                                 kv_heads x its own number of chunks), or NULL: workgroup w takes pair w / n_chunks,
                                 chunk w % n_chunks */
    lng_k_row first;          /* row 0 when rows == NULL; row i: q/out advance by one row, start by i */
    uint32_t n_rows;
    uint32_t heads;
    uint32_t kv_heads;
    uint32_t dim;
    uint32_t chunk;           /* positions per workgroup along the cache (multiple of 128): a row of v visible positions
                                 has ceil(v / chunk) workgroups per kv head, which share its groups of 128 positions */
    uint32_t n_chunks;        /* chunks of the longest visible run = ceil(it / chunk): the partials keep this many slots per (row, kv head) */
    uint32_t dtype;           /* lng_dtype of q, k, v, out */
    uint32_t fused;           /* split-K: 1 = the last workgroup of a row merges, 0 = lng_decode_merge follows */
    float scale;
} lng_k_attn;

/* Most chunks one row may be split into: bounds the merge's LDS weight table. */
#define LNG_MAX_CHUNKS 256

/* Prompt pass: t query rows from `start`, one cache. */
typedef struct lng_k_prefill {
    const char *q;
    const char *k;
    const char *v;
    char *out;
    const float *sinks; /* NULL when absent */
    uint64_t t;
    uint64_t start;
    uint64_t window;
    uint64_t slots;
    uint32_t heads;
    uint32_t kv_heads;
    uint32_t dim;
    uint32_t q_tiles;   /* ceil(t / rows per workgroup) */
    float scale;
    uint32_t splits;    /* workgroups that share one (query tile, kv head), each with a run of its key tiles; 1: none */
    uint32_t dtype;     /* LNG_F32 / LNG_BF16: element type of q, k, v and out */
    float *partial_o;   /* splits > 1: [row][kv_head][split][group][dim] f32, unnormalised */
    float *partial_ml;  /* splits > 1: [row][kv_head][split][group][2] f32 (max in the log2 domain, sum) */
    uint32_t *second_passes; /* NULL, or a counter: +1 for every query tile of a long causal pass whose fixed-maximum
                                pass failed its range check and was made again with the maximum tracked */
} lng_k_prefill;

typedef struct lng_k_copy {
    const char *src;
    char *dst;
    uint64_t rows;
    uint64_t width;
    uint64_t src_stride;
    uint64_t dst_stride;
    uint32_t src_dtype;
    uint32_t dst_dtype;
} lng_k_copy;

typedef struct lng_k_fill {
    char *dst;
    uint64_t n;      /* elements */
    uint64_t seed;
    uint64_t period; /* 0: none */
    float factor;    /* scale / LNG_SYNTH_STD */
    uint32_t dtype;
} lng_k_fill;

/* XOR of every 16-byte word of src[0 .. n16): lng_checksum leaves one 16-byte word per workgroup in `parts`,
 * lng_checksum_fold (one workgroup) folds the n_parts of them into dst. */
typedef struct lng_k_checksum {
    const char *src;
    uint32_t *parts;
    uint32_t *dst;
    uint64_t n16; /* 16-byte words */
    uint32_t n_parts;
    uint32_t pad_;
} lng_k_checksum;

/* dst[r][i] += src[r * src_stride + i], f32. */
typedef struct lng_k_add {
    float *dst;
    const float *src;
    uint64_t rows;
    uint64_t width;
    uint64_t src_stride;
} lng_k_add;

/* In place: the first d floats of each row (stride floats apart) times w / sqrt(mean of squares + eps). */
typedef struct lng_k_rmsnorm {
    float *v;
    const float *w;
    uint32_t rows;
    uint32_t d;
    uint32_t stride;
    float eps;
} lng_k_rmsnorm;

/* In-place rotation by halves of x[rows][heads][dim], f32. */
typedef struct lng_k_rotate {
    float *x;
    const float *table; /* [rows][rotary/2][2] */
    uint64_t rows;
    uint32_t heads;
    uint32_t dim;
    uint32_t rotary;
    uint32_t pad;
} lng_k_rotate;

/* Bias + rotation + narrowing + cache append for a table of items (or the one item `first`). */
typedef struct lng_k_prepare {
    const char *q, *k, *v;   /* bases of the projection buffers */
    const float *q_bias, *k_bias, *v_bias; /* NULL when absent */
    const char *table;
    char *q_out, *k_cache, *v_cache;
    const lng_prepare_item *items; /* device table of n_items, or NULL: the one item is `first` */
    lng_prepare_item first;
    uint32_t n_items;
    uint32_t heads;
    uint32_t kv_heads;
    uint32_t dim;
    uint32_t rotary;
    uint32_t out_dtype;
    uint32_t units_per_row;  /* work units of `vec` elements (pairs, for rotated parts) per row */
    uint32_t vec;            /* 1 or 4 */
} lng_k_prepare;

/* x[n][x_stride] f32 -> two bf16 planes [n_pad][cols]: hi = nearest bf16 of x, lo = nearest bf16
 * of x - hi; rows n..n_pad are zero. */
typedef struct lng_k_q8_split {
    const float *x;
    uint16_t *hi;
    uint16_t *lo;
    uint32_t n;
    uint32_t n_pad;
    uint32_t cols;
    uint32_t x_stride;
} lng_k_q8_split;

/* y[p][r] = sum over blocks b of scale[r][b] * sum_i codes[r][32b+i] * x[p][32b+i]. */
typedef struct lng_k_q8 {
    const int8_t *codes;     /* [rows][cols] */
    const uint16_t *scales;  /* [rows][cols/32] binary16 */
    const float *x;          /* [n][x_stride] (few positions: split in registers) */
    const uint16_t *x_hi;    /* [n_pad][cols] bf16 (many positions: the planes lng_q8_split_x wrote) */
    const uint16_t *x_lo;
    float *y;                /* [n][y_stride] */
    uint32_t rows;
    uint32_t cols;
    uint32_t n;
    uint32_t x_stride;
    uint32_t y_stride;
    uint32_t plane_stride;   /* elements between positions of x_hi / x_lo: cols for the split planes; x's own stride
                                when the positions are bf16 already (x_hi = x, no x_lo, n rows only) */
    /* Few positions only: further matrices of the same dispatch, multiplied by the same x (same cols, n).
     * Workgroups from `first_tile` (in units of 16 rows) on belong to matrix more[i]; first_tile ascends. */
    uint32_t n_more;         /* 0..LNG_Q8_MORE */
    float eps;               /* of the RMS norm, when norm_w is set */
    /* Few positions only. norm_w: x is RMS-normalised on the way in, x'[c] = (x[c] / sqrt(mean(x^2) + eps)) * norm_w[c]
     * (cols <= 12288). bias: y gets bias[row] added. accumulate: the result is added to what y holds (a residual). */
    const float *norm_w;
    const float *bias;
    uint32_t accumulate;
    uint32_t pad_;
    struct lng_k_q8_more {
        const int8_t *codes;
        const uint16_t *scales;
        float *y;
        uint32_t rows;
        uint32_t y_stride;
        uint32_t first_tile;
        uint32_t pad_;
    } more[3];
} lng_k_q8;
#define LNG_Q8_MORE 3

/* Synthetic element i: z = splitmix64 finaliser of (i' + seed * 0x9E3779B97F4A7C15) with
 * i' = period ? i % period : i; s = sum of the four 16-bit fields of z; value =
 * (float)(s - 131070) * factor, one f32 multiply, then narrowed if the dtype is bf16.
 * The sum of four independent uniform 16-bit integers has standard deviation
 * sqrt(4 * (65536^2 - 1) / 12). */
#define LNG_SYNTH_STD 37837.227f

#endif /* LNG_KERNEL_ARGS_H */
