/*
 * TEST INFRASTRUCTURE — NOT PRODUCT CODE.
 *
 * CPU restatement of the grouped-query attention with sinks and sliding window that
 * jaylauffer/loadngo runs on the CPU. Only tests, the smoke check and the benchmark's
 * cpu_baseline leg may link or call this file; the shipped HIP path never does.
 *
 * The reference is Rust and cannot be built where this file is built (no rustc), so
 * this is a restatement, function by function, of:
 *
 *   gpt-oss/src/model.rs:434-464            f32 attention of Model::step (the parity target)
 *   gpt-oss/src/config.rs:99-103            even layers slide, odd layers see everything
 *   metal-compute/tests/attention_grouped.rs:65-100   float64 definition (t, start, window, sinks)
 *   metal-compute/tests/attention_grouped.rs:25-35    xorshift input generator `values`
 *   metal-compute/tests/attention_grouped.rs:47-63    ring layout of a cache (`ring`)
 *   metal-compute/src/apple.rs:1243-1256,1356-1369    accepted / rejected shapes
 *   weights/src/dtype.rs:95-116             bf16 widen / round-to-nearest-even narrow
 *   gpt-oss/src/model.rs:282-286,389-404,427-433      bias add, rotation by halves, cache append
 *   gpt-oss/src/gpu.rs:690-697,733-759      rotary table; the same step as GPU dispatches
 *
 * What pins each function (tests/test_oracle_*.py): the three literal bf16 vectors and the
 * round trip over all codes from dtype.rs:183-202; the integer generator reproduced
 * independently in Python; the f32 restatement against the f64 definition; the f64
 * definition against torch's scaled_dot_product_attention with an explicit mask and with
 * the sink written as one extra key of value zero; closed forms (zero queries, constant
 * values, window of one); ring independence; NaN poisoning of rows outside the window;
 * the rotation against complex multiplication in float64, its composition law and norm; and,
 * end to end, the reference's tiny-model fixture (transformers' logits within 2e-3) with this
 * file's attention and pre-attention step inside a numpy restatement of the rest of the model.
 *
 * Build: make -C oracle   (gcc -O2 -fno-fast-math -ffp-contract=off -fopenmp)
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define LNG_ORACLE_FULL UINT64_MAX

/* ---- weights/src/dtype.rs:95-97 ------------------------------------------------------ */
float lng_oracle_bf16_to_f32(uint16_t bits) {
    uint32_t wide = (uint32_t)bits << 16;
    float out;
    memcpy(&out, &wide, 4);
    return out;
}

/* ---- weights/src/dtype.rs:101-109: nearest, ties to even; NaN stays a quiet NaN ------- */
uint16_t lng_oracle_f32_to_bf16(float value) {
    uint32_t bits;
    memcpy(&bits, &value, 4);
    if (value != value) {
        return (uint16_t)((bits >> 16) | 0x40);
    }
    uint32_t bias = 0x7fffu + ((bits >> 16) & 1u);
    return (uint16_t)((bits + bias) >> 16);
}

void lng_oracle_widen(const uint16_t *src, float *dst, size_t n) {
    for (size_t i = 0; i < n; ++i) dst[i] = lng_oracle_bf16_to_f32(src[i]);
}

void lng_oracle_narrow(const float *src, uint16_t *dst, size_t n) {
    for (size_t i = 0; i < n; ++i) dst[i] = lng_oracle_f32_to_bf16(src[i]);
}

/* ---- metal-compute/tests/attention_grouped.rs:25-35 ---------------------------------- */
void lng_oracle_values(uint64_t seed, size_t n, float *out) {
    uint64_t s = seed | 1u;
    for (size_t i = 0; i < n; ++i) {
        s ^= s << 13;
        s ^= s >> 7;
        s ^= s << 17;
        out[i] = (float)(s >> 40) / (float)((uint64_t)1 << 23) - 1.0f;
    }
}

/*
 * ---- metal-compute/tests/attention_grouped.rs:47-63 ----------------------------------
 * `all` holds a row of `row` floats for every absolute position below start + t. `out`
 * receives the cache a decoder would hold after reaching start + t: position p in row
 * p % slots. Rows the plain operator must never read are NaN; the tiled operator's padded
 * rows are zero. Returns the number of rows written (rows * row floats must fit `out`).
 */
size_t lng_oracle_ring_rows(uint64_t t, uint64_t start, uint64_t slots, int tiled) {
    uint64_t end = start + t;
    if (!tiled) return slots < end ? slots : end;
    if (slots < end) return slots;
    return (end + 31) / 32 * 32;
}

size_t lng_oracle_ring(const float *all, size_t row, uint64_t t, uint64_t start,
                       uint64_t slots, int tiled, float *out) {
    uint64_t end = start + t;
    size_t rows = lng_oracle_ring_rows(t, start, slots, tiled);
    float fill = tiled ? 0.0f : NAN;
    for (size_t i = 0; i < rows * row; ++i) out[i] = fill;
    uint64_t from = end > slots ? end - slots : 0;
    for (uint64_t p = from; p < end; ++p) {
        memcpy(out + (p % slots) * row, all + p * row, row * sizeof(float));
    }
    return rows;
}

/*
 * ---- metal-compute/src/apple.rs:1243-1256 (plain) and 1356-1369 (tiled) ---------------
 * 1 when the reference would record the dispatch, 0 when it answers Error::Dispatch.
 */
int lng_oracle_accepts(uint64_t t, uint64_t start, uint64_t heads, uint64_t kv_heads,
                       uint64_t dim, uint64_t window, uint64_t slots, int tiled) {
    uint64_t end = start + t;
    uint64_t need = window > UINT64_MAX - t ? UINT64_MAX : window + t; /* saturating_add */
    if (t == 0 || kv_heads == 0 || heads % kv_heads != 0 || dim == 0 || dim > 512 ||
        window == 0 || slots == 0) {
        return 0;
    }
    if (!tiled) {
        if (dim % 32 != 0) return 0;
        if (slots < end && slots < need) return 0;
    } else {
        if (dim % 16 != 0) return 0;
        if (slots < end && (slots % 32 != 0 || slots < need)) return 0;
    }
    /* apple.rs:1257-1272: every count must fit u32 */
    uint64_t win = window < end ? window : end;
    uint64_t groups = tiled ? (t + 31) / 32 * heads : t * heads;
    if (t > UINT32_MAX || start > UINT32_MAX || heads > UINT32_MAX || kv_heads > UINT32_MAX ||
        win > UINT32_MAX || slots > UINT32_MAX || groups > UINT32_MAX) {
        return 0;
    }
    return 1;
}

/*
 * ---- gpt-oss/src/model.rs:434-464, generalised to (t, start, window, slots) -----------
 * q   [t][heads][dim] f32
 * k,v [rows][kv_heads][dim] f32, position p in row p % slots (a flat Vec in model.rs,
 *     i.e. slots = infinity; the ring is how metal-compute's callers hold it)
 * sinks [heads] or NULL (NULL: the sink logit is -inf, exp(-inf) = 0)
 * out [t][heads][dim] f32
 *
 * Operation order is the reference's: the score is a sequential f32 sum over the head
 * dimension, times scale (445-448); max folds from the sink (449-450); total starts at
 * exp(sink - max) and adds exp(score - max) in position order (451-455); each output
 * element accumulates weight / total * value in position order from 0 (456-463).
 * `threads` > 1 spreads (query, head) pairs over OpenMP threads without changing any
 * per-pair arithmetic; the reference itself walks heads on one thread.
 */
static void attend_f32(const float *query, const float *k, const float *v, const float *sink_at,
                       float *target, uint64_t pos, uint64_t kv, uint64_t kv_heads, uint64_t dim,
                       uint64_t window, uint64_t slots, float scale) {
    const uint64_t first = (window == LNG_ORACLE_FULL || pos + 1 <= window) ? 0 : pos + 1 - window;
    const uint64_t count = pos + 1 - first;
    float *scores = (float *)malloc(count * sizeof(float));
    for (uint64_t p = first; p <= pos; ++p) {
        const float *key = k + ((p % slots) * kv_heads + kv) * dim;
        float sum = 0.0f;
        for (uint64_t d = 0; d < dim; ++d) sum += query[d] * key[d];
        scores[p - first] = sum * scale;
    }
    const float sink = sink_at ? *sink_at : -INFINITY;
    float max = sink;
    for (uint64_t j = 0; j < count; ++j) max = fmaxf(max, scores[j]);
    float total = expf(sink - max);
    for (uint64_t j = 0; j < count; ++j) {
        scores[j] = expf(scores[j] - max);
        total += scores[j];
    }
    for (uint64_t d = 0; d < dim; ++d) target[d] = 0.0f;
    for (uint64_t p = first; p <= pos; ++p) {
        const float *value = v + ((p % slots) * kv_heads + kv) * dim;
        const float weight = scores[p - first];
        for (uint64_t d = 0; d < dim; ++d) target[d] += weight / total * value[d];
    }
    free(scores);
}

void lng_oracle_attention_f32(const float *q, const float *k, const float *v,
                              const float *sinks, float *out, uint64_t t, uint64_t start,
                              uint64_t heads, uint64_t kv_heads, uint64_t dim, uint64_t window,
                              uint64_t slots, float scale, int threads) {
    const uint64_t group = heads / kv_heads;
    const int64_t pairs = (int64_t)(t * heads);
    if (threads < 1) threads = 1;
#pragma omp parallel for schedule(dynamic, 1) num_threads(threads) if (threads > 1)
    for (int64_t pair = 0; pair < pairs; ++pair) {
        const uint64_t i = (uint64_t)pair / heads;
        const uint64_t head = (uint64_t)pair % heads;
        attend_f32(q + (i * heads + head) * dim, k, v, sinks ? sinks + head : NULL,
                   out + (i * heads + head) * dim, start + i, head / group, kv_heads, dim, window,
                   slots, scale);
    }
}

/*
 * ---- metal-compute/tests/attention_grouped.rs:65-100 ---------------------------------
 * The float64 definition the reference's operator tests compare against; same layouts as
 * above (the test indexes a flat array of all positions; slots >= start + t gives that).
 * Every term is exp(x - m) / z * v in f64, summed in position order, then cast to f32.
 */
void lng_oracle_attention_f64(const float *q, const float *k, const float *v,
                              const float *sinks, float *out, uint64_t t, uint64_t start,
                              uint64_t heads, uint64_t kv_heads, uint64_t dim, uint64_t window,
                              uint64_t slots, float scale, int threads) {
    const uint64_t group = heads / kv_heads;
    const int64_t pairs = (int64_t)(t * heads);
    if (threads < 1) threads = 1;
#pragma omp parallel for schedule(dynamic, 1) num_threads(threads) if (threads > 1)
    for (int64_t pair = 0; pair < pairs; ++pair) {
        const uint64_t i = (uint64_t)pair / heads;
        const uint64_t h = (uint64_t)pair % heads;
        const uint64_t last = start + i;
        const uint64_t first = (window == LNG_ORACLE_FULL || last + 1 <= window) ? 0 : last + 1 - window;
        const uint64_t g = h / group;
        const float *qt = q + (i * heads + h) * dim;
        const uint64_t count = last + 1 - first;
        double *scores = (double *)malloc(count * sizeof(double));
        for (uint64_t p = first; p <= last; ++p) {
            const float *kr = k + ((p % slots) * kv_heads + g) * dim;
            double sum = 0.0;
            for (uint64_t d = 0; d < dim; ++d) sum += (double)qt[d] * (double)kr[d];
            scores[p - first] = sum * (double)scale;
        }
        const double sink = sinks ? (double)sinks[h] : -INFINITY;
        double m = sink;
        for (uint64_t j = 0; j < count; ++j) m = fmax(m, scores[j]);
        double z = 0.0;
        for (uint64_t j = 0; j < count; ++j) z += exp(scores[j] - m);
        z += exp(sink - m);
        /* exp(x - m) / z does not depend on d: evaluated once per position, same value */
        for (uint64_t j = 0; j < count; ++j) scores[j] = exp(scores[j] - m) / z;
        for (uint64_t d = 0; d < dim; ++d) {
            double acc = 0.0;
            for (uint64_t p = first; p <= last; ++p) {
                acc += scores[p - first] * (double)v[((p % slots) * kv_heads + g) * dim + d];
            }
            out[(i * heads + h) * dim + d] = (float)acc;
        }
        free(scores);
    }
}

/*
 * bf16 in, bf16 out, f32 accumulate: inputs are widened exactly (dtype.rs:95-97), the f32
 * restatement above runs on them, and the output is rounded to nearest even
 * (dtype.rs:101-109). `rows` is the number of cache rows behind k and v. Sinks stay f32.
 */
void lng_oracle_attention_bf16(const uint16_t *q, const uint16_t *k, const uint16_t *v,
                               const float *sinks, uint16_t *out, uint64_t rows, uint64_t t,
                               uint64_t start, uint64_t heads, uint64_t kv_heads, uint64_t dim,
                               uint64_t window, uint64_t slots, float scale, int threads) {
    const size_t nq = (size_t)(t * heads * dim);
    const size_t nk = (size_t)(rows * kv_heads * dim);
    float *qf = (float *)malloc(nq * sizeof(float));
    float *kf = (float *)malloc(nk * sizeof(float));
    float *vf = (float *)malloc(nk * sizeof(float));
    float *of = (float *)malloc(nq * sizeof(float));
    lng_oracle_widen(q, qf, nq);
    lng_oracle_widen(k, kf, nk);
    lng_oracle_widen(v, vf, nk);
    lng_oracle_attention_f32(qf, kf, vf, sinks, of, t, start, heads, kv_heads, dim, window, slots,
                             scale, threads);
    lng_oracle_narrow(of, out, nq);
    free(qf);
    free(kf);
    free(vf);
    free(of);
}

/*
 * The same, for a subset of query rows: row i of the output is the attention of query row
 * i at absolute position positions[i] (each its own `start`, t = 1). Lets a long prefill be
 * checked, and timed as a CPU baseline, on a sample of rows instead of all of them.
 */
void lng_oracle_attention_rows_f32(const float *q, const float *k, const float *v,
                                   const float *sinks, float *out, const uint64_t *positions,
                                   uint64_t n_rows, uint64_t heads, uint64_t kv_heads, uint64_t dim,
                                   uint64_t window, uint64_t slots, float scale, int threads) {
    const uint64_t group = heads / kv_heads;
    if (threads < 1) threads = 1;
    const int64_t pairs = (int64_t)(n_rows * heads);
#pragma omp parallel for schedule(dynamic, 1) num_threads(threads) if (threads > 1)
    for (int64_t pair = 0; pair < pairs; ++pair) {
        const uint64_t i = (uint64_t)pair / heads;
        const uint64_t head = (uint64_t)pair % heads;
        attend_f32(q + (i * heads + head) * dim, k, v, sinks ? sinks + head : NULL,
                   out + (i * heads + head) * dim, positions[i], head / group, kv_heads, dim,
                   window, slots, scale);
    }
}

/* ------------------------------------------------------------------------------------------
 * The step before attention (gpt-oss/src/gpu.rs:733-759; CPU form gpt-oss/src/model.rs:427-433):
 * biases on the projections, rotary position embedding by halves on q and k, new k/v rows
 * appended to the cache at row position % slots.
 * ------------------------------------------------------------------------------------------ */

/* metal-compute/src/kernels.metal:1648-1660, apple.rs:1886-1911 (model.rs:282-286 `add`):
 * dst[r][i] += src[r * src_stride + i]; a stride of 0 adds one row, a bias, to every row. */
void lng_oracle_add_rows(float *dst, const float *src, uint64_t rows, uint64_t width,
                         uint64_t src_stride) {
    for (uint64_t r = 0; r < rows; ++r)
        for (uint64_t i = 0; i < width; ++i) dst[r * width + i] += src[r * src_stride + i];
}

/* gpt-oss/src/gpu.rs:690-697 (same numbers as model.rs:393-398): per position dim/2 pairs
 * (cos, sin) of position * inv_freq[i], computed in f64, times the YaRN factor, rounded to f32. */
void lng_oracle_rope_table(float *table, const double *inv_freq, uint64_t half, double scale,
                           uint64_t start, uint64_t n) {
    for (uint64_t p = 0; p < n; ++p)
        for (uint64_t i = 0; i < half; ++i) {
            const double angle = (double)(start + p) * inv_freq[i];
            table[(p * half + i) * 2] = (float)(cos(angle) * scale);
            table[(p * half + i) * 2 + 1] = (float)(sin(angle) * scale);
        }
}

/* model.rs:389-404 on rows, with the partial form of kernels.metal:1673-1690 / apple.rs:1929-1955:
 * x is [rows][heads][dim]; element i of the first half of a head's first `rotary` dimensions
 * turns with element i of their second half by the row's pair i; dimensions from `rotary` on
 * stay. Four products, one difference, one sum, each rounded to f32 (no fused multiply-add:
 * this file is compiled with -ffp-contract=off). */
void lng_oracle_rotate_halves(float *x, const float *table, uint64_t rows, uint64_t heads,
                              uint64_t dim, uint64_t rotary) {
    const uint64_t half = rotary / 2;
    for (uint64_t r = 0; r < rows; ++r)
        for (uint64_t h = 0; h < heads; ++h) {
            float *head = x + (r * heads + h) * dim;
            for (uint64_t i = 0; i < half; ++i) {
                const float c = table[(r * half + i) * 2], s = table[(r * half + i) * 2 + 1];
                const float a = head[i], b = head[i + half];
                head[i] = a * c - b * s;
                head[i + half] = b * c + a * s;
            }
        }
}

/* gpu.rs:733-759 as one function: q, k, v are the projections of n positions from `start`
 * ([n][heads*dim], [n][kv_heads*dim]); biases may be NULL. Writes the prepared queries to
 * q_out[n][heads*dim] and the prepared k/v rows of position start + r to cache row
 * (start + r) % slots. bf16 != 0: outputs are bf16 (weights/src/dtype.rs:103-116 rounding of the
 * f32 results), else f32. */
void lng_oracle_prepare(const float *q, const float *k, const float *v, const float *q_bias,
                        const float *k_bias, const float *v_bias, const float *table, void *q_out,
                        void *k_cache, void *v_cache, uint64_t n, uint64_t start, uint64_t slots,
                        uint64_t heads, uint64_t kv_heads, uint64_t dim, uint64_t rotary, int bf16) {
    const uint64_t qw = heads * dim, kw = kv_heads * dim;
    float *row = (float *)malloc((qw > kw ? qw : kw) * sizeof(float));
    for (uint64_t r = 0; r < n; ++r) {
        const uint64_t slot = (start + r) % slots;
        const float *pair = table + r * (rotary / 2) * 2;
        memcpy(row, q + r * qw, qw * sizeof(float));
        if (q_bias) lng_oracle_add_rows(row, q_bias, 1, qw, 0);
        lng_oracle_rotate_halves(row, pair, 1, heads, dim, rotary);
        if (bf16) lng_oracle_narrow(row, (uint16_t *)q_out + r * qw, qw);
        else memcpy((float *)q_out + r * qw, row, qw * sizeof(float));
        memcpy(row, k + r * kw, kw * sizeof(float));
        if (k_bias) lng_oracle_add_rows(row, k_bias, 1, kw, 0);
        lng_oracle_rotate_halves(row, pair, 1, kv_heads, dim, rotary);
        if (bf16) lng_oracle_narrow(row, (uint16_t *)k_cache + slot * kw, kw);
        else memcpy((float *)k_cache + slot * kw, row, kw * sizeof(float));
        memcpy(row, v + r * kw, kw * sizeof(float));
        if (v_bias) lng_oracle_add_rows(row, v_bias, 1, kw, 0);
        if (bf16) lng_oracle_narrow(row, (uint16_t *)v_cache + slot * kw, kw);
        else memcpy((float *)v_cache + slot * kw, row, kw * sizeof(float));
    }
    free(row);
}

/* ------------------------------------------------------------------------------------------
 * Q8_0 projections (the products either side of attention: gpt-oss/src/gpu.rs:99-138,724-732,
 * 807-817; CPU form weights/src/q8_0.rs).
 * ------------------------------------------------------------------------------------------ */

/* weights/src/dtype.rs:123-145: IEEE binary16 bits to f32, exact (subnormals renormalised). */
float lng_oracle_f16_to_f32(uint16_t bits) {
    const uint32_t sign = (uint32_t)(bits >> 15) << 31;
    const uint32_t exponent = (bits >> 10) & 0x1f;
    uint32_t mantissa = bits & 0x3ff;
    uint32_t out;
    if (exponent == 0 && mantissa == 0) {
        out = sign;
    } else if (exponent == 0) {
        int unbiased = -14;
        while ((mantissa & 0x400) == 0) {
            mantissa <<= 1;
            unbiased -= 1;
        }
        out = sign | ((uint32_t)(unbiased + 127) << 23) | ((mantissa & 0x3ff) << 13);
    } else if (exponent == 0x1f) {
        out = sign | 0x7f800000u | (mantissa << 13);
    } else {
        out = sign | ((exponent + 127 - 15) << 23) | (mantissa << 13);
    }
    float f;
    memcpy(&f, &out, 4);
    return f;
}

/* weights/src/q8_0.rs:17-31 split_blocks: ggml blocks (2-byte binary16 scale + 32 signed bytes)
 * into the codes, in order, and the scales, in order: the layout the GPU kernels take. */
void lng_oracle_q8_split_blocks(const uint8_t *blocks, size_t n_blocks, int8_t *codes, uint16_t *scales) {
    for (size_t b = 0; b < n_blocks; ++b) {
        scales[b] = (uint16_t)(blocks[34 * b] | (blocks[34 * b + 1] << 8));
        memcpy(codes + 32 * b, blocks + 34 * b + 2, 32);
    }
}

/* weights/src/q8_0.rs:103-123 mul_rows on the split layout, for n positions (the CPU model calls
 * it once per position): per block the 32 products code * x are summed in f32 in order, the
 * block sum is scaled once by d and added to the row's f32 accumulator.
 * x: n rows x_stride apart, y: n rows y_stride apart (metal-compute/src/apple.rs:987-1013). */
void lng_oracle_q8_mul(const int8_t *codes, const uint16_t *scales, const float *x, float *y,
                       uint64_t rows, uint64_t cols, uint64_t n, uint64_t x_stride, uint64_t y_stride) {
    const uint64_t blocks = cols / 32;
#pragma omp parallel for schedule(static)
    for (uint64_t r = 0; r < rows; ++r)
        for (uint64_t p = 0; p < n; ++p) {
            float acc = 0.0f;
            for (uint64_t b = 0; b < blocks; ++b) {
                const float d = lng_oracle_f16_to_f32(scales[r * blocks + b]);
                float sum = 0.0f;
                for (int i = 0; i < 32; ++i)
                    sum += (float)codes[r * cols + 32 * b + i] * x[p * x_stride + 32 * b + i];
                acc += d * sum;
            }
            y[p * y_stride + r] = acc;
        }
}

/* The float64 definition the reference's GPU tests hold the products to
 * (metal-compute/tests/q8_0_and_gpt_oss_glue.rs:139-149): element = scale * code, y = sum in f64. */
void lng_oracle_q8_mul_f64(const int8_t *codes, const uint16_t *scales, const float *x, double *y,
                           uint64_t rows, uint64_t cols, uint64_t n, uint64_t x_stride, uint64_t y_stride) {
    const uint64_t blocks = cols / 32;
#pragma omp parallel for schedule(static)
    for (uint64_t r = 0; r < rows; ++r)
        for (uint64_t p = 0; p < n; ++p) {
            double acc = 0.0;
            for (uint64_t c = 0; c < cols; ++c)
                acc += (double)lng_oracle_f16_to_f32(scales[r * blocks + c / 32]) * (double)codes[r * cols + c] *
                       (double)x[p * x_stride + c];
            y[p * y_stride + r] = acc;
        }
}

/* gpt-oss/src/model.rs:274-280 rms_norm over rows (the GPU operator's strided form,
 * metal-compute/src/apple.rs:1731-1758, in place on the first d floats of each row): the mean of
 * squares in f64, scale = (1 / sqrt(mean + eps)) rounded to f32, each element (v * scale) * w. */
void lng_oracle_rms_norm_rows(float *v, const float *w, uint64_t rows, uint64_t d, uint64_t stride, float eps) {
    for (uint64_t r = 0; r < rows; ++r) {
        float *x = v + r * stride;
        double ss = 0.0;
        for (uint64_t i = 0; i < d; ++i) ss += (double)x[i] * (double)x[i];
        const float scale = (float)(1.0 / sqrt(ss / (double)d + (double)eps));
        for (uint64_t i = 0; i < d; ++i) x[i] = x[i] * scale * w[i];
    }
}
