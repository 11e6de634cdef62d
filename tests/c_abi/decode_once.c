/* The C ABI used from plain C, the way a foreign-function binding would: one decoding query of
 * the gpt-oss shapes over a small bf16 cache, committed with a completion callback, and the same
 * query again through the batched entry point; prints both outputs' checksums (they must agree)
 * and the refusal message of a bad shape. Exit code 0 on success. */
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "lng_hip.h"

#define CHECK(call)                                                                      \
    do {                                                                                 \
        int rc_ = (call);                                                                \
        if (rc_ != LNG_OK) {                                                             \
            fprintf(stderr, "%s -> %d: %s\n", #call, rc_, lng_hip_last_error());         \
            return 1;                                                                    \
        }                                                                                \
    } while (0)

static uint16_t bf16(float x) { /* round to nearest even */
    uint32_t b;
    memcpy(&b, &x, 4);
    return (uint16_t)((b + 0x7fffu + ((b >> 16) & 1u)) >> 16);
}
static float widen(uint16_t h) {
    uint32_t b = (uint32_t)h << 16;
    float x;
    memcpy(&x, &b, 4);
    return x;
}

static volatile int g_done = 0;
static double g_seconds = -1.0;
static void on_done(const lng_completed *done, void *user) {
    g_seconds = done->status == LNG_OK ? done->gpu_seconds : -1.0;
    *(volatile int *)user = 1;
}

int main(void) {
    enum { H = 64, G = 8, D = 64, CTX = 700 };
    lng_gpu *gpu = NULL;
    CHECK(lng_hip_open(0, &gpu));
    uint16_t *q = malloc(H * D * 2), *k = malloc(CTX * G * D * 2), *v = malloc(CTX * G * D * 2);
    float sinks[H];
    uint64_t s = 88172645463325252ull;
    for (int i = 0; i < H * D + 2 * CTX * G * D + H; ++i) {
        s ^= s << 13; s ^= s >> 7; s ^= s << 17;
        const float x = (float)(s >> 40) / 8388608.0f - 1.0f;
        if (i < H * D) q[i] = bf16(x);
        else if (i < H * D + CTX * G * D) k[i - H * D] = bf16(x);
        else if (i < H * D + 2 * CTX * G * D) v[i - H * D - CTX * G * D] = bf16(x);
        else sinks[i - H * D - 2 * CTX * G * D] = x;
    }
    lng_buffer *bq, *bk, *bv, *bo, *bo2, *bs;
    CHECK(lng_hip_buffer(gpu, H * D * 2, &bq));
    CHECK(lng_hip_buffer(gpu, CTX * G * D * 2, &bk));
    CHECK(lng_hip_buffer(gpu, CTX * G * D * 2, &bv));
    CHECK(lng_hip_buffer(gpu, H * D * 2, &bo));
    CHECK(lng_hip_buffer(gpu, H * D * 2, &bo2));
    CHECK(lng_hip_resident(gpu, sinks, sizeof sinks, &bs));
    CHECK(lng_hip_upload(bq, 0, q, H * D * 2));
    CHECK(lng_hip_upload(bk, 0, k, CTX * G * D * 2));
    CHECK(lng_hip_upload(bv, 0, v, CTX * G * D * 2));

    lng_buffer *owned[] = {bq, bk, bv, bo, bo2};
    lng_batch *batch = NULL;
    CHECK(lng_hip_batch(gpu, owned, 5, &batch));
    lng_slice sink_slice;
    CHECK(lng_hip_batch_attach(batch, bs, &sink_slice));
    const lng_slice sq = {0, 0, H * D * 2}, sk = {1, 0, CTX * G * D * 2}, sv = {2, 0, CTX * G * D * 2},
                    so = {3, 0, H * D * 2};
    lng_grouped_shape shape = {1, CTX - 1, H, G, D, 128, CTX, 0.125f};
    lng_grouped_shape bad = shape;
    bad.heads = 60; /* not a multiple of the kv heads */
    if (lng_hip_attention_grouped(batch, sq, sk, sv, so, &sink_slice, &bad, LNG_BF16) != LNG_ERR_DISPATCH) return 2;
    printf("refused: %s\n", lng_hip_last_error());
    CHECK(lng_hip_attention_grouped(batch, sq, sk, sv, so, &sink_slice, &shape, LNG_BF16));
    const lng_decode_item item = {0, 0, 0, 0, 0, CTX - 1, 128, CTX};
    CHECK(lng_hip_attention_decode_batched(batch, 0, 1, 2, 4, sink_slice.buffer, &item, 1, H, G, D, 0.125f, LNG_BF16));
    CHECK(lng_hip_batch_commit(batch, on_done, (void *)&g_done));
    CHECK(lng_hip_batch_wait(batch, NULL));
    if (!g_done || g_seconds <= 0.0) return 3; /* wait returns after the callback has run */
    lng_hip_batch_drop(batch);

    uint16_t out[H * D], out2[H * D];
    CHECK(lng_hip_download(bo, 0, out, sizeof out));
    CHECK(lng_hip_download(bo2, 0, out2, sizeof out2));
    double sum = 0.0, sum2 = 0.0;
    for (int i = 0; i < H * D; ++i) {
        if (isnan(widen(out[i]))) return 4;
        sum += widen(out[i]);
        sum2 += widen(out2[i]);
    }
    printf("gpu %.1f us, checksum %.6f, batched checksum %.6f\n", g_seconds * 1e6, sum, sum2);
    if (memcmp(out, out2, sizeof out) != 0) return 5;
    lng_buffer *all[] = {bq, bk, bv, bo, bo2, bs};
    for (int i = 0; i < 6; ++i) CHECK(lng_hip_buffer_free(all[i]));
    lng_hip_close(gpu);
    free(q); free(k); free(v);
    return 0;
}
