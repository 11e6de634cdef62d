// Prompt-pass kernels for head widths 128, 256 and 512 (DS = width / 64 slices of 64 dimensions), f32 and bf16,
// up to 16 query heads per kv head. Part of lng_kernels.hip (included at its end; uses its helpers).
//
// What they compute is the tiled operator of metal-compute (apple.rs:1311-1401, kernels.metal:588-720), whose
// kernel is generic in the head width; the reference's own tiled tests and its only published kernel times are
// at widths 256 and 512 (metal-compute/tests/attention_grouped.rs:210-221, 281-358).
//
// The head-width-64 kernels keep a whole K tile, a whole V tile and the wavefront's queries where the matrix
// unit reads them (LDS, registers). At width 512 a tile of 64 keys is 128 KiB in f32 and 32 queries are 64 KiB:
// neither fits. So the head is walked in slices of 64 dimensions, as the decode kernels of these widths do:
//
//   per tile of 64 keys:   S^T[key][query]  = sum over slices s of  K_s . Q_s^T       (DS stages)
//                          online softmax, one query per lane
//                          O_s^T[dim][query] += V_s^T . P^T  for every slice s        (DS stages)
//
// A stage is one [64 keys][64 dims] slice of K or of V, double buffered in LDS: the loads of stage u + 1 are
// issued before the products of stage u and stored after them, one barrier per stage. The queries of a slice
// come straight from memory (they are re-read once per key tile and stay in the caches: 32 rows x 256 bytes per
// wavefront and slice against 64 x 32 x 64 products), one slice ahead. The output accumulators are the state that
// stays: 32 x DS registers per lane, which is why a workgroup is four wavefronts, one per SIMD, with the whole
// register file of 512 to each.
//
// A workgroup takes HW = 1, 2 or 4 query heads of one kv head (as many as the group has, up to four) and 4 / HW
// blocks of 32 query rows, so groups of one or two heads (32 heads over 16 kv heads, the reference's other model)
// still fill their wavefronts; groups of more than four heads take several workgroups per kv head. Splits of the
// key tiles between workgroups, partials and lng_prefill_merge as in the width-64 kernels.
#define PWD_THREADS 256
#define PWD_STAGE_F32 (64 * 72) // floats per stage buffer: K rows 68 floats apart, V rows 72 (see lng_prefill_f32_d64)

struct wide_geometry {
    uint32_t g, hb, split, qtile;     // kv head, block of heads within it, split of the key tiles, query tile
    uint32_t group, hw, bm;           // heads per kv head; heads and query rows per workgroup
    uint32_t hslot, qb;               // this wavefront's head within the group and its block of 32 rows
    bool wave_active;
};

__device__ __forceinline__ wide_geometry wide_geometry_of(const lng_k_prefill &a, uint32_t wave) {
    wide_geometry w;
    w.group = a.heads / a.kv_heads;
    w.hw = w.group >= 3u ? 4u : w.group;
    w.bm = 32u * (4u / w.hw);
    const uint32_t head_blocks = (w.group + w.hw - 1u) / w.hw;
    uint32_t id = blockIdx.x;
    w.g = id % a.kv_heads;
    id /= a.kv_heads;
    w.hb = id % head_blocks;
    id /= head_blocks;
    w.split = id % a.splits;
    w.qtile = a.q_tiles - 1u - id / a.splits;
    w.hslot = w.hb * w.hw + (wave & (w.hw - 1u));
    w.qb = wave / w.hw;
    w.wave_active = w.hslot < w.group;
    return w;
}

template <int DS> __device__ __forceinline__ void prefill_wide_f32(const lng_k_prefill a) {
    __shared__ __attribute__((aligned(16))) float s_kv[2][PWD_STAGE_F32];
    constexpr uint32_t WIDTH = 64u * DS;

    const uint32_t tid = threadIdx.x;
    const uint32_t lane = tid & 63u;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t n = lane & 31u; // query within the wavefront's block
    const uint32_t hh = lane >> 5; // which of the two k slots of the matrix instruction
    const wide_geometry w = wide_geometry_of(a, wave);
    const uint32_t g = w.g, group = w.group, split = w.split;

    const uint32_t t = (uint32_t)a.t, start = (uint32_t)a.start;
    const uint32_t q0 = w.qtile * w.bm;
    const uint32_t rows_here = t - q0 < w.bm ? t - q0 : w.bm;
    const uint32_t end = start + t;
    const uint32_t pos_first = start + q0;
    const uint32_t pos_last = pos_first + rows_here - 1;
    const bool windowed = a.window != LNG_WINDOW_FULL;
    const uint32_t window = windowed ? (uint32_t)a.window : 0u;
    const uint32_t kfirst = (windowed && pos_first + 1 > window) ? pos_first + 1 - window : 0u;
    const uint32_t tile0 = kfirst & ~63u;
    const uint32_t all_tiles = (pos_last - tile0) / 64u + 1;
    const bool partial = a.splits > 1u;
    const uint32_t first_tile = (uint32_t)((uint64_t)all_tiles * split / a.splits);
    const uint32_t n_tiles = (uint32_t)((uint64_t)all_tiles * (split + 1u) / a.splits);
    const bool ring = a.slots < end;
    const uint32_t slots = (uint32_t)a.slots;
    const uint64_t row_bytes = (uint64_t)a.kv_heads * (WIDTH * 4u);

    // this wavefront's 32 queries; a lane past the last row reads the last row and stores nothing
    const uint32_t my_row = q0 + 32u * w.qb + n;
    const uint32_t my_pos = start + my_row;
    const bool row_ok = my_row < t;
    const uint32_t wpos_first = pos_first + 32u * w.qb;                         // first and last position of the wavefront's rows
    const uint32_t wpos_last = wpos_first + 31u < pos_last ? wpos_first + 31u : pos_last;
    const uint32_t wkfirst = (windowed && wpos_first + 1 > window) ? wpos_first + 1 - window : 0u;
    const uint32_t head = g * group + (w.wave_active ? w.hslot : 0u);
    const char *qbase = a.q + (((uint64_t)(row_ok ? my_row : t - 1u) * a.heads + head) * WIDTH + 4u * hh) * 4u;
    float4 qs[2][8]; // the slice in use and the next one
    auto fetch_q = [&](int slice, float4 (&dst)[8]) {
#pragma unroll
        for (int j = 0; j < 8; ++j) dst[j] = *(const float4 *)(qbase + (64u * slice + 8u * j) * 4u);
    };

    const float sl2 = a.scale * LNG_LOG2E;
    const bool sink_here = a.sinks && !partial;
    float m = sink_here ? a.sinks[head] * LNG_LOG2E : LNG_NEG_INF;
    float l = (sink_here && hh == 0) ? 1.0f : 0.0f;
    floatx16 ot[DS][2];
#pragma unroll
    for (int s = 0; s < DS; ++s) {
#pragma unroll
        for (int db = 0; db < 2; ++db) {
#pragma unroll
            for (int i = 0; i < 16; ++i) ot[s][db][i] = 0.0f;
        }
    }

    // ---- stage loader: four 16-byte pieces per thread (keys ld_key + 16 r) -------------------------------------
    const uint32_t ld_key = tid >> 4;    // 0..15
    const uint32_t ld_chunk = tid & 15u; // 16-byte piece of the slice's 256-byte row
    const char *kbase = a.k + (uint64_t)g * (WIDTH * 4u) + ld_chunk * 16u;
    const char *vbase = a.v + (uint64_t)g * (WIDTH * 4u) + ld_chunk * 16u;
    uint64_t roff0, roff1, roff2, roff3; // byte offsets of the tile's four rows of this thread
    auto row_offset = [&](uint32_t p) {
        p = p > pos_last ? pos_last : p; // rows outside [first visible, last] are masked, and may not exist
        p = p < kfirst ? kfirst : p;
        return (uint64_t)(ring ? p % slots : p) * row_bytes;
    };
    auto rows_of = [&](uint32_t tile) {
        const uint32_t p = tile0 + tile * 64u + ld_key;
        roff0 = row_offset(p);
        roff1 = row_offset(p + 16u);
        roff2 = row_offset(p + 32u);
        roff3 = row_offset(p + 48u);
    };
    uint4 r0, r1, r2, r3;
    auto fetch = [&](const char *base, int slice) {
        const char *b = base + 256u * slice;
        r0 = *(const uint4 *)(b + roff0);
        r1 = *(const uint4 *)(b + roff1);
        r2 = *(const uint4 *)(b + roff2);
        r3 = *(const uint4 *)(b + roff3);
    };
    auto stash = [&](uint32_t buf, uint32_t stride) {
        float *dst = &s_kv[buf][ld_key * stride + ld_chunk * 4u];
        *(uint4 *)(dst) = r0;
        *(uint4 *)(dst + 16u * stride) = r1;
        *(uint4 *)(dst + 32u * stride) = r2;
        *(uint4 *)(dst + 48u * stride) = r3;
    };
    if (first_tile < n_tiles) {
        rows_of(first_tile);
        fetch(kbase, 0);
        fetch_q(0, qs[0]);
        stash(0u, 68u);
    }
    __syncthreads();

    const uint32_t k_lane_off = n * 68u + 4u * hh; // + kb*32*68 + 8j
    const uint32_t v_lane_off = 4u * hh * 72u + n; // + (kb*32 + 8a + e)*72 + 32db

    // One loop for every tile: the masks of edge and diagonal tiles sit behind a uniform branch (a few dozen
    // compares beside hundreds of matrix instructions; separate loops made the compiler keep several copies of
    // the accumulators).
    for (uint32_t tile = first_tile; tile < n_tiles; ++tile) {
        const uint32_t kt0 = tile0 + tile * 64u;
        const bool more = tile + 1 < n_tiles;
        const bool masked = kt0 + 63u > pos_first || (windowed && kt0 + window < pos_first + w.bm);
        bool see[2]; // a block of 32 keys that no query of the wavefront sees is skipped
#pragma unroll
        for (int kb = 0; kb < 2; ++kb) {
            const uint32_t b0 = kt0 + 32u * kb;
            see[kb] = w.wave_active && !(b0 > wpos_last || b0 + 31u < wkfirst);
        }
        floatx16 st[2];
#pragma unroll
        for (int kb = 0; kb < 2; ++kb) {
#pragma unroll
            for (int i = 0; i < 16; ++i) st[kb][i] = 0.0f;
        }
        // ---- S^T = sum over slices of K_s . Q_s^T: stage s of the tile, in buffer s & 1 ---------------------------
#pragma unroll
        for (int s = 0; s < DS; ++s) {
            if (s + 1 < DS) fetch(kbase, s + 1); else fetch(vbase, 0);
            fetch_q((s + 1) % DS, qs[(s + 1) & 1]);
#pragma unroll
            for (int kb = 0; kb < 2; ++kb) {
                if (!see[kb]) continue;
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    const float4 ka = *(const float4 *)(&s_kv[s & 1][k_lane_off + kb * 32 * 68 + 8 * j]);
                    const float4 qv = qs[s & 1][j];
                    st[kb] = __builtin_amdgcn_mfma_f32_32x32x2f32(ka.x, qv.x, st[kb], 0, 0, 0);
                    st[kb] = __builtin_amdgcn_mfma_f32_32x32x2f32(ka.y, qv.y, st[kb], 0, 0, 0);
                    st[kb] = __builtin_amdgcn_mfma_f32_32x32x2f32(ka.z, qv.z, st[kb], 0, 0, 0);
                    st[kb] = __builtin_amdgcn_mfma_f32_32x32x2f32(ka.w, qv.w, st[kb], 0, 0, 0);
                }
            }
            stash((s + 1) & 1, s + 1 < DS ? 68u : 72u);
            __syncthreads();
        }
        // ---- online softmax, one query per lane. One maximum per tile; it moves only when it grows by PF_TAU. The
        // accumulators are rescaled on every tile, by 1 when it did not move: a branch around the rescaling makes the
        // register allocator hold the accumulators in vector registers across it (512 spilled registers at width 512),
        // and 32 DS multiplies per tile beside 128 DS matrix instructions are cheaper than that.
        float tmax = LNG_NEG_INF;
#pragma unroll
        for (int kb = 0; kb < 2; ++kb) {
            if (masked || !see[kb]) {
#pragma unroll
                for (int i = 0; i < 16; ++i) {
                    const uint32_t kp = kt0 + 32u * kb + 8u * (i >> 2) + 4u * hh + (i & 3);
                    const bool vis = see[kb] && kp <= my_pos && (!windowed || kp + window > my_pos);
                    st[kb][i] = vis ? st[kb][i] : LNG_NEG_INF;
                }
            }
#pragma unroll
            for (int i = 0; i < 16; ++i) tmax = fmaxf(tmax, st[kb][i]);
        }
        tmax = other_half_max(tmax) * sl2;
        const float m_new = tmax > m + PF_TAU ? tmax : m;
        const float m_safe = m_new == LNG_NEG_INF ? 0.0f : m_new;
        const float alpha = m_new == m ? 1.0f : __builtin_amdgcn_exp2f(m - m_safe);
        m = m_new;
        l *= alpha;
#pragma unroll
        for (int s = 0; s < DS; ++s) {
#pragma unroll
            for (int db = 0; db < 2; ++db) {
#pragma unroll
                for (int i = 0; i < 16; ++i) ot[s][db][i] *= alpha;
            }
        }
#pragma unroll
        for (int kb = 0; kb < 2; ++kb) {
            if (!see[kb]) continue;
            float psum = 0.0f;
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                st[kb][i] = __builtin_amdgcn_exp2f(__builtin_fmaf(st[kb][i], sl2, -m_safe));
                psum += st[kb][i];
            }
            l += psum;
        }
        // ---- O_s^T += V_s^T . P^T: stage DS + s of the tile, in buffer s & 1 (DS is even) ----------------------------
#pragma unroll
        for (int s = 0; s < DS; ++s) {
            const bool next = s + 1 < DS || more;
            if (s + 1 < DS) {
                fetch(vbase, s + 1);
            } else if (more) {
                rows_of(tile + 1);
                fetch(kbase, 0);
            }
#pragma unroll
            for (int kb = 0; kb < 2; ++kb) {
                if (!see[kb]) continue;
#pragma unroll
                for (int i = 0; i < 16; ++i) {
                    const float *vp = &s_kv[s & 1][v_lane_off + (kb * 32 + 8 * (i >> 2) + (i & 3)) * 72];
                    ot[s][0] = __builtin_amdgcn_mfma_f32_32x32x2f32(vp[0], st[kb][i], ot[s][0], 0, 0, 0);
                    ot[s][1] = __builtin_amdgcn_mfma_f32_32x32x2f32(vp[32], st[kb][i], ot[s][1], 0, 0, 0);
                }
            }
            if (next) stash((s + 1) & 1, s + 1 < DS ? 72u : 68u);
            __syncthreads();
        }
    }

    if (!w.wave_active || !row_ok) return;
    const float total = l + __shfl_xor(l, 32, 64);
    if (partial) { // (max, sum, unnormalised output) for lng_prefill_merge, which also adds the sink
        const uint64_t slot = (((uint64_t)my_row * a.kv_heads + g) * a.splits + split) * group + w.hslot;
        float *po = a.partial_o + slot * WIDTH;
#pragma unroll
        for (int s = 0; s < DS; ++s) {
#pragma unroll
            for (int db = 0; db < 2; ++db) {
#pragma unroll
                for (int blk = 0; blk < 4; ++blk) {
                    *(float4 *)(po + 64 * s + 32 * db + 8 * blk + 4 * hh) =
                        make_float4(ot[s][db][4 * blk + 0], ot[s][db][4 * blk + 1], ot[s][db][4 * blk + 2], ot[s][db][4 * blk + 3]);
                }
            }
        }
        if (hh == 0) *(float2 *)(a.partial_ml + slot * 2u) = make_float2(m, total);
        return;
    }
    const float inv = total > 0.0f ? 1.0f / total : 0.0f;
    float *op = (float *)a.out + ((uint64_t)my_row * a.heads + head) * WIDTH;
#pragma unroll
    for (int s = 0; s < DS; ++s) {
#pragma unroll
        for (int db = 0; db < 2; ++db) {
#pragma unroll
            for (int blk = 0; blk < 4; ++blk) {
                *(float4 *)(op + 64 * s + 32 * db + 8 * blk + 4 * hh) =
                    make_float4(ot[s][db][4 * blk + 0] * inv, ot[s][db][4 * blk + 1] * inv, ot[s][db][4 * blk + 2] * inv,
                                ot[s][db][4 * blk + 3] * inv);
            }
        }
    }
}

extern "C" __global__ __launch_bounds__(PWD_THREADS) void lng_prefill_f32_w128(lng_k_prefill a) { prefill_wide_f32<2>(a); }
extern "C" __global__ __launch_bounds__(PWD_THREADS) void lng_prefill_f32_w256(lng_k_prefill a) { prefill_wide_f32<4>(a); }
extern "C" __global__ __launch_bounds__(PWD_THREADS) void lng_prefill_f32_w512(lng_k_prefill a) { prefill_wide_f32<8>(a); }

// bf16 in and out, f32 accumulation: the same walk on v_mfma_f32_32x32x16_bf16, operand layouts as in
// lng_prefill_bf16_d64_h1 (K rows read with ds_read_b128, V^T with the transposing read, weights narrowed to
// bf16 where they are the B operand of the second product, the normaliser summed from the same rounded weights).
#define PWD_STAGE_BF16 (64 * PF_VSTRIDE) // bf16 elements per stage buffer: K rows PF_KSTRIDE apart, V rows PF_VSTRIDE

template <int DS> __device__ __forceinline__ void prefill_wide_bf16(const lng_k_prefill a) {
    __shared__ __attribute__((aligned(16))) uint16_t s_kv[2][PWD_STAGE_BF16];
    constexpr uint32_t WIDTH = 64u * DS;

    const uint32_t tid = threadIdx.x;
    const uint32_t lane = tid & 63u;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t n = lane & 31u;
    const uint32_t hh = lane >> 5;
    const wide_geometry w = wide_geometry_of(a, wave);
    const uint32_t g = w.g, group = w.group, split = w.split;

    const uint32_t t = (uint32_t)a.t, start = (uint32_t)a.start;
    const uint32_t q0 = w.qtile * w.bm;
    const uint32_t rows_here = t - q0 < w.bm ? t - q0 : w.bm;
    const uint32_t end = start + t;
    const uint32_t pos_first = start + q0;
    const uint32_t pos_last = pos_first + rows_here - 1;
    const bool windowed = a.window != LNG_WINDOW_FULL;
    const uint32_t window = windowed ? (uint32_t)a.window : 0u;
    const uint32_t kfirst = (windowed && pos_first + 1 > window) ? pos_first + 1 - window : 0u;
    const uint32_t tile0 = kfirst & ~63u;
    const uint32_t all_tiles = (pos_last - tile0) / 64u + 1;
    const bool partial = a.splits > 1u;
    const uint32_t first_tile = (uint32_t)((uint64_t)all_tiles * split / a.splits);
    const uint32_t n_tiles = (uint32_t)((uint64_t)all_tiles * (split + 1u) / a.splits);
    const bool ring = a.slots < end;
    const uint32_t slots = (uint32_t)a.slots;
    const uint64_t row_bytes = (uint64_t)a.kv_heads * (WIDTH * 2u);

    const uint32_t my_row = q0 + 32u * w.qb + n;
    const uint32_t my_pos = start + my_row;
    const bool row_ok = my_row < t;
    const uint32_t wpos_first = pos_first + 32u * w.qb;
    const uint32_t wpos_last = wpos_first + 31u < pos_last ? wpos_first + 31u : pos_last;
    const uint32_t wkfirst = (windowed && wpos_first + 1 > window) ? wpos_first + 1 - window : 0u;
    const uint32_t head = g * group + (w.wave_active ? w.hslot : 0u);
    const char *qbase = a.q + (((uint64_t)(row_ok ? my_row : t - 1u) * a.heads + head) * WIDTH + 8u * hh) * 2u;
    uint4 qs[2][4];
    auto fetch_q = [&](int slice, uint4 (&dst)[4]) {
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) dst[ks] = *(const uint4 *)(qbase + (64u * slice + 16u * ks) * 2u);
    };

    const float sl2 = a.scale * LNG_LOG2E;
    const bool sink_here = a.sinks && !partial;
    float m = sink_here ? a.sinks[head] * LNG_LOG2E : LNG_NEG_INF;
    float l = (sink_here && hh == 0) ? 1.0f : 0.0f;
    floatx16 ot[DS][2];
#pragma unroll
    for (int s = 0; s < DS; ++s) {
#pragma unroll
        for (int db = 0; db < 2; ++db) {
#pragma unroll
            for (int i = 0; i < 16; ++i) ot[s][db][i] = 0.0f;
        }
    }
    bf16x2 ones2;
    ones2[0] = (__bf16)1.0f;
    ones2[1] = (__bf16)1.0f;

    // ---- stage loader: two 16-byte pieces per thread (keys ld_key and ld_key + 32) ----------------------------
    const uint32_t ld_key = tid >> 3;   // 0..31
    const uint32_t ld_chunk = tid & 7u; // 16-byte piece of the slice's 128-byte row
    const char *kbase = a.k + (uint64_t)g * (WIDTH * 2u) + ld_chunk * 16u;
    const char *vbase = a.v + (uint64_t)g * (WIDTH * 2u) + ld_chunk * 16u;
    uint64_t roff0, roff1;
    auto row_offset = [&](uint32_t p) {
        p = p > pos_last ? pos_last : p;
        p = p < kfirst ? kfirst : p;
        return (uint64_t)(ring ? p % slots : p) * row_bytes;
    };
    auto rows_of = [&](uint32_t tile) {
        const uint32_t p = tile0 + tile * 64u + ld_key;
        roff0 = row_offset(p);
        roff1 = row_offset(p + 32u);
    };
    uint4 r0, r1;
    auto fetch = [&](const char *base, int slice) {
        const char *b = base + 128u * slice;
        r0 = *(const uint4 *)(b + roff0);
        r1 = *(const uint4 *)(b + roff1);
    };
    auto stash = [&](uint32_t buf, uint32_t stride) {
        uint16_t *dst = &s_kv[buf][ld_key * stride + ld_chunk * 8u];
        *(uint4 *)(dst) = r0;
        *(uint4 *)(dst + 32u * stride) = r1;
    };
    if (first_tile < n_tiles) {
        rows_of(first_tile);
        fetch(kbase, 0);
        fetch_q(0, qs[0]);
        stash(0u, PF_KSTRIDE);
    }
    __syncthreads();

    const uint32_t k_lane_off = n * PF_KSTRIDE + 8u * hh; // + kb*32*KSTRIDE + 16*ks
    const uint32_t L = lane & 15u;
    const uint32_t blk16 = lane >> 4;
    const uint32_t v_lane_off = (4u * (blk16 >> 1) + (L >> 2)) * PF_VSTRIDE + 16u * (blk16 & 1u) + 4u * (L & 3u);

    for (uint32_t tile = first_tile; tile < n_tiles; ++tile) {
        const uint32_t kt0 = tile0 + tile * 64u;
        const bool more = tile + 1 < n_tiles;
        const bool masked = kt0 + 63u > pos_first || (windowed && kt0 + window < pos_first + w.bm);
        bool see[2];
#pragma unroll
        for (int kb = 0; kb < 2; ++kb) {
            const uint32_t b0 = kt0 + 32u * kb;
            see[kb] = w.wave_active && !(b0 > wpos_last || b0 + 31u < wkfirst);
        }
        floatx16 st[2];
#pragma unroll
        for (int kb = 0; kb < 2; ++kb) {
#pragma unroll
            for (int i = 0; i < 16; ++i) st[kb][i] = 0.0f;
        }
#pragma unroll
        for (int s = 0; s < DS; ++s) {
            if (s + 1 < DS) fetch(kbase, s + 1); else fetch(vbase, 0);
            fetch_q((s + 1) % DS, qs[(s + 1) & 1]);
#pragma unroll
            for (int kb = 0; kb < 2; ++kb) {
                if (!see[kb]) continue;
#pragma unroll
                for (int ks = 0; ks < 4; ++ks) {
                    const bf16x8 ka = as_bf16x8(*(const uint4 *)(&s_kv[s & 1][k_lane_off + kb * 32 * PF_KSTRIDE + 16 * ks]));
                    st[kb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ka, as_bf16x8(qs[s & 1][ks]), st[kb], 0, 0, 0);
                }
            }
            stash((s + 1) & 1, s + 1 < DS ? PF_KSTRIDE : PF_VSTRIDE);
            __syncthreads();
        }
        bf16x8 pb[2][2]; // [key block][16 keys]: the weights as the second product's B operand
        float tmax = LNG_NEG_INF;
#pragma unroll
        for (int kb = 0; kb < 2; ++kb) {
            if (masked || !see[kb]) {
                const uint32_t b0 = kt0 + 32u * kb;
                const int dist = see[kb] ? (int)(my_pos - (b0 + 4u * hh)) : -1;
                const int below = windowed ? dist - (int)window : -0x40000000;
#pragma unroll
                for (int i = 0; i < 16; ++i) {
                    const int o = 8 * (i >> 2) + (i & 3);
                    st[kb][i] = (o <= dist && o > below) ? st[kb][i] : LNG_NEG_INF;
                }
            }
#pragma unroll
            for (int i = 0; i < 16; ++i) tmax = fmaxf(tmax, st[kb][i]);
        }
        tmax = other_half_max(tmax) * sl2;
        const float m_new = tmax > m + PF_TAU ? tmax : m;
        const float m_safe = m_new == LNG_NEG_INF ? 0.0f : m_new;
        const float alpha = m_new == m ? 1.0f : __builtin_amdgcn_exp2f(m - m_safe);
        m = m_new;
        l *= alpha;
#pragma unroll
        for (int s = 0; s < DS; ++s) {
#pragma unroll
            for (int db = 0; db < 2; ++db) {
#pragma unroll
                for (int i = 0; i < 16; ++i) ot[s][db][i] *= alpha;
            }
        }
#pragma unroll
        for (int kb = 0; kb < 2; ++kb) {
            if (!see[kb]) continue;
            float psum[2] = {0.0f, 0.0f};
#pragma unroll
            for (int jj = 0; jj < 2; ++jj) {
#pragma unroll
                for (int e = 0; e < 8; e += 2) {
                    bf16x2 pr;
                    pr[0] = (__bf16)__builtin_amdgcn_exp2f(__builtin_fmaf(st[kb][8 * jj + e], sl2, -m_safe));
                    pr[1] = (__bf16)__builtin_amdgcn_exp2f(__builtin_fmaf(st[kb][8 * jj + e + 1], sl2, -m_safe));
                    pb[kb][jj][e] = pr[0];
                    pb[kb][jj][e + 1] = pr[1];
                    psum[jj] = __builtin_amdgcn_fdot2_f32_bf16(pr, ones2, psum[jj], false);
                }
            }
            l += psum[0] + psum[1];
        }
#pragma unroll
        for (int s = 0; s < DS; ++s) {
            const bool next = s + 1 < DS || more;
            if (s + 1 < DS) {
                fetch(vbase, s + 1);
            } else if (more) {
                rows_of(tile + 1);
                fetch(kbase, 0);
            }
#pragma unroll
            for (int kb = 0; kb < 2; ++kb) {
                if (!see[kb]) continue;
#pragma unroll
                for (int jj = 0; jj < 2; ++jj) {
#pragma unroll
                    for (int db = 0; db < 2; ++db) {
                        const uint16_t *vp = &s_kv[s & 1][v_lane_off + (32 * kb + 16 * jj) * PF_VSTRIDE + 32 * db];
                        const bf16x8 va = lds_read_tr8(vp, vp + 8 * PF_VSTRIDE);
                        ot[s][db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(va, pb[kb][jj], ot[s][db], 0, 0, 0);
                    }
                }
            }
            if (next) stash((s + 1) & 1, s + 1 < DS ? PF_VSTRIDE : PF_KSTRIDE);
            __syncthreads();
        }
    }

    if (!w.wave_active || !row_ok) return;
    const float total = l + __shfl_xor(l, 32, 64);
    if (partial) {
        const uint64_t slot = (((uint64_t)my_row * a.kv_heads + g) * a.splits + split) * group + w.hslot;
        float *po = a.partial_o + slot * WIDTH;
#pragma unroll
        for (int s = 0; s < DS; ++s) {
#pragma unroll
            for (int db = 0; db < 2; ++db) {
#pragma unroll
                for (int blk = 0; blk < 4; ++blk) {
                    *(float4 *)(po + 64 * s + 32 * db + 8 * blk + 4 * hh) =
                        make_float4(ot[s][db][4 * blk + 0], ot[s][db][4 * blk + 1], ot[s][db][4 * blk + 2], ot[s][db][4 * blk + 3]);
                }
            }
        }
        if (hh == 0) *(float2 *)(a.partial_ml + slot * 2u) = make_float2(m, total);
        return;
    }
    const float inv = total > 0.0f ? 1.0f / total : 0.0f;
    uint16_t *op = (uint16_t *)a.out + ((uint64_t)my_row * a.heads + head) * WIDTH;
#pragma unroll
    for (int s = 0; s < DS; ++s) {
#pragma unroll
        for (int db = 0; db < 2; ++db) {
#pragma unroll
            for (int blk = 0; blk < 4; ++blk) {
                bf16x4 o; // narrowed by the conversion instruction (round to nearest even)
#pragma unroll
                for (int i = 0; i < 4; ++i) o[i] = (__bf16)(ot[s][db][4 * blk + i] * inv);
                *(bf16x4 *)(op + 64 * s + 32 * db + 8 * blk + 4 * hh) = o;
            }
        }
    }
}

extern "C" __global__ __launch_bounds__(PWD_THREADS) void lng_prefill_bf16_w128(lng_k_prefill a) { prefill_wide_bf16<2>(a); }
extern "C" __global__ __launch_bounds__(PWD_THREADS) void lng_prefill_bf16_w256(lng_k_prefill a) { prefill_wide_bf16<4>(a); }
extern "C" __global__ __launch_bounds__(PWD_THREADS) void lng_prefill_bf16_w512(lng_k_prefill a) { prefill_wide_bf16<8>(a); }
