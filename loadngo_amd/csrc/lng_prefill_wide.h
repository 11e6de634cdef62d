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
// A stage is two slices ([64 keys][128 dims]) of K or of V, double buffered in LDS: the loads of stage u + 1 are
// issued before the products of stage u and stored after them, one barrier per stage (a wavefront is alone on its
// SIMD, so whatever it waits for at a barrier is lost: with one slice per stage the pass took 5 % longer). Up to
// width 256 a wavefront's queries stay in registers; at width 512 they do not fit and come straight from memory
// (re-read once per key tile, from the caches: 32 rows x 256 bytes per wavefront and slice against 64 x 32 x 64
// products), one slice ahead. The output accumulators are the state that stays: 32 x DS registers per lane, which
// is why a workgroup is four wavefronts, one per SIMD, with the whole register file of 512 to each.
//
// A workgroup takes HW = 1, 2 or 4 query heads of one kv head (as many as the group has, up to four) and 4 / HW
// blocks of 32 query rows, so groups of one or two heads (32 heads over 16 kv heads, the reference's other model)
// still fill their wavefronts; groups of more than four heads take several workgroups per kv head. Splits of the
// key tiles between workgroups, partials and lng_prefill_merge as in the width-64 kernels.
#define PWD_THREADS 256
#define PWD_KS_F32 132 // floats between K rows of a stage in LDS: 16-byte reads of 16 consecutive rows cover all 64 banks
#define PWD_VS_F32 136 // between V rows: the rows 4 apart that the two halves of a wavefront read fall 32 banks apart
#define PWD_STAGE_F32 (64 * PWD_VS_F32)

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

// What both element types share: the tile range of the workgroup and the rows its threads load.
struct wide_tiles {
    uint32_t t, start, q0, end, pos_first, pos_last, window, kfirst, tile0, first_tile, n_tiles, slots;
    bool windowed, partial, ring;
};

__device__ __forceinline__ wide_tiles wide_tiles_of(const lng_k_prefill &a, const wide_geometry &w) {
    wide_tiles x;
    x.t = (uint32_t)a.t;
    x.start = (uint32_t)a.start;
    x.q0 = w.qtile * w.bm;
    const uint32_t rows_here = x.t - x.q0 < w.bm ? x.t - x.q0 : w.bm;
    x.end = x.start + x.t;
    x.pos_first = x.start + x.q0;
    x.pos_last = x.pos_first + rows_here - 1;
    x.windowed = a.window != LNG_WINDOW_FULL;
    x.window = x.windowed ? (uint32_t)a.window : 0u;
    x.kfirst = (x.windowed && x.pos_first + 1 > x.window) ? x.pos_first + 1 - x.window : 0u;
    x.tile0 = x.kfirst & ~63u;
    const uint32_t all_tiles = (x.pos_last - x.tile0) / 64u + 1;
    x.partial = a.splits > 1u;
    x.first_tile = (uint32_t)((uint64_t)all_tiles * w.split / a.splits);
    x.n_tiles = (uint32_t)((uint64_t)all_tiles * (w.split + 1u) / a.splits);
    x.ring = a.slots < x.end;
    x.slots = (uint32_t)a.slots;
    return x;
}

template <int DS> __device__ __forceinline__ void prefill_wide_f32(const lng_k_prefill a) {
    __shared__ __attribute__((aligned(16))) float s_kv[2][PWD_STAGE_F32];
    constexpr uint32_t WIDTH = 64u * DS;
    constexpr int NST = DS / 2; // stages of K, and of V, per tile of 64 keys

    const uint32_t tid = threadIdx.x;
    const uint32_t lane = tid & 63u;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t n = lane & 31u; // query within the wavefront's block
    const uint32_t hh = lane >> 5; // which of the two k slots of the matrix instruction
    const wide_geometry w = wide_geometry_of(a, wave);
    const wide_tiles x = wide_tiles_of(a, w);
    const uint32_t g = w.g, group = w.group, split = w.split, t = x.t;
    const uint64_t row_bytes = (uint64_t)a.kv_heads * (WIDTH * 4u);

    // this wavefront's 32 queries; a lane past the last row reads the last row and stores nothing
    const uint32_t my_row = x.q0 + 32u * w.qb + n;
    const uint32_t my_pos = x.start + my_row;
    const bool row_ok = my_row < t;
    const uint32_t head = g * group + (w.wave_active ? w.hslot : 0u);
    const char *qbase = a.q + (((uint64_t)(row_ok ? my_row : t - 1u) * a.heads + head) * WIDTH + 4u * hh) * 4u;
    // Up to width 256 the queries stay in registers for the whole pass (32 DS of them); at width 512 they do not fit
    // beside 256 accumulators: the slice in use and the next one.
    constexpr bool Q_STAYS = DS <= 4;
    constexpr int QN = Q_STAYS ? DS : 2;
    float4 qs[QN][8];
    auto fetch_q = [&](int slice, float4 (&dst)[8]) {
#pragma unroll
        for (int j = 0; j < 8; ++j) dst[j] = *(const float4 *)(qbase + (64u * slice + 8u * j) * 4u);
    };

    const float sl2 = a.scale * LNG_LOG2E;
    const bool sink_here = a.sinks && !x.partial;
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

    // ---- stage loader: eight 16-byte pieces per thread (keys ld_key + 16 r, pieces ld_chunk and ld_chunk + 16) -------
    const uint32_t ld_key = tid >> 4;    // 0..15
    const uint32_t ld_chunk = tid & 15u; // 16-byte piece of each of the stage's two 256-byte slice rows
    const char *kbase = a.k + (uint64_t)g * (WIDTH * 4u) + ld_chunk * 16u;
    const char *vbase = a.v + (uint64_t)g * (WIDTH * 4u) + ld_chunk * 16u;
    // (plain scalars: arrays indexed inside the lambdas end up in scratch memory, every load waited for at once)
    uint64_t roff0, roff1, roff2, roff3; // byte offsets of the tile's four rows of this thread
    auto row_offset = [&](uint32_t p) {
        p = p > x.pos_last ? x.pos_last : p; // rows outside [first visible, last] are masked, and may not exist
        p = p < x.kfirst ? x.kfirst : p;
        return (uint64_t)(x.ring ? p % x.slots : p) * row_bytes;
    };
    auto rows_of = [&](uint32_t tile) {
        const uint32_t p = x.tile0 + tile * 64u + ld_key;
        roff0 = row_offset(p);
        roff1 = row_offset(p + 16u);
        roff2 = row_offset(p + 32u);
        roff3 = row_offset(p + 48u);
    };
    uint4 l0a, l0b, l1a, l1b, l2a, l2b, l3a, l3b;
    auto fetch = [&](const char *base, int stage) {
        const char *b = base + 512u * stage;
        l0a = *(const uint4 *)(b + roff0);
        l0b = *(const uint4 *)(b + roff0 + 256u);
        l1a = *(const uint4 *)(b + roff1);
        l1b = *(const uint4 *)(b + roff1 + 256u);
        l2a = *(const uint4 *)(b + roff2);
        l2b = *(const uint4 *)(b + roff2 + 256u);
        l3a = *(const uint4 *)(b + roff3);
        l3b = *(const uint4 *)(b + roff3 + 256u);
    };
    auto stash = [&](uint32_t buf, uint32_t stride) {
        float *dst = &s_kv[buf][ld_key * stride + ld_chunk * 4u];
        *(uint4 *)(dst) = l0a;
        *(uint4 *)(dst + 64u) = l0b;
        *(uint4 *)(dst + 16u * stride) = l1a;
        *(uint4 *)(dst + 16u * stride + 64u) = l1b;
        *(uint4 *)(dst + 32u * stride) = l2a;
        *(uint4 *)(dst + 32u * stride + 64u) = l2b;
        *(uint4 *)(dst + 48u * stride) = l3a;
        *(uint4 *)(dst + 48u * stride + 64u) = l3b;
    };
    if (x.first_tile < x.n_tiles) {
        rows_of(x.first_tile);
        fetch(kbase, 0);
        if constexpr (Q_STAYS) {
#pragma unroll
            for (int s = 0; s < DS; ++s) fetch_q(s, qs[s]);
        } else {
            fetch_q(0, qs[0]);
        }
        stash(0u, PWD_KS_F32);
    }
    __syncthreads();

    const uint32_t k_lane_off = n * PWD_KS_F32 + 4u * hh; // + kb*32*KS + 64*half + 8j
    const uint32_t v_lane_off = 4u * hh * PWD_VS_F32 + n; // + (kb*32 + 8a + e)*VS + 64*half + 32db

    // One loop for every tile and no branch in it but the one around the masks of edge and diagonal tiles (a few
    // dozen compares beside hundreds of matrix instructions): with a loop per kind of tile, or with blocks of keys
    // skipped behind branches, the compiler keeps copies of the accumulators and moves them about. A wavefront
    // therefore also multiplies the blocks of an edge tile that none of its queries sees (their weights are zero).
    // Operands come from LDS two groups of matrix instructions ahead of their use; the scheduling fences keep them
    // there (left alone, the compiler reads each operand right before the instructions that need it and waits).
    for (uint32_t tile = x.first_tile; tile < x.n_tiles; ++tile) {
        const uint32_t kt0 = x.tile0 + tile * 64u;
        const bool more = tile + 1 < x.n_tiles;
        const bool masked = kt0 + 63u > x.pos_first || (x.windowed && kt0 + x.window < x.pos_first + w.bm);
        floatx16 st[2];
#pragma unroll
        for (int kb = 0; kb < 2; ++kb) {
#pragma unroll
            for (int i = 0; i < 16; ++i) st[kb][i] = 0.0f;
        }
        // ---- S^T = sum over slices of K_s . Q_s^T: K stage u of the tile (slices 2u, 2u + 1), in buffer u & 1 -----------
#pragma unroll
        for (int u = 0; u < NST; ++u) {
            if (u + 1 < NST) fetch(kbase, u + 1); else fetch(vbase, 0);
            const float *kp = &s_kv[u & 1][k_lane_off];
            float4 ka[3][2];
            auto read_k = [&](int gi, float4 (&dst)[2]) { // group gi of the stage: slice half gi / 8, dims 8 (gi % 8) ..
                const float *p = kp + 64 * (gi >> 3) + 8 * (gi & 7);
                dst[0] = *(const float4 *)p;
                dst[1] = *(const float4 *)(p + 32 * PWD_KS_F32);
            };
            read_k(0, ka[0]);
            read_k(1, ka[1]);
#pragma unroll
            for (int gi = 0; gi < 16; ++gi) {
                __builtin_amdgcn_sched_barrier(0);
                const int slice = 2 * u + (gi >> 3);
                if constexpr (!Q_STAYS) {
                    if ((gi & 7) == 0) fetch_q((slice + 1) % DS, qs[(slice + 1) & 1]);
                }
                if (gi + 2 < 16) read_k(gi + 2, ka[(gi + 2) % 3]);
                const float4 k0 = ka[gi % 3][0], k1 = ka[gi % 3][1], qv = qs[Q_STAYS ? slice : (slice & 1)][gi & 7];
                st[0] = __builtin_amdgcn_mfma_f32_32x32x2f32(k0.x, qv.x, st[0], 0, 0, 0);
                st[1] = __builtin_amdgcn_mfma_f32_32x32x2f32(k1.x, qv.x, st[1], 0, 0, 0);
                st[0] = __builtin_amdgcn_mfma_f32_32x32x2f32(k0.y, qv.y, st[0], 0, 0, 0);
                st[1] = __builtin_amdgcn_mfma_f32_32x32x2f32(k1.y, qv.y, st[1], 0, 0, 0);
                st[0] = __builtin_amdgcn_mfma_f32_32x32x2f32(k0.z, qv.z, st[0], 0, 0, 0);
                st[1] = __builtin_amdgcn_mfma_f32_32x32x2f32(k1.z, qv.z, st[1], 0, 0, 0);
                st[0] = __builtin_amdgcn_mfma_f32_32x32x2f32(k0.w, qv.w, st[0], 0, 0, 0);
                st[1] = __builtin_amdgcn_mfma_f32_32x32x2f32(k1.w, qv.w, st[1], 0, 0, 0);
            }
            __builtin_amdgcn_sched_barrier(0);
            stash((u + 1) & 1, u + 1 < NST ? PWD_KS_F32 : PWD_VS_F32);
            __syncthreads();
        }
        // ---- online softmax, one query per lane. One maximum per tile; it moves only when it grows by PF_TAU. The
        // accumulators are rescaled on every tile, by 1 when it did not move: a branch around the rescaling makes the
        // register allocator hold the accumulators in vector registers across it (hundreds of spilled registers at
        // width 512), and 32 DS multiplies per tile beside 128 DS matrix instructions are cheaper than that.
        float tmax = LNG_NEG_INF;
#pragma unroll
        for (int kb = 0; kb < 2; ++kb) {
            if (masked) {
#pragma unroll
                for (int i = 0; i < 16; ++i) {
                    const uint32_t kp = kt0 + 32u * kb + 8u * (i >> 2) + 4u * hh + (i & 3);
                    const bool vis = kp <= my_pos && (!x.windowed || kp + x.window > my_pos);
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
        float psum = 0.0f;
#pragma unroll
        for (int kb = 0; kb < 2; ++kb) {
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                st[kb][i] = __builtin_amdgcn_exp2f(__builtin_fmaf(st[kb][i], sl2, -m_safe));
                psum += st[kb][i];
            }
        }
        l += psum;
        // ---- O_s^T += V_s^T . P^T: V stage u of the tile, in buffer (NST + u) & 1 ----------------------------------------
#pragma unroll
        for (int u = 0; u < NST; ++u) {
            const bool next = u + 1 < NST || more;
            if (u + 1 < NST) {
                fetch(vbase, u + 1);
            } else if (more) {
                rows_of(tile + 1);
                fetch(kbase, 0);
            }
            const float *vq = &s_kv[(NST + u) & 1][v_lane_off];
            float va[3][4]; // [ring][key block x half of the slice]
            auto read_v = [&](int gi, float (&dst)[4]) { // group gi: slice half gi / 16, key i = gi % 16 of both blocks
                const int i = gi & 15;
                const float *vp = vq + 64 * (gi >> 4) + (8 * (i >> 2) + (i & 3)) * PWD_VS_F32;
                dst[0] = vp[0];
                dst[1] = vp[32];
                dst[2] = vp[32 * PWD_VS_F32];
                dst[3] = vp[32 * PWD_VS_F32 + 32];
            };
            read_v(0, va[0]);
            read_v(1, va[1]);
#pragma unroll
            for (int gi = 0; gi < 32; ++gi) {
                __builtin_amdgcn_sched_barrier(0);
                if (gi + 2 < 32) read_v(gi + 2, va[(gi + 2) % 3]);
                const int s = 2 * u + (gi >> 4), i = gi & 15;
                ot[s][0] = __builtin_amdgcn_mfma_f32_32x32x2f32(va[gi % 3][0], st[0][i], ot[s][0], 0, 0, 0);
                ot[s][1] = __builtin_amdgcn_mfma_f32_32x32x2f32(va[gi % 3][1], st[0][i], ot[s][1], 0, 0, 0);
                ot[s][0] = __builtin_amdgcn_mfma_f32_32x32x2f32(va[gi % 3][2], st[1][i], ot[s][0], 0, 0, 0);
                ot[s][1] = __builtin_amdgcn_mfma_f32_32x32x2f32(va[gi % 3][3], st[1][i], ot[s][1], 0, 0, 0);
            }
            __builtin_amdgcn_sched_barrier(0);
            if (next) stash((NST + u + 1) & 1, u + 1 < NST ? PWD_VS_F32 : PWD_KS_F32);
            __syncthreads();
        }
    }

    if (!w.wave_active || !row_ok) return;
    const float total = l + __shfl_xor(l, 32, 64);
    if (x.partial) { // (max, sum, unnormalised output) for lng_prefill_merge, which also adds the sink
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
#define PWD_KS_BF16 136 // bf16 elements between K rows of a stage (272 bytes): conflict-free 16-byte row reads
#define PWD_VS_BF16 160 // between V rows (320 bytes): the four keys x 64 bytes that half a wavefront reads transposed fall in 64 banks
#define PWD_STAGE_BF16 (64 * PWD_VS_BF16)

template <int DS> __device__ __forceinline__ void prefill_wide_bf16(const lng_k_prefill a) {
    __shared__ __attribute__((aligned(16))) uint16_t s_kv[2][PWD_STAGE_BF16];
    constexpr uint32_t WIDTH = 64u * DS;
    constexpr int NST = DS / 2;

    const uint32_t tid = threadIdx.x;
    const uint32_t lane = tid & 63u;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t n = lane & 31u;
    const uint32_t hh = lane >> 5;
    const wide_geometry w = wide_geometry_of(a, wave);
    const wide_tiles x = wide_tiles_of(a, w);
    const uint32_t g = w.g, group = w.group, split = w.split, t = x.t;
    const uint64_t row_bytes = (uint64_t)a.kv_heads * (WIDTH * 2u);

    const uint32_t my_row = x.q0 + 32u * w.qb + n;
    const uint32_t my_pos = x.start + my_row;
    const bool row_ok = my_row < t;
    const uint32_t head = g * group + (w.wave_active ? w.hslot : 0u);
    const char *qbase = a.q + (((uint64_t)(row_ok ? my_row : t - 1u) * a.heads + head) * WIDTH + 8u * hh) * 2u;
    constexpr bool Q_STAYS = DS <= 4;
    constexpr int QN = Q_STAYS ? DS : 2;
    uint4 qs[QN][4];
    auto fetch_q = [&](int slice, uint4 (&dst)[4]) {
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) dst[ks] = *(const uint4 *)(qbase + (64u * slice + 16u * ks) * 2u);
    };

    const float sl2 = a.scale * LNG_LOG2E;
    const bool sink_here = a.sinks && !x.partial;
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

    // ---- stage loader: four 16-byte pieces per thread (keys ld_key + 16 r) -------------------------------------
    const uint32_t ld_key = tid >> 4;    // 0..15
    const uint32_t ld_chunk = tid & 15u; // 16-byte piece of the stage's 256-byte row (two slices)
    const char *kbase = a.k + (uint64_t)g * (WIDTH * 2u) + ld_chunk * 16u;
    const char *vbase = a.v + (uint64_t)g * (WIDTH * 2u) + ld_chunk * 16u;
    uint64_t roff0, roff1, roff2, roff3;
    auto row_offset = [&](uint32_t p) {
        p = p > x.pos_last ? x.pos_last : p;
        p = p < x.kfirst ? x.kfirst : p;
        return (uint64_t)(x.ring ? p % x.slots : p) * row_bytes;
    };
    auto rows_of = [&](uint32_t tile) {
        const uint32_t p = x.tile0 + tile * 64u + ld_key;
        roff0 = row_offset(p);
        roff1 = row_offset(p + 16u);
        roff2 = row_offset(p + 32u);
        roff3 = row_offset(p + 48u);
    };
    uint4 l0, l1, l2, l3;
    auto fetch = [&](const char *base, int stage) {
        const char *b = base + 256u * stage;
        l0 = *(const uint4 *)(b + roff0);
        l1 = *(const uint4 *)(b + roff1);
        l2 = *(const uint4 *)(b + roff2);
        l3 = *(const uint4 *)(b + roff3);
    };
    auto stash = [&](uint32_t buf, uint32_t stride) {
        uint16_t *dst = &s_kv[buf][ld_key * stride + ld_chunk * 8u];
        *(uint4 *)(dst) = l0;
        *(uint4 *)(dst + 16u * stride) = l1;
        *(uint4 *)(dst + 32u * stride) = l2;
        *(uint4 *)(dst + 48u * stride) = l3;
    };
    if (x.first_tile < x.n_tiles) {
        rows_of(x.first_tile);
        fetch(kbase, 0);
        if constexpr (Q_STAYS) {
#pragma unroll
            for (int s = 0; s < DS; ++s) fetch_q(s, qs[s]);
        } else {
            fetch_q(0, qs[0]);
        }
        stash(0u, PWD_KS_BF16);
    }
    __syncthreads();

    const uint32_t k_lane_off = n * PWD_KS_BF16 + 8u * hh; // + kb*32*KS + 64*half + 16*ks
    const uint32_t L = lane & 15u;
    const uint32_t blk16 = lane >> 4;
    const uint32_t v_lane_off = (4u * (blk16 >> 1) + (L >> 2)) * PWD_VS_BF16 + 16u * (blk16 & 1u) + 4u * (L & 3u);

    // (one loop, no branches but the one around the masks, operands two groups ahead: see prefill_wide_f32)
    for (uint32_t tile = x.first_tile; tile < x.n_tiles; ++tile) {
        const uint32_t kt0 = x.tile0 + tile * 64u;
        const bool more = tile + 1 < x.n_tiles;
        const bool masked = kt0 + 63u > x.pos_first || (x.windowed && kt0 + x.window < x.pos_first + w.bm);
        floatx16 st[2];
#pragma unroll
        for (int kb = 0; kb < 2; ++kb) {
#pragma unroll
            for (int i = 0; i < 16; ++i) st[kb][i] = 0.0f;
        }
#pragma unroll
        for (int u = 0; u < NST; ++u) {
            if (u + 1 < NST) fetch(kbase, u + 1); else fetch(vbase, 0);
            const uint16_t *kp = &s_kv[u & 1][k_lane_off];
            // groups of eight matrix instructions (one slice: 4 steps of 16 dims x 2 key blocks), operands a group ahead
            uint4 ka[2][4][2];
            auto read_k = [&](int half, uint4 (&dst)[4][2]) {
#pragma unroll
                for (int ks = 0; ks < 4; ++ks) {
                    const uint16_t *p = kp + 64 * half + 16 * ks;
                    dst[ks][0] = *(const uint4 *)p;
                    dst[ks][1] = *(const uint4 *)(p + 32 * PWD_KS_BF16);
                }
            };
            read_k(0, ka[0]);
#pragma unroll
            for (int half = 0; half < 2; ++half) {
                __builtin_amdgcn_sched_barrier(0);
                const int slice = 2 * u + half;
                if constexpr (!Q_STAYS) fetch_q((slice + 1) % DS, qs[(slice + 1) & 1]);
                if (half == 0) read_k(1, ka[1]);
#pragma unroll
                for (int ks = 0; ks < 4; ++ks) {
                    const bf16x8 qv = as_bf16x8(qs[Q_STAYS ? slice : (slice & 1)][ks]);
                    st[0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(as_bf16x8(ka[half][ks][0]), qv, st[0], 0, 0, 0);
                    st[1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(as_bf16x8(ka[half][ks][1]), qv, st[1], 0, 0, 0);
                }
            }
            __builtin_amdgcn_sched_barrier(0);
            stash((u + 1) & 1, u + 1 < NST ? PWD_KS_BF16 : PWD_VS_BF16);
            __syncthreads();
        }
        bf16x8 pb[2][2]; // [key block][16 keys]: the weights as the second product's B operand
        float tmax = LNG_NEG_INF;
#pragma unroll
        for (int kb = 0; kb < 2; ++kb) {
            if (masked) {
                const uint32_t b0 = kt0 + 32u * kb;
                const int dist = (int)(my_pos - (b0 + 4u * hh));
                const int below = x.windowed ? dist - (int)x.window : -0x40000000;
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
        float psum[2] = {0.0f, 0.0f};
#pragma unroll
        for (int kb = 0; kb < 2; ++kb) {
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
        }
        l += psum[0] + psum[1];
#pragma unroll
        for (int u = 0; u < NST; ++u) {
            const bool next = u + 1 < NST || more;
            if (u + 1 < NST) {
                fetch(vbase, u + 1);
            } else if (more) {
                rows_of(tile + 1);
                fetch(kbase, 0);
            }
            const uint16_t *vq = &s_kv[(NST + u) & 1][v_lane_off];
            bf16x8 va[2][4][2]; // [slice half][key block x its two groups of 16 keys][half of the slice's dims]
            auto read_v = [&](int half, bf16x8 (&dst)[4][2]) {
#pragma unroll
                for (int c = 0; c < 4; ++c) {
                    const uint16_t *vp = vq + 16 * c * PWD_VS_BF16 + 64 * half;
                    dst[c][0] = lds_read_tr8(vp, vp + 8 * PWD_VS_BF16);
                    dst[c][1] = lds_read_tr8(vp + 32, vp + 32 + 8 * PWD_VS_BF16);
                }
            };
            read_v(0, va[0]);
#pragma unroll
            for (int half = 0; half < 2; ++half) {
                __builtin_amdgcn_sched_barrier(0);
                if (half == 0) read_v(1, va[1]);
                const int s = 2 * u + half;
#pragma unroll
                for (int c = 0; c < 4; ++c) {
                    ot[s][0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(va[half][c][0], pb[c >> 1][c & 1], ot[s][0], 0, 0, 0);
                    ot[s][1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(va[half][c][1], pb[c >> 1][c & 1], ot[s][1], 0, 0, 0);
                }
            }
            __builtin_amdgcn_sched_barrier(0);
            if (next) stash((NST + u + 1) & 1, u + 1 < NST ? PWD_VS_BF16 : PWD_KS_BF16);
            __syncthreads();
        }
    }

    if (!w.wave_active || !row_ok) return;
    const float total = l + __shfl_xor(l, 32, 64);
    if (x.partial) {
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
