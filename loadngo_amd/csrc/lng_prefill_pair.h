// =============================================================================================
// Prompt pass, bf16, head width 64, for calls with too few query rows to give every compute unit a
// (64-row query tile, kv head) of its own - the reference feeds a prompt 512 rows at a time
// (gpt-oss/src/engine.rs:51): 64 such pairs on 256 units.
//
// A workgroup takes 64 query rows, one kv head and ONE PAIR of that kv head's query heads, and deals the KEYS out
// among its wavefronts: wavefront w works on query block w & 1 (32 rows), both heads, and every fourth sub-tile of
// 64 keys (kq = w >> 1 of each 256 staged per barrier). There are four times as many workgroups as (query tile, kv
// head) pairs, each as long as before in arithmetic per wavefront (two heads x 64 keys x 32 rows per barrier), and
// what a split between workgroups has to send through memory - a partial output row per split, a merge dispatch that
// reads them back - stays inside the workgroup: at the end the four wavefronts that share a query block exchange
// (maximum, sum, accumulator) through LDS, and each normalises and stores one quarter (head, half of the width).
// The price is K and V staged four times as often (each workgroup stages every key for only two heads): 64 KiB per
// barrier, by loads that write LDS directly and need no registers; the ids put the kv head fastest, so what the 32
// workgroups of a kv head ask for lies in one XCD's L2.
//
// The two staging buffers are two arrays, and the interior loop takes two steps a turn with each buffer named outright:
// with one array and a computed index the compiler cannot tell the rows a direct load is writing from the rows being
// read, and makes the first LDS read after the loads wait for all of them (s_waitcnt vmcnt(0)) - the step after next
// would then arrive before this one's arithmetic starts instead of during it.
//
// LDS rows are 128 bytes, unpadded (a direct load puts lane l's 16 bytes at base + 16 l), swizzled as in
// lng_prefill_bf16_d64_h1w: piece c of K row r at c ^ ((r >> 1) & 7), piece c of V row r at c ^ (((r >> 1) & 1) << 2).
// The arithmetic of a block of 32 keys is lng_prefill_bf16_d64's (two heads per wavefront), with the same three
// modes: maximum tracked; fixed after the first interior sub-tile; fixed at zero when every maximum is moderate -
// and the same range check with a second, tracked attempt when it fails.
// =============================================================================================
#define PP_SUB 64u          // keys per sub-tile (one wavefront's share of a step)
#define PP_STEP 256u        // keys staged per barrier
#define PP_TILE_ELEMS (PP_STEP * 64u)
#define PP_ML_OFF (4u * PP_TILE_ELEMS * 2u)             // bytes: after the four tile buffers (128 KiB)
#define PP_OUT_OFF (PP_ML_OFF + 8u * 2u * 32u * 8u)     // bytes: after the (maximum, sum) table (4 KiB)
#define PP_OUT_STRIDE 40u   // bf16 elements between staged output rows (32 used)
#define PP_LDS_BYTES (PP_OUT_OFF + 8u * 32u * PP_OUT_STRIDE * 2u)

// A 64-bit value that is the same in every lane, as a pointer the compiler knows to be scalar: a load from it plus a
// lane's 32-bit offset takes its base from scalar registers and one vector register for the offset.
__device__ __forceinline__ const char *scalar64(uint64_t x) {
    const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)x), hi = __builtin_amdgcn_readfirstlane((uint32_t)(x >> 32));
    return (const char *)(((uint64_t)hi << 32) | lo);
}

extern "C" __global__ __launch_bounds__(PF_THREADS) void lng_prefill_bf16_d64_pair(lng_k_prefill a) {
    constexpr int NH = 2;
    // [buffer][K, V][256 rows x 64]; after the last step: the accumulators being exchanged, then the table of
    // (maximum, sum) and the outputs on their way to whole-row stores
    // Two arrays, not one with an index: where a step's buffers are named outright the compiler can tell that the rows a
    // direct load is writing are not the rows being read, and does not make every LDS read wait for the loads in flight.
    __shared__ __attribute__((aligned(16))) uint16_t s_buf0[2u * PP_TILE_ELEMS]; // K then V of the even steps (64 KiB)
    __shared__ __attribute__((aligned(16))) uint16_t s_buf1[2u * PP_TILE_ELEMS]; // of the odd steps
    __shared__ __attribute__((aligned(16))) uint16_t s_tail[(PP_LDS_BYTES - PP_ML_OFF) / 2u];
    __shared__ uint32_t s_far, s_again;

    const uint32_t group = a.heads / a.kv_heads;
    const uint32_t pairs = (group + 1u) / 2u;
    const uint32_t g = blockIdx.x % a.kv_heads;
    const uint32_t above = blockIdx.x / a.kv_heads;
    const uint32_t hp = above % pairs;
    const uint32_t qtile = a.q_tiles - 1u - above / pairs;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t qb = wave & 1u;  // block of 32 query rows
    const uint32_t kq = wave >> 1;  // which sub-tile of every four
    // What a lane derives from its number, worked out again where it is needed after the loops (a register that lives
    // across a loop without being used in it is spilled, and a reload waits for every load in flight).
    uint32_t lane, n, hh, k_lane_off, v_lane_off, v_flip, k_ask_off, v_ask_off;
    const uint32_t row_bytes = a.kv_heads * 128u;
    auto lane_values = [&]() __attribute__((always_inline)) {
        uint32_t z = 0u;
        asm volatile("" : "+v"(z));
        lane = __builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, z));
        n = lane & 31u;
        hh = lane >> 5;
        k_lane_off = n * 64u + ((hh ^ ((n >> 1) & 7u)) << 3); // ^ 16 ks, + 2048 per block of 32 keys
        const uint32_t L = lane & 15u;
        const uint32_t blk16 = lane >> 4;
        // transposing read: source lane L names key (L>>2) of its group and dims 4*(L&3).. of the block's 16
        v_lane_off = (4u * (blk16 >> 1) + (L >> 2)) * 64u + 16u * (blk16 & 1u) + 4u * (L & 3u);
        v_flip = (L >> 3) & 1u; // rows two apart within a group of four have their 64-byte halves exchanged
        // asking: a wavefront's 64 lanes fill 8 whole rows; rows 64 i + 8 w + (lane >> 3) of a step, so
        // (row >> 1) & 7 = (4 (w & 1) + (lane >> 4)) & 7 whatever i is
        const uint32_t ld_row = 8u * (wave & 1u) + (lane >> 3), ld_chunk = lane & 7u;
        k_ask_off = (lane >> 3) * row_bytes + ((ld_chunk ^ ((ld_row >> 1) & 7u)) << 4);
        v_ask_off = (lane >> 3) * row_bytes + ((ld_chunk ^ (((ld_row >> 1) & 1u) << 2)) << 4);
    };
    lane_values();
    s_far = 0u; // (every thread, the same value; the first barrier is ahead of their first use)
    s_again = 0u;

    // Positions fit 32 bits (the host refuses shapes whose counts do not).
    const uint32_t t = (uint32_t)a.t, start = (uint32_t)a.start;
    const uint32_t q0 = qtile * 64u;
    const uint32_t rows_here = t - q0 < 64u ? t - q0 : 64u;
    const uint32_t end = start + t;
    const uint32_t pos_first = start + q0;
    const uint32_t pos_last = pos_first + rows_here - 1u;
    const bool windowed = a.window != LNG_WINDOW_FULL; // the host maps window >= end to FULL
    const uint32_t window = windowed ? (uint32_t)a.window : 0u;
    const uint32_t kfirst = (windowed && pos_first + 1u > window) ? pos_first + 1u - window : 0u;
    const uint32_t tile0 = kfirst & ~(PP_SUB - 1u);
    const uint32_t all_tiles = (pos_last - tile0) / PP_SUB + 1u; // sub-tiles of the run
    const uint32_t n_steps = (all_tiles + 3u) / 4u;
    const bool ring = a.slots < end;
    const uint32_t slots = (uint32_t)a.slots;

    uint32_t my_row, my_pos;
    bool row_ok;
    auto row_values = [&]() __attribute__((always_inline)) {
        my_row = q0 + 32u * qb + n;
        my_pos = start + my_row;
        row_ok = my_row < t;
    };
    row_values();
    const bool second_ok = hp * 2u + 1u < group; // an odd group's last pair: the second head repeats the first and is not stored
    uint32_t head[NH];
    head[0] = g * group + hp * 2u;
    head[1] = second_ok ? head[0] + 1u : head[0];
    bf16x8 qreg[NH][4];
    float m[NH], l[NH];
    floatx16 ot[NH][2];
    const float sl2 = a.scale * LNG_LOG2E;
#pragma unroll
    for (int h = 0; h < NH; ++h) {
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) {
            uint4 raw = make_uint4(0, 0, 0, 0);
            if (row_ok) raw = *(const uint4 *)(a.q + (((uint64_t)my_row * a.heads + head[h]) * 64u + 16u * ks + 8u * hh) * 2u);
            // scale * log2(e) goes into the query operand, once (see lng_prefill_bf16_d64)
            bf16x8 qv = as_bf16x8(raw);
#pragma unroll
            for (int e = 0; e < 8; ++e) qv[e] = (__bf16)((float)qv[e] * sl2);
            qreg[h][ks] = qv;
        }
    }
    bf16x2 ones2;
    ones2[0] = (__bf16)1.0f;
    ones2[1] = (__bf16)1.0f;

    // ---- the 256 rows of step s, K and V, into buffer s & 1: four direct loads of each per wavefront --------------
    typedef __attribute__((address_space(1))) const void *gptr;
    typedef __attribute__((address_space(3))) void *lptr;
    auto buf_of = [&](uint32_t s) __attribute__((always_inline)) { return (s & 1u) ? &s_buf1[0] : &s_buf0[0]; };
    auto ask = [&](uint32_t s, uint16_t *dst) __attribute__((always_inline)) {
        const uint32_t kdst = wave * 512u, vdst = kdst + PP_TILE_ELEMS; // elements of dst
        const uint32_t p0 = tile0 + PP_STEP * s;
        if (!ring && p0 >= kfirst && p0 + (PP_STEP - 1u) <= pos_last) {
            // every row is there and wanted: one base per load, worked out by the scalar unit, plus the lane's offset
            const uint64_t kb = (uint64_t)a.k + (uint64_t)g * 128u + (uint64_t)(p0 + 8u * wave) * row_bytes;
            const uint64_t vb = (uint64_t)a.v + (uint64_t)g * 128u + (uint64_t)(p0 + 8u * wave) * row_bytes;
#pragma unroll
            for (uint32_t i = 0; i < PP_STEP / 64u; ++i) { // eight wavefronts x eight rows at a time
                const uint64_t ko = kb + (uint64_t)(64u * i) * row_bytes, vo = vb + (uint64_t)(64u * i) * row_bytes;
                __builtin_amdgcn_global_load_lds((gptr)(scalar64(ko) + k_ask_off), (lptr)&dst[kdst + i * 4096u], 16, 0, 0);
                __builtin_amdgcn_global_load_lds((gptr)(scalar64(vo) + v_ask_off), (lptr)&dst[vdst + i * 4096u], 16, 0, 0);
            }
        } else {
            const uint32_t kc = k_ask_off - (lane >> 3) * row_bytes, vc = v_ask_off - (lane >> 3) * row_bytes;
#pragma unroll
            for (uint32_t i = 0; i < PP_STEP / 64u; ++i) { // eight wavefronts x eight rows at a time
                uint32_t p = p0 + 64u * i + 8u * wave + (lane >> 3);
                p = p > pos_last ? pos_last : p; // rows past the last needed position are masked or never used,
                p = p < kfirst ? kfirst : p;     // and so are rows before the first one (a ring may not hold them any more)
                const uint32_t r = ring ? p % slots : p;
                __builtin_amdgcn_global_load_lds((gptr)(a.k + (uint64_t)g * 128u + (uint64_t)r * row_bytes + kc), (lptr)&dst[kdst + i * 4096u], 16, 0, 0);
                __builtin_amdgcn_global_load_lds((gptr)(a.v + (uint64_t)g * 128u + (uint64_t)r * row_bytes + vc), (lptr)&dst[vdst + i * 4096u], 16, 0, 0);
            }
        }
    };
    auto landed = [&]() __attribute__((always_inline)) {
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); // this wavefront's rows are in LDS
        __syncthreads();
    };

    floatx4 lacc[NH];
    auto selector = [&]() __attribute__((always_inline)) { // built where it is used (see lng_prefill_bf16_d64)
        uint32_t z = 0u;
        asm volatile("" : "+v"(z));
        const uint32_t l31 = __builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, z)) & 31u;
        const uint32_t w = (l31 == 0u || l31 == 17u) ? 0x3f803f80u : 0u;
        return as_bf16x8(make_uint4(w, w, w, w));
    };
    // Three ways to make the pass, each a fallback of the one before: (0) every step at the reference point zero, with no
    // maxima at all, when the run begins with interior steps - the range check below is all that correctness needs (a
    // softmax does not depend on its reference point, only the number range does), and it passes whenever a row's
    // largest score is between about -70 and 80 in the exponent's units; (1) the first interior step with the maxima
    // tracked, the rest fixed there; (2) the maxima tracked throughout.
    constexpr int ATTEMPTS = 3;
    for (int attempt = 0; attempt < ATTEMPTS; ++attempt) {
    const bool optimistic = attempt < 2;
#pragma unroll
    for (int h = 0; h < NH; ++h) {
        m[h] = LNG_NEG_INF; // the sink joins when the wavefronts' states are put together (0 below, for way (0))
        l[h] = 0.0f;
        lacc[h] = floatx4{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int db = 0; db < 2; ++db) {
#pragma unroll
            for (int i = 0; i < 16; ++i) ot[h][db][i] = 0.0f;
        }
    }
    ask(0, s_buf0);
    landed();

    // One block of 32 keys (kb = 0, 1 of the wavefront's sub-tile of step s) for both heads.
    // MODE 0: the running maximum is tracked. MODE 1: it is fixed. MODE 2: it is fixed at zero.
    auto block = [&](auto mask_tag, auto mode_tag, const uint16_t *src, uint32_t s, int kb) __attribute__((always_inline)) {
        constexpr bool MASK = decltype(mask_tag)::value;
        constexpr int MODE = decltype(mode_tag)::value;
        constexpr bool FIXED = MODE != 0;
        const uint32_t kt = kq * 4096u + kb * 2048, vt = kt + PP_TILE_ELEMS; // elements of src
        bf16x8 ka[4];
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) ka[ks] = as_bf16x8(*(const uint4 *)(&src[kt + (k_lane_off ^ (16u * ks))]));
        floatx16 st[NH];
#pragma unroll
        for (int h = 0; h < NH; ++h) {
#pragma unroll
            for (int i = 0; i < 16; ++i) st[h][i] = 0.0f;
        }
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) {
            st[0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ka[ks], qreg[0][ks], st[0], 0, 0, 0);
            st[1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ka[ks], qreg[1][ks], st[1], 0, 0, 0);
        }
        bf16x8 va[2][2];
#pragma unroll
        for (int jj = 0; jj < 2; ++jj) {
#pragma unroll
            for (int db = 0; db < 2; ++db) {
                const uint16_t *vp = &src[vt + v_lane_off + (16 * jj) * 64u + 32 * (db ^ v_flip)];
                va[jj][db] = lds_read_tr8(vp, vp + 8 * 64);
            }
        }
        bf16x8 pb[NH][2];
#pragma unroll
        for (int h = 0; h < NH; ++h) {
            if constexpr (MASK) {
                // key kp = b0 + 4 hh + o_i is visible when 0 <= my_pos - kp < window
                const uint32_t b0 = tile0 + PP_STEP * s + PP_SUB * kq + 32u * kb;
                const int dist = (int)(my_pos - (b0 + 4u * hh));
                const int below = windowed ? dist - (int)window : -0x40000000;
#pragma unroll
                for (int i = 0; i < 16; ++i) {
                    const int o = 8 * (i >> 2) + (i & 3);
                    st[h][i] = (o <= dist && o > below) ? st[h][i] : LNG_NEG_INF;
                }
            }
            float m_safe = 0.0f;
            if constexpr (FIXED) {
                m_safe = m[h];
            } else {
                float tmax = LNG_NEG_INF;
#pragma unroll
                for (int i = 0; i < 16; ++i) tmax = fmaxf(tmax, st[h][i]);
                tmax = other_half_max(tmax);
                const float m_new = tmax > m[h] + PF_TAU ? tmax : m[h];
                m_safe = m_new == LNG_NEG_INF ? 0.0f : m_new;
                if (__builtin_amdgcn_ballot_w64(m_new != m[h]) != 0) {
                    const float alpha = __builtin_amdgcn_exp2f(m[h] - m_safe);
                    l[h] *= alpha;
#pragma unroll
                    for (int db = 0; db < 2; ++db) {
#pragma unroll
                        for (int i = 0; i < 16; ++i) ot[h][db][i] *= alpha;
                    }
                    m[h] = m_new;
                }
            }
            float psum[2] = {0.0f, 0.0f};
#pragma unroll
            for (int jj = 0; jj < 2; ++jj) {
#pragma unroll
                for (int e = 0; e < 8; e += 2) {
                    const float s0 = st[h][8 * jj + e], s1 = st[h][8 * jj + e + 1];
                    const float p0 = __builtin_amdgcn_exp2f(MODE == 2 ? s0 : s0 - m_safe);
                    const float p1 = __builtin_amdgcn_exp2f(MODE == 2 ? s1 : s1 - m_safe);
                    bf16x2 pr;
                    pr[0] = (__bf16)p0;
                    pr[1] = (__bf16)p1;
                    pb[h][jj][e] = pr[0];
                    pb[h][jj][e + 1] = pr[1];
                    // the normaliser sums the same rounded weights the product uses
                    if constexpr (!FIXED) psum[jj] = __builtin_amdgcn_fdot2_f32_bf16(pr, ones2, psum[jj], false);
                }
            }
            if constexpr (!FIXED) l[h] += psum[0] + psum[1];
        }
        if constexpr (FIXED) { // the matrix unit sums the normaliser (see lng_prefill_bf16_d64)
            const bf16x8 sel = selector();
#pragma unroll
            for (int jj = 0; jj < 2; ++jj) {
#pragma unroll
                for (int h = 0; h < NH; ++h) lacc[h] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(sel, pb[h][jj], lacc[h], 0, 0, 0);
            }
        }
#pragma unroll
        for (int jj = 0; jj < 2; ++jj) {
#pragma unroll
            for (int db = 0; db < 2; ++db) {
                ot[0][db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(va[jj][db], pb[0][jj], ot[0][db], 0, 0, 0);
                ot[1][db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(va[jj][db], pb[1][jj], ot[1][db], 0, 0, 0);
            }
        }
    };
    // a sub-tile some query of the workgroup sees only in part: the window's edge or the diagonal
    auto edge = [&](uint32_t j) __attribute__((always_inline)) {
        const uint32_t kt0 = tile0 + j * PP_SUB;
        return kt0 + (PP_SUB - 1u) > pos_first || (windowed && kt0 + window < pos_first + 64u);
    };
    // a step whose four sub-tiles every query sees whole (edges lie at the two ends of the run only)
    auto interior = [&](uint32_t s) __attribute__((always_inline)) { return 4u * s + 3u < all_tiles && !edge(4u * s) && !edge(4u * s + 3u); };
    using tracked = std::integral_constant<int, 0>;
    using fixed_at_m = std::integral_constant<int, 1>;
    using fixed_at_zero = std::integral_constant<int, 2>;
    // a step of any kind, the maximum tracked: each wavefront looks at its own sub-tile
    auto any_step = [&](uint32_t s) __attribute__((always_inline)) {
        if (s + 1u < n_steps) ask(s + 1u, buf_of(s + 1u));
        const uint32_t j = 4u * s + kq;
        if (j < all_tiles) {
            if (edge(j)) {
                block(std::true_type{}, tracked{}, buf_of(s), s, 0);
                block(std::true_type{}, tracked{}, buf_of(s), s, 1);
            } else {
                block(std::false_type{}, tracked{}, buf_of(s), s, 0);
                block(std::false_type{}, tracked{}, buf_of(s), s, 1);
            }
        }
    };
    auto fixed_step = [&](auto mode_tag, uint32_t s) __attribute__((always_inline)) {
        if (s + 1u < n_steps) ask(s + 1u, buf_of(s + 1u));
        block(std::false_type{}, mode_tag, buf_of(s), s, 0);
        block(std::false_type{}, mode_tag, buf_of(s), s, 1);
        landed();
    };
    uint32_t s = 0;
    bool frozen = false, at_zero = false;
    const bool speculate = attempt == 0 && interior(0) && interior(1);
    if (speculate) {
        frozen = true;
        at_zero = true;
#pragma unroll
        for (int h = 0; h < NH; ++h) m[h] = 0.0f;
    } else {
    for (; s < n_steps && !(optimistic && interior(s)); ++s) { // all of a tracked attempt; else up to the first interior step
        any_step(s);
        landed();
    }
    if (optimistic && s + 1u < n_steps && interior(s + 1u)) {
        // the first interior step sets every wavefront's maxima from real scores; from the second on they are fixed -
        // at zero when all of them, in all of the workgroup, are moderate (|m| <= 40 in the exponent's units)
        any_step(s);
        ++s;
        frozen = true;
        bool moderate = true;
#pragma unroll
        for (int h = 0; h < NH; ++h) {
            m[h] = m[h] == LNG_NEG_INF ? 0.0f : m[h];
            moderate = moderate && __builtin_fabsf(m[h]) <= 40.0f;
        }
        if (__builtin_amdgcn_ballot_w64(!moderate) != 0) s_far = 1u;
        landed();
        at_zero = s_far == 0u; // (never cleared: what it says of the scores holds for a later attempt as well)
        if (at_zero) {
#pragma unroll
            for (int h = 0; h < NH; ++h) {
                const float up = __builtin_amdgcn_exp2f(m[h]);
                l[h] *= up;
#pragma unroll
                for (int db = 0; db < 2; ++db) {
#pragma unroll
                    for (int i = 0; i < 16; ++i) ot[h][db][i] *= up;
                }
                m[h] = 0.0f;
            }
        }
    }
    }
    if (frozen) { // loops of their own: one path through each
        if (at_zero) {
            if ((s & 1u) && s < n_steps && interior(s)) { // to an even step first
                fixed_step(fixed_at_zero{}, s);
                ++s;
            }
            for (; s + 1u < n_steps && interior(s + 1u); s += 2u) { // two steps a turn, their buffers named outright
                ask(s + 1u, s_buf1);
                block(std::false_type{}, fixed_at_zero{}, s_buf0, s, 0);
                block(std::false_type{}, fixed_at_zero{}, s_buf0, s, 1);
                landed();
                if (s + 2u < n_steps) ask(s + 2u, s_buf0);
                block(std::false_type{}, fixed_at_zero{}, s_buf1, s + 1u, 0);
                block(std::false_type{}, fixed_at_zero{}, s_buf1, s + 1u, 1);
                landed();
            }
            for (; s < n_steps && interior(s); ++s) fixed_step(fixed_at_zero{}, s);
            // the step of the diagonal at the same reference point and ahead of the check, which then covers it (a
            // masked score is 2^-inf = 0; every sub-tile through the masks, so that there is one more form of the block only)
            for (; s < n_steps; ++s) {
                if (s + 1u < n_steps) ask(s + 1u, buf_of(s + 1u));
                if (4u * s + kq < all_tiles) {
                    block(std::true_type{}, fixed_at_zero{}, buf_of(s), s, 0);
                    block(std::true_type{}, fixed_at_zero{}, buf_of(s), s, 1);
                }
                landed();
            }
        } else {
            for (; s < n_steps && interior(s); ++s) fixed_step(fixed_at_m{}, s);
        }
    }
    lane_values();
    row_values();
    bool again = false;
    if (frozen) { // uniform over the workgroup
        // query n's sum is in lane n % 16, register n / 16; l[] is per (query, half) and the halves are added at the
        // end, so the whole of it goes to the first half
        int bad = 0;
#pragma unroll
        for (int h = 0; h < NH; ++h) {
            const float lo = __shfl(lacc[h][0], (int)(n & 15u), 64);
            const float hi = __shfl(lacc[h][1], (int)(n & 15u), 64);
            if (hh == 0u) l[h] += n < 16u ? lo : hi;
            lacc[h] = floatx4{0.0f, 0.0f, 0.0f, 0.0f};
            const float total = l[h] + __shfl_xor(l[h], 32, 64);
            uint32_t top = 0;
#pragma unroll
            for (int db = 0; db < 2; ++db) {
#pragma unroll
                for (int i = 0; i < 16; ++i) top = max(top, __float_as_uint(ot[h][db][i]) & 0x7fffffffu);
            }
            // 2^-90 .. 2^100 and every accumulator finite (a NaN fails the comparison)
            bad |= !(total >= 8.0779357e-28f && total <= 1.2676506e30f) || top >= 0x7f800000u;
        }
        bad = row_ok ? bad : 0;
        if (__builtin_amdgcn_ballot_w64(bad != 0) != 0) s_again = 1u;
        __syncthreads();
        again = s_again != 0u;
        if (again) {
            __syncthreads(); // everyone has read it
            s_again = 0u;    // for the next attempt's check: its barriers lie between
            if (a.second_passes && wave == 0u && lane == 0u) __hip_atomic_fetch_add(a.second_passes, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            if (!speculate) attempt = 1; // fixing the maxima after a tracked step has failed: track them throughout
        }
    }
    if (!again) {
        for (; s < n_steps; ++s) { // the diagonal
            any_step(s);
            landed();
        }
        break;
    }
    }

    // ---- the four wavefronts of a query block put their states together ------------------------------------------
    // Every wavefront lays down its (maximum, sum) per row and head and its four accumulator pieces (head, half of the
    // width: 32 rows x 32 dims, a lane's 16 values as four 16-byte words, word-major so that the 64 lanes of a store
    // or load are consecutive); wavefront kq then owns piece kq = 2 head + half. The last step's barrier has passed:
    // nobody reads K or V any more.
    lane_values();
    row_values();
    float *const xch = (float *)(qb ? &s_buf1[0] : &s_buf0[0]); // a query block's 64 KiB
    float2 *const ml = (float2 *)&s_tail[0];
#pragma unroll
    for (int h = 0; h < NH; ++h) {
        const float total = l[h] + __shfl_xor(l[h], 32, 64);
        if (hh == 0u) ml[((qb * 4u + kq) * 2u + h) * 32u + n] = make_float2(m[h], total);
#pragma unroll
        for (int db = 0; db < 2; ++db) {
            float *const dst = xch + (((((2u * h + db)) * 4u + kq) * 4u) * 64u + lane) * 4u;
#pragma unroll
            for (int blk = 0; blk < 4; ++blk) {
                *(float4 *)(dst + blk * 256u) = make_float4(ot[h][db][4 * blk + 0], ot[h][db][4 * blk + 1], ot[h][db][4 * blk + 2], ot[h][db][4 * blk + 3]);
            }
        }
    }
    __syncthreads();
    const uint32_t h_own = kq >> 1, db_own = kq & 1u;
    if (h_own == 1u && !second_ok) return;
    const uint32_t head_own = head[0] + h_own;
    const float sink = a.sinks ? a.sinks[head_own] * LNG_LOG2E : LNG_NEG_INF;
    float mk[4], lk[4], top = sink;
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        const float2 e = ml[((qb * 4u + k) * 2u + h_own) * 32u + n];
        mk[k] = e.x;
        lk[k] = e.y;
        top = fmaxf(top, e.x);
    }
    float total = (a.sinks && top != LNG_NEG_INF) ? __builtin_amdgcn_exp2f(sink - top) : 0.0f;
    float w[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        w[k] = mk[k] == LNG_NEG_INF ? 0.0f : __builtin_amdgcn_exp2f(mk[k] - top);
        total += lk[k] * w[k];
    }
    const float inv = total > 0.0f ? 1.0f / total : 0.0f;
    uint16_t *const stage = &s_tail[(PP_OUT_OFF - PP_ML_OFF) / 2u + wave * (32u * PP_OUT_STRIDE)];
#pragma unroll
    for (int blk = 0; blk < 4; ++blk) {
        float4 sum = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            const float4 piece = *(const float4 *)(xch + (((kq * 4u + k) * 4u + blk) * 64u + lane) * 4u);
            const float wk = w[k] * inv;
            // (a wavefront that saw no key left zeros and has weight 0: no NaN from 0 x inf, its piece is finite)
            sum.x = __builtin_fmaf(piece.x, wk, sum.x);
            sum.y = __builtin_fmaf(piece.y, wk, sum.y);
            sum.z = __builtin_fmaf(piece.z, wk, sum.z);
            sum.w = __builtin_fmaf(piece.w, wk, sum.w);
        }
        bf16x4 o; // narrowed by the conversion instruction (round to nearest even)
        o[0] = (__bf16)sum.x;
        o[1] = (__bf16)sum.y;
        o[2] = (__bf16)sum.z;
        o[3] = (__bf16)sum.w;
        *(bf16x4 *)(stage + n * PP_OUT_STRIDE + 8 * blk + 4 * hh) = o;
    }
    __builtin_amdgcn_wave_barrier();
    // four lanes store the 64 bytes this wavefront has of a row
#pragma unroll
    for (int pass = 0; pass < 2; ++pass) {
        const uint32_t r = 16u * pass + (lane >> 2), ch = lane & 3u;
        const uint4 piece = *(const uint4 *)(stage + r * PP_OUT_STRIDE + 8u * ch);
        const uint32_t row = q0 + 32u * qb + r;
        if (row < t) *(uint4 *)((uint16_t *)a.out + ((uint64_t)row * a.heads + head_own) * 64u + 32u * db_own + 8u * ch) = piece;
    }
}
