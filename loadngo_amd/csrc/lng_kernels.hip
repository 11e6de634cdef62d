// gfx950 (CDNA4) kernels of the grouped-attention operator: compiled to one code object
// (hipcc --genco) that the host library embeds and loads with hipModuleLoadData.
//
// What every kernel here computes is the operator of metal-compute (apple.rs:1199-1401,
// kernels.metal:500-720 and 1944-2032), itself the GPU twin of gpt-oss/src/model.rs:434-464:
//   for each query i at absolute position last = start + i, head h, kv head g = h / (H/G):
//     first = max(0, last + 1 - window);  s_p = (q . k_p) * scale for p in first..=last
//     m = max(sink, max_p s_p);  Z = exp(sink - m) + sum_p exp(s_p - m)
//     out = sum_p exp(s_p - m) / Z * v_p                      (position p is in row p % slots)
// The kernels that carry the load (head widths 64, 128, 256 and 512, groups of up to 16 query heads per kv head)
// choose their work split, layouts and reductions for 64-wide wavefronts, MFMA and HBM streaming: K and V are read
// once per kv head, long rows are cut into chunks. One kernel keeps the reference's own split of a workgroup per
// (row, head) - lng_attn_generic_* - and serves only what is left: other widths, larger groups, scales that are
// not positive, operands off 16-byte boundaries.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <type_traits>

#include "lng_kernel_args.h"

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef float floatx16 __attribute__((ext_vector_type(16)));

#define LNG_LOG2E 1.4426950408889634f
#define LNG_NEG_INF (-__builtin_huge_valf())

// ---- element helpers (weights/src/dtype.rs:95-116: widen is a shift, narrow is RNE) --------
__device__ __forceinline__ float bf16_bits_to_f32(uint16_t bits) {
    return __uint_as_float((uint32_t)bits << 16);
}

__device__ __forceinline__ uint16_t f32_to_bf16_bits(float value) {
    uint32_t bits = __float_as_uint(value);
    if (value != value) return (uint16_t)((bits >> 16) | 0x40);
    uint32_t bias = 0x7fffu + ((bits >> 16) & 1u);
    return (uint16_t)((bits + bias) >> 16);
}

template <typename T> __device__ __forceinline__ float load_elem(const T *p);
template <> __device__ __forceinline__ float load_elem<float>(const float *p) { return *p; }
template <> __device__ __forceinline__ float load_elem<uint16_t>(const uint16_t *p) {
    return bf16_bits_to_f32(*p);
}
template <typename T> __device__ __forceinline__ void store_elem(T *p, float x);
template <> __device__ __forceinline__ void store_elem<float>(float *p, float x) { *p = x; }
template <> __device__ __forceinline__ void store_elem<uint16_t>(uint16_t *p, float x) {
    *p = f32_to_bf16_bits(x);
}

__device__ __forceinline__ lng_k_row row_of(const lng_k_attn &a, uint32_t r) {
    if (a.rows) return a.rows[r];
    lng_k_row it = a.first;
    const uint64_t step = (uint64_t)a.heads * a.dim * (a.dtype == LNG_BF16 ? 2u : 4u);
    it.q_offset += r * step;
    it.out_offset += r * step;
    it.start += r;
    return it;
}

__device__ __forceinline__ uint64_t first_visible(uint64_t last, uint64_t window) {
    return (window != LNG_WINDOW_FULL && last + 1 > window) ? last + 1 - window : 0;
}

// Which (row, kv head) pair and which chunk of its visible run a decode workgroup takes. With rows of
// unequal length the host gives cum[r] = workgroups of the rows before r (cum[n_rows] = the grid), so
// that no workgroup is launched only to return: workgroup w finds the last r with cum[r] <= w by a
// 64-way search (every lane looks at one entry, a ballot counts), in one step for up to 64 rows and
// one more per factor of 64; within the row its workgroups go kv head by kv head, chunks the fast
// index. Without the table: a rectangle of n_chunks per pair, chunks the fast index.
struct work_item {
    uint32_t pair;
    uint32_t chunk;
};
__device__ __forceinline__ work_item work_of(const lng_k_attn &a) {
    work_item w;
    if (a.work) {
        const uint32_t lane = threadIdx.x & 63u;
        uint32_t lo = 0, n = a.n_rows; // the row is in [lo, lo + n)
        while (n > 64u) {
            const uint32_t stride = (n + 63u) / 64u;
            const uint32_t i = lo + lane * stride;
            const bool here = lane * stride < n && a.work[i] <= blockIdx.x;
            const uint32_t cnt = (uint32_t)__builtin_popcountll(__builtin_amdgcn_ballot_w64(here)); // >= 1: cum[lo] <= w
            const uint32_t step = (cnt - 1u) * stride;
            n = n - step < stride ? n - step : stride;
            lo += step;
        }
        const bool here = lane < n && a.work[lo + lane] <= blockIdx.x;
        const uint32_t row = lo + (uint32_t)__builtin_popcountll(__builtin_amdgcn_ballot_w64(here)) - 1u;
        const uint32_t c0 = a.work[row], c1 = a.work[row + 1u];
        const uint32_t live = (c1 - c0) / a.kv_heads; // chunks of this row
        const uint32_t local = blockIdx.x - c0;
        w.pair = row * a.kv_heads + local / live;
        w.chunk = local % live;
    } else {
        w.pair = blockIdx.x / a.n_chunks;
        w.chunk = blockIdx.x % a.n_chunks;
    }
    w.pair = __builtin_amdgcn_readfirstlane(w.pair);
    w.chunk = __builtin_amdgcn_readfirstlane(w.chunk);
    return w;
}

// Sum over the 64 lanes, in every lane: four steps inside each row of 16 lanes with data-parallel
// primitives (neighbour, pair, mirrored half row, mirrored row), then the two lane-swap instructions
// across rows. All VALU: the shuffle form goes through the LDS crossbar six times, one after the other.
__device__ __forceinline__ float wave_sum(float x) {
    auto dpp = [](float v, auto ctrl) {
        return __uint_as_float((uint32_t)__builtin_amdgcn_update_dpp(0, (int)__float_as_uint(v), decltype(ctrl)::value, 0xf, 0xf, true));
    };
    x += dpp(x, std::integral_constant<int, 0xB1>{});  // quad_perm [1,0,3,2]
    x += dpp(x, std::integral_constant<int, 0x4E>{});  // quad_perm [2,3,0,1]
    x += dpp(x, std::integral_constant<int, 0x141>{}); // row_half_mirror
    x += dpp(x, std::integral_constant<int, 0x140>{}); // row_mirror
    const auto a = __builtin_amdgcn_permlane16_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    x = __uint_as_float(a[0]) + __uint_as_float(a[1]);
    const auto b = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    return __uint_as_float(b[0]) + __uint_as_float(b[1]);
}

// =============================================================================================
// Generic kernel: any element type, any head width up to 512, any group size. One workgroup
// per (row, head) (the reference's split, kernels.metal:500-560: each query head reads its kv head's
// rows again); its four wavefronts take every fourth position, lanes split the head
// dimension; per-wavefront online softmax, merged in LDS with the sink joining the merge.
// The remainder kernel: head widths other than 64, 128, 256, 512, groups of more than 16 query heads,
// f32 with a scale that is not positive, operands off 16-byte boundaries. Accurate exp/divide.
// =============================================================================================
template <typename T>
__device__ __forceinline__ void attn_generic(const lng_k_attn &a) {
    __shared__ float s_m[4];
    __shared__ float s_l[4];
    __shared__ float s_acc[4][512];
    const uint32_t row = blockIdx.x / a.heads;
    const uint32_t head = blockIdx.x % a.heads;
    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t wave = threadIdx.x >> 6;
    const lng_k_row it = row_of(a, row);
    const uint32_t dim = a.dim;
    const uint32_t g = head / (a.heads / a.kv_heads);
    const T *q = (const T *)(a.q + it.q_offset) + (uint64_t)head * dim;
    const T *kb = (const T *)(a.k + it.k_offset) + (uint64_t)g * dim;
    const T *vb = (const T *)(a.v + it.v_offset) + (uint64_t)g * dim;
    const uint64_t stride = (uint64_t)a.kv_heads * dim;
    const uint64_t last = it.start;
    const uint64_t first = first_visible(last, it.window);

    float qv[8], acc[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const uint32_t d = lane + 64u * i;
        qv[i] = d < dim ? load_elem<T>(q + d) : 0.0f;
        acc[i] = 0.0f;
    }
    float m = LNG_NEG_INF, l = 0.0f;
    uint64_t p = first + wave;
    if (dim <= 64u) {
        // One element per lane and row: sixteen of the wavefront's positions at a time, all their K and V
        // loads in flight together (one position per turn is a chain of memory latencies, 1 ms for 4,096
        // keys), then one block step of the online softmax.
        constexpr int U = 16;
        const bool mine = lane < dim;
        for (; p <= last; p += 4u * U) {
            float kx[U], vx[U], sc[U];
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const uint64_t pu = p + 4u * u;
                const uint64_t r = (pu <= last ? pu : last) % it.slots;
                kx[u] = mine ? load_elem<T>(kb + r * stride + lane) : 0.0f;
                vx[u] = mine ? load_elem<T>(vb + r * stride + lane) : 0.0f;
            }
            float top = LNG_NEG_INF;
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const float s = wave_sum(qv[0] * kx[u]) * a.scale;
                sc[u] = p + 4u * u <= last ? s : LNG_NEG_INF;
                top = fmaxf(top, sc[u]);
            }
            const float next = fmaxf(m, top); // the first position of the block is always a real one
            const float keep = m == LNG_NEG_INF ? 0.0f : expf(m - next);
            l *= keep;
            acc[0] *= keep;
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const float w = sc[u] == LNG_NEG_INF ? 0.0f : expf(sc[u] - next);
                l += w;
                acc[0] += w * vx[u];
            }
            m = next;
        }
    }
    for (; p <= last; p += 4) {
        const uint64_t r = p % it.slots;
        const T *kr = kb + r * stride;
        const T *vr = vb + r * stride;
        float part = 0.0f;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const uint32_t d = lane + 64u * i;
            if (d < dim) part += qv[i] * load_elem<T>(kr + d);
        }
        const float s = wave_sum(part) * a.scale;
        const float next = fmaxf(m, s);
        const float keep = m == LNG_NEG_INF ? 0.0f : expf(m - next);
        const float w = expf(s - next);
        l = l * keep + w;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const uint32_t d = lane + 64u * i;
            if (d < dim) acc[i] = acc[i] * keep + w * load_elem<T>(vr + d);
        }
        m = next;
    }
    if (lane == 0) {
        s_m[wave] = m;
        s_l[wave] = l;
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const uint32_t d = lane + 64u * i;
        if (d < dim) s_acc[wave][d] = acc[i];
    }
    __syncthreads();
    const float sink = it.sinks_offset != LNG_NO_SINKS
                           ? ((const float *)(a.sinks + it.sinks_offset))[head]
                           : LNG_NEG_INF;
    float top = sink;
#pragma unroll
    for (int w = 0; w < 4; ++w) top = fmaxf(top, s_m[w]);
    float total = sink == LNG_NEG_INF ? 0.0f : expf(sink - top);
    float weight[4];
#pragma unroll
    for (int w = 0; w < 4; ++w) {
        weight[w] = s_m[w] == LNG_NEG_INF ? 0.0f : expf(s_m[w] - top);
        total += s_l[w] * weight[w];
    }
    T *o = (T *)(a.out + it.out_offset) + (uint64_t)head * dim;
    for (uint32_t d = threadIdx.x; d < dim; d += 256) {
        float sum = 0.0f;
#pragma unroll
        for (int w = 0; w < 4; ++w) sum += s_acc[w][d] * weight[w];
        store_elem<T>(o + d, sum / total);
    }
}

extern "C" __global__ __launch_bounds__(256) void lng_attn_generic_f32(lng_k_attn a) {
    attn_generic<float>(a);
}

extern "C" __global__ __launch_bounds__(256) void lng_attn_generic_bf16(lng_k_attn a) {
    attn_generic<uint16_t>(a);
}

// =============================================================================================
// Decode kernel, bf16, head width 64, up to 16 query heads per kv head.
//
// Grid: one workgroup per (row, kv head, chunk), see work_of; a row of v visible positions has
// ceil(v / a.chunk) chunks, and chunk c of n is the groups of 128 positions c, c + n, c + 2n, ... of the
// row. A workgroup serves ALL query heads of its kv head at once, so each cached K and V row is read
// from HBM once per group instead of once per query head. Its four wavefronts take a tile of 32
// positions of each group. Everything is lane-local between the three MFMA stages:
//
//   S^T[tok][head] = K[tok][:] . Q[head][:]        2x2 v_mfma_f32_16x16x32_bf16 per tile
//       lane (n = lane%16, j = lane/16) loads, for token half*16 + n, the 16 bytes at
//       step*64 + j*16 of the 128-byte K row (global_load_dwordx4): the four lanes of a token
//       read one contiguous 64-byte half row per instruction, both halves make the 128-byte
//       run. Q is loaded with the same (step, j) -> bytes rule, so the contraction order is
//       consistent whatever order the hardware gives the 32 k-slots.
//       Result: lane holds S^T[half*16 + 4j + i][head n], i = 0..3.
//   V^T block[dim][tok]: V rows are loaded exactly like K rows (row-major, coalesced) and
//       transposed on the matrix unit: D = V[tok][k-slots] . E, E a 0/1 selection matrix,
//       gives lane (n, j) the values V[half*16 + 4j + i][16m + n]: four positions of one
//       dimension, exact because 1.0 * bf16 accumulates exactly in f32.
//   O^T[dim][head] += V^T[dim][tok] . P^T[tok][head]: the A operand is the lane's own
//       transposed V values, the B operand the lane's own exp'd scores, both narrowed to bf16.
//
// Online softmax state per lane: running max of its head (log2 domain), its share of the
// running sum, and 16 accumulators O^T[16m + 4j + i][n]. Wavefronts merge through LDS; with
// one chunk the workgroup writes the output (sink folded into the normaliser), otherwise it
// writes (max, sum, O) partials; these are merged by the workgroup that finishes last (small
// grids, where a second dispatch would cost more than the chunks themselves) or by
// lng_decode_merge as the next dispatch (large grids).
// =============================================================================================
__device__ __forceinline__ bf16x8 as_bf16x8(uint4 x) { return __builtin_bit_cast(bf16x8, x); }

__device__ __forceinline__ bf16x8 narrow8(floatx4 lo, floatx4 hi) {
    bf16x8 r;
    r[0] = (__bf16)lo[0];
    r[1] = (__bf16)lo[1];
    r[2] = (__bf16)lo[2];
    r[3] = (__bf16)lo[3];
    r[4] = (__bf16)hi[0];
    r[5] = (__bf16)hi[1];
    r[6] = (__bf16)hi[2];
    r[7] = (__bf16)hi[3];
    return r;
}

// Merges the split-K partials of one (row, kv head): 16 threads per head first turn the chunks'
// (max, sum) pairs into weights in LDS and the head's normaliser; then each thread owns outputs
// (head, dim) and streams the chunks' partial rows with independent loads. The sink joins here,
// once: exp(sink - max) in the normaliser and no value. COHERENT: the partials were written by
// other workgroups of the same dispatch and are read with device-coherent loads.
template <bool COHERENT> __device__ __forceinline__ float load_partial(const float *p) {
    if (COHERENT) return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    return *p;
}

template <bool COHERENT>
__device__ __forceinline__ void merge_chunks(const lng_k_attn &a, const lng_k_row &it, uint32_t pair, uint32_t g,
                                             uint32_t group, uint32_t row_chunks) {
    __shared__ float s_w[16][LNG_MAX_CHUNKS];
    __shared__ float s_z[16];
    {
        const uint32_t h = threadIdx.x >> 4, t16 = threadIdx.x & 15u;
        if (h < group) {
            const uint32_t head = g * group + h;
            const uint64_t slot0 = ((uint64_t)pair * a.n_chunks) * group + h;
            const float sink2 = it.sinks_offset != LNG_NO_SINKS
                                    ? ((const float *)(a.sinks + it.sinks_offset))[head] * LNG_LOG2E
                                    : LNG_NEG_INF;
            float top = sink2;
            for (uint32_t c = t16; c < row_chunks; c += 16u) {
                const float mc = load_partial<COHERENT>(&a.partial_ml[(slot0 + (uint64_t)c * group) * 2u]);
                s_w[h][c] = mc;
                top = fmaxf(top, mc);
            }
#pragma unroll
            for (int s = 8; s >= 1; s >>= 1) top = fmaxf(top, __shfl_xor(top, s, 64));
            float z = 0.0f;
            for (uint32_t c = t16; c < row_chunks; c += 16u) {
                const float lc = load_partial<COHERENT>(&a.partial_ml[(slot0 + (uint64_t)c * group) * 2u + 1u]);
                const float mc = s_w[h][c];
                const float wt = mc == LNG_NEG_INF ? 0.0f : __builtin_amdgcn_exp2f(mc - top);
                s_w[h][c] = wt;
                z += lc * wt;
            }
#pragma unroll
            for (int s = 8; s >= 1; s >>= 1) z += __shfl_xor(z, s, 64);
            if (t16 == 0) s_z[h] = z + (sink2 == LNG_NEG_INF ? 0.0f : __builtin_amdgcn_exp2f(sink2 - top));
        }
    }
    __syncthreads();
    for (uint32_t idx = threadIdx.x; idx < group * 64u; idx += 256u) {
        const uint32_t h = idx >> 6;
        const uint32_t d = idx & 63u;
        const float *po = a.partial_o + (((uint64_t)pair * a.n_chunks) * group + h) * 64u + d;
        const uint64_t step = (uint64_t)group * 64u;
        // sixteen loads in flight per turn: the merge is a chain of memory latencies otherwise
        float o0 = 0.0f, o1 = 0.0f, o2 = 0.0f, o3 = 0.0f;
        uint32_t c = 0;
        for (; c + 16 <= row_chunks; c += 16) {
            float x[16];
#pragma unroll
            for (int u = 0; u < 16; ++u) x[u] = load_partial<COHERENT>(po + (c + u) * step);
#pragma unroll
            for (int u = 0; u < 16; u += 4) {
                o0 += x[u] * s_w[h][c + u];
                o1 += x[u + 1] * s_w[h][c + u + 1];
                o2 += x[u + 2] * s_w[h][c + u + 2];
                o3 += x[u + 3] * s_w[h][c + u + 3];
            }
        }
        for (; c + 4 <= row_chunks; c += 4) {
            const float x0 = load_partial<COHERENT>(po + (c + 0) * step);
            const float x1 = load_partial<COHERENT>(po + (c + 1) * step);
            const float x2 = load_partial<COHERENT>(po + (c + 2) * step);
            const float x3 = load_partial<COHERENT>(po + (c + 3) * step);
            o0 += x0 * s_w[h][c];
            o1 += x1 * s_w[h][c + 1];
            o2 += x2 * s_w[h][c + 2];
            o3 += x3 * s_w[h][c + 3];
        }
        for (; c < row_chunks; ++c) o0 += load_partial<COHERENT>(po + c * step) * s_w[h][c];
        const float res = ((o0 + o1) + (o2 + o3)) / s_z[h];
        const uint64_t at = ((uint64_t)g * group + h) * 64u + d;
        if (a.dtype == LNG_F32) {
            ((float *)(a.out + it.out_offset))[at] = res;
        } else {
            ((uint16_t *)(a.out + it.out_offset))[at] = f32_to_bf16_bits(res);
        }
    }
}

struct kv_tile {
    uint4 k[2][2]; // [position half][k step]
    uint4 v[2][2];
};

__device__ __forceinline__ void decode_bf16_d64_body(const lng_k_attn a) {
    __shared__ float s_m[4][16];
    __shared__ float s_l[4][16];
    __shared__ float s_o[4][16][65];

    const work_item wi = work_of(a);
    const uint32_t row = wi.pair / a.kv_heads;
    const uint32_t g = wi.pair % a.kv_heads;
    const lng_k_row it = row_of(a, row);
    const uint64_t last = it.start;
    const uint64_t first = first_visible(last, it.window);
    const uint64_t base = first & ~(uint64_t)31;
    const uint32_t row_chunks = (uint32_t)((last + 1 - base + a.chunk - 1) / a.chunk);
    if (wi.chunk >= row_chunks) return; // this row has fewer chunks than the longest one
    // The row's workgroups take interleaved groups of 128 positions (workgroup c: groups c, c + chunks, ...), not
    // a run of a.chunk positions each: together they sweep one window of the row, and every workgroup of a row
    // has the same number of groups to within one, however the row's length divides.
    const uint64_t c0 = base + (uint64_t)wi.chunk * 128u;
    const uint64_t c1 = last + 1;
    const uint64_t tile_stride = 128ull * row_chunks;

    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t wave = threadIdx.x >> 6;
    const uint32_t n = lane & 15u;
    const uint32_t j = lane >> 4;
    const uint32_t group = a.heads / a.kv_heads;
    const bool wraps = it.slots <= last;
    const uint64_t row_bytes = (uint64_t)a.kv_heads * 128u;
    const char *kb = a.k + it.k_offset + (uint64_t)g * 128u + j * 16u;
    const char *vb = a.v + it.v_offset + (uint64_t)g * 128u + j * 16u;

    // Q^T operand: head n of this group, the lane's 8 k-slots of each step.
    bf16x8 qb[2];
    {
        uint4 q0 = make_uint4(0, 0, 0, 0), q1 = q0;
        if (n < group) {
            const char *qp = a.q + it.q_offset + ((uint64_t)g * group + n) * 128u + j * 16u;
            q0 = *(const uint4 *)qp;
            q1 = *(const uint4 *)(qp + 64);
        }
        qb[0] = as_bf16x8(q0);
        qb[1] = as_bf16x8(q1);
    }
    // Selection operands of the transposing product: slot (j, e) of a 32-wide step holds
    // dimension 8j + e; column n of block parity b wants dimension 16b + n.
    bf16x8 sel[2];
#pragma unroll
    for (int b = 0; b < 2; ++b) {
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            sel[b][e] = (8u * j + (uint32_t)e == 16u * (uint32_t)b + n) ? (__bf16)1.0f : (__bf16)0.0f;
        }
    }

    auto load_tile = [&](uint64_t tp, kv_tile &t) {
#pragma unroll
        for (int half = 0; half < 2; ++half) {
            uint64_t p = tp + (uint64_t)(half * 16) + n;
            p = p < first ? first : p;
            p = p > last ? last : p;
            const uint64_t r = wraps ? p % it.slots : p;
            const uint64_t off = r * row_bytes;
            t.k[half][0] = *(const uint4 *)(kb + off);
            t.k[half][1] = *(const uint4 *)(kb + off + 64);
            t.v[half][0] = *(const uint4 *)(vb + off);
            t.v[half][1] = *(const uint4 *)(vb + off + 64);
        }
    };

    const float sl2 = a.scale * LNG_LOG2E;
    float m = LNG_NEG_INF; // running max of head n, log2 domain
    float l = 0.0f;        // this lane's share of the running sum
    floatx4 ot[4];         // O^T[16mm + 4j + i][head n]
#pragma unroll
    for (int mm = 0; mm < 4; ++mm) ot[mm] = (floatx4){0.f, 0.f, 0.f, 0.f};
    const floatx4 zero4 = (floatx4){0.f, 0.f, 0.f, 0.f};

    kv_tile cur, nxt;
    uint64_t tp = c0 + (uint64_t)wave * 32u;
    if (tp < c1) load_tile(tp, cur);
    for (; tp < c1; tp += tile_stride) {
        const uint64_t tn = tp + tile_stride;
        if (tn < c1) load_tile(tn, nxt);

        floatx4 st[2];
#pragma unroll
        for (int half = 0; half < 2; ++half) {
            st[half] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(cur.k[half][0]), qb[0], zero4, 0, 0, 0);
            st[half] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(cur.k[half][1]), qb[1], st[half], 0, 0, 0);
        }
        float tmax = LNG_NEG_INF;
#pragma unroll
        for (int half = 0; half < 2; ++half) {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const uint64_t p = tp + (uint64_t)(half * 16 + i) + 4u * j;
                const float x = (p >= first && p <= last) ? st[half][i] * sl2 : LNG_NEG_INF;
                st[half][i] = x;
                tmax = fmaxf(tmax, x);
            }
        }
        tmax = fmaxf(tmax, __shfl_xor(tmax, 16, 64));
        tmax = fmaxf(tmax, __shfl_xor(tmax, 32, 64));
        const float m_new = fmaxf(m, tmax);
        const float m_safe = m_new == LNG_NEG_INF ? 0.0f : m_new;
        const float alpha = __builtin_amdgcn_exp2f(m - m_safe);
        float psum = 0.0f;
#pragma unroll
        for (int half = 0; half < 2; ++half) {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const float pw = __builtin_amdgcn_exp2f(st[half][i] - m_safe);
                st[half][i] = pw;
                psum += pw;
            }
        }
        l = l * alpha + psum;
        m = m_new;
        const bf16x8 pb = narrow8(st[0], st[1]);
#pragma unroll
        for (int mm = 0; mm < 4; ++mm) {
            const floatx4 t0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(cur.v[0][mm >> 1]), sel[mm & 1], zero4, 0, 0, 0);
            const floatx4 t1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(cur.v[1][mm >> 1]), sel[mm & 1], zero4, 0, 0, 0);
            const bf16x8 va = narrow8(t0, t1);
            ot[mm] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(va, pb, ot[mm] * alpha, 0, 0, 0);
        }
        cur = nxt;
    }

    // ---- merge the four wavefronts ---------------------------------------------------------
    {
        float lt = l + __shfl_xor(l, 16, 64);
        lt += __shfl_xor(lt, 32, 64);
        if (j == 0) {
            s_m[wave][n] = m;
            s_l[wave][n] = lt;
        }
#pragma unroll
        for (int mm = 0; mm < 4; ++mm) {
#pragma unroll
            for (int i = 0; i < 4; ++i) s_o[wave][n][16 * mm + 4 * j + i] = ot[mm][i];
        }
    }
    __syncthreads();
    for (uint32_t idx = threadIdx.x; idx < group * 64u; idx += 256u) {
        const uint32_t h = idx >> 6;
        const uint32_t d = idx & 63u;
        float top = LNG_NEG_INF;
#pragma unroll
        for (int w = 0; w < 4; ++w) top = fmaxf(top, s_m[w][h]);
        float sum = 0.0f, o = 0.0f;
#pragma unroll
        for (int w = 0; w < 4; ++w) {
            const float wt = s_m[w][h] == LNG_NEG_INF ? 0.0f : __builtin_amdgcn_exp2f(s_m[w][h] - top);
            sum += s_l[w][h] * wt;
            o += s_o[w][h][d] * wt;
        }
        if (row_chunks == 1) {
            const uint32_t head = g * group + h;
            const float sink2 = it.sinks_offset != LNG_NO_SINKS
                                    ? ((const float *)(a.sinks + it.sinks_offset))[head] * LNG_LOG2E
                                    : LNG_NEG_INF;
            const float all = fmaxf(top, sink2);
            const float keep = __builtin_amdgcn_exp2f(top - all);
            const float z = sum * keep + (sink2 == LNG_NEG_INF ? 0.0f : __builtin_amdgcn_exp2f(sink2 - all));
            uint16_t *op = (uint16_t *)(a.out + it.out_offset) + (uint64_t)head * 64u + d;
            *op = f32_to_bf16_bits(o * keep / z);
        } else {
            const uint64_t slot = ((uint64_t)wi.pair * a.n_chunks + wi.chunk) * group + h;
            if (a.fused) {
                // device-coherent stores: visible to every XCD once acknowledged, no cache write-back
                __hip_atomic_store(&a.partial_o[slot * 64u + d], o, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                if (d == 0) {
                    __hip_atomic_store(&a.partial_ml[slot * 2u], top, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    __hip_atomic_store(&a.partial_ml[slot * 2u + 1u], sum, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                }
            } else { // lng_decode_merge runs as the next dispatch and sees ordinary stores
                a.partial_o[slot * 64u + d] = o;
                if (d == 0) {
                    a.partial_ml[slot * 2u] = top;
                    a.partial_ml[slot * 2u + 1u] = sum;
                }
            }
        }
    }
    if (row_chunks == 1 || !a.fused) return;

    // ---- split-K: the workgroup that finishes last for this (row, kv head) merges the partials ----
    // Publication without a cache-wide write-back (an agent-scope release fence writes back this XCD's
    // whole L2 from every workgroup: measured 35 us instead of 9 us on a 504-workgroup dispatch):
    //  - the partials above are agent-scope atomic stores: they write through to where every XCD sees
    //    them, and the store counter only falls when that has happened;
    //  - every thread waits for its own store counter to reach zero (the explicit s_waitcnt below; the
    //    "memory" clobber keeps the compiler from moving the stores past it), then the workgroup meets;
    //  - only then one thread takes the ticket (an agent-scope read-modify-write);
    //  - whoever draws the last ticket has, through the two barriers, that read-modify-write's result
    //    before any of its loads issue (the hardware issues a wave's memory instructions in order and
    //    the branch depends on the result), and reads the partials with agent-scope atomic loads, which
    //    do not take a stale line from this XCD's L2.
    // The ticket counter returns to zero for the next dispatch (dispatches run in stream order).
    __shared__ uint32_t s_ticket;
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    if (threadIdx.x == 0) s_ticket = __hip_atomic_fetch_add(&a.tickets[wi.pair], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __syncthreads();
    if (s_ticket != row_chunks - 1u) return;
    asm volatile("" ::: "memory");
    if (threadIdx.x == 0) __hip_atomic_store(&a.tickets[wi.pair], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);

    merge_chunks<true>(a, it, wi.pair, g, group, row_chunks);
}

// Two builds of the same body: 130 registers and three wavefronts per SIMD for long chunks (what a long context
// streams best with), 125 registers and four for dispatches of many workgroups with chunks under 2,048 positions
// (a table of sequences), where workgroups are short-lived and a fourth one per compute unit hides more of their
// start-up (32 sequences 65 -> 62 us, 128 sequences 243 -> 236 us; on 4,096-position chunks it is 1.7 % slower).
extern "C" __global__ __launch_bounds__(256, 2) void lng_decode_bf16_d64(lng_k_attn a) { decode_bf16_d64_body(a); }
extern "C" __global__ __launch_bounds__(256, 4) void lng_decode_bf16_d64_o4(lng_k_attn a) { decode_bf16_d64_body(a); }

// =============================================================================================
// Decode kernel, f32 (the reference's own element type), head width 64, up to 16 query heads per
// kv head: the bf16 kernel's grid, chunks, partials and lane roles on the f32 matrix instruction
// v_mfma_f32_16x16x4_f32 (A: lane (n, j) gives row n, k-slot j; B: k-slot j, column n; the lane
// receives rows 4j + i of column n).
//
//   S^T[tok][head] = K[tok][:] . Q[head][:]   16 instructions per 16 positions: lane (n, j) loads the
//       four floats at dims 16s + 4j of position n's K row (16 bytes, the four lanes of a position
//       read 64 contiguous bytes) and of head n's query; step (s, e) contracts dim 16s + 4j + e.
//   O^T[dim][head] += V^T[dim][tok] . P^T[tok][head]   16 per 16 positions: step i of block mm takes the
//       lane's own weight of position 4j + i as B and V[position 4j + i][dim 16mm + n] as A, a
//       4-byte load whose 16 lanes read 64 contiguous bytes of one V row: V arrives transposed
//       straight from memory, every byte read once.
// 64 cycles of the matrix pipe per position and wavefront, a third of what reading the rows takes
// at full memory rate, so the kernel is bound by memory like the bf16 one; nothing is rounded below
// f32. Rows of a ring are found without a division per lane: the tile's first row is uniform.
// =============================================================================================
struct kv_tile_f32 {
    float4 k[2][4];  // [position half][dim step]
    float v[2][16];  // [position half][4 * i + mm]: position 4j + i, dim 16mm + n
};

extern "C" __global__ __launch_bounds__(256, 2) void lng_decode_f32_d64(lng_k_attn a) {
    __shared__ float s_m[4][16];
    __shared__ float s_l[4][16];
    __shared__ float s_o[4][16][65];

    const work_item wi = work_of(a);
    const uint32_t row = wi.pair / a.kv_heads;
    const uint32_t g = wi.pair % a.kv_heads;
    const lng_k_row it = row_of(a, row);
    // positions and slots fit 32 bits (the host refuses shapes whose counts do not)
    const uint32_t last = (uint32_t)it.start;
    const uint32_t first = (uint32_t)first_visible(it.start, it.window);
    const uint32_t base = first & ~31u;
    const uint32_t row_chunks = (uint32_t)(((uint64_t)last + 1u - base + a.chunk - 1u) / a.chunk);
    if (wi.chunk >= row_chunks) return; // this row has fewer chunks than the longest one
    // interleaved groups of 128 positions, as in the bf16 kernel; the host keeps last below 2^32 - 65,536, so
    // neither last + 1 nor a position plus the stride (at most 256 chunks x 128) leaves 32 bits
    const uint32_t c0 = base + wi.chunk * 128u;
    const uint32_t c1 = last + 1u;
    const uint32_t tile_stride = 128u * row_chunks;

    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t n = lane & 15u;
    const uint32_t j = lane >> 4;
    const uint32_t group = a.heads / a.kv_heads;
    const uint32_t slots = (uint32_t)(it.slots > 0xffffffffull ? 0xffffffffull : it.slots);
    const bool wraps = it.slots <= last;
    const bool small_ring = slots < 32u;
    const uint64_t row_floats = (uint64_t)a.kv_heads * 64u;
    const float *kb = (const float *)(a.k + it.k_offset) + (uint64_t)g * 64u + 4u * j;
    const float *vb = (const float *)(a.v + it.v_offset) + (uint64_t)g * 64u + n;

    float4 qv[4];
#pragma unroll
    for (int s = 0; s < 4; ++s) {
        qv[s] = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
        if (n < group) qv[s] = *(const float4 *)((const float *)(a.q + it.q_offset) + ((uint64_t)g * group + n) * 64u + 16u * s + 4u * j);
    }

    // cache row of position tp + off (off < 32), clamped into [first, last] so that it exists and is finite
    auto row_of_pos = [&](uint32_t tp, uint32_t rbase, uint32_t off) -> uint64_t {
        uint32_t p = tp + off;
        p = p < first ? first : p;
        p = p > last ? last : p;
        uint32_t r = rbase + (p - tp);
        if (small_ring) {
            r %= slots;
        } else {
            r = r >= slots ? r - slots : r;
        }
        return (uint64_t)r * row_floats;
    };
    auto load_tile = [&](uint32_t tp, kv_tile_f32 &t) {
        const uint32_t rbase = wraps ? tp % slots : tp; // uniform over the wavefront
#pragma unroll
        for (int half = 0; half < 2; ++half) {
            const float *kp = kb + row_of_pos(tp, rbase, 16u * half + n);
#pragma unroll
            for (int s = 0; s < 4; ++s) t.k[half][s] = *(const float4 *)(kp + 16 * s);
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const float *vp = vb + row_of_pos(tp, rbase, 16u * half + 4u * j + i);
#pragma unroll
                for (int mm = 0; mm < 4; ++mm) t.v[half][4 * i + mm] = vp[16 * mm];
            }
        }
    };

    const float sl2 = a.scale * LNG_LOG2E;
    float m = LNG_NEG_INF; // running max of head n, log2 domain
    float l = 0.0f;        // this lane's share of the running sum
    floatx4 ot[4];         // O^T[16mm + 4j + i][head n]
#pragma unroll
    for (int mm = 0; mm < 4; ++mm) ot[mm] = (floatx4){0.f, 0.f, 0.f, 0.f};

    kv_tile_f32 cur, nxt;
    uint32_t tp = c0 + wave * 32u;
    if (tp < c1) load_tile(tp, cur);
    for (; tp < c1; tp += tile_stride) {
        if (c1 - tp > tile_stride) load_tile(tp + tile_stride, nxt);

        floatx4 st[2];
#pragma unroll
        for (int half = 0; half < 2; ++half) {
            st[half] = (floatx4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int s = 0; s < 4; ++s) {
                st[half] = __builtin_amdgcn_mfma_f32_16x16x4f32(cur.k[half][s].x, qv[s].x, st[half], 0, 0, 0);
                st[half] = __builtin_amdgcn_mfma_f32_16x16x4f32(cur.k[half][s].y, qv[s].y, st[half], 0, 0, 0);
                st[half] = __builtin_amdgcn_mfma_f32_16x16x4f32(cur.k[half][s].z, qv[s].z, st[half], 0, 0, 0);
                st[half] = __builtin_amdgcn_mfma_f32_16x16x4f32(cur.k[half][s].w, qv[s].w, st[half], 0, 0, 0);
            }
        }
        float tmax = LNG_NEG_INF;
#pragma unroll
        for (int half = 0; half < 2; ++half) {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const uint32_t off = (uint32_t)(half * 16 + i) + 4u * j;
                const bool seen = off < c1 - tp && tp + off >= first; // c1 <= last + 1
                const float x = seen ? st[half][i] : LNG_NEG_INF;
                st[half][i] = x;
                tmax = fmaxf(tmax, x);
            }
        }
        tmax = fmaxf(tmax, __shfl_xor(tmax, 16, 64));
        tmax = fmaxf(tmax, __shfl_xor(tmax, 32, 64));
        const float m_new = fmaxf(m, tmax * sl2); // scale > 0: the maximum commutes with it
        const float m_safe = m_new == LNG_NEG_INF ? 0.0f : m_new;
        const float alpha = __builtin_amdgcn_exp2f(m - m_safe);
        float psum = 0.0f;
#pragma unroll
        for (int half = 0; half < 2; ++half) {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                // one rounding, of the small difference (not of the scaled score and then of the difference)
                const float pw = __builtin_amdgcn_exp2f(__builtin_fmaf(st[half][i], sl2, -m_safe));
                st[half][i] = pw;
                psum += pw;
            }
        }
        l = l * alpha + psum;
        m = m_new;
#pragma unroll
        for (int mm = 0; mm < 4; ++mm) {
            ot[mm] = ot[mm] * alpha;
#pragma unroll
            for (int half = 0; half < 2; ++half) {
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    ot[mm] = __builtin_amdgcn_mfma_f32_16x16x4f32(cur.v[half][4 * i + mm], st[half][i], ot[mm], 0, 0, 0);
                }
            }
        }
        cur = nxt;
    }

    // ---- merge the four wavefronts ---------------------------------------------------------
    {
        float lt = l + __shfl_xor(l, 16, 64);
        lt += __shfl_xor(lt, 32, 64);
        if (j == 0) {
            s_m[wave][n] = m;
            s_l[wave][n] = lt;
        }
#pragma unroll
        for (int mm = 0; mm < 4; ++mm) {
#pragma unroll
            for (int i = 0; i < 4; ++i) s_o[wave][n][16 * mm + 4 * j + i] = ot[mm][i];
        }
    }
    __syncthreads();
    for (uint32_t idx = threadIdx.x; idx < group * 64u; idx += 256u) {
        const uint32_t h = idx >> 6;
        const uint32_t d = idx & 63u;
        float top = LNG_NEG_INF;
#pragma unroll
        for (int w = 0; w < 4; ++w) top = fmaxf(top, s_m[w][h]);
        float sum = 0.0f, o = 0.0f;
#pragma unroll
        for (int w = 0; w < 4; ++w) {
            const float wt = s_m[w][h] == LNG_NEG_INF ? 0.0f : __builtin_amdgcn_exp2f(s_m[w][h] - top);
            sum += s_l[w][h] * wt;
            o += s_o[w][h][d] * wt;
        }
        if (row_chunks == 1) {
            const uint32_t head = g * group + h;
            const float sink = it.sinks_offset != LNG_NO_SINKS
                                   ? ((const float *)(a.sinks + it.sinks_offset))[head] * LNG_LOG2E
                                   : LNG_NEG_INF;
            const float all = fmaxf(top, sink);
            const float keep = top == LNG_NEG_INF ? 0.0f : __builtin_amdgcn_exp2f(top - all);
            const float z = sum * keep + (sink == LNG_NEG_INF ? 0.0f : __builtin_amdgcn_exp2f(sink - all));
            ((float *)(a.out + it.out_offset))[(uint64_t)head * 64u + d] = o * keep / z;
        } else { // lng_decode_merge follows
            const uint64_t slot = ((uint64_t)wi.pair * a.n_chunks + wi.chunk) * group + h;
            a.partial_o[slot * 64u + d] = o;
            if (d == 0) {
                a.partial_ml[slot * 2u] = top;
                a.partial_ml[slot * 2u + 1u] = sum;
            }
        }
    }
}

// =============================================================================================
// Decode kernels for head widths 128, 256 and 512 (DS slices of 64 dimensions): the plan of the two
// kernels above - one workgroup per (row, kv head, chunk) serves every query head of the group, so K
// and V are read once per kv head; chunks, partials and lng_decode_merge are shared - with the head
// dimension walked in slices. Scores accumulate over the slices of K on the matrix unit; after the
// softmax each slice of V gives its 64 output dimensions. Loads run one batch ahead of the
// arithmetic (a batch = two slices of K or of V for bf16, one for f32), across tiles too.
// Callers: the reference's other user of this operator has 32 heads over 16 kv heads of width 256
// (decider/src/gpu.rs:878-893), its own tests go to width 512 (attention_grouped.rs:187-199).
// =============================================================================================
template <int DS> __device__ __forceinline__ void decode_wide_bf16(const lng_k_attn a) {
    __shared__ float s_m[4][16];
    __shared__ float s_l[4][16];
    __shared__ float s_o[4][16][65];
    constexpr int SB = DS >= 4 ? 4 : 2; // slices per batch of loads (512 contiguous bytes per row from width 256 on)
    constexpr int KBATCH = DS / SB;    // batches of K per tile, and as many of V
    constexpr int NBATCH = 2 * KBATCH;

    const work_item wi = work_of(a);
    const uint32_t row = wi.pair / a.kv_heads;
    const uint32_t g = wi.pair % a.kv_heads;
    const lng_k_row it = row_of(a, row);
    const uint64_t last = it.start;
    const uint64_t first = first_visible(last, it.window);
    const uint64_t base = first & ~(uint64_t)31;
    // (a run of a.chunk positions per workgroup: with 256 bytes and more per position and kv head the interleaved
    // groups of the head-width-64 kernel measured 4-5 % slower here)
    const uint64_t c0 = base + (uint64_t)wi.chunk * a.chunk;
    if (c0 > last) return;
    const uint64_t c1 = (c0 + a.chunk < last + 1) ? c0 + a.chunk : last + 1;
    const uint32_t row_chunks = (uint32_t)((last + 1 - base + a.chunk - 1) / a.chunk);

    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t n = lane & 15u;
    const uint32_t j = lane >> 4;
    const uint32_t group = a.heads / a.kv_heads;
    const bool wraps = it.slots <= last;
    constexpr uint32_t head_bytes = 128u * DS;
    const uint64_t row_bytes = (uint64_t)a.kv_heads * head_bytes;
    const char *kb = a.k + it.k_offset + (uint64_t)g * head_bytes + j * 16u;
    const char *vb = a.v + it.v_offset + (uint64_t)g * head_bytes + j * 16u;

    bf16x8 qb[DS][2]; // head n of this group: the lane's 8 k-slots of each step of each slice
#pragma unroll
    for (int s = 0; s < DS; ++s) {
        uint4 q0 = make_uint4(0, 0, 0, 0), q1 = q0;
        if (n < group) {
            const char *qp = a.q + it.q_offset + ((uint64_t)g * group + n) * head_bytes + s * 128u + j * 16u;
            q0 = *(const uint4 *)qp;
            q1 = *(const uint4 *)(qp + 64);
        }
        qb[s][0] = as_bf16x8(q0);
        qb[s][1] = as_bf16x8(q1);
    }
    bf16x8 sel[2];
#pragma unroll
    for (int b = 0; b < 2; ++b) {
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            sel[b][e] = (8u * j + (uint32_t)e == 16u * (uint32_t)b + n) ? (__bf16)1.0f : (__bf16)0.0f;
        }
    }

    struct batch {
        uint4 x[2][SB][2]; // [position half][slice of the batch][k step]
    };
    struct rows2 {
        uint64_t lo, hi; // byte offsets of the cache rows of the lane's two positions of a tile
    };
    auto row_at = [&](uint64_t p) -> uint64_t {
        p = p < first ? first : p;
        p = p > last ? last : p;
        return (wraps ? p % it.slots : p) * row_bytes;
    };
    auto offsets = [&](uint64_t tp) -> rows2 { return rows2{row_at(tp + n), row_at(tp + 16u + n)}; };
    auto load_batch = [&](const rows2 &off, int b, batch &t) {
        const char *from = (b < KBATCH ? kb : vb) + (uint32_t)((b % KBATCH) * SB) * 128u;
#pragma unroll
        for (int half = 0; half < 2; ++half) {
            const char *at = from + (half ? off.hi : off.lo);
#pragma unroll
            for (int u = 0; u < SB; ++u) {
                t.x[half][u][0] = *(const uint4 *)(at + u * 128);
                t.x[half][u][1] = *(const uint4 *)(at + u * 128 + 64);
            }
        }
    };

    const float sl2 = a.scale * LNG_LOG2E;
    float m = LNG_NEG_INF, l = 0.0f;
    floatx4 ot[DS][4]; // O^T[64s + 16mm + 4j + i][head n]
#pragma unroll
    for (int s = 0; s < DS; ++s) {
#pragma unroll
        for (int mm = 0; mm < 4; ++mm) ot[s][mm] = (floatx4){0.f, 0.f, 0.f, 0.f};
    }
    const floatx4 zero4 = (floatx4){0.f, 0.f, 0.f, 0.f};

    batch cur, nxt;
    rows2 off = {0, 0}, off_next = {0, 0};
    uint64_t tp = c0 + (uint64_t)wave * 32u;
    if (tp < c1) {
        off = offsets(tp);
        load_batch(off, 0, cur);
    }
    for (; tp < c1; tp += 128u) {
        const bool more = tp + 128u < c1;
        if (more) off_next = offsets(tp + 128u);
        floatx4 st[2] = {zero4, zero4};
        float alpha = 1.0f;
        bf16x8 pb;
#pragma unroll
        for (int b = 0; b < NBATCH; ++b) {
            if (b + 1 < NBATCH) {
                load_batch(off, b + 1, nxt);
            } else if (more) {
                load_batch(off_next, 0, nxt);
            }
            if (b < KBATCH) {
#pragma unroll
                for (int u = 0; u < SB; ++u) {
#pragma unroll
                    for (int half = 0; half < 2; ++half) {
                        st[half] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(cur.x[half][u][0]), qb[b * SB + u][0], st[half], 0, 0, 0);
                        st[half] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(cur.x[half][u][1]), qb[b * SB + u][1], st[half], 0, 0, 0);
                    }
                }
                if (b == KBATCH - 1) { // every slice of K is in: the tile's softmax
                    float tmax = LNG_NEG_INF;
#pragma unroll
                    for (int half = 0; half < 2; ++half) {
#pragma unroll
                        for (int i = 0; i < 4; ++i) {
                            const uint64_t p = tp + (uint64_t)(half * 16 + i) + 4u * j;
                            const float x = (p >= first && p <= last) ? st[half][i] * sl2 : LNG_NEG_INF;
                            st[half][i] = x;
                            tmax = fmaxf(tmax, x);
                        }
                    }
                    tmax = fmaxf(tmax, __shfl_xor(tmax, 16, 64));
                    tmax = fmaxf(tmax, __shfl_xor(tmax, 32, 64));
                    const float m_new = fmaxf(m, tmax);
                    const float m_safe = m_new == LNG_NEG_INF ? 0.0f : m_new;
                    alpha = __builtin_amdgcn_exp2f(m - m_safe);
                    float psum = 0.0f;
#pragma unroll
                    for (int half = 0; half < 2; ++half) {
#pragma unroll
                        for (int i = 0; i < 4; ++i) {
                            const float pw = __builtin_amdgcn_exp2f(st[half][i] - m_safe);
                            st[half][i] = pw;
                            psum += pw;
                        }
                    }
                    l = l * alpha + psum;
                    m = m_new;
                    pb = narrow8(st[0], st[1]);
                }
            } else {
#pragma unroll
                for (int u = 0; u < SB; ++u) {
                    const int s = (b - KBATCH) * SB + u;
#pragma unroll
                    for (int mm = 0; mm < 4; ++mm) {
                        const floatx4 t0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(cur.x[0][u][mm >> 1]), sel[mm & 1], zero4, 0, 0, 0);
                        const floatx4 t1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(cur.x[1][u][mm >> 1]), sel[mm & 1], zero4, 0, 0, 0);
                        const bf16x8 va = narrow8(t0, t1);
                        ot[s][mm] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(va, pb, ot[s][mm] * alpha, 0, 0, 0);
                    }
                }
            }
            cur = nxt;
        }
        off = off_next;
    }

    // ---- merge the four wavefronts, 64 output dimensions at a time ---------------------------------
    {
        float lt = l + __shfl_xor(l, 16, 64);
        lt += __shfl_xor(lt, 32, 64);
        if (j == 0) {
            s_m[wave][n] = m;
            s_l[wave][n] = lt;
        }
    }
#pragma unroll
    for (int s = 0; s < DS; ++s) {
        if (s) __syncthreads(); // the previous slice has been read
#pragma unroll
        for (int mm = 0; mm < 4; ++mm) {
#pragma unroll
            for (int i = 0; i < 4; ++i) s_o[wave][n][16 * mm + 4 * j + i] = ot[s][mm][i];
        }
        __syncthreads();
        for (uint32_t idx = threadIdx.x; idx < group * 64u; idx += 256u) {
            const uint32_t h = idx >> 6;
            const uint32_t d = idx & 63u;
            float top = LNG_NEG_INF;
#pragma unroll
            for (int w = 0; w < 4; ++w) top = fmaxf(top, s_m[w][h]);
            float sum = 0.0f, o = 0.0f;
#pragma unroll
            for (int w = 0; w < 4; ++w) {
                const float wt = s_m[w][h] == LNG_NEG_INF ? 0.0f : __builtin_amdgcn_exp2f(s_m[w][h] - top);
                sum += s_l[w][h] * wt;
                o += s_o[w][h][d] * wt;
            }
            if (row_chunks == 1) {
                const uint32_t head = g * group + h;
                const float sink2 = it.sinks_offset != LNG_NO_SINKS
                                        ? ((const float *)(a.sinks + it.sinks_offset))[head] * LNG_LOG2E
                                        : LNG_NEG_INF;
                const float all = fmaxf(top, sink2);
                const float keep = __builtin_amdgcn_exp2f(top - all);
                const float z = sum * keep + (sink2 == LNG_NEG_INF ? 0.0f : __builtin_amdgcn_exp2f(sink2 - all));
                uint16_t *op = (uint16_t *)(a.out + it.out_offset) + (uint64_t)head * (64u * DS) + 64u * s + d;
                *op = f32_to_bf16_bits(o * keep / z);
            } else { // lng_decode_merge runs as the next dispatch
                const uint64_t slot = ((uint64_t)wi.pair * a.n_chunks + wi.chunk) * group + h;
                a.partial_o[slot * (64u * DS) + 64u * s + d] = o;
                if (s == 0 && d == 0) {
                    a.partial_ml[slot * 2u] = top;
                    a.partial_ml[slot * 2u + 1u] = sum;
                }
            }
        }
    }
}

extern "C" __global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2))) void lng_decode_bf16_w128(lng_k_attn a) { decode_wide_bf16<2>(a); }
// (width 256: batches of four slices at one wavefront per SIMD measured 1.37 ms against 1.55 ms for batches of two at
// two wavefronts, 16 sequences of 32,768 positions at 32/16 heads)
extern "C" __global__ __launch_bounds__(256) void lng_decode_bf16_w256(lng_k_attn a) { decode_wide_bf16<4>(a); }
extern "C" __global__ __launch_bounds__(256) void lng_decode_bf16_w512(lng_k_attn a) { decode_wide_bf16<8>(a); }

// f32 (the reference's element type): lng_decode_f32_d64's products (v_mfma_f32_16x16x4_f32, V arriving transposed
// straight from memory), one or two slices of 64 dimensions per batch of loads. The queries wait in LDS (16 heads x 512 floats
// would not fit the registers beside 128 accumulators).
template <int DS> __device__ __forceinline__ void decode_wide_f32(const lng_k_attn a) {
    __shared__ float s_m[4][16];
    __shared__ float s_l[4][16];
    __shared__ float s_o[4][16][65];
    __shared__ __attribute__((aligned(16))) float s_q[16][64 * DS + 4];
    constexpr int SB = DS == 4 ? 2 : 1; // slices per batch of loads (width 256: 512 contiguous bytes per row, 1.54 against 1.60 ms
                                        // on 16 sequences of 16,384 positions; at width 512 two slices no longer fit the registers)
    constexpr int KBATCH = DS / SB;                    // batches of K per tile, and as many of V
    constexpr int NBATCH = 2 * KBATCH;

    const work_item wi = work_of(a);
    const uint32_t row = wi.pair / a.kv_heads;
    const uint32_t g = wi.pair % a.kv_heads;
    const lng_k_row it = row_of(a, row);
    const uint64_t last = it.start;
    const uint64_t first = first_visible(last, it.window);
    const uint64_t base = first & ~(uint64_t)31;
    const uint32_t row_chunks = (uint32_t)((last + 1 - base + a.chunk - 1) / a.chunk);
    if (wi.chunk >= row_chunks) return; // this row has fewer chunks than the longest one
    // The row's workgroups take interleaved groups of 128 positions (workgroup c: groups c, c + chunks, ...), not
    // a run of a.chunk positions each: together they sweep one window of the row, and every workgroup of a row
    // has the same number of groups to within one, however the row's length divides.
    const uint64_t c0 = base + (uint64_t)wi.chunk * 128u;
    const uint64_t c1 = last + 1;
    const uint64_t tile_stride = 128ull * row_chunks;

    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t n = lane & 15u;
    const uint32_t j = lane >> 4;
    const uint32_t group = a.heads / a.kv_heads;
    const bool wraps = it.slots <= last;
    constexpr uint32_t D = 64u * DS;
    const uint64_t row_floats = (uint64_t)a.kv_heads * D;
    const float *kb = (const float *)(a.k + it.k_offset) + (uint64_t)g * D + 4u * j;
    const float *vb = (const float *)(a.v + it.v_offset) + (uint64_t)g * D + n;

    for (uint32_t idx = threadIdx.x; idx < 16u * D; idx += 256u) { // heads past the group: zero queries
        const uint32_t h = idx / D, d = idx % D;
        s_q[h][d] = h < group ? ((const float *)(a.q + it.q_offset))[((uint64_t)g * group + h) * D + d] : 0.0f;
    }
    __syncthreads();

    struct batch {
        float4 k[SB][2][4]; // K: [slice of the batch][position half][dim step of the slice]
    };                      // V reuses the registers: [slice][half][i] = position 4j + i, .x .y .z .w = dims 16mm + n of the slice
    auto row_of_pos = [&](uint64_t p) -> uint64_t {
        p = p < first ? first : p;
        p = p > last ? last : p;
        return (wraps ? p % it.slots : p) * row_floats;
    };
    auto load_batch = [&](uint64_t tp, int b, batch &t) {
        if (b < KBATCH) {
#pragma unroll
            for (int half = 0; half < 2; ++half) {
                const float *kp = kb + row_of_pos(tp + 16u * half + n) + 64 * SB * b;
#pragma unroll
                for (int u = 0; u < SB; ++u) {
#pragma unroll
                    for (int s = 0; s < 4; ++s) t.k[u][half][s] = *(const float4 *)(kp + 64 * u + 16 * s);
                }
            }
        } else {
#pragma unroll
            for (int half = 0; half < 2; ++half) {
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const float *vp = vb + row_of_pos(tp + 16u * half + 4u * j + i) + 64 * SB * (b - KBATCH);
#pragma unroll
                    for (int u = 0; u < SB; ++u) {
                        float4 x;
                        x.x = vp[64 * u];
                        x.y = vp[64 * u + 16];
                        x.z = vp[64 * u + 32];
                        x.w = vp[64 * u + 48];
                        t.k[u][half][i] = x; // .x .y .z .w = dim blocks mm = 0..3
                    }
                }
            }
        }
    };

    const float sl2 = a.scale * LNG_LOG2E;
    float m = LNG_NEG_INF, l = 0.0f;
    floatx4 ot[DS][4];
#pragma unroll
    for (int s = 0; s < DS; ++s) {
#pragma unroll
        for (int mm = 0; mm < 4; ++mm) ot[s][mm] = (floatx4){0.f, 0.f, 0.f, 0.f};
    }

    batch cur, nxt;
    uint64_t tp = c0 + (uint64_t)wave * 32u;
    if (tp < c1) load_batch(tp, 0, cur);
    for (; tp < c1; tp += tile_stride) {
        const bool more = tp + tile_stride < c1;
        floatx4 st[2] = {(floatx4){0.f, 0.f, 0.f, 0.f}, (floatx4){0.f, 0.f, 0.f, 0.f}};
        float alpha = 1.0f;
#pragma unroll
        for (int b = 0; b < NBATCH; ++b) {
            if (b + 1 < NBATCH) {
                load_batch(tp, b + 1, nxt);
            } else if (more) {
                load_batch(tp + tile_stride, 0, nxt);
            }
            if (b < KBATCH) {
#pragma unroll
                for (int u = 0; u < SB; ++u) {
#pragma unroll
                    for (int s = 0; s < 4; ++s) {
                        const float4 qv = *(const float4 *)(&s_q[n][64 * (SB * b + u) + 16 * s + 4 * j]);
#pragma unroll
                        for (int half = 0; half < 2; ++half) {
                            st[half] = __builtin_amdgcn_mfma_f32_16x16x4f32(cur.k[u][half][s].x, qv.x, st[half], 0, 0, 0);
                            st[half] = __builtin_amdgcn_mfma_f32_16x16x4f32(cur.k[u][half][s].y, qv.y, st[half], 0, 0, 0);
                            st[half] = __builtin_amdgcn_mfma_f32_16x16x4f32(cur.k[u][half][s].z, qv.z, st[half], 0, 0, 0);
                            st[half] = __builtin_amdgcn_mfma_f32_16x16x4f32(cur.k[u][half][s].w, qv.w, st[half], 0, 0, 0);
                        }
                    }
                }
                if (b == KBATCH - 1) {
                    float tmax = LNG_NEG_INF;
#pragma unroll
                    for (int half = 0; half < 2; ++half) {
#pragma unroll
                        for (int i = 0; i < 4; ++i) {
                            const uint64_t p = tp + (uint64_t)(half * 16 + i) + 4u * j;
                            const float x = (p >= first && p <= last) ? st[half][i] : LNG_NEG_INF;
                            st[half][i] = x;
                            tmax = fmaxf(tmax, x);
                        }
                    }
                    tmax = fmaxf(tmax, __shfl_xor(tmax, 16, 64));
                    tmax = fmaxf(tmax, __shfl_xor(tmax, 32, 64));
                    const float m_new = fmaxf(m, tmax * sl2); // scale > 0: the maximum commutes with it
                    const float m_safe = m_new == LNG_NEG_INF ? 0.0f : m_new;
                    alpha = __builtin_amdgcn_exp2f(m - m_safe);
                    float psum = 0.0f;
#pragma unroll
                    for (int half = 0; half < 2; ++half) {
#pragma unroll
                        for (int i = 0; i < 4; ++i) {
                            const float pw = __builtin_amdgcn_exp2f(__builtin_fmaf(st[half][i], sl2, -m_safe));
                            st[half][i] = pw;
                            psum += pw;
                        }
                    }
                    l = l * alpha + psum;
                    m = m_new;
                }
            } else {
#pragma unroll
                for (int u = 0; u < SB; ++u) {
                    const int s = SB * (b - KBATCH) + u;
#pragma unroll
                    for (int mm = 0; mm < 4; ++mm) {
                        ot[s][mm] = ot[s][mm] * alpha;
#pragma unroll
                        for (int half = 0; half < 2; ++half) {
#pragma unroll
                            for (int i = 0; i < 4; ++i) {
                                const float4 x = cur.k[u][half][i];
                                const float vx = mm == 0 ? x.x : mm == 1 ? x.y : mm == 2 ? x.z : x.w;
                                ot[s][mm] = __builtin_amdgcn_mfma_f32_16x16x4f32(vx, st[half][i], ot[s][mm], 0, 0, 0);
                            }
                        }
                    }
                }
            }
            cur = nxt;
        }
    }

    {
        float lt = l + __shfl_xor(l, 16, 64);
        lt += __shfl_xor(lt, 32, 64);
        if (j == 0) {
            s_m[wave][n] = m;
            s_l[wave][n] = lt;
        }
    }
#pragma unroll
    for (int s = 0; s < DS; ++s) {
        if (s) __syncthreads();
#pragma unroll
        for (int mm = 0; mm < 4; ++mm) {
#pragma unroll
            for (int i = 0; i < 4; ++i) s_o[wave][n][16 * mm + 4 * j + i] = ot[s][mm][i];
        }
        __syncthreads();
        for (uint32_t idx = threadIdx.x; idx < group * 64u; idx += 256u) {
            const uint32_t h = idx >> 6;
            const uint32_t d = idx & 63u;
            float top = LNG_NEG_INF;
#pragma unroll
            for (int w = 0; w < 4; ++w) top = fmaxf(top, s_m[w][h]);
            float sum = 0.0f, o = 0.0f;
#pragma unroll
            for (int w = 0; w < 4; ++w) {
                const float wt = s_m[w][h] == LNG_NEG_INF ? 0.0f : __builtin_amdgcn_exp2f(s_m[w][h] - top);
                sum += s_l[w][h] * wt;
                o += s_o[w][h][d] * wt;
            }
            if (row_chunks == 1) {
                const uint32_t head = g * group + h;
                const float sink = it.sinks_offset != LNG_NO_SINKS
                                       ? ((const float *)(a.sinks + it.sinks_offset))[head] * LNG_LOG2E
                                       : LNG_NEG_INF;
                const float all = fmaxf(top, sink);
                const float keep = top == LNG_NEG_INF ? 0.0f : __builtin_amdgcn_exp2f(top - all);
                const float z = sum * keep + (sink == LNG_NEG_INF ? 0.0f : __builtin_amdgcn_exp2f(sink - all));
                ((float *)(a.out + it.out_offset))[(uint64_t)head * D + 64u * s + d] = o * keep / z;
            } else {
                const uint64_t slot = ((uint64_t)wi.pair * a.n_chunks + wi.chunk) * group + h;
                a.partial_o[slot * D + 64u * s + d] = o;
                if (s == 0 && d == 0) {
                    a.partial_ml[slot * 2u] = top;
                    a.partial_ml[slot * 2u + 1u] = sum;
                }
            }
        }
    }
}

extern "C" __global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2))) void lng_decode_f32_w128(lng_k_attn a) { decode_wide_f32<2>(a); }
extern "C" __global__ __launch_bounds__(256) void lng_decode_f32_w256(lng_k_attn a) { decode_wide_f32<4>(a); }
extern "C" __global__ __launch_bounds__(256) void lng_decode_f32_w512(lng_k_attn a) { decode_wide_f32<8>(a); }

// The merge as its own dispatch, for large grids (there a workgroup that waits for its coherent stores and
// its ticket holds a compute unit's slot that another chunk could use) and for the f32 kernel. One workgroup
// per (row, kv head, query head), the query head the fast index of the grid: thread c turns chunk c's (max, sum) into a weight, then thread (dim, quarter)
// adds every fourth chunk's partial output and the quarters meet in LDS: eight times the workgroups of a
// merge per (row, kv head) and a quarter of the chain of loads per thread.
extern "C" __global__ __launch_bounds__(256) void lng_decode_merge(lng_k_attn a) {
    __shared__ float s_w[LNG_MAX_CHUNKS];
    __shared__ float s_red[2][4];
    __shared__ float s_acc[4][64];
    const uint32_t group = a.heads / a.kv_heads, h = blockIdx.x % group, pair = blockIdx.x / group;
    const uint32_t row = pair / a.kv_heads;
    const uint32_t g = pair % a.kv_heads;
    const lng_k_row it = row_of(a, row);
    const uint64_t last = it.start;
    const uint64_t base = first_visible(last, it.window) & ~(uint64_t)31;
    const uint32_t row_chunks = (uint32_t)((last + 1 - base + a.chunk - 1) / a.chunk);
    if (row_chunks == 1) return; // the decode kernel already wrote this row
    const uint32_t head = g * group + h;
    const uint32_t tid = threadIdx.x, wave = tid >> 6;
    const uint64_t slot0 = ((uint64_t)pair * a.n_chunks) * group + h;
    const float sink2 = it.sinks_offset != LNG_NO_SINKS ? ((const float *)(a.sinks + it.sinks_offset))[head] * LNG_LOG2E
                                                         : LNG_NEG_INF;
    float mc = LNG_NEG_INF, lc = 0.0f;
    if (tid < row_chunks) {
        const float2 ml = *(const float2 *)(a.partial_ml + (slot0 + (uint64_t)tid * group) * 2u);
        mc = ml.x;
        lc = ml.y;
    }
    float top = fmaxf(mc, sink2);
#pragma unroll
    for (int s = 32; s >= 1; s >>= 1) top = fmaxf(top, __shfl_xor(top, s, 64));
    if ((tid & 63u) == 0) s_red[0][wave] = top;
    __syncthreads();
    top = fmaxf(fmaxf(s_red[0][0], s_red[0][1]), fmaxf(s_red[0][2], s_red[0][3]));
    const float wt = mc == LNG_NEG_INF ? 0.0f : __builtin_amdgcn_exp2f(mc - top);
    if (tid < row_chunks) s_w[tid] = wt;
    float z = lc * wt;
#pragma unroll
    for (int s = 32; s >= 1; s >>= 1) z += __shfl_xor(z, s, 64);
    if ((tid & 63u) == 0) s_red[1][wave] = z;
    __syncthreads();
    z = (s_red[1][0] + s_red[1][1]) + (s_red[1][2] + s_red[1][3]) +
        (sink2 == LNG_NEG_INF ? 0.0f : __builtin_amdgcn_exp2f(sink2 - top));
    const uint32_t d = tid & 63u;
    const uint64_t step = (uint64_t)group * a.dim;
    for (uint32_t db = 0; db < a.dim; db += 64u) { // 64 dimensions at a time (one turn at the gpt-oss head width)
        const float *po = a.partial_o + slot0 * a.dim + db + d;
        float o = 0.0f;
        uint32_t c = wave;
        for (; c + 28u < row_chunks; c += 32u) { // eight loads in flight per turn
            float x[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) x[u] = po[(c + 4u * u) * step];
#pragma unroll
            for (int u = 0; u < 8; ++u) o += x[u] * s_w[c + 4u * u];
        }
        for (; c < row_chunks; c += 4u) o += po[c * step] * s_w[c];
        if (db) __syncthreads(); // the previous turn's sums have been read
        s_acc[wave][d] = o;
        __syncthreads();
        if (wave == 0) {
            const float res = ((s_acc[0][d] + s_acc[1][d]) + (s_acc[2][d] + s_acc[3][d])) / z;
            const uint64_t at = (uint64_t)head * a.dim + db + d;
            if (a.dtype == LNG_F32) {
                ((float *)(a.out + it.out_offset))[at] = res;
            } else {
                ((uint16_t *)(a.out + it.out_offset))[at] = f32_to_bf16_bits(res);
            }
        }
    }
}

// The same merge when no row has more than LNG_MERGE_FEW chunks (many rows in the dispatch: a table of sequences): a
// wavefront per (row, kv head, query head), four to a workgroup, no LDS and no barrier - the lanes hold the
// chunks' (max, sum), a lane per dimension adds the partial outputs, asked for eight at a time before the weights
// are known. A quarter of the workgroups of lng_decode_merge, which at thousands of rows costs more to launch than
// to run (128 sequences, up to eight chunks: 5.5 us against 17 us).
#define LNG_MERGE_FEW 32u
extern "C" __global__ __launch_bounds__(256) void lng_decode_merge_few(lng_k_attn a) {
    const uint32_t group = a.heads / a.kv_heads;
    const uint32_t per_pair = (group + 3u) / 4u; // workgroups per (row, kv head)
    const uint32_t pair = blockIdx.x / per_pair;
    const uint32_t lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
    const uint32_t h = 4u * (blockIdx.x % per_pair) + wave;
    if (h >= group) return;
    const uint32_t row = pair / a.kv_heads;
    const uint32_t g = pair % a.kv_heads;
    const lng_k_row it = row_of(a, row);
    const uint64_t last = it.start;
    const uint64_t base = first_visible(last, it.window) & ~(uint64_t)31;
    const uint32_t row_chunks = (uint32_t)((last + 1 - base + a.chunk - 1) / a.chunk); // <= n_chunks <= LNG_MERGE_FEW
    if (row_chunks == 1) return; // the decode kernel already wrote this row
    const uint64_t step = (uint64_t)group * a.dim;
    const uint32_t head = g * group + h;
    const uint64_t slot0 = ((uint64_t)pair * a.n_chunks) * group + h;
    const float *po = a.partial_o + slot0 * a.dim + lane;
    float x[8]; // the first 64 dimensions' partial outputs of the first eight chunks, asked for before the weights are known
#pragma unroll
    for (int u = 0; u < 8; ++u) x[u] = (uint32_t)u < row_chunks ? po[(uint64_t)u * step] : 0.0f;
    const float sink2 = it.sinks_offset != LNG_NO_SINKS ? ((const float *)(a.sinks + it.sinks_offset))[head] * LNG_LOG2E
                                                         : LNG_NEG_INF;
    const uint32_t c = lane & (LNG_MERGE_FEW - 1u); // both halves of the wavefront hold the same chunks
    float mc = LNG_NEG_INF, lc = 0.0f;
    if (c < row_chunks) {
        const float2 ml = *(const float2 *)(a.partial_ml + (slot0 + (uint64_t)c * group) * 2u);
        mc = ml.x;
        lc = ml.y;
    }
    float top = fmaxf(mc, sink2);
#pragma unroll
    for (int s = 16; s >= 1; s >>= 1) top = fmaxf(top, __shfl_xor(top, s, 64));
    const float wt = mc == LNG_NEG_INF ? 0.0f : __builtin_amdgcn_exp2f(mc - top);
    float z = lc * wt;
#pragma unroll
    for (int s = 16; s >= 1; s >>= 1) z += __shfl_xor(z, s, 64);
    z += sink2 == LNG_NEG_INF ? 0.0f : __builtin_amdgcn_exp2f(sink2 - top);
    for (uint32_t db = 0; db < a.dim; db += 64u) {
        float o0 = 0.0f, o1 = 0.0f;
        for (uint32_t c0 = 0; c0 < row_chunks; c0 += 8u) { // uniform: one turn up to eight chunks
            if (db || c0) {
#pragma unroll
                for (int u = 0; u < 8; ++u) x[u] = c0 + (uint32_t)u < row_chunks ? po[db + (uint64_t)(c0 + u) * step] : 0.0f;
            }
#pragma unroll
            for (int u = 0; u < 8; u += 2) {
                o0 += x[u] * __shfl(wt, (int)(c0 + u), 64);
                o1 += x[u + 1] * __shfl(wt, (int)(c0 + u + 1), 64);
            }
        }
        const float res = (o0 + o1) / z;
        const uint64_t at = (uint64_t)head * a.dim + db + lane;
        if (a.dtype == LNG_F32) {
            ((float *)(a.out + it.out_offset))[at] = res;
        } else {
            ((uint16_t *)(a.out + it.out_offset))[at] = f32_to_bf16_bits(res);
        }
    }
}

// =============================================================================================
// Row copy with optional conversion (Batch::copy_rows, apple.rs:1762; kernels.metal:1127-1138):
// how new K and V rows enter a cache. One thread per element.
// =============================================================================================
extern "C" __global__ __launch_bounds__(256) void lng_copy_rows(lng_k_copy a) {
    const uint64_t gid = (uint64_t)blockIdx.x * 256u + threadIdx.x;
    if (gid >= a.rows * a.width) return;
    const uint64_t r = gid / a.width;
    const uint64_t i = gid % a.width;
    const uint64_t si = r * a.src_stride + i;
    const uint64_t di = r * a.dst_stride + i;
    if (a.src_dtype == a.dst_dtype) {
        if (a.src_dtype == LNG_F32) {
            ((uint32_t *)a.dst)[di] = ((const uint32_t *)a.src)[si];
        } else {
            ((uint16_t *)a.dst)[di] = ((const uint16_t *)a.src)[si];
        }
    } else if (a.src_dtype == LNG_F32) {
        ((uint16_t *)a.dst)[di] = f32_to_bf16_bits(((const float *)a.src)[si]);
    } else {
        ((float *)a.dst)[di] = bf16_bits_to_f32(((const uint16_t *)a.src)[si]);
    }
}

// =============================================================================================
// The step before attention (gpt-oss/src/gpu.rs:733-759): biases, rotation by halves, append.
// The arithmetic is the CPU model's (model.rs:282-286, 389-404): one f32 add for the bias, then
// four products, one difference and one sum, each rounded on its own, so fused multiply-add
// is switched off in these functions.
// =============================================================================================

// Batch::rmsnorm_rows (apple.rs:1731-1758; kernels.metal:1087-1117; CPU form model.rs:274-280),
// in place. One wavefront per row: squares summed in f32 (four partial sums per lane, then across
// the lanes), scale = 1 / sqrt(mean + eps), each element (v * scale) * w as the CPU form orders it.
extern "C" __global__ __launch_bounds__(256) void lng_rmsnorm_rows(lng_k_rmsnorm a) {
#pragma clang fp contract(off)
    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t row = blockIdx.x * 4u + (threadIdx.x >> 6);
    if (row >= a.rows) return;
    float *x = a.v + (uint64_t)row * a.stride;
    float s0 = 0.0f, s1 = 0.0f, s2 = 0.0f, s3 = 0.0f;
    uint32_t i = lane;
    for (; i + 192u < a.d; i += 256u) {
        const float v0 = x[i], v1 = x[i + 64u], v2 = x[i + 128u], v3 = x[i + 192u];
        s0 += v0 * v0;
        s1 += v1 * v1;
        s2 += v2 * v2;
        s3 += v3 * v3;
    }
    for (; i < a.d; i += 64u) s0 += x[i] * x[i];
    float ss = (s0 + s1) + (s2 + s3);
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) ss += __shfl_xor(ss, off, 64);
    const float scale = 1.0f / sqrtf(ss / (float)a.d + a.eps);
    for (i = lane; i < a.d; i += 64u) x[i] = x[i] * scale * a.w[i];
}

// The same operator with a workgroup per row, for rows of 257..4096 floats: every thread requests its (up to 16)
// elements and weights at once and keeps the elements in registers between the sum and the scaling, so a row
// costs two memory round trips instead of one per 64 elements (one decoding row of 2,880 floats: 14 -> 7 us).
extern "C" __global__ __launch_bounds__(256) void lng_rmsnorm_row_wg(lng_k_rmsnorm a) {
#pragma clang fp contract(off)
    __shared__ float s_part[4];
    float *x = a.v + (uint64_t)blockIdx.x * a.stride;
    float v[16], w[16];
    float ss = 0.0f;
#pragma unroll
    for (int u = 0; u < 16; ++u) {
        const uint32_t i = threadIdx.x + 256u * u;
        v[u] = i < a.d ? x[i] : 0.0f;
        w[u] = i < a.d ? a.w[i] : 0.0f;
    }
#pragma unroll
    for (int u = 0; u < 16; ++u) ss += v[u] * v[u];
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) ss += __shfl_xor(ss, off, 64);
    if ((threadIdx.x & 63u) == 0) s_part[threadIdx.x >> 6] = ss;
    __syncthreads();
    ss = (s_part[0] + s_part[1]) + (s_part[2] + s_part[3]);
    const float scale = 1.0f / sqrtf(ss / (float)a.d + a.eps);
#pragma unroll
    for (int u = 0; u < 16; ++u) {
        const uint32_t i = threadIdx.x + 256u * u;
        if (i < a.d) x[i] = v[u] * scale * w[u];
    }
}

// Batch::add_rows (apple.rs:1886-1911; kernels.metal:1648-1660). One thread per element.
extern "C" __global__ __launch_bounds__(256) void lng_add_rows(lng_k_add a) {
    const uint64_t gid = (uint64_t)blockIdx.x * 256u + threadIdx.x;
    if (gid >= a.rows * a.width) return;
    const uint64_t r = gid / a.width;
    const uint64_t i = gid % a.width;
    a.dst[gid] += a.src[r * a.src_stride + i];
}

// Batch::rotate_halves_partial (apple.rs:1929-1955; kernels.metal:1673-1690), in place.
// One thread per rotated pair.
extern "C" __global__ __launch_bounds__(256) void lng_rotate_halves(lng_k_rotate a) {
#pragma clang fp contract(off)
    const uint32_t half = a.rotary / 2;
    const uint64_t gid = (uint64_t)blockIdx.x * 256u + threadIdx.x;
    if (gid >= a.rows * a.heads * half) return;
    const uint32_t i = (uint32_t)(gid % half);
    const uint64_t row_head = gid / half;
    const uint64_t row = row_head / a.heads;
    float *h = a.x + row_head * a.dim;
    const float c = a.table[(row * half + i) * 2], s = a.table[(row * half + i) * 2 + 1];
    const float x0 = h[i], x1 = h[i + half];
    h[i] = x0 * c - x1 * s;
    h[i + half] = x1 * c + x0 * s;
}

template <int W> struct prep_vec;
template <> struct prep_vec<1> {
    static __device__ void load(const float *p, float (&x)[1]) { x[0] = *p; }
    static __device__ void store_f32(float *p, const float (&x)[1]) { *p = x[0]; }
    static __device__ void store_bf16(uint16_t *p, const float (&x)[1]) { *p = f32_to_bf16_bits(x[0]); }
};
template <> struct prep_vec<4> {
    static __device__ void load(const float *p, float (&x)[4]) {
        const float4 t = *(const float4 *)p;
        x[0] = t.x; x[1] = t.y; x[2] = t.z; x[3] = t.w;
    }
    static __device__ void store_f32(float *p, const float (&x)[4]) {
        *(float4 *)p = make_float4(x[0], x[1], x[2], x[3]);
    }
    static __device__ void store_bf16(uint16_t *p, const float (&x)[4]) {
        uint2 t;
        t.x = (uint32_t)f32_to_bf16_bits(x[0]) | ((uint32_t)f32_to_bf16_bits(x[1]) << 16);
        t.y = (uint32_t)f32_to_bf16_bits(x[2]) | ((uint32_t)f32_to_bf16_bits(x[3]) << 16);
        *(uint2 *)p = t;
    }
};

// One work unit = W consecutive pairs of a head's rotated part (reads and writes W elements
// in each half), or W consecutive elements of a head's unrotated tail or of a v row.
// Grid: x over (row, unit) of the longest item, y = item.
template <int W> static __device__ __forceinline__ void prepare_body(const lng_k_prepare &a) {
#pragma clang fp contract(off)
    const lng_prepare_item it = a.items ? a.items[blockIdx.y] : a.first;
    const uint32_t idx = blockIdx.x * 256u + threadIdx.x;
    const uint32_t r = idx / a.units_per_row;
    if (r >= it.n) return;
    uint32_t u = idx % a.units_per_row;
    const uint32_t half = a.rotary / 2, ru = half / W, uph = ru + (a.dim - a.rotary) / W;
    const uint32_t qw = a.heads * a.dim, kw = a.kv_heads * a.dim;
    const uint64_t slot = (it.start + r) % it.slots;
    const bool bf16 = a.out_dtype == LNG_BF16;
    const uint32_t es = bf16 ? 2u : 4u;

    const float *src, *bias;
    char *dst;
    if (u < (a.heads + a.kv_heads) * uph) {
        const bool is_q = u < a.heads * uph;
        if (!is_q) u -= a.heads * uph;
        const uint32_t head = u / uph, w = u % uph;
        if (is_q) {
            src = (const float *)(a.q + it.q_offset) + (uint64_t)r * qw + head * a.dim;
            bias = a.q_bias ? a.q_bias + head * a.dim : nullptr;
            dst = a.q_out + it.q_out_offset + ((uint64_t)r * qw + head * a.dim) * es;
        } else {
            src = (const float *)(a.k + it.k_offset) + (uint64_t)r * kw + head * a.dim;
            bias = a.k_bias ? a.k_bias + head * a.dim : nullptr;
            dst = a.k_cache + it.k_cache_offset + (slot * kw + head * a.dim) * es;
        }
        if (w < ru) {
            const uint32_t i = w * W;
            float x0[W], x1[W], cs[2][W], y0[W], y1[W];
            prep_vec<W>::load(src + i, x0);
            prep_vec<W>::load(src + i + half, x1);
            if (bias) {
                float b0[W], b1[W];
                prep_vec<W>::load(bias + i, b0);
                prep_vec<W>::load(bias + i + half, b1);
#pragma unroll
                for (int e = 0; e < W; ++e) {
                    x0[e] += b0[e];
                    x1[e] += b1[e];
                }
            }
            const float *t = (const float *)(a.table + it.table_offset) + ((uint64_t)r * half + i) * 2;
            if constexpr (W == 4) {
                float lo[4], hi[4];
                prep_vec<4>::load(t, lo);
                prep_vec<4>::load(t + 4, hi);
                cs[0][0] = lo[0]; cs[1][0] = lo[1]; cs[0][1] = lo[2]; cs[1][1] = lo[3];
                cs[0][2] = hi[0]; cs[1][2] = hi[1]; cs[0][3] = hi[2]; cs[1][3] = hi[3];
            } else {
                cs[0][0] = t[0];
                cs[1][0] = t[1];
            }
#pragma unroll
            for (int e = 0; e < W; ++e) {
                y0[e] = x0[e] * cs[0][e] - x1[e] * cs[1][e];
                y1[e] = x1[e] * cs[0][e] + x0[e] * cs[1][e];
            }
            if (bf16) {
                prep_vec<W>::store_bf16((uint16_t *)dst + i, y0);
                prep_vec<W>::store_bf16((uint16_t *)dst + i + half, y1);
            } else {
                prep_vec<W>::store_f32((float *)dst + i, y0);
                prep_vec<W>::store_f32((float *)dst + i + half, y1);
            }
            return;
        }
        const uint32_t j = a.rotary + (w - ru) * W;
        src += j;
        if (bias) bias += j;
        dst += (uint64_t)j * es;
    } else {
        u -= (a.heads + a.kv_heads) * uph;
        const uint32_t j = u * W;
        src = (const float *)(a.v + it.v_offset) + (uint64_t)r * kw + j;
        bias = a.v_bias ? a.v_bias + j : nullptr;
        dst = a.v_cache + it.v_cache_offset + (slot * kw + j) * es;
    }
    float x[W];
    prep_vec<W>::load(src, x);
    if (bias) {
        float b[W];
        prep_vec<W>::load(bias, b);
#pragma unroll
        for (int e = 0; e < W; ++e) x[e] += b[e];
    }
    if (bf16) prep_vec<W>::store_bf16((uint16_t *)dst, x);
    else prep_vec<W>::store_f32((float *)dst, x);
}

extern "C" __global__ __launch_bounds__(256) void lng_prepare_v4(lng_k_prepare a) { prepare_body<4>(a); }
extern "C" __global__ __launch_bounds__(256) void lng_prepare_v1(lng_k_prepare a) { prepare_body<1>(a); }

// =============================================================================================
// Q8_0 products (Batch::gemv_q8_0 / gemm_q8_0 / gemm_q8_0_tiled, apple.rs:1812-1883):
// y[p] = W x[p], W = signed bytes with one binary16 scale per 32 of a row, x and y f32.
//
// The bytes are exact in bf16 and one 16x16x32 product spans exactly one block of a row, so the
// matrix unit computes each block's sum of code * x and the block's scale multiplies it once,
// as the CPU form does (weights/src/q8_0.rs:103-123). x is split into two bf16 values,
// hi + lo = x to 16 significant bits (in registers for few positions, into two planes by
// lng_q8_split_x beforehand for many), and both go through the matrix unit: the
// result is within 1e-5 of the float64 definition relative to the largest |y|, the bound the
// reference holds its own kernels to.
// =============================================================================================
extern "C" __global__ __launch_bounds__(256) void lng_q8_split_x(lng_k_q8_split a) {
    const uint32_t per_row = a.cols / 4;
    const uint32_t idx = blockIdx.x * 256u + threadIdx.x;
    if (idx >= a.n_pad * per_row) return;
    const uint32_t p = idx / per_row, c = (idx % per_row) * 4u;
    float4 v = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
    if (p < a.n) v = *(const float4 *)(a.x + (uint64_t)p * a.x_stride + c);
    const float x[4] = {v.x, v.y, v.z, v.w};
    uint16_t hi[4], lo[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        hi[e] = f32_to_bf16_bits(x[e]);
        lo[e] = f32_to_bf16_bits(x[e] - bf16_bits_to_f32(hi[e]));
    }
    const uint64_t at = (uint64_t)p * a.cols + c;
    *(uint2 *)(a.hi + at) = make_uint2((uint32_t)hi[0] | ((uint32_t)hi[1] << 16), (uint32_t)hi[2] | ((uint32_t)hi[3] << 16));
    *(uint2 *)(a.lo + at) = make_uint2((uint32_t)lo[0] | ((uint32_t)lo[1] << 16), (uint32_t)lo[2] | ((uint32_t)lo[3] << 16));
}

// Eight signed bytes as eight bf16 values (exact: |code| <= 128 has at most 8 significant bits, so
// the upper half of its f32 form is the whole number).
__device__ __forceinline__ bf16x8 q8_codes_to_bf16(uint2 raw) {
    uint32_t w[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const uint32_t word = i < 2 ? raw.x : raw.y;
        const float f0 = (float)(int8_t)(word >> (16 * (i & 1)));
        const float f1 = (float)(int8_t)(word >> (16 * (i & 1) + 8));
        w[i] = (__float_as_uint(f0) >> 16) | (__float_as_uint(f1) & 0xffff0000u);
    }
    return as_bf16x8(make_uint4(w[0], w[1], w[2], w[3]));
}

__device__ __forceinline__ float f16_bits_to_f32(uint16_t bits) {
    return (float)__builtin_bit_cast(_Float16, bits);
}

// hi + lo = x to 16 significant bits, both bf16.
__device__ __forceinline__ void q8_split8(const float (&x)[8], bf16x8 &hi, bf16x8 &lo) {
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        const __bf16 h = (__bf16)x[e];
        hi[e] = h;
        lo[e] = (__bf16)(x[e] - (float)h);
    }
}

// Few positions (one pass of the matrix per 16; bound by reading the matrix, in practice by the
// number of load instructions a compute unit can take: some 40 cycles each): a workgroup takes
// 16 rows, its sixteen wavefronts take every sixteenth block of the rows and their partial sums
// meet in LDS. Lane l holds row l % 16 and, of each block, the 8 columns of group l / 16 - the B
// operand; positions are the A operand, read as f32 and split in registers. All loads of up to
// eight blocks are issued before the first product; blocks past the end are skipped, loads and
// all (the test is the same for the whole wavefront); the rows' scales come through LDS. ONE: a
// single position, whose x the
// workgroup first copies to LDS with 16-byte loads (a wavefront's two x loads per block become
// two LDS reads; x must fit Q8S_X1 floats). Grid: x = 16-row tiles, y = 16-position tiles.
#define Q8S_WAVES 16
#define Q8S_UNROLL 8 // blocks in flight per wavefront: 128 blocks (4096 columns) in one turn
#define Q8S_X1 12288 // floats of x held in LDS by the one-position form (48 KB)
#define Q8S_SC_BLOCKS 512 // rows of up to this many blocks (16,384 columns) have their scales staged through LDS
// The matrix a workgroup of a several-matrix dispatch works on becomes the one `a` names; returns its row tile.
__device__ __forceinline__ uint32_t q8_select_matrix(lng_k_q8 &a) {
    uint32_t tile = blockIdx.x;
#pragma unroll
    for (int i = 0; i < LNG_Q8_MORE; ++i) {
        if ((uint32_t)i < a.n_more && blockIdx.x >= a.more[i].first_tile) { // uniform: scalar selects
            a.codes = a.more[i].codes;
            a.scales = a.more[i].scales;
            a.y = a.more[i].y;
            a.rows = a.more[i].rows;
            a.y_stride = a.more[i].y_stride;
            tile = blockIdx.x - a.more[i].first_tile;
        }
    }
    return tile;
}

// WAVES wavefronts share the blocks of a row tile (16; 8 for the one-position form when two workgroups per compute
// unit cover the row tiles in one round instead of two).
template <bool ONE, bool XBF16 = false, int WAVES = Q8S_WAVES>
__device__ __forceinline__ void q8_stream_body(const lng_k_q8 &a, uint32_t tile) {
    static_assert(ONE || WAVES == 16, "the several-position forms map wavefront w to position w of 16");
    __shared__ float s_part[Q8S_WAVES - 1][4][64];
    // ONE: the position's x (normalised there, if asked); otherwise the weights of the RMS norm, if asked
    __shared__ __attribute__((aligned(16))) float s_x1[(ONE || !XBF16) ? Q8S_X1 : 4];
    __shared__ __attribute__((aligned(4))) uint16_t s_sc[16 * Q8S_SC_BLOCKS];
    __shared__ float s_norm[16]; // ONE: partial sums of squares; otherwise the 16 positions' scales
    const bool normed = !XBF16 && a.norm_w != nullptr; // uniform
    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t j = lane & 15u, kg = lane >> 4;
    const uint32_t r0 = tile * 16u, p0 = blockIdx.y * 16u;
    const uint32_t row = r0 + j < a.rows ? r0 + j : a.rows - 1u;
    const uint32_t pos = p0 + j < a.n ? p0 + j : a.n - 1u; // rows of the product past n are not stored
    const uint32_t blocks = a.cols / 32u;
    const int8_t *wrow = a.codes + (uint64_t)row * a.cols + 8u * kg;
    const uint16_t *srow = a.scales + (uint64_t)row * blocks;
    const float *xrow = a.x + (uint64_t)pos * a.x_stride + 8u * kg;
    const uint16_t *xrow16 = a.x_hi + (uint64_t)pos * a.plane_stride + 8u * kg; // XBF16: positions in bf16
    floatx4 y = {0.0f, 0.0f, 0.0f, 0.0f};
    const floatx4 zero4 = {0.0f, 0.0f, 0.0f, 0.0f};
    // The scales of the workgroup's 16 rows are one contiguous run (rows follow each other): copied to
    // LDS a dword per thread, instead of 2-byte loads from 16 different rows per block and wavefront.
    const bool sc_staged = blocks <= Q8S_SC_BLOCKS && r0 + 16u <= a.rows && ((uintptr_t)a.scales & 3u) == 0;
    if (!ONE && normed) { // wavefront w works out the scale of position p0 + w (there are 16 of each)
        const uint32_t pw = p0 + wave < a.n ? p0 + wave : a.n - 1u;
        const float *xp = a.x + (uint64_t)pw * a.x_stride;
        float ss = 0.0f;
        for (uint32_t c = 4u * lane; c < a.cols; c += 256u) {
            const float4 v = *(const float4 *)(xp + c);
            ss += v.x * v.x + v.y * v.y + v.z * v.z + v.w * v.w;
        }
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) ss += __shfl_xor(ss, off, 64);
        if (lane == 0) s_norm[wave] = 1.0f / sqrtf(ss / (float)a.cols + a.eps);
    }
    bool staged = false;
    floatx4 y0 = zero4; // stream 0's sum (wavefront 0)
    for (uint32_t stream = wave; stream < Q8S_WAVES; stream += WAVES) {
    y = zero4;
    for (uint32_t b0 = stream; b0 < blocks || !staged; b0 += Q8S_UNROLL * Q8S_WAVES) {
        uint2 raw[Q8S_UNROLL];
        uint16_t scale[Q8S_UNROLL];
        float4 xa[Q8S_UNROLL], xb[Q8S_UNROLL];
#pragma unroll
        for (int u = 0; u < Q8S_UNROLL; ++u) {
            const uint32_t b = b0 + u * Q8S_WAVES;
            raw[u] = make_uint2(0, 0);
            scale[u] = 0;
            xa[u] = xb[u] = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
            if (b < blocks) { // the same for every lane of the wavefront
                raw[u] = *(const uint2 *)(wrow + 32u * b);
                if (!sc_staged) scale[u] = srow[b];
                if (XBF16) {
                    xa[u] = *(const float4 *)(xrow16 + 32u * b); // eight bf16 values, used as they are
                } else if (!ONE) {
                    xa[u] = *(const float4 *)(xrow + 32u * b);
                    xb[u] = *(const float4 *)(xrow + 32u * b + 4u);
                }
            }
        }
        if (!staged) { // every wavefront comes here exactly once, in its first turn
            if (ONE) {
                float ss = 0.0f;
                for (uint32_t i = 4u * threadIdx.x; i < a.cols; i += 4u * 64u * WAVES) {
                    const float4 v = *(const float4 *)(a.x + i);
                    *(float4 *)(&s_x1[i]) = v;
                    ss += v.x * v.x + v.y * v.y + v.z * v.z + v.w * v.w;
                }
                if (normed) { // every thread normalises the elements it has just written
#pragma unroll
                    for (int off = 32; off > 0; off >>= 1) ss += __shfl_xor(ss, off, 64);
                    if (lane == 0) s_norm[wave] = ss;
                    __syncthreads();
                    float total = 0.0f;
#pragma unroll
                    for (int w = 0; w < WAVES; ++w) total += s_norm[w];
                    const float scale = 1.0f / sqrtf(total / (float)a.cols + a.eps);
                    for (uint32_t i = 4u * threadIdx.x; i < a.cols; i += 4u * 64u * WAVES) {
                        float4 v = *(const float4 *)(&s_x1[i]);
                        const float4 nw = *(const float4 *)(a.norm_w + i);
                        v.x = v.x * scale * nw.x;
                        v.y = v.y * scale * nw.y;
                        v.z = v.z * scale * nw.z;
                        v.w = v.w * scale * nw.w;
                        *(float4 *)(&s_x1[i]) = v;
                    }
                }
            } else if (normed) {
                for (uint32_t i = 4u * threadIdx.x; i < a.cols; i += 4u * 64u * WAVES) {
                    *(float4 *)(&s_x1[i]) = *(const float4 *)(a.norm_w + i);
                }
            }
            if (sc_staged) { // 16 * blocks * 2 bytes from a 32-byte boundary
                const uint32_t *src = (const uint32_t *)(a.scales + (uint64_t)r0 * blocks);
                for (uint32_t i = threadIdx.x; i < 8u * blocks; i += 64u * WAVES) ((uint32_t *)s_sc)[i] = src[i];
            }
            __syncthreads();
            staged = true;
        }
#pragma unroll
        for (int u = 0; u < Q8S_UNROLL; ++u) {
            const uint32_t b = b0 + u * Q8S_WAVES;
            if (b < blocks) {
                if (ONE) {
                    xa[u] = *(const float4 *)(&s_x1[32u * b + 8u * kg]);
                    xb[u] = *(const float4 *)(&s_x1[32u * b + 8u * kg + 4u]);
                }
                const bf16x8 wb = q8_codes_to_bf16(raw[u]);
                floatx4 acc;
                if (XBF16) {
                    acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, xa[u]), wb, zero4, 0, 0, 0);
                } else {
                    float xs[8] = {xa[u].x, xa[u].y, xa[u].z, xa[u].w, xb[u].x, xb[u].y, xb[u].z, xb[u].w};
                    if (!ONE && normed) {
                        const float sp = s_norm[j];
                        const float4 wa = *(const float4 *)(&s_x1[32u * b + 8u * kg]);
                        const float4 wb2 = *(const float4 *)(&s_x1[32u * b + 8u * kg + 4u]);
                        const float nw[8] = {wa.x, wa.y, wa.z, wa.w, wb2.x, wb2.y, wb2.z, wb2.w};
#pragma unroll
                        for (int e = 0; e < 8; ++e) xs[e] = xs[e] * sp * nw[e];
                    }
                    bf16x8 hi, lo;
                    q8_split8(xs, hi, lo);
                    acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(hi, wb, zero4, 0, 0, 0);
                    acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(lo, wb, acc, 0, 0, 0);
                }
                const float sc = f16_bits_to_f32(sc_staged ? s_sc[j * blocks + b] : scale[u]);
#pragma unroll
                for (int i = 0; i < 4; ++i) y[i] = __builtin_fmaf(sc, acc[i], y[i]);
            }
        }
    }
    if (stream != 0) {
#pragma unroll
        for (int i = 0; i < 4; ++i) s_part[stream - 1][i][lane] = y[i];
    } else {
        y0 = y;
    }
    }
    __syncthreads();
    if (wave != 0) return;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        float sum = y0[i];
#pragma unroll
        for (int w = 0; w < Q8S_WAVES - 1; ++w) sum += s_part[w][i][lane];
        const uint32_t p = p0 + 4u * kg + i; // accumulator row = position, column = matrix row
        if (p < a.n && r0 + j < a.rows) {
            float *yp = a.y + (uint64_t)p * a.y_stride + r0 + j;
            if (a.bias) sum = sum + a.bias[r0 + j];
            if (a.accumulate) sum = *yp + sum; // the residual: h + ((W x) + bias), each sum rounded as the separate dispatches round it
            *yp = sum;
        }
    }
}

extern "C" __global__ __launch_bounds__(64 * Q8S_WAVES) void lng_q8_stream(lng_k_q8 a) {
    const uint32_t tile = q8_select_matrix(a);
    q8_stream_body<false>(a, tile);
}

extern "C" __global__ __launch_bounds__(64 * Q8S_WAVES) void lng_q8_stream_one(lng_k_q8 a) {
    const uint32_t tile = q8_select_matrix(a);
    q8_stream_body<true>(a, tile);
}

// the same with 8 wavefronts: half the LDS partials and threads, two workgroups per compute unit
extern "C" __global__ __launch_bounds__(512) void lng_q8_stream_one_w8(lng_k_q8 a) {
    const uint32_t tile = q8_select_matrix(a);
    q8_stream_body<true, false, 8>(a, tile);
}

// positions already in bf16 (the output of a bf16 attention): one matrix instruction per block
extern "C" __global__ __launch_bounds__(64 * Q8S_WAVES) void lng_q8_stream_bf16(lng_k_q8 a) {
    const uint32_t tile = q8_select_matrix(a);
    q8_stream_body<false, true>(a, tile);
}

// Many positions (bound by the matrix unit): a workgroup of eight wavefronts takes 256 rows x 128
// positions, wavefront (w % 4, w / 4) the 64 x 64 corner of it: four 16-row B operands of codes
// (as bf16, in which every code is exact), four 16-position A operands per plane of x. Codes,
// planes and block scales are staged in LDS 64 columns (two blocks) at a time, double buffered:
// the loads of stage s + 1 are issued before stage s is computed and stored to LDS after it, so
// every byte of the matrix is fetched once per workgroup, in 64-byte runs. The thread that
// fetched 16 codes widens them to bf16 on the way into LDS, once per workgroup, rather than
// every wavefront that uses them doing so in its inner loop. Rows of both tiles are 128 bytes,
// unpadded; the 16-byte chunk c of row r is kept at chunk c ^ ((r >> 1) & 7), which makes the
// 16 rows that one operand read touches fall in different banks; rows of codes add r & 1 to
// that, so that the eight lanes that store two rows' even (or odd) chunks together, 128 bytes a
// cycle, also hit eight different places. (Loads that go from global
// memory straight into LDS were tried for the staging: the compiler then waits for every
// outstanding one before the first LDS read of a stage, which undoes the overlap.) Every
// (rows, positions) pair of operands gives one block sum per lane-held output; the row's block
// scale multiplies it into the f32 result.
#define Q8T_POS 128
#define Q8T_ROWS 256
#define Q8T_PLANE (Q8T_POS * 64) // bf16 elements of one plane of one stage
__device__ __forceinline__ bf16x8 q8_codes_to_bf16_perm(uint2 raw) {
    uint32_t w[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const uint32_t word = i < 2 ? raw.x : raw.y;
        const float f0 = (float)(int8_t)(word >> (16 * (i & 1)));
        const float f1 = (float)(int8_t)(word >> (16 * (i & 1) + 8));
        w[i] = __builtin_amdgcn_perm(__float_as_uint(f1), __float_as_uint(f0), 0x07060302u); // upper halves
    }
    return as_bf16x8(make_uint4(w[0], w[1], w[2], w[3]));
}

// WAVES wavefronts per workgroup: 8 (64 x 64 outputs each, two per SIMD) is what is launched; 16 (64 rows x
// 32 positions each, four per SIMD with half the registers) measures the same and is not instantiated.
// PLANES: 2 for f32 positions split into hi and lo bf16 planes; 1 when the positions are bf16 already
// (x_hi is then x itself, its rows plane_stride apart and only n of them: rows past n repeat the last).
template <int WAVES, int PLANES = 2> __device__ __forceinline__ void q8_tiled_body(const lng_k_q8 &a) {
    constexpr int MT = WAVES == 8 ? 4 : 2;       // groups of 16 positions per wavefront
    constexpr int XQ = 16 * PLANES / WAVES;      // x loads per wavefront and stage (PLANES x 16 groups of 8 positions in all)
    constexpr int WQ = 16 / WAVES;               // code loads (16 in all: groups of 16 rows)
    __shared__ __attribute__((aligned(16))) uint16_t s_x[2][PLANES][Q8T_PLANE]; // [stage % 2][plane]
    __shared__ __attribute__((aligned(16))) uint16_t s_w[2][Q8T_ROWS * 64];  // [stage % 2]: 64 codes per row as bf16
    __shared__ uint16_t s_sc[2][Q8T_ROWS * 2];                               // [stage % 2]: two block scales per row
    const uint32_t tid = threadIdx.x, lane = tid & 63u;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t j = lane & 15u, kg = lane >> 4;
    const uint32_t rw = 64u * (wave & 3u); // this wavefront's rows within the tile
    const uint32_t pw = 16u * MT * (wave >> 2); // and its positions
    // Which tile: workgroup ids go round the eight XCDs, each with an L2 of its own, and a few dozen
    // consecutive ids of one XCD run at a time. With eight position tiles or more, XCD k takes the
    // position tiles k, k + 8, ..; its ids walk blocks of 8 row tiles x 4 position tiles, so what
    // runs together reads 4 tiles of x and 8 of the matrix, every x tile is read through one L2
    // only, and the fetches from beyond L2 are about half of what row-major ids cost. The grid is
    // rounded up to whole blocks; a workgroup whose tile does not exist leaves at once.
    const uint32_t row_tiles = (a.rows + Q8T_ROWS - 1u) / Q8T_ROWS;
    const uint32_t pos_tiles = (a.n + Q8T_POS - 1u) / Q8T_POS;
    uint32_t row_tile, pos_tile;
    if (pos_tiles >= 8u) {
        const uint32_t xcd = blockIdx.x & 7u, seq = blockIdx.x >> 3;
        const uint32_t per_xcd = (pos_tiles + 7u) / 8u;
        const uint32_t row_blocks = (row_tiles + 7u) / 8u;
        const uint32_t blk = seq >> 5, within = seq & 31u;
        row_tile = (blk % row_blocks) * 8u + (within & 7u);
        const uint32_t pi = (blk / row_blocks) * 4u + (within >> 3);
        pos_tile = pi * 8u + xcd;
        if (row_tile >= row_tiles || pi >= per_xcd || pos_tile >= pos_tiles) return;
    } else {
        row_tile = blockIdx.x % row_tiles;
        pos_tile = blockIdx.x / row_tiles;
    }
    const uint32_t r0 = row_tile * Q8T_ROWS;
    const uint32_t p0 = pos_tile * Q8T_POS;
    const uint32_t blocks = a.cols / 32u;
    const uint32_t stages = (blocks + 1u) / 2u;
    const bool rows_here = r0 + rw < a.rows; // wavefronts past the last row only help staging

    // x staging: wavefront w issues XQ loads per stage; load q covers plane idx / 16 and the 8 positions
    // of group idx % 16, idx = XQ * w + q; lane l brings position 8 * group + l / 8, physical chunk l % 8.
    const uint16_t *x_src[XQ];
    uint32_t x_chunk[XQ];
#pragma unroll
    for (int q = 0; q < XQ; ++q) {
        const uint32_t idx = XQ * wave + q;
        const uint32_t pos = 8u * (idx & 15u) + (lane >> 3);
        x_chunk[q] = (lane & 7u) ^ ((pos >> 1) & 7u); // the logical chunk kept at this physical place
        const uint16_t *plane = (idx >> 4) ? a.x_lo : a.x_hi;
        const uint32_t at = PLANES == 2 || p0 + pos < a.n ? p0 + pos : a.n - 1u; // split planes are padded to whole tiles
        x_src[q] = plane + (uint64_t)at * a.plane_stride;
    }
    // code staging: WQ loads per stage; load q covers the 16 rows of group WQ * w + q; lane l brings row
    // 16 * group + l / 4 and its codes 16 * (l % 4) .. + 15, which become the row's bf16 chunks
    // 2 * (l % 4) and 2 * (l % 4) + 1.
    const int8_t *w_src[WQ];
    uint32_t w_to[WQ][2]; // element index in s_w[buf] of the two chunks
#pragma unroll
    for (int q = 0; q < WQ; ++q) {
        const uint32_t row = 16u * (WQ * wave + q) + (lane >> 2);
        const uint32_t r = r0 + row < a.rows ? r0 + row : a.rows - 1u;
        w_src[q] = a.codes + (uint64_t)r * a.cols;
#pragma unroll
        for (int h = 0; h < 2; ++h) w_to[q][h] = row * 64u + 8u * ((2u * (lane & 3u) + h) ^ ((row >> 1) & 7u) ^ (row & 1u));
    }
    // scale staging: thread t < 512 brings the scale of row t / 2, block t % 2 of the stage
    const bool sc_mine = WAVES == 8 || wave < 8u;
    const uint32_t sc_t = tid & 511u;
    const uint32_t sc_row = r0 + (sc_t >> 1) < a.rows ? r0 + (sc_t >> 1) : a.rows - 1u;
    const uint16_t *sc_src = a.scales + (uint64_t)sc_row * blocks;
    auto x_col = [&](uint32_t stage, int q) {
        const uint32_t col = stage * 64u + 8u * x_chunk[q];
        return col < a.cols ? col : col - 32u; // odd block count: the last stage's second block repeats its first
    };
    auto w_col = [&](uint32_t stage) { // the same, for this lane's 16 codes (col >= cols >= 32 where it applies)
        const uint32_t col = stage * 64u + 16u * (lane & 3u);
        return col < a.cols ? col : col - 32u;
    };
    // Two sets of staging registers: the loads of stage s + 2 are issued when stage s starts and
    // stored to LDS when stage s + 1 ends, two stages of time for a fetch that misses L2 (with one
    // stage, nearly every stage had some wavefront waiting out a miss before the barrier).
    // (plain scalars: arrays of staged values end up in scratch memory)
    const uint4 zero_u4 = make_uint4(0, 0, 0, 0);
    uint4 ax0 = zero_u4, ax1 = zero_u4, ax2 = zero_u4, ax3 = zero_u4, aw0 = zero_u4, aw1 = zero_u4;
    uint4 bx0 = zero_u4, bx1 = zero_u4, bx2 = zero_u4, bx3 = zero_u4, bw0 = zero_u4, bw1 = zero_u4;
    uint16_t asc = 0, bsc = 0;
    auto fetch = [&](uint32_t stage, uint4 &x0, uint4 &x1, uint4 &x2, uint4 &x3, uint4 &w0, uint4 &w1, uint16_t &sc) {
        x0 = *(const uint4 *)(x_src[0] + x_col(stage, 0));
        x1 = *(const uint4 *)(x_src[1] + x_col(stage, 1));
        if constexpr (XQ == 4) {
            x2 = *(const uint4 *)(x_src[2] + x_col(stage, 2));
            x3 = *(const uint4 *)(x_src[3] + x_col(stage, 3));
        }
        const uint32_t wc = w_col(stage);
        w0 = *(const uint4 *)(w_src[0] + wc);
        if constexpr (WQ == 2) w1 = *(const uint4 *)(w_src[1] + wc);
        const uint32_t b = 2u * stage + (tid & 1u);
        if (sc_mine) sc = b < blocks ? sc_src[b] : (uint16_t)0; // a block past the end counts for nothing
    };
    auto x_slot = [&](uint32_t buf, uint32_t q) {
        const uint32_t idx = XQ * wave + q;
        return (uint4 *)(&s_x[buf][idx >> 4][(idx & 15u) * 512u + 8u * lane]);
    };
    auto widen = [&](uint32_t buf, int q, const uint4 &codes) {
        *(bf16x8 *)(&s_w[buf][w_to[q][0]]) = q8_codes_to_bf16_perm(make_uint2(codes.x, codes.y));
        *(bf16x8 *)(&s_w[buf][w_to[q][1]]) = q8_codes_to_bf16_perm(make_uint2(codes.z, codes.w));
    };
    auto stash = [&](uint32_t buf, const uint4 &x0, const uint4 &x1, const uint4 &x2, const uint4 &x3, const uint4 &w0,
                     const uint4 &w1, uint16_t sc) {
        *x_slot(buf, 0) = x0;
        *x_slot(buf, 1) = x1;
        if constexpr (XQ == 4) {
            *x_slot(buf, 2) = x2;
            *x_slot(buf, 3) = x3;
        }
        widen(buf, 0, w0);
        if constexpr (WQ == 2) widen(buf, 1, w1);
        if (sc_mine) s_sc[buf][sc_t] = sc;
    };

    floatx4 y[4][MT];
#pragma unroll
    for (int nt = 0; nt < 4; ++nt) {
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) y[nt][mt] = floatx4{0.0f, 0.0f, 0.0f, 0.0f};
    }
    const floatx4 zero4 = {0.0f, 0.0f, 0.0f, 0.0f};
    // per-lane parts of the operand reads: row (position or matrix row) t * 16 + j, logical chunk 4 kb + kg
    uint32_t x_at[MT], x_sw[MT], w_at[4], w_sw[4];
#pragma unroll
    for (int t = 0; t < MT; ++t) {
        const uint32_t pos = pw + 16u * t + j;
        x_at[t] = pos * 64u;
        x_sw[t] = (pos >> 1) & 7u;
    }
#pragma unroll
    for (int t = 0; t < 4; ++t) {
        const uint32_t row = rw + 16u * t + j;
        w_at[t] = row * 64u;
        w_sw[t] = ((row >> 1) & 7u) ^ (row & 1u);
    }
    auto compute = [&](uint32_t buf) {
#pragma unroll
        for (int kb = 0; kb < 2; ++kb) {
            bf16x8 xh[MT], xl[MT];
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) {
                const uint32_t at = x_at[mt] + 8u * ((4u * kb + kg) ^ x_sw[mt]);
                xh[mt] = as_bf16x8(*(const uint4 *)(&s_x[buf][0][at]));
                if constexpr (PLANES == 2) xl[mt] = as_bf16x8(*(const uint4 *)(&s_x[buf][PLANES - 1][at]));
            }
#pragma unroll
            for (int nt = 0; nt < 4; ++nt) {
                const bf16x8 wb = as_bf16x8(*(const uint4 *)(&s_w[buf][w_at[nt] + 8u * ((4u * kb + kg) ^ w_sw[nt])]));
                const float scale = f16_bits_to_f32(s_sc[buf][2u * (rw + 16u * nt + j) + kb]);
                floatx4 acc[MT];
#pragma unroll
                for (int mt = 0; mt < MT; ++mt) acc[mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(xh[mt], wb, zero4, 0, 0, 0);
                if constexpr (PLANES == 2) {
#pragma unroll
                    for (int mt = 0; mt < MT; ++mt) acc[mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(xl[mt], wb, acc[mt], 0, 0, 0);
                }
#pragma unroll
                for (int mt = 0; mt < MT; ++mt) {
#pragma unroll
                    for (int i = 0; i < 4; ++i) y[nt][mt][i] = __builtin_fmaf(scale, acc[mt][i], y[nt][mt][i]);
                }
            }
        }
    };

    fetch(0, ax0, ax1, ax2, ax3, aw0, aw1, asc);
    stash(0, ax0, ax1, ax2, ax3, aw0, aw1, asc);
    __syncthreads();
    if (stages > 1u) fetch(1, bx0, bx1, bx2, bx3, bw0, bw1, bsc);
    for (uint32_t stage = 0; stage < stages; stage += 2u) {
        // even stage, in buffer 0: stage + 1 waits in set b, stage + 2 goes to set a
        if (stage + 2u < stages) fetch(stage + 2u, ax0, ax1, ax2, ax3, aw0, aw1, asc);
        if (rows_here) compute(0);
        if (stage + 1u < stages) stash(1, bx0, bx1, bx2, bx3, bw0, bw1, bsc);
        __syncthreads();
        if (stage + 1u >= stages) break;
        // odd stage, in buffer 1: stage + 2 waits in set a, stage + 3 goes to set b
        if (stage + 3u < stages) fetch(stage + 3u, bx0, bx1, bx2, bx3, bw0, bw1, bsc);
        if (rows_here) compute(1);
        if (stage + 2u < stages) stash(0, ax0, ax1, ax2, ax3, aw0, aw1, asc);
        __syncthreads();
    }
    if (!rows_here) return;
#pragma unroll
    for (int nt = 0; nt < 4; ++nt) {
        const uint32_t r = r0 + rw + 16u * nt + j;
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const uint32_t p = p0 + pw + 16u * mt + 4u * kg + i;
                if (p < a.n && r < a.rows) a.y[(uint64_t)p * a.y_stride + r] = y[nt][mt][i];
            }
        }
    }
}

extern "C" __global__ __launch_bounds__(512) void lng_q8_tiled(lng_k_q8 a) {
    q8_tiled_body<8>(a);
}

// positions already in bf16: one plane, half the matrix instructions, no split kernel before it
extern "C" __global__ __launch_bounds__(512) void lng_q8_tiled_bf16(lng_k_q8 a) {
    q8_tiled_body<8, 1>(a);
}

// Synthetic data (see LNG_SYNTH_STD in lng_kernel_args.h for the exact integers).
// A plain streaming read: the XOR of every 16-byte word of a buffer. Consecutive lanes read consecutive 16-byte
// words (a wavefront instruction = eight whole 128-byte lines), four loads in flight per lane and turn; the yardstick
// for what the memory system delivers to a kernel that does nothing but read.
extern "C" __global__ __launch_bounds__(256) void lng_checksum(lng_k_checksum a) {
    const uint64_t stride = (uint64_t)gridDim.x * 256u;
    uint64_t i = (uint64_t)blockIdx.x * 256u + threadIdx.x;
    const uint4 *src = (const uint4 *)a.src;
    uint4 x = make_uint4(0, 0, 0, 0);
    for (; i + 3u * stride < a.n16; i += 4u * stride) {
        const uint4 p0 = src[i], p1 = src[i + stride], p2 = src[i + 2u * stride], p3 = src[i + 3u * stride];
        x.x ^= p0.x ^ p1.x ^ p2.x ^ p3.x;
        x.y ^= p0.y ^ p1.y ^ p2.y ^ p3.y;
        x.z ^= p0.z ^ p1.z ^ p2.z ^ p3.z;
        x.w ^= p0.w ^ p1.w ^ p2.w ^ p3.w;
    }
    for (; i < a.n16; i += stride) {
        const uint4 p = src[i];
        x.x ^= p.x, x.y ^= p.y, x.z ^= p.z, x.w ^= p.w;
    }
#pragma unroll
    for (int s = 32; s >= 1; s >>= 1) {
        x.x ^= __shfl_xor(x.x, s, 64);
        x.y ^= __shfl_xor(x.y, s, 64);
        x.z ^= __shfl_xor(x.z, s, 64);
        x.w ^= __shfl_xor(x.w, s, 64);
    }
    __shared__ uint4 s_x[4];
    if ((threadIdx.x & 63u) == 0) s_x[threadIdx.x >> 6] = x;
    __syncthreads();
    if (threadIdx.x == 0) {
        uint4 r = s_x[0];
#pragma unroll
        for (int w = 1; w < 4; ++w) r.x ^= s_x[w].x, r.y ^= s_x[w].y, r.z ^= s_x[w].z, r.w ^= s_x[w].w;
        ((uint4 *)a.parts)[blockIdx.x] = r;
    }
}

extern "C" __global__ __launch_bounds__(256) void lng_checksum_fold(lng_k_checksum a) {
    uint4 x = make_uint4(0, 0, 0, 0);
    for (uint32_t i = threadIdx.x; i < a.n_parts; i += 256u) {
        const uint4 p = ((const uint4 *)a.parts)[i];
        x.x ^= p.x, x.y ^= p.y, x.z ^= p.z, x.w ^= p.w;
    }
#pragma unroll
    for (int s = 32; s >= 1; s >>= 1) {
        x.x ^= __shfl_xor(x.x, s, 64);
        x.y ^= __shfl_xor(x.y, s, 64);
        x.z ^= __shfl_xor(x.z, s, 64);
        x.w ^= __shfl_xor(x.w, s, 64);
    }
    __shared__ uint4 s_x[4];
    if ((threadIdx.x & 63u) == 0) s_x[threadIdx.x >> 6] = x;
    __syncthreads();
    if (threadIdx.x == 0) {
        uint4 r = s_x[0];
#pragma unroll
        for (int w = 1; w < 4; ++w) r.x ^= s_x[w].x, r.y ^= s_x[w].y, r.z ^= s_x[w].z, r.w ^= s_x[w].w;
        *(uint4 *)a.dst = r;
    }
}

extern "C" __global__ __launch_bounds__(256) void lng_fill_synthetic(lng_k_fill a) {
    const uint64_t stride = (uint64_t)gridDim.x * 256u;
    for (uint64_t i = (uint64_t)blockIdx.x * 256u + threadIdx.x; i < a.n; i += stride) {
        const uint64_t e = a.period ? i % a.period : i;
        uint64_t z = e + a.seed * 0x9E3779B97F4A7C15ull;
        z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
        z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
        z ^= z >> 31;
        const int s = (int)(z & 0xffff) + (int)((z >> 16) & 0xffff) + (int)((z >> 32) & 0xffff) +
                      (int)(z >> 48) - 131070;
        const float x = (float)s * a.factor;
        if (a.dtype == LNG_F32) {
            ((float *)a.dst)[i] = x;
        } else {
            ((uint16_t *)a.dst)[i] = f32_to_bf16_bits(x);
        }
    }
}

// =============================================================================================
// Prompt-pass kernel, bf16, head width 64, up to 8 query heads per kv head.
//
// A workgroup (8 wavefronts) takes 64 consecutive query positions and ALL query heads of one
// kv head: wavefront w handles query block w&1 (32 positions) and head pair w>>1, so every
// K/V tile staged in LDS is used by every head of the group. Workgroup ids put the kv head
// fastest (id % kv_heads): consecutive ids go to different XCDs, so each XCD's L2 keeps one kv
// head's K and V; the longest (latest) query tiles are issued first.
//
// Per 64-key tile, everything per query is lane-local: the products are computed transposed,
//   S^T[key][query] = K . Q^T   (v_mfma_f32_32x32x16_bf16; A = K rows read from LDS with
//                                ds_read_b128, B = Q^T held in registers for the whole pass)
// so lane l owns query l%32 and 16 of each 32 keys; the row maximum and sum need one exchange
// with lane l^32 only. exp'd scores narrowed to bf16 are directly the B operand of
//   O^T[dim][query] += V^T . P^T (A = V^T read from the row-major V tile with the transposing
//                                LDS read ds_read_b64_tr_b16: a 16-lane block reads 4 keys x 16
//                                dims and each lane receives 4 keys of one dim)
// and the accumulator column, like the softmax state, belongs to the lane's query. The sink
// initialises the running maximum and contributes 1 to the running sum (it is one more logit
// with no value); tiles wholly outside the causal/window band are never visited.
// =============================================================================================
// PF_BM query rows per workgroup = 32 * (8 wavefronts / (8 / NH) head slots): 64 with two heads per
// wavefront, 32 with one.
#define PF_BN 64
#define PF_THREADS 512
#define PF_KSTRIDE 72 // bf16 elements per LDS row (144 bytes): conflict-free 16-byte row reads
#define PF_VSTRIDE 96 // 192-byte rows: the four keys x 64 bytes that half a wavefront reads transposed fall in 64 different banks

#define PF_TAU 8.0f
typedef short short4v __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));

// max of x over lanes l and l^32, without LDS: swap the upper half of one copy with the
// lower half of another, then both copies hold one half's value in every lane.
__device__ __forceinline__ float other_half_max(float x) {
    const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}

__device__ __forceinline__ bf16x8 lds_read_tr8(const uint16_t *p0, const uint16_t *p1) {
    // two transposing reads: slots 0..3 and 4..7 of the lane's k-group
    const short4v lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) short4v *)p0);
    const short4v hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) short4v *)p1);
    typedef short short8v __attribute__((ext_vector_type(8)));
    const short8v both = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
    return __builtin_bit_cast(bf16x8, both);
}

// NH = heads per wavefront. NH = 2: 64 query rows per workgroup, wavefront = (32-row block, head pair);
// every K/V operand read from LDS feeds two products, which is what a long causal pass needs.
// NH = 1: 32 query rows per workgroup, wavefront = head; half the registers, so two workgroups share a
// compute unit (4 wavefronts per SIMD) and short, latency-bound passes (a 128-token window) overlap.
template <int NH> __device__ __forceinline__ void prefill_body(const lng_k_prefill &a) {
    constexpr uint32_t PF_BM = NH == 2 ? 64u : 32u;
    __shared__ __attribute__((aligned(16))) uint16_t s_k[2][PF_BN * PF_KSTRIDE];
    __shared__ __attribute__((aligned(16))) uint16_t s_v[2][PF_BN * PF_VSTRIDE];
    __shared__ uint32_t s_again; // the outcome of the range check (two heads per wavefront)

    const bool partial = a.splits > 1u;
    const uint32_t g = blockIdx.x % a.kv_heads;
    const uint32_t above = blockIdx.x / a.kv_heads;
    const uint32_t split = partial ? above % a.splits : 0u;        // an unsplit pass pays for no division by splits
    const uint32_t qtile = a.q_tiles - 1u - (partial ? above / a.splits : above);
    const uint32_t group = a.heads / a.kv_heads;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6); // scalar: branches on it are uniform
    // What a lane derives from its number: n = query within the wave's block, hh = which half of the k-slots / of each
    // 8 accumulator rows, the chunk of a tile it loads, its LDS offsets. With two heads per wavefront (256 registers
    // in use in the loops) these are worked out again after the loops instead of kept: a register that lives across a
    // loop without being used in it is spilled, a spill goes out to memory and its reload waits for every load in
    // flight. The lane number comes from mbcnt behind an empty asm statement, which the compiler cannot trace back
    // to the first copy.
    uint32_t lane, tid, n, hh, ld_key, ld_chunk, k_lane_off, v_lane_off;
    const char *kbase, *vbase;
    auto lane_values = [&]() {
        uint32_t z = 0u;
        asm volatile("" : "+v"(z));
        lane = __builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, z));
        tid = wave * 64u + lane;
        n = lane & 31u;
        hh = lane >> 5;
        ld_key = tid >> 3;  // 0..63
        ld_chunk = tid & 7u;
        kbase = a.k + (uint64_t)g * 128u + ld_chunk * 16u;
        vbase = a.v + (uint64_t)g * 128u + ld_chunk * 16u;
        // per-lane constant parts of the LDS addresses
        k_lane_off = n * PF_KSTRIDE + 8u * hh;                 // + kb*32*KSTRIDE + 16*ks
        const uint32_t L = lane & 15u;
        const uint32_t blk16 = lane >> 4;                                     // 16-lane block 0..3
        // transposing read: source lane L names key (L>>2) of its group and dims 4*(L&3).. of the block's 16
        v_lane_off = (4u * (blk16 >> 1) + (L >> 2)) * PF_VSTRIDE + 16u * (blk16 & 1u) + 4u * (L & 3u);
    };
    lane_values();
    if constexpr (NH == 2) s_again = 0u; // (every thread, the same value; the first barrier is ahead of its first use)
    const uint32_t qb = NH == 2 ? (wave & 1u) : 0u;
    const uint32_t hp = NH == 2 ? (wave >> 1) : wave; // first head slot of the wavefront is hp * NH

    // Positions fit 32 bits (the host refuses shapes whose counts do not).
    const uint32_t t = (uint32_t)a.t, start = (uint32_t)a.start;
    const uint32_t q0 = qtile * PF_BM;                         // first query row of the workgroup
    const uint32_t rows_here = t - q0 < PF_BM ? t - q0 : PF_BM;
    const uint32_t end = start + t;                            // positions in the cache
    const uint32_t pos_first = start + q0;                     // position of the first query row
    const uint32_t pos_last = pos_first + rows_here - 1;       // of the last real one
    const bool windowed = a.window != LNG_WINDOW_FULL;         // the host maps window >= end to FULL
    const uint32_t window = windowed ? (uint32_t)a.window : 0u;
    const uint32_t kfirst = (windowed && pos_first + 1 > window) ? pos_first + 1 - window : 0u;
    const uint32_t tile0 = kfirst & ~(uint32_t)(PF_BN - 1);
    const uint32_t all_tiles = (pos_last - tile0) / PF_BN + 1;
    // With splits, this workgroup takes tiles [first_tile, n_tiles) of the query tile's run (possibly
    // none) and leaves (max, sum, unnormalised output) for lng_prefill_merge, which also adds the sink.
    const uint32_t first_tile = partial ? (uint32_t)((uint64_t)all_tiles * split / a.splits) : 0u;
    const uint32_t n_tiles = partial ? (uint32_t)((uint64_t)all_tiles * (split + 1u) / a.splits) : all_tiles;
    const bool ring = a.slots < end;
    const uint32_t slots = (uint32_t)a.slots;
    const uint64_t row_bytes = (uint64_t)a.kv_heads * 128u;

    // ---- this wavefront's queries and its two heads -------------------------------------------
    // A wavefront whose second head slot is past the group computes its first head twice and
    // stores it once; one whose first slot is past the group only helps loading tiles.
    uint32_t my_row, my_pos;
    bool row_ok;
    auto row_values = [&]() {
        my_row = q0 + 32u * qb + n;      // query row of this lane
        my_pos = start + my_row;         // its absolute position
        row_ok = my_row < t;
    };
    row_values();
    const bool wave_active = hp * NH < group;
    const bool second_ok = NH == 2 && hp * 2u + 1u < group;
    uint32_t head[NH];
    head[0] = g * group + (wave_active ? hp * NH : 0u);
    if constexpr (NH == 2) head[1] = second_ok ? head[0] + 1u : head[0];
    bf16x8 qreg[NH][4];
    float m[NH], l[NH];
    floatx16 ot[NH][2];
    const float sl2 = a.scale * LNG_LOG2E;
#pragma unroll
    for (int h = 0; h < NH; ++h) {
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) {
            uint4 raw = make_uint4(0, 0, 0, 0);
            if (row_ok) {
                raw = *(const uint4 *)(a.q + (((uint64_t)my_row * a.heads + head[h]) * 64u + 16u * ks + 8u * hh) * 2u);
            }
            // Two heads per wavefront: scale * log2(e) goes into the query operand, once; the products then come out
            // of the matrix unit in the exponent's own units (one more bf16 rounding of q: 2^-9 relative per element,
            // a few 1e-4 on a score, an order below the rounding of the weights to bf16), and a pass whose maximum is
            // fixed at zero has nothing left to do but the exponential. One head per wavefront always tracks the
            // maximum: there the factor rides in the multiply-add that subtracts the maximum, and the 80
            // instructions that rescale the queries are saved.
            bf16x8 qv = as_bf16x8(raw);
            if constexpr (NH == 2) {
#pragma unroll
                for (int e = 0; e < 8; ++e) qv[e] = (__bf16)((float)qv[e] * sl2);
            }
            qreg[h][ks] = qv;
        }
    }
    bf16x2 ones2;
    ones2[0] = (__bf16)1.0f;
    ones2[1] = (__bf16)1.0f;

    // ---- tile loader: one 16-byte chunk of K and of V per thread --------------------------------
    auto fetch = [&](uint32_t tile, uint4 &kr, uint4 &vr) {
        uint32_t p = tile0 + tile * PF_BN + ld_key;
        p = p > pos_last ? pos_last : p; // rows past the last needed position are masked anyway,
        p = p < kfirst ? kfirst : p;     // and so are rows before the first one (a ring may not hold them any more)
        const uint32_t r = ring ? p % slots : p;
        kr = *(const uint4 *)(kbase + (uint64_t)r * row_bytes);
        vr = *(const uint4 *)(vbase + (uint64_t)r * row_bytes);
    };
    auto stash = [&](uint32_t buf, const uint4 &kr, const uint4 &vr) {
        *(uint4 *)(&s_k[buf][ld_key * PF_KSTRIDE + ld_chunk * 8u]) = kr;
        *(uint4 *)(&s_v[buf][ld_key * PF_VSTRIDE + ld_chunk * 8u]) = vr;
    };


    // With two heads per wavefront (long causal runs) the pass is first made optimistically: once a
    // first interior tile has set the running maximum from real scores, the remaining interior
    // tiles keep it FIXED and compute neither maxima nor rescalings (a softmax does not depend on
    // its reference point, only the number range does). Before the diagonal tile the workgroup
    // checks that every normaliser stayed in a range that rules out overflow and any underflow
    // that could matter, and that every accumulator is finite; if not, the pass is made again
    // with the maximum tracked throughout.
    constexpr int ATTEMPTS = NH == 2 ? 2 : 1;
    uint4 kr, vr;
    // With the maximum fixed the normaliser needs no rescaling, and the matrix unit sums it: the weights of 16 keys
    // x 32 queries as they lie in registers for the value product, read as the B operand of a 16x16x32 product, are
    // 16 columns x 32 slots, column c holding query c in slots 0-7 and 16-23 and query c + 16 in slots 8-15 and
    // 24-31; an A operand of ones in row 0 at the first and in row 1 at the second set of slots leaves the two sums
    // in rows 0 and 1 of column c (lanes 0..15, registers 0 and 1). (The sum instruction of the vector unit,
    // v_dot2c_f32_bf16, runs at two fifths of its rate beside another wavefront's matrix instructions.)
    floatx4 lacc[NH];
    auto selector = [&]() { // built where it is used: four registers less to keep (or spill) across the loops
        uint32_t z = 0u;
        asm volatile("" : "+v"(z));
        const uint32_t l31 = __builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, z)) & 31u;
        const uint32_t w = (l31 == 0u || l31 == 17u) ? 0x3f803f80u : 0u;
        return as_bf16x8(make_uint4(w, w, w, w));
    };
    for (int attempt = 0; attempt < ATTEMPTS; ++attempt) {
    const bool optimistic = NH == 2 && attempt == 0;
#pragma unroll
    for (int h = 0; h < NH; ++h) {
        const bool sink_here = a.sinks && !partial;
        m[h] = sink_here ? a.sinks[head[h]] * LNG_LOG2E : LNG_NEG_INF;
        l[h] = (sink_here && hh == 0) ? 1.0f : 0.0f;
        lacc[h] = floatx4{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int db = 0; db < 2; ++db) {
#pragma unroll
            for (int i = 0; i < 16; ++i) ot[h][db][i] = 0.0f;
        }
    }
    if (first_tile < n_tiles) {
        fetch(first_tile, kr, vr);
        stash(first_tile & 1u, kr, vr);
    }
    __syncthreads();

    // MODE 0: the running maximum is tracked. MODE 1: it is fixed (weights = 2^(score - m)). MODE 2: it is
    // fixed at zero (weights = 2^score: nothing but the exponential, the narrowing and the sum per score).
    // One block of 32 keys (kb = 0, 1 of a tile) for every head of the wavefront.
    auto block = [&](auto mask_tag, auto mode_tag, uint32_t tile, int kb) {
        constexpr bool MASK = decltype(mask_tag)::value;
        constexpr int MODE = decltype(mode_tag)::value;
        constexpr bool FIXED = MODE != 0;
        constexpr bool RAW = NH == 1; // the products are plain q.k: the factor is applied with the maximum
        const uint32_t buf = tile & 1u;
        const uint32_t kt0 = tile0 + tile * PF_BN; // position of the tile's first key
            {
                {
                // ---- S^T = K . Q^T, both heads ------------------------------------------------------
                bf16x8 ka[4];
#pragma unroll
                for (int ks = 0; ks < 4; ++ks) {
                    ka[ks] = as_bf16x8(*(const uint4 *)(&s_k[buf][k_lane_off + kb * 32 * PF_KSTRIDE + 16 * ks]));
                }
                floatx16 st[NH];
#pragma unroll
                for (int h = 0; h < NH; ++h) {
#pragma unroll
                    for (int i = 0; i < 16; ++i) st[h][i] = 0.0f;
                }
#pragma unroll
                for (int ks = 0; ks < 4; ++ks) {
                    st[0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ka[ks], qreg[0][ks], st[0], 0, 0, 0);
                    if constexpr (NH == 2) st[1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ka[ks], qreg[1][ks], st[1], 0, 0, 0);
                }
                // V^T operands of this block: two groups of 16 keys x two halves of the head width;
                // issued now, their LDS latency hides behind the softmax arithmetic
                bf16x8 va[2][2];
                auto read_v = [&]() {
#pragma unroll
                    for (int jj = 0; jj < 2; ++jj) {
#pragma unroll
                        for (int db = 0; db < 2; ++db) {
                            const uint16_t *vp = &s_v[buf][v_lane_off + (32 * kb + 16 * jj) * PF_VSTRIDE + 32 * db];
                            va[jj][db] = lds_read_tr8(vp, vp + 8 * PF_VSTRIDE);
                        }
                    }
                };
                read_v();
                // ---- online softmax, one query per lane -----------------------------------------------
                // The running maximum only moves when the block's maximum exceeds it by PF_TAU (log2
                // domain): weights then stay below 2^PF_TAU, and the accumulators are rescaled only
                // on the rare blocks where some lane's maximum moved. The normaliser uses the same
                // maximum, so the result is the same softmax.
                bf16x8 pb[NH][2];
#pragma unroll
                for (int h = 0; h < NH; ++h) {
                    if constexpr (MASK) {
                        // key kp = kt0 + 32 kb + 4 hh + o_i is visible when 0 <= my_pos - kp < window, i.e. when the
                        // constant o_i lies in (dist - window, dist]: two compares against per-block bounds
                        // With one head per wavefront (windows), a block of an edge tile that every query of the
                        // workgroup sees whole skips the masks: a uniform branch around them (three of the five
                        // blocks of a 128-position window).
                        const uint32_t b0 = kt0 + 32u * kb;
                        const bool cut = NH == 2 || b0 + 31u > pos_first || (windowed && b0 + window < pos_first + PF_BM);
                        if (cut) {
                            const int dist = (int)(my_pos - (b0 + 4u * hh));
                            const int below = windowed ? dist - (int)window : -0x40000000;
#pragma unroll
                            for (int i = 0; i < 16; ++i) {
                                const int o = 8 * (i >> 2) + (i & 3);
                                st[h][i] = (o <= dist && o > below) ? st[h][i] : LNG_NEG_INF;
                            }
                        }
                    }
                    float m_safe = 0.0f;
                    if constexpr (FIXED) {
                        m_safe = m[h]; // not -inf once frozen
                    } else {
                        float tmax = LNG_NEG_INF;
#pragma unroll
                        for (int i = 0; i < 16; ++i) tmax = fmaxf(tmax, st[h][i]);
                        tmax = other_half_max(tmax);
                        if constexpr (RAW) tmax *= sl2; // the host sends only positive factors this way
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
                    float psum[2] = {0.0f, 0.0f}; // two chains of four dependent sums instead of one of eight
#pragma unroll
                    for (int jj = 0; jj < 2; ++jj) {
#pragma unroll
                        for (int e = 0; e < 8; e += 2) {
                            const float s0 = st[h][8 * jj + e], s1 = st[h][8 * jj + e + 1];
                            const float p0 = __builtin_amdgcn_exp2f(RAW ? __builtin_fmaf(s0, sl2, MODE == 2 ? 0.0f : -m_safe) : MODE == 2 ? s0 : s0 - m_safe);
                            const float p1 = __builtin_amdgcn_exp2f(RAW ? __builtin_fmaf(s1, sl2, MODE == 2 ? 0.0f : -m_safe) : MODE == 2 ? s1 : s1 - m_safe);
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
                if constexpr (FIXED) {
                    const bf16x8 sel = selector();
#pragma unroll
                    for (int jj = 0; jj < 2; ++jj) {
#pragma unroll
                        for (int h = 0; h < NH; ++h) lacc[h] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(sel, pb[h][jj], lacc[h], 0, 0, 0);
                    }
                }
                // ---- O^T += V^T . P^T ---------------------------------------------------------------------
#pragma unroll
                for (int jj = 0; jj < 2; ++jj) {
#pragma unroll
                    for (int db = 0; db < 2; ++db) {
                        ot[0][db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(va[jj][db], pb[0][jj], ot[0][db], 0, 0, 0);
                        if constexpr (NH == 2) ot[1][db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(va[jj][db], pb[1][jj], ot[1][db], 0, 0, 0);
                    }
                }
            }
        }
    };
    // One tile step. Edge tiles (MASK) are a separate instantiation so that the interior loop
    // carries no position arithmetic at all.
    auto step = [&](auto mask_tag, auto mode_tag, uint32_t tile) {
        const uint32_t buf = tile & 1u;
        if (tile + 1 < n_tiles) fetch(tile + 1, kr, vr);
        if (wave_active) {
#pragma unroll
            for (int kb = 0; kb < 2; ++kb) {
                if constexpr (decltype(mask_tag)::value && NH == 1) {
                    const uint32_t b0 = tile0 + tile * PF_BN + 32u * kb;
                    if (b0 > pos_last || b0 + 31u < kfirst) continue; // windows: a block no query of the workgroup sees
                }
                block(mask_tag, mode_tag, tile, kb);
            }
        }
        if (tile + 1 < n_tiles) stash(buf ^ 1u, kr, vr);
        __syncthreads();
    };
    // interior tiles need no mask: every key visible to every query of the workgroup
    auto edge = [&](uint32_t tile) {
        const uint32_t kt0 = tile0 + tile * PF_BN;
        return kt0 + (PF_BN - 1) > pos_first || (windowed && kt0 + window < pos_first + PF_BM);
    };
    using tracked = std::integral_constant<int, 0>;
    using fixed_at_m = std::integral_constant<int, 1>;
    using fixed_at_zero = std::integral_constant<int, 2>;
    uint32_t tile = first_tile;
    bool frozen = false;
    {
    for (; tile < n_tiles && edge(tile); ++tile) step(std::true_type{}, tracked{}, tile); // window edge
    if (optimistic) {                                                                      // interior
        bool at_zero = false;
        if (tile < n_tiles && !edge(tile)) {
            step(std::false_type{}, tracked{}, tile); // sets the maximum from real scores
            ++tile;
            frozen = true;
            // Maxima of moderate size (|m| <= 40 in the exponent's units, for every query of the wavefront): move
            // the reference point to zero once, and the loop below has no subtraction left either.
            bool moderate = true;
#pragma unroll
            for (int h = 0; h < NH; ++h) {
                m[h] = m[h] == LNG_NEG_INF ? 0.0f : m[h];
                moderate = moderate && __builtin_fabsf(m[h]) <= 40.0f;
            }
            at_zero = __builtin_amdgcn_ballot_w64(!moderate) == 0;
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
        // loops of their own: one path through each, so their registers need no reconciling copies
        if (at_zero) {
            for (; tile < n_tiles && !edge(tile); ++tile) step(std::false_type{}, fixed_at_zero{}, tile);
        } else {
            for (; tile < n_tiles && !edge(tile); ++tile) step(std::false_type{}, fixed_at_m{}, tile);
        }
    } else {
        for (; tile < n_tiles && !edge(tile); ++tile) step(std::false_type{}, tracked{}, tile);
    }
    }
    if constexpr (NH == 2) {
        lane_values();
        row_values();
    }
    bool again = false;
    if (NH == 2 && frozen) { // frozen is uniform over the workgroup
        if (wave_active) {
            // query n's sum is in lane n % 16, register n / 16; l[] is per (query, half) and the halves are added at
            // the end, so the whole of it goes to the first half
#pragma unroll
            for (int h = 0; h < NH; ++h) {
                const float lo = __shfl(lacc[h][0], (int)(n & 15u), 64);
                const float hi = __shfl(lacc[h][1], (int)(n & 15u), 64);
                if (hh == 0u) l[h] += n < 16u ? lo : hi;
            }
        }
        int bad = 0;
        if (wave_active) {
#pragma unroll
            for (int h = 0; h < NH; ++h) {
                const float total = l[h] + __shfl_xor(l[h], 32, 64);
                uint32_t top = 0;
#pragma unroll
                for (int db = 0; db < 2; ++db) {
#pragma unroll
                    for (int i = 0; i < 16; ++i) top = max(top, __float_as_uint(ot[h][db][i]) & 0x7fffffffu);
                }
                // 2^-90 .. 2^100: terms lost below 2^-126 are then under 2^-19 of the total even for 2^17
                // keys, and nothing overflowed (a NaN fails the comparison)
                bad |= !(total >= 8.0779357e-28f && total <= 1.2676506e30f) || top >= 0x7f800000u;
            }
            bad = row_ok ? bad : 0;
        }
        // (the workgroup's OR through a word of LDS: the library routine works out a thread number from the three
        // thread indices, which live in registers from the kernel's start and are spilled by now)
        if (__builtin_amdgcn_ballot_w64(bad != 0) != 0) s_again = 1u;
        __syncthreads();
        again = s_again != 0u;
        __syncthreads(); // everyone has read it
        s_again = 0u;    // for the second attempt's check: its barriers lie between
        if (again && a.second_passes && wave == 0u && lane == 0u) __hip_atomic_fetch_add(a.second_passes, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    if (!again) {
        for (; tile < n_tiles; ++tile) step(std::true_type{}, tracked{}, tile);                    // diagonal
        break;
    }
    }


    if constexpr (NH == 2) {
        lane_values();
        row_values();
    }
    // ---- with splits: leave the partial state, lane holds dims 32db + 8blk + 4hh + i of its query. Through LDS
    // like the outputs below, 32 dimensions (128 bytes of f32) of 32 rows at a time: eight lanes store a whole line.
    if (partial) {
        if (wave_active) {
            float *stage = (float *)(wave < 4u ? &s_k[0][0] + wave * (32u * 72u) : &s_v[0][0] + (wave - 4u) * (32u * 72u));
#pragma unroll
            for (int h = 0; h < NH; ++h) {
                if (h == 1 && !second_ok) continue;
                const float total = l[h] + __shfl_xor(l[h], 32, 64);
                const uint64_t slot = (((uint64_t)my_row * a.kv_heads + g) * a.splits + split) * group + (head[h] - g * group);
                if (hh == 0 && row_ok) *(float2 *)(a.partial_ml + slot * 2u) = make_float2(m[h], total);
#pragma unroll
                for (int db = 0; db < 2; ++db) {
#pragma unroll
                    for (int blk = 0; blk < 4; ++blk) {
                        *(float4 *)(stage + n * 36u + 8 * blk + 4 * hh) = make_float4(ot[h][db][4 * blk + 0], ot[h][db][4 * blk + 1],
                                                                                      ot[h][db][4 * blk + 2], ot[h][db][4 * blk + 3]);
                    }
                    __builtin_amdgcn_wave_barrier();
#pragma unroll
                    for (int pass = 0; pass < 4; ++pass) {
                        const uint32_t r = 8u * pass + (lane >> 3), ch = lane & 7u;
                        const float4 piece = *(const float4 *)(stage + r * 36u + 4u * ch);
                        const uint32_t row = q0 + 32u * qb + r;
                        const uint64_t rslot = (((uint64_t)row * a.kv_heads + g) * a.splits + split) * group + (head[h] - g * group);
                        if (row < t) *(float4 *)(a.partial_o + rslot * 64u + 32 * db + 4u * ch) = piece;
                    }
                    __builtin_amdgcn_wave_barrier();
                }
            }
        }
        return;
    }

    // ---- normalise and store. A lane holds 8-byte pieces of its query's row (dims 32db + 8blk + 4hh + i), and 32
    // such pieces from 32 rows make a poor store: 16 partial writes to every 128-byte line. Through LDS (the K/V
    // buffers, which nobody reads after the last tile's barrier; 32 rows of 144 bytes per wavefront) eight lanes
    // write one whole 128-byte head row. No workgroup barrier: a wavefront's LDS operations run in order.
    if (wave_active) {
        uint16_t *stage = wave < 4u ? &s_k[0][0] + wave * (32u * 72u) : &s_v[0][0] + (wave - 4u) * (32u * 72u);
#pragma unroll
        for (int h = 0; h < NH; ++h) {
            if (h == 1 && !second_ok) continue;
            const float total = l[h] + __shfl_xor(l[h], 32, 64);
            const float inv = total > 0.0f ? 1.0f / total : 0.0f;
#pragma unroll
            for (int db = 0; db < 2; ++db) {
#pragma unroll
                for (int blk = 0; blk < 4; ++blk) {
                    bf16x4 w; // narrowed by the conversion instruction (round to nearest even)
#pragma unroll
                    for (int i = 0; i < 4; ++i) w[i] = (__bf16)(ot[h][db][4 * blk + i] * inv);
                    *(bf16x4 *)(stage + n * 72u + 32 * db + 8 * blk + 4 * hh) = w;
                }
            }
            __builtin_amdgcn_wave_barrier();
#pragma unroll
            for (int pass = 0; pass < 4; ++pass) {
                const uint32_t r = 8u * pass + (lane >> 3), ch = lane & 7u;
                const uint4 piece = *(const uint4 *)(stage + r * 72u + 8u * ch);
                const uint32_t row = q0 + 32u * qb + r;
                if (row < t) *(uint4 *)((uint16_t *)a.out + ((uint64_t)row * a.heads + head[h]) * 64u + 8u * ch) = piece;
            }
            __builtin_amdgcn_wave_barrier();
        }
    }
}

extern "C" __global__ __launch_bounds__(PF_THREADS) void lng_prefill_bf16_d64(lng_k_prefill a) {
    prefill_body<2>(a);
}

extern "C" __global__ __launch_bounds__(PF_THREADS, 4) void lng_prefill_bf16_d64_h1(lng_k_prefill a) {
    prefill_body<1>(a);
}

// Windows of at most 160 positions (unsplit passes): lng_prefill_bf16_d64_h1's arithmetic, block for block, with
// every K and V row of the workgroup requested at its start. A workgroup of eight wavefronts (a head each) takes 32
// query rows; they see at most 160 + 31 keys, which lie in at most seven blocks of 32 rows from a multiple of 32 (five
// for a window of 128 at a start that is a multiple of 32: 160 rows; whole tiles of 64 from a multiple of 64 were 256).
// These rows are asked for together with the queries by loads that write LDS directly (global_load_lds_dwordx4: no registers in between, so nothing limits how
// many are in flight); there is one barrier when they have landed, and the blocks of 32 keys then run without any
// further wait for memory - tile by tile, such a pass spends a memory round trip per tile: the loads of tile i+1
// leave when tile i's arithmetic starts and take longer than it does. A load of this kind puts the 16 bytes of
// lane l at base + 16 l, so rows cannot be padded; instead each lane fetches the piece that belongs at its place in
// a swizzled row: piece c (16 bytes) of K row r sits at c ^ ((r >> 1) & 7) - the 16-byte reads of 16 consecutive
// rows then fall in 16 different 16-byte bank groups - and piece c of V row r at c ^ (((r >> 1) & 1) << 2): the
// four rows x 64 bytes that half a wavefront reads transposed fall in four different quarters of the banks.
// After the last block a barrier says that nobody reads K and V any more, and each wavefront lays its rows down
// there so that eight lanes store a whole 128-byte row. 56 KiB of LDS: two workgroups per compute unit.
// (Measured and not kept: a first pass around zero - weights 2^score, no maxima, the sums on the matrix unit, a range
// check and the tracked pass again when it fails: 40 % fewer vector instructions per block, same time; workgroups of
// four wavefronts with two heads each, three to a compute unit with 48 KiB of LDS each: same time; 64 query rows per
// workgroup as two blocks of 32, one after the other, over the same K and V rows: 42 against 39 us.)
#define PW_BLOCKS 7 // blocks of 32 keys a workgroup may see: a window of 160, 32 rows, and up to 31 keys before the first
extern "C" __global__ __launch_bounds__(PF_THREADS, 4) void lng_prefill_bf16_d64_h1w(lng_k_prefill a) {
    __shared__ __attribute__((aligned(16))) uint16_t s_k[PW_BLOCKS * 32 * 64];
    __shared__ __attribute__((aligned(16))) uint16_t s_v[PW_BLOCKS * 32 * 64];
    const uint32_t g = blockIdx.x % a.kv_heads;
    const uint32_t qtile = a.q_tiles - 1u - blockIdx.x / a.kv_heads;
    const uint32_t group = a.heads / a.kv_heads;
    const uint32_t tid = threadIdx.x;
    const uint32_t lane = tid & 63u;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t n = lane & 31u;  // query within the block of 32
    const uint32_t hh = lane >> 5;  // which half of the k-slots / of each 8 accumulator rows
    const uint32_t t = (uint32_t)a.t, start = (uint32_t)a.start;
    const uint32_t q0 = qtile * 32u;
    const uint32_t rows_here = t - q0 < 32u ? t - q0 : 32u;
    const uint32_t end = start + t;
    const uint32_t pos_first = start + q0;
    const uint32_t pos_last = pos_first + rows_here - 1u;
    const uint32_t window = (uint32_t)a.window; // the host sends windows of 1..160 only
    const uint32_t kfirst = pos_first + 1u > window ? pos_first + 1u - window : 0u;
    const uint32_t blk0 = kfirst & ~31u; // the rows in LDS begin at a multiple of 32: 160 of them for a window of 128
    const uint32_t n_blocks = min((pos_last - blk0) / 32u + 1u, (uint32_t)PW_BLOCKS);
    const bool ring = a.slots < end;
    const uint32_t slots = (uint32_t)a.slots;
    const uint64_t row_bytes = (uint64_t)a.kv_heads * 128u;
    const float sl2 = a.scale * LNG_LOG2E;
    const bool wave_active = wave < group; // a wavefront past the group only helps loading
    const uint32_t head = g * group + (wave_active ? wave : 0u);

    // the head's sink: asked for here, with everything else (after the barrier it would be a memory round trip of its own)
    const float sink_l2 = a.sinks ? a.sinks[head] * LNG_LOG2E : LNG_NEG_INF;
    // the queries as they are: scale x log2(e) rides with the maximum
    const uint32_t my_pos = pos_first + n;
    bf16x8 qreg[4];
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) {
        uint4 raw = make_uint4(0, 0, 0, 0);
        if (q0 + n < t) raw = *(const uint4 *)(a.q + (((uint64_t)(q0 + n) * a.heads + head) * 64u + 16u * ks + 8u * hh) * 2u);
        qreg[ks] = as_bf16x8(raw);
    }
    // every K and V row of the workgroup: a wavefront's 64 lanes fill 8 whole rows of a tile
    {
        const uint32_t ld_row = 8u * wave + (lane >> 3), ld_chunk = lane & 7u;
        const uint32_t ck = ld_chunk ^ ((ld_row >> 1) & 7u), cv = ld_chunk ^ (((ld_row >> 1) & 1u) << 2);
        typedef __attribute__((address_space(1))) const void *gptr;
        typedef __attribute__((address_space(3))) void *lptr;
        // (eight wavefronts x eight rows at a time; a wavefront whose eight rows lie past the last block asks for nothing)
        for (uint32_t i = 0; 64u * i + 8u * wave < 32u * n_blocks; ++i) {
            uint32_t p = blk0 + 64u * i + ld_row;
            p = p > pos_last ? pos_last : p; // rows past the last needed position are masked anyway,
            p = p < kfirst ? kfirst : p;     // and so are rows before the first one (a ring may not hold them any more)
            const uint32_t r = ring ? p % slots : p;
            __builtin_amdgcn_global_load_lds((gptr)(a.k + (uint64_t)g * 128u + (uint64_t)r * row_bytes + ck * 16u),
                                             (lptr)(s_k + i * 4096u + wave * 512u), 16, 0, 0);
            __builtin_amdgcn_global_load_lds((gptr)(a.v + (uint64_t)g * 128u + (uint64_t)r * row_bytes + cv * 16u),
                                             (lptr)(s_v + i * 4096u + wave * 512u), 16, 0, 0);
        }
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); // this wavefront's rows are in LDS, its queries in registers
    __syncthreads();

    const uint32_t k_lane_off = n * 64u + ((hh ^ ((n >> 1) & 7u)) << 3); // ^ 16 ks, + 2048 b
    const uint32_t L = lane & 15u;
    const uint32_t blk16 = lane >> 4;
    // transposing read: source lane L names key (L>>2) of its group and dims 4*(L&3).. of the block's 16
    const uint32_t v_lane_off = (4u * (blk16 >> 1) + (L >> 2)) * 64u + 16u * (blk16 & 1u) + 4u * (L & 3u);
    const uint32_t v_flip = (L >> 3) & 1u; // rows two apart within a group of four have their 64-byte halves exchanged
    bf16x2 ones2;
    ones2[0] = (__bf16)1.0f;
    ones2[1] = (__bf16)1.0f;
    floatx16 ot[2];
    float l = 0.0f;
    if (wave_active) {
        float m = sink_l2;
        l = (a.sinks && hh == 0) ? 1.0f : 0.0f;
#pragma unroll
        for (int db = 0; db < 2; ++db) {
#pragma unroll
            for (int i = 0; i < 16; ++i) ot[db][i] = 0.0f;
        }
        // blocks of 32 keys from the one that holds the first visible key to the one that holds the last
        for (uint32_t b = 0; b < n_blocks; ++b) {
            bf16x8 ka[4];
#pragma unroll
            for (int ks = 0; ks < 4; ++ks) ka[ks] = as_bf16x8(*(const uint4 *)(&s_k[(k_lane_off ^ (16u * ks)) + b * 2048u]));
            floatx16 st;
#pragma unroll
            for (int i = 0; i < 16; ++i) st[i] = 0.0f;
#pragma unroll
            for (int ks = 0; ks < 4; ++ks) st = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ka[ks], qreg[ks], st, 0, 0, 0);
            // V^T operands: issued now, their LDS latency hides behind the softmax arithmetic
            bf16x8 va[2][2];
#pragma unroll
            for (int jj = 0; jj < 2; ++jj) {
#pragma unroll
                for (int db = 0; db < 2; ++db) {
                    const uint16_t *vp = &s_v[v_lane_off + (32u * b + 16 * jj) * 64u + 32 * (db ^ v_flip)];
                    va[jj][db] = lds_read_tr8(vp, vp + 8 * 64);
                }
            }
            // key kp = b0 + 4 hh + o_i is visible when 0 <= my_pos - kp < window; a block every row sees whole skips it
            const uint32_t b0 = blk0 + 32u * b;
            if (b0 + 31u > pos_first || b0 + window < pos_first + 32u) {
                const int dist = (int)(my_pos - (b0 + 4u * hh));
                const int below = dist - (int)window;
#pragma unroll
                for (int i = 0; i < 16; ++i) {
                    const int o = 8 * (i >> 2) + (i & 3);
                    st[i] = (o <= dist && o > below) ? st[i] : LNG_NEG_INF;
                }
            }
            // the running maximum only moves when the block's exceeds it by PF_TAU (see prefill_body)
            float tmax = LNG_NEG_INF;
#pragma unroll
            for (int i = 0; i < 16; ++i) tmax = fmaxf(tmax, st[i]);
            tmax = other_half_max(tmax) * sl2; // the host sends only positive factors this way
            const float m_new = tmax > m + PF_TAU ? tmax : m;
            const float m_safe = m_new == LNG_NEG_INF ? 0.0f : m_new;
            if (__builtin_amdgcn_ballot_w64(m_new != m) != 0) {
                const float alpha = __builtin_amdgcn_exp2f(m - m_safe);
                l *= alpha;
#pragma unroll
                for (int db = 0; db < 2; ++db) {
#pragma unroll
                    for (int i = 0; i < 16; ++i) ot[db][i] *= alpha;
                }
                m = m_new;
            }
            bf16x8 pb[2];
            float psum[2] = {0.0f, 0.0f};
#pragma unroll
            for (int jj = 0; jj < 2; ++jj) {
#pragma unroll
                for (int e = 0; e < 8; e += 2) {
                    bf16x2 pr;
                    pr[0] = (__bf16)__builtin_amdgcn_exp2f(__builtin_fmaf(st[8 * jj + e], sl2, -m_safe));
                    pr[1] = (__bf16)__builtin_amdgcn_exp2f(__builtin_fmaf(st[8 * jj + e + 1], sl2, -m_safe));
                    pb[jj][e] = pr[0];
                    pb[jj][e + 1] = pr[1];
                    psum[jj] = __builtin_amdgcn_fdot2_f32_bf16(pr, ones2, psum[jj], false); // the sum of the rounded weights
                }
            }
            l += psum[0] + psum[1];
#pragma unroll
            for (int jj = 0; jj < 2; ++jj) {
#pragma unroll
                for (int db = 0; db < 2; ++db) ot[db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(va[jj][db], pb[jj], ot[db], 0, 0, 0);
            }
        }
    }
    __syncthreads(); // K and V are dead: the outputs go through their place (32 rows of 144 bytes per wavefront)
    if (!wave_active) return;
    const float total = l + __shfl_xor(l, 32, 64);
    const float inv = total > 0.0f ? 1.0f / total : 0.0f;
    uint16_t *stage = wave < 4u ? s_k + wave * (32u * 72u) : s_v + (wave - 4u) * (32u * 72u);
#pragma unroll
    for (int db = 0; db < 2; ++db) {
#pragma unroll
        for (int blk = 0; blk < 4; ++blk) {
            bf16x4 w; // narrowed by the conversion instruction (round to nearest even)
#pragma unroll
            for (int i = 0; i < 4; ++i) w[i] = (__bf16)(ot[db][4 * blk + i] * inv);
            *(bf16x4 *)(stage + n * 72u + 32 * db + 8 * blk + 4 * hh) = w;
        }
    }
    __builtin_amdgcn_wave_barrier();
#pragma unroll
    for (int pass = 0; pass < 4; ++pass) {
        const uint32_t r = 8u * pass + (lane >> 3), ch = lane & 7u;
        const uint4 piece = *(const uint4 *)(stage + r * 72u + 8u * ch);
        const uint32_t row = q0 + r;
        if (row < t) *(uint4 *)((uint16_t *)a.out + ((uint64_t)row * a.heads + head) * 64u + 8u * ch) = piece;
    }
}

// =============================================================================================
// The long full-causal prompt pass (no window, no ring, keys not split): lng_prefill_bf16_d64's
// arithmetic, tile for tile, in a workgroup that STAYS on its compute unit and walks several
// query tiles.
//
// Why: with one workgroup per (query tile, kv head) a compute unit runs about four workgroups one
// after the other on an 8192-position pass, and each pays about 20 us that no other work hides (it is
// alone on its unit): the dispatch gap, a round trip for its queries and another for its first K/V
// tile, the one-off tiles, the scattered stores - a tenth of the pass - and the units finish up to
// 60 us apart. Here the grid is one workgroup per compute unit (kv head = id % kv_heads, so the ids
// of one kv head share an XCD and its L2), and workgroup c of the C that share a kv head takes query
// tiles c, 2C-1-c, 2C+c, 4C-1-c, ... counted from the longest: every unit gets the same number of key
// tiles to within one per round. Queries and the first two K/V tiles of a query tile arrive in one
// round trip.
//
// K/V tiles go through THREE LDS buffers: tile i + 2 is fetched into registers during tile i and
// stored at its end, so when a tile starts, the next one is already visible, and the K operands of
// the next tile's first block are read before the barrier, under the last products of this one
// (with two buffers every tile began by waiting for its first LDS reads with the matrix unit idle).
// =============================================================================================
// (Measured and not kept: two four-wavefront workgroups of 32 rows per compute unit, which share no barrier:
// 565 us against 521 us; tiles of 128 keys per barrier: 546 us.)
extern "C" __global__ __launch_bounds__(PF_THREADS) void lng_prefill_bf16_d64_stream(lng_k_prefill a) {
    constexpr int NH = 2;
    constexpr int QB = 2;                    // blocks of 32 query rows per workgroup
    constexpr uint32_t PF_BM = 32u * QB;
    constexpr int KB = 2;                    // blocks of 32 keys per tile, i.e. per barrier
    constexpr uint32_t SBN = 32u * KB;       // keys per tile
    constexpr int LD = (int)SBN / (32 * QB); // keys of a tile each thread loads
    __shared__ __attribute__((aligned(16))) uint16_t s_k[3][SBN * PF_KSTRIDE];
    __shared__ __attribute__((aligned(16))) uint16_t s_v[3][SBN * PF_VSTRIDE];
    __shared__ uint32_t s_again; // the outcome of the range check, see below

    const uint32_t c = blockIdx.x / a.kv_heads;   // this workgroup among the C of its kv head
    const uint32_t C = gridDim.x / a.kv_heads;
    const uint32_t group = a.heads / a.kv_heads;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    // What a lane derives from its number (its query, its half, its LDS and cache offsets) is cheap to work out and
    // expensive to keep: registers that live across the interior loop without being used in it are spilled, a spill
    // goes out to memory, and its reload waits for every load in flight. These are therefore worked out again at the
    // top of a query tile, after its interior loop and before its outputs, from a lane number the compiler cannot
    // follow (so that it does not keep the first copy instead).
    uint32_t lane, tid, n, hh, ld_key, ld_chunk, k_lane_off, v_lane_off;
    const char *kbase, *vbase;
    const uint32_t g = blockIdx.x % a.kv_heads;
    auto lane_values = [&]() {
        uint32_t z = 0u;
        asm volatile("" : "+v"(z));
        lane = __builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, z));
        tid = wave * 64u + lane;
        n = lane & 31u;
        hh = lane >> 5;
        ld_key = tid >> 3; // a thread's further keys are 32 * QB apart
        ld_chunk = tid & 7u;
        kbase = a.k + (uint64_t)g * 128u + ld_chunk * 16u;
        vbase = a.v + (uint64_t)g * 128u + ld_chunk * 16u;
        k_lane_off = n * PF_KSTRIDE + 8u * hh;
        const uint32_t L = lane & 15u;
        const uint32_t blk16 = lane >> 4;
        v_lane_off = (4u * (blk16 >> 1) + (L >> 2)) * PF_VSTRIDE + 16u * (blk16 & 1u) + 4u * (L & 3u);
    };
    lane_values();
    s_again = 0u; // (every thread, the same value; the first barrier below is ahead of its first use)
    const uint32_t qb = QB == 2 ? (wave & 1u) : 0u;
    const uint32_t hp = QB == 2 ? (wave >> 1) : wave;
    const uint32_t t = (uint32_t)a.t, start = (uint32_t)a.start;
    const uint64_t row_bytes = (uint64_t)a.kv_heads * 128u;

    const bool wave_active = hp * NH < group;
    const bool second_ok = hp * 2u + 1u < group;
    uint32_t head[NH];
    head[0] = g * group + (wave_active ? hp * NH : 0u);
    head[1] = second_ok ? head[0] + 1u : head[0];
    const float sl2 = a.scale * LNG_LOG2E;
    float sink2[NH]; // read once, not per query tile (and both in one trip)
#pragma unroll
    for (int h = 0; h < NH; ++h) sink2[h] = LNG_NEG_INF;
    if (a.sinks) {
        float raw[NH];
#pragma unroll
        for (int h = 0; h < NH; ++h) raw[h] = a.sinks[head[h]];
#pragma unroll
        for (int h = 0; h < NH; ++h) sink2[h] = raw[h] * LNG_LOG2E;
    }
    bf16x2 ones2;
    ones2[0] = (__bf16)1.0f;
    ones2[1] = (__bf16)1.0f;


    using tracked = std::integral_constant<int, 0>;
    using fixed_at_m = std::integral_constant<int, 1>;
    using fixed_at_zero = std::integral_constant<int, 2>;

    for (uint32_t round = 0;; ++round) {
        const uint32_t idx = round * C + ((round & 1u) ? C - 1u - c : c);
        if (idx >= a.q_tiles) break; // idx grows with the round for every c: nothing later either
        const uint32_t qtile = a.q_tiles - 1u - idx;
        const uint32_t q0 = qtile * PF_BM;
        const uint32_t rows_here = t - q0 < PF_BM ? t - q0 : PF_BM;
        const uint32_t pos_first = start + q0;
        const uint32_t pos_last = pos_first + rows_here - 1;
        const uint32_t n_tiles = pos_last / SBN + 1;
        const uint32_t n_interior = (pos_first + 1u) / SBN; // tiles whose every key every query of the tile sees
        uint32_t my_row, my_pos;
        bool row_ok;
        auto row_values = [&]() {
            lane_values();
            my_row = q0 + 32u * qb + n;
            my_pos = start + my_row;
            row_ok = my_row < t;
        };
        row_values();

        auto fetch = [&](uint32_t tile, uint4 (&kr)[LD], uint4 (&vr)[LD]) {
#pragma unroll
            for (int u = 0; u < LD; ++u) {
                uint32_t p = tile * SBN + ld_key + (32u * QB) * u;
                p = p > pos_last ? pos_last : p; // rows past the last needed position are masked anyway
                kr[u] = *(const uint4 *)(kbase + (uint64_t)p * row_bytes);
                vr[u] = *(const uint4 *)(vbase + (uint64_t)p * row_bytes);
            }
        };
        auto stash = [&](uint32_t buf, const uint4 (&kr)[LD], const uint4 (&vr)[LD]) {
#pragma unroll
            for (int u = 0; u < LD; ++u) {
                *(uint4 *)(&s_k[buf][(ld_key + (32u * QB) * u) * PF_KSTRIDE + ld_chunk * 8u]) = kr[u];
                *(uint4 *)(&s_v[buf][(ld_key + (32u * QB) * u) * PF_VSTRIDE + ld_chunk * 8u]) = vr[u];
            }
        };
        auto read_k = [&](uint32_t buf, int kb, bf16x8 (&ka)[4]) {
#pragma unroll
            for (int ks = 0; ks < 4; ++ks) {
                ka[ks] = as_bf16x8(*(const uint4 *)(&s_k[buf][k_lane_off + kb * 32 * PF_KSTRIDE + 16 * ks]));
            }
        };

        // ---- queries (scaled once, see lng_prefill_bf16_d64) and the first two tiles: one round trip ----
        bf16x8 qreg[NH][4];
        {
            uint4 raw[NH][4];
#pragma unroll
            for (int h = 0; h < NH; ++h) {
#pragma unroll
                for (int ks = 0; ks < 4; ++ks) {
                    raw[h][ks] = make_uint4(0, 0, 0, 0);
                    if (row_ok) {
                        raw[h][ks] = *(const uint4 *)(a.q + (((uint64_t)my_row * a.heads + head[h]) * 64u + 16u * ks + 8u * hh) * 2u);
                    }
                }
            }
            uint4 k0[LD], v0[LD], k1[LD], v1[LD];
            fetch(0, k0, v0);
            fetch(n_tiles > 1u ? 1u : 0u, k1, v1);
            stash(0, k0, v0);
            stash(1, k1, v1);
#pragma unroll
            for (int h = 0; h < NH; ++h) {
#pragma unroll
                for (int ks = 0; ks < 4; ++ks) {
                    bf16x8 qv = as_bf16x8(raw[h][ks]);
#pragma unroll
                    for (int e = 0; e < 8; ++e) qv[e] = (__bf16)((float)qv[e] * sl2);
                    qreg[h][ks] = qv;
                }
            }
        }
        __syncthreads();

        float m[NH], l[NH];
        floatx16 ot[NH][2];
        uint4 kr[LD], vr[LD];
        bf16x8 ka0[4];       // K operands of the coming tile's first block of 32 keys
        uint32_t buf = 0;    // LDS buffer of the coming tile; tile + 1 is in buf + 1, tile + 2 goes to buf + 2 (mod 3)

        auto step = [&](auto mask_tag, auto mode_tag, uint32_t tile) {
            constexpr bool MASK = decltype(mask_tag)::value;
            constexpr int MODE = decltype(mode_tag)::value;
            constexpr bool FIXED = MODE != 0;
            const uint32_t nxt = buf == 2u ? 0u : buf + 1u;
            const uint32_t after = nxt == 2u ? 0u : nxt + 1u;
            fetch(tile + 2, kr, vr); // (past the last tile: its rows again, stored where nobody reads them)
            if (wave_active) {
                const uint32_t kt0 = tile * SBN;
#pragma unroll
                for (int kb = 0; kb < KB; ++kb) {
                    if constexpr (MASK) { // a block of keys past the last row of the tile: nobody sees it
                        if (kt0 + 32u * kb > pos_last) continue;
                    }
                    bf16x8 ka[4];
                    if (kb == 0) {
#pragma unroll
                        for (int ks = 0; ks < 4; ++ks) ka[ks] = ka0[ks];
                    } else {
                        read_k(buf, kb, ka);
                    }
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
                            const uint16_t *vp = &s_v[buf][v_lane_off + (32 * kb + 16 * jj) * PF_VSTRIDE + 32 * db];
                            va[jj][db] = lds_read_tr8(vp, vp + 8 * PF_VSTRIDE);
                        }
                    }
                    // the next tile's first operands, under this block's arithmetic and products (after the last
                    // tile this reads a buffer that nobody uses: no branch in the middle of the tile)
                    if (kb == KB - 1) read_k(nxt, 0, ka0);
                    bf16x8 pb[NH][2];
#pragma unroll
                    for (int h = 0; h < NH; ++h) {
                        if constexpr (MASK) {
#pragma unroll
                            for (int i = 0; i < 16; ++i) {
                                const uint32_t kp = kt0 + 32u * kb + 8u * (i >> 2) + 4u * hh + (i & 3);
                                st[h][i] = kp <= my_pos ? st[h][i] : LNG_NEG_INF;
                            }
                        }
                        float m_safe;
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
                                const float p0 = __builtin_amdgcn_exp2f(MODE == 2 ? st[h][8 * jj + e] : st[h][8 * jj + e] - m_safe);
                                const float p1 = __builtin_amdgcn_exp2f(MODE == 2 ? st[h][8 * jj + e + 1] : st[h][8 * jj + e + 1] - m_safe);
                                bf16x2 pr;
                                pr[0] = (__bf16)p0;
                                pr[1] = (__bf16)p1;
                                pb[h][jj][e] = pr[0];
                                pb[h][jj][e + 1] = pr[1];
                                psum[jj] = __builtin_amdgcn_fdot2_f32_bf16(pr, ones2, psum[jj], false);
                            }
                        }
                        l[h] += psum[0] + psum[1];
                    }
#pragma unroll
                    for (int jj = 0; jj < 2; ++jj) {
#pragma unroll
                        for (int db = 0; db < 2; ++db) {
                            ot[0][db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(va[jj][db], pb[0][jj], ot[0][db], 0, 0, 0);
                            ot[1][db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(va[jj][db], pb[1][jj], ot[1][db], 0, 0, 0);
                        }
                    }
                }
            }
            stash(after, kr, vr);
            __syncthreads();
            buf = nxt;
        };

        // ---- the interior tiles with the maximum fixed at zero: matrix and arithmetic phases, the two wavefronts
        // of a SIMD one phase apart ----------------------------------------------------------------------------
        // Per block of 32 keys a wavefront (two heads) has a MATRIX phase - the 8 score products of the block, the 8
        // value products and 4 normaliser products of the block before, then the LDS reads of the next operands -
        // and an ARITHMETIC phase - 32 exponentials and 16 narrowings, nothing else. A wavefront that issues both
        // kinds side by side overlaps them only partly on this part, and two wavefronts that are in the same phase
        // at the same time share one pipe while the other idles; a wavefront in its matrix phase beside one in its
        // arithmetic phase keeps both busy. The tile barrier would put all wavefronts in the same phase, so the
        // second wavefront of every SIMD (w + 4) passes it one phase earlier in its own sequence: after the second
        // matrix phase of the tile, where the first passes it after the second arithmetic phase. Both make the
        // same phases in the same order and pass one barrier per tile.
        // LDS: every read of a tile's buffer is issued before the barrier that ends the tile (the late wavefronts
        // have read the second block's V operands and the next tile's first K operands by then); the buffer is
        // written again two tiles later. K/V rows are asked for a whole tile before they are stored to LDS: a
        // barrier waits for the slowest load of 512 threads.
        auto pipe = [&](uint32_t &tile) {
            const bool late = wave >= 4u;
            floatx16 st[NH];
            bf16x8 pb[NH][2];   // weights of the last block, their value products pending
            // The normaliser is summed by the matrix unit as well: the weights of 16 keys x 32 queries, as they lie in
            // registers for the value product (lane = query n, half hh = keys 8hh..8hh+7), read as the B operand of a
            // 16x16x32 product are 16 columns x 32 slots, column c holding query c in slots 0-7 and 16-23 and query
            // c + 16 in slots 8-15 and 24-31. An A operand with ones in row 0 at the first and row 1 at the second set of
            // slots leaves the sums of queries c and c + 16 in rows 0 and 1 of column c: lanes 0..15, registers 0 and 1.
            floatx4 lacc[NH];
#pragma unroll
            for (int h = 0; h < NH; ++h) lacc[h] = floatx4{0.0f, 0.0f, 0.0f, 0.0f};
            // (built where it is used, from a lane mask: four registers that would otherwise be spilled and reloaded
            // in the loop, and a reload there waits for the K/V loads in flight)
            auto selector = [&]() {
                uint32_t z = 0u;
                asm volatile("" : "+v"(z)); // not a loop invariant: nothing of this is kept in a register between uses
                const uint32_t l31 = __builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, z)) & 31u;
                const uint32_t w = (l31 == 0u || l31 == 17u) ? 0x3f803f80u : 0u; // rows 0 / 1 at slot groups 0, 2 / 1, 3
                return as_bf16x8(make_uint4(w, w, w, w));
            };
            bf16x8 va[2][2];    // and its V^T operands
            auto zero16 = [&]() {
                floatx16 z;
#pragma unroll
                for (int i = 0; i < 16; ++i) z[i] = 0.0f;
                return z;
            };
            // nothing pending yet: weights of zero against any finite operands
#pragma unroll
            for (int jj = 0; jj < 2; ++jj) {
#pragma unroll
                for (int h = 0; h < NH; ++h) {
#pragma unroll
                    for (int e = 0; e < 8; ++e) pb[h][jj][e] = (__bf16)0.0f;
                }
#pragma unroll
                for (int db = 0; db < 2; ++db) va[jj][db] = pb[0][jj];
            }
            // matrix phase of block kb of the tile in `b`: scores of the block, values and weight sums of the block
            // before, then the operands of the next matrix phase (K of the next block, V of this one)
            auto matrix = [&](uint32_t b, uint32_t b_next, int kb) {
                const bf16x8 sel = selector();
                __builtin_amdgcn_sched_barrier(0);
                st[0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ka0[0], qreg[0][0], zero16(), 0, 0, 0);
                st[1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ka0[0], qreg[1][0], zero16(), 0, 0, 0);
#pragma unroll
                for (int ks = 1; ks < 4; ++ks) {
                    st[0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ka0[ks], qreg[0][ks], st[0], 0, 0, 0);
                    st[1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ka0[ks], qreg[1][ks], st[1], 0, 0, 0);
                }
#pragma unroll
                for (int jj = 0; jj < 2; ++jj) {
#pragma unroll
                    for (int db = 0; db < 2; ++db) {
                        ot[0][db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(va[jj][db], pb[0][jj], ot[0][db], 0, 0, 0);
                        ot[1][db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(va[jj][db], pb[1][jj], ot[1][db], 0, 0, 0);
                    }
                    lacc[0] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(sel, pb[0][jj], lacc[0], 0, 0, 0);
                    lacc[1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(sel, pb[1][jj], lacc[1], 0, 0, 0);
                }
                __builtin_amdgcn_sched_barrier(0);
                if (kb + 1 < KB) {
                    read_k(b, kb + 1, ka0);
                } else {
                    read_k(b_next, 0, ka0);
                }
#pragma unroll
                for (int jj = 0; jj < 2; ++jj) {
#pragma unroll
                    for (int db = 0; db < 2; ++db) {
                        const uint16_t *vp = &s_v[b][v_lane_off + (32 * kb + 16 * jj) * PF_VSTRIDE + 32 * db];
                        va[jj][db] = lds_read_tr8(vp, vp + 8 * PF_VSTRIDE);
                    }
                }
                __builtin_amdgcn_sched_barrier(0);
            };
            // (the empty asm statements keep the phase where it is written: its arithmetic has no side effects, and
            // the compiler would otherwise move parts of it behind the matrix phase and the barrier that follow)
            auto arithmetic = [&]() {
#pragma unroll
                for (int h = 0; h < NH; ++h) asm volatile("" : "+v"(st[h]));
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int h = 0; h < NH; ++h) {
#pragma unroll
                    for (int jj = 0; jj < 2; ++jj) {
#pragma unroll
                        for (int e = 0; e < 8; e += 2) {
                            const float p0 = __builtin_amdgcn_exp2f(st[h][8 * jj + e]);
                            const float p1 = __builtin_amdgcn_exp2f(st[h][8 * jj + e + 1]);
                            pb[h][jj][e] = (__bf16)p0;
                            pb[h][jj][e + 1] = (__bf16)p1;
                        }
                    }
                }
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int h = 0; h < NH; ++h) asm volatile("" : "+v"(pb[h][0]), "+v"(pb[h][1]));
            };
            auto publish = [&](uint32_t after) { // the tile after next goes to LDS, the one after that is asked for; the tile ends
                stash(after, kr, vr);
                fetch(tile + 3, kr, vr); // a whole tile before it is stored (past the last tile: its rows again, never stored)
                __builtin_amdgcn_s_waitcnt(0xC07F); // lgkmcnt(0)
                __builtin_amdgcn_s_barrier();
            };
            // (the first operands are read here again rather than taken from the step before: carried across the
            // rescaling to zero they were spilled and reloaded, sixteen registers per query tile)
            read_k(buf, 0, ka0);
            fetch(tile + 2, kr, vr);
            auto loop = [&](auto active_tag) {
                constexpr bool ACTIVE = decltype(active_tag)::value;
                for (; tile < n_interior; ++tile) {
                    const uint32_t nxt = buf == 2u ? 0u : buf + 1u;
                    const uint32_t after = nxt == 2u ? 0u : nxt + 1u;
                    if constexpr (ACTIVE) {
#pragma unroll
                        for (int kb = 0; kb + 1 < KB; ++kb) {
                            matrix(buf, nxt, kb);
                            arithmetic();
                        }
                        matrix(buf, nxt, KB - 1);
                        if (late) publish(after);
                        arithmetic();
                        if (!late) publish(after);
                    } else {
                        publish(after);
                    }
                    buf = nxt;
                }
            };
            if (wave_active) {
                loop(std::true_type{});
            } else {
                loop(std::false_type{});
            }
            if (wave_active) { // the last block's values
                const bf16x8 sel = selector();
#pragma unroll
                for (int jj = 0; jj < 2; ++jj) {
#pragma unroll
                    for (int db = 0; db < 2; ++db) {
                        ot[0][db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(va[jj][db], pb[0][jj], ot[0][db], 0, 0, 0);
                        ot[1][db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(va[jj][db], pb[1][jj], ot[1][db], 0, 0, 0);
                    }
                    lacc[0] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(sel, pb[0][jj], lacc[0], 0, 0, 0);
                    lacc[1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(sel, pb[1][jj], lacc[1], 0, 0, 0);
                }
                // query n's sum is in lane n % 16, register n / 16; l[] is per (query, half) and the halves are added
                // at the end, so the whole of it goes to the first half
#pragma unroll
                for (int h = 0; h < NH; ++h) {
                    const float lo = __shfl(lacc[h][0], (int)(n & 15u), 64);
                    const float hi = __shfl(lacc[h][1], (int)(n & 15u), 64);
                    if (hh == 0u) l[h] += n < 16u ? lo : hi;
                }
            }
        };

        for (int attempt = 0; attempt < 2; ++attempt) {
            const bool optimistic = attempt == 0;
#pragma unroll
            for (int h = 0; h < NH; ++h) {
                m[h] = sink2[h];
                l[h] = (a.sinks && hh == 0) ? 1.0f : 0.0f;
#pragma unroll
                for (int db = 0; db < 2; ++db) {
#pragma unroll
                    for (int i = 0; i < 16; ++i) ot[h][db][i] = 0.0f;
                }
            }
            if (attempt != 0) { // the tiles again from the first: the buffers hold later ones by now
                uint4 k0[LD], v0[LD], k1[LD], v1[LD];
                fetch(0, k0, v0);
                fetch(n_tiles > 1u ? 1u : 0u, k1, v1);
                stash(0, k0, v0);
                stash(1, k1, v1);
                __syncthreads();
            }
            buf = 0;
            if (wave_active) read_k(0, 0, ka0);
            uint32_t tile = 0;
            bool frozen = false;
            if (optimistic) {
                bool at_zero = false;
                if (n_interior > 0u) {
                    step(std::false_type{}, tracked{}, tile); // sets the maximum from real scores
                    ++tile;
                    frozen = true;
                    bool moderate = true;
#pragma unroll
                    for (int h = 0; h < NH; ++h) {
                        m[h] = m[h] == LNG_NEG_INF ? 0.0f : m[h];
                        moderate = moderate && __builtin_fabsf(m[h]) <= 40.0f;
                    }
                    at_zero = __builtin_amdgcn_ballot_w64(!moderate) == 0;
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
                if (at_zero) {
                    pipe(tile);
                    row_values();
                    // the diagonal at the same fixed reference point (a masked score is 2^-inf = 0), before the check
                    for (; tile < n_tiles; ++tile) step(std::true_type{}, fixed_at_zero{}, tile);
                } else {
                    for (; tile < n_interior; ++tile) step(std::false_type{}, fixed_at_m{}, tile);
                }
            } else {
                for (; tile < n_interior; ++tile) step(std::false_type{}, tracked{}, tile);
            }
            bool again = false;
            if (frozen) { // uniform over the workgroup
                int bad = 0;
                if (wave_active) {
#pragma unroll
                    for (int h = 0; h < NH; ++h) {
                        const float total = l[h] + __shfl_xor(l[h], 32, 64);
                        uint32_t top = 0;
#pragma unroll
                        for (int db = 0; db < 2; ++db) {
#pragma unroll
                            for (int i = 0; i < 16; ++i) top = max(top, __float_as_uint(ot[h][db][i]) & 0x7fffffffu);
                        }
                        bad |= !(total >= 8.0779357e-28f && total <= 1.2676506e30f) || top >= 0x7f800000u;
                    }
                    bad = row_ok ? bad : 0;
                }
                // (the workgroup's OR through a word of LDS: the library routine works out a thread number from the
                // three thread indices, which live in registers from the kernel's start and had been spilled by now -
                // two trips to memory per query tile)
                if (__builtin_amdgcn_ballot_w64(bad != 0) != 0) s_again = 1u;
                __syncthreads();
                again = s_again != 0u;
                __syncthreads(); // everyone has read it
                s_again = 0u;    // for the next query tile: its first barrier is ahead of the next check
                if (again && a.second_passes && wave == 0u && lane == 0u) __hip_atomic_fetch_add(a.second_passes, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
            if (!again) {
                for (; tile < n_tiles; ++tile) step(std::true_type{}, tracked{}, tile); // the diagonal, where not done yet
                break;
            }
        }

        row_values();
        // ---- normalise and store: lane holds dims 32db + 8blk + 4hh + i of its query ------------------
        if (wave_active && row_ok) {
#pragma unroll
            for (int h = 0; h < NH; ++h) {
                if (h == 1 && !second_ok) continue;
                const float total = l[h] + __shfl_xor(l[h], 32, 64);
                const float inv = total > 0.0f ? 1.0f / total : 0.0f;
                uint16_t *op = (uint16_t *)a.out + ((uint64_t)my_row * a.heads + head[h]) * 64u;
#pragma unroll
                for (int db = 0; db < 2; ++db) {
#pragma unroll
                    for (int blk = 0; blk < 4; ++blk) {
                        bf16x4 w; // narrowed by the conversion instruction (round to nearest even)
#pragma unroll
                        for (int i = 0; i < 4; ++i) w[i] = (__bf16)(ot[h][db][4 * blk + i] * inv);
                        *(bf16x4 *)(op + 32 * db + 8 * blk + 4 * hh) = w;
                    }
                }
            }
        }
        // (the last step of this query tile ended with a barrier: every wavefront is done with the buffers)
    }
}

// =============================================================================================
// Prompt-pass kernel, f32 (the reference's own element type), head width 64, up to 8 query heads
// per kv head: the bf16 kernel's plan on the f32 matrix instruction.
//
// A workgroup (8 wavefronts) takes 32 consecutive query positions and all query heads of one kv
// head, one head per wavefront; K/V tiles of 64 keys go through LDS as f32. Per 32-key block
//   S^T[key][query] = K . Q^T    32 x v_mfma_f32_32x32x2_f32: lane (query n, half hh) feeds dims
//                                8j + 4hh + e of its key row (ds_read_b128) and of its query (registers)
//   O^T[dim][query] += V^T . P^T 32 x the same instruction: lane (n, hh) holds the weights of keys
//                                8a + 4hh + e, which is how the first product left them, and reads
//                                V[that key][dim 32db + n] with ds_read_b32
// so softmax state and output column are lane-local exactly as in the bf16 kernel, and the
// arithmetic is f32 throughout (products are not rounded to a narrower type anywhere). The kernel
// is bound by the f32 matrix rate (64 FLOP per clock and SIMD, a sixteenth of bf16).
// =============================================================================================
#define PF32_BM 32u
#define PF32_KSTRIDE 68 // floats per LDS row of K: 16-byte reads of 16 consecutive rows cover all 64 banks
#define PF32_VSTRIDE 72 // of V: the rows 4 apart that the two halves of a wavefront read fall 32 banks apart

__device__ __forceinline__ void prefill_f32_body(const lng_k_prefill &a) {
    __shared__ __attribute__((aligned(16))) float s_k[2][PF_BN * PF32_KSTRIDE];
    __shared__ __attribute__((aligned(16))) float s_v[2][PF_BN * PF32_VSTRIDE];

    const uint32_t g = blockIdx.x % a.kv_heads;
    const uint32_t split = (blockIdx.x / a.kv_heads) % a.splits;
    const uint32_t qtile = a.q_tiles - 1u - blockIdx.x / a.kv_heads / a.splits;
    const uint32_t group = a.heads / a.kv_heads;
    const uint32_t tid = threadIdx.x;
    const uint32_t lane = tid & 63u;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t n = lane & 31u; // query within the workgroup's block
    const uint32_t hh = lane >> 5; // which of the two k slots of the matrix instruction

    const uint32_t t = (uint32_t)a.t, start = (uint32_t)a.start;
    const uint32_t q0 = qtile * PF32_BM;
    const uint32_t rows_here = t - q0 < PF32_BM ? t - q0 : PF32_BM;
    const uint32_t end = start + t;
    const uint32_t pos_first = start + q0;
    const uint32_t pos_last = pos_first + rows_here - 1;
    const bool windowed = a.window != LNG_WINDOW_FULL;
    const uint32_t window = windowed ? (uint32_t)a.window : 0u;
    const uint32_t kfirst = (windowed && pos_first + 1 > window) ? pos_first + 1 - window : 0u;
    const uint32_t tile0 = kfirst & ~(uint32_t)(PF_BN - 1);
    const uint32_t all_tiles = (pos_last - tile0) / PF_BN + 1;
    const bool partial = a.splits > 1u;
    const uint32_t first_tile = (uint32_t)((uint64_t)all_tiles * split / a.splits);
    const uint32_t n_tiles = (uint32_t)((uint64_t)all_tiles * (split + 1u) / a.splits);
    const bool ring = a.slots < end;
    const uint32_t slots = (uint32_t)a.slots;
    const uint64_t row_bytes = (uint64_t)a.kv_heads * 256u;

    const uint32_t my_row = q0 + n;
    const uint32_t my_pos = start + my_row;
    const bool row_ok = my_row < t;
    const bool wave_active = wave < group; // the others only help loading tiles
    const uint32_t head = g * group + (wave_active ? wave : 0u);
    float4 qreg[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        qreg[j] = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
        if (row_ok) qreg[j] = *(const float4 *)(a.q + (((uint64_t)my_row * a.heads + head) * 64u + 8u * j + 4u * hh) * 4u);
    }
    const float sl2 = a.scale * LNG_LOG2E;
    const bool sink_here = a.sinks && !partial;
    float m = sink_here ? a.sinks[head] * LNG_LOG2E : LNG_NEG_INF;
    float l = (sink_here && hh == 0) ? 1.0f : 0.0f;
    floatx16 ot[2];
#pragma unroll
    for (int db = 0; db < 2; ++db) {
#pragma unroll
        for (int i = 0; i < 16; ++i) ot[db][i] = 0.0f;
    }

    // ---- tile loader: two 16-byte chunks of K and of V per thread (keys ld_key and ld_key + 32) ----
    const uint32_t ld_key = tid >> 4;  // 0..31
    const uint32_t ld_chunk = tid & 15u;
    const char *kbase = a.k + (uint64_t)g * 256u + ld_chunk * 16u;
    const char *vbase = a.v + (uint64_t)g * 256u + ld_chunk * 16u;
    uint4 kr0, kr1, vr0, vr1; // plain scalars: arrays indexed inside the lambdas end up in scratch memory
    auto fetch_row = [&](uint32_t p, uint4 &kr, uint4 &vr) {
        p = p > pos_last ? pos_last : p; // rows outside [first visible, last] are masked, and may not exist
        p = p < kfirst ? kfirst : p;
        const uint32_t row = ring ? p % slots : p;
        kr = *(const uint4 *)(kbase + (uint64_t)row * row_bytes);
        vr = *(const uint4 *)(vbase + (uint64_t)row * row_bytes);
    };
    auto fetch = [&](uint32_t tile) {
        fetch_row(tile0 + tile * PF_BN + ld_key, kr0, vr0);
        fetch_row(tile0 + tile * PF_BN + 32u + ld_key, kr1, vr1);
    };
    auto stash = [&](uint32_t buf) {
        *(uint4 *)(&s_k[buf][ld_key * PF32_KSTRIDE + ld_chunk * 4u]) = kr0;
        *(uint4 *)(&s_v[buf][ld_key * PF32_VSTRIDE + ld_chunk * 4u]) = vr0;
        *(uint4 *)(&s_k[buf][(32u + ld_key) * PF32_KSTRIDE + ld_chunk * 4u]) = kr1;
        *(uint4 *)(&s_v[buf][(32u + ld_key) * PF32_VSTRIDE + ld_chunk * 4u]) = vr1;
    };
    if (first_tile < n_tiles) {
        fetch(first_tile);
        stash(first_tile & 1u);
    }
    __syncthreads();

    const uint32_t k_lane_off = n * PF32_KSTRIDE + 4u * hh; // + kb*32*KSTRIDE + 8j
    const uint32_t v_lane_off = 4u * hh * PF32_VSTRIDE + n; // + (kb*32 + 8a + e)*VSTRIDE + 32db

    auto step = [&](auto mask_tag, uint32_t tile) {
        constexpr bool MASK = decltype(mask_tag)::value;
        const uint32_t buf = tile & 1u;
        if (tile + 1 < n_tiles) fetch(tile + 1);
        if (wave_active) {
            const uint32_t kt0 = tile0 + tile * PF_BN;
#pragma unroll
            for (int kb = 0; kb < 2; ++kb) {
                if constexpr (MASK) { // a block no query of the workgroup sees
                    const uint32_t b0 = kt0 + 32u * kb;
                    if (b0 > pos_last || b0 + 31u < kfirst) continue;
                }
                floatx16 st;
#pragma unroll
                for (int i = 0; i < 16; ++i) st[i] = 0.0f;
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    const float4 ka = *(const float4 *)(&s_k[buf][k_lane_off + kb * 32 * PF32_KSTRIDE + 8 * j]);
                    st = __builtin_amdgcn_mfma_f32_32x32x2f32(ka.x, qreg[j].x, st, 0, 0, 0);
                    st = __builtin_amdgcn_mfma_f32_32x32x2f32(ka.y, qreg[j].y, st, 0, 0, 0);
                    st = __builtin_amdgcn_mfma_f32_32x32x2f32(ka.z, qreg[j].z, st, 0, 0, 0);
                    st = __builtin_amdgcn_mfma_f32_32x32x2f32(ka.w, qreg[j].w, st, 0, 0, 0);
                }
                if constexpr (MASK) {
#pragma unroll
                    for (int i = 0; i < 16; ++i) {
                        const uint32_t kp = kt0 + 32u * kb + 8u * (i >> 2) + 4u * hh + (i & 3);
                        const bool vis = kp <= my_pos && (!windowed || kp + window > my_pos);
                        st[i] = vis ? st[i] : LNG_NEG_INF;
                    }
                }
                // online softmax, one query per lane; the maximum moves only when it grows by PF_TAU
                float tmax = LNG_NEG_INF;
#pragma unroll
                for (int i = 0; i < 16; ++i) tmax = fmaxf(tmax, st[i]);
                tmax = other_half_max(tmax) * sl2;
                const float m_new = tmax > m + PF_TAU ? tmax : m;
                const float m_safe = m_new == LNG_NEG_INF ? 0.0f : m_new;
                if (__builtin_amdgcn_ballot_w64(m_new != m) != 0) {
                    const float alpha = __builtin_amdgcn_exp2f(m - m_safe);
                    l *= alpha;
#pragma unroll
                    for (int db = 0; db < 2; ++db) {
#pragma unroll
                        for (int i = 0; i < 16; ++i) ot[db][i] *= alpha;
                    }
                    m = m_new;
                }
                float psum = 0.0f;
#pragma unroll
                for (int i = 0; i < 16; ++i) {
                    st[i] = __builtin_amdgcn_exp2f(__builtin_fmaf(st[i], sl2, -m_safe));
                    psum += st[i];
                }
                l += psum;
                // O^T += V^T . P^T: step i of the 16 multiplies keys 8(i>>2) + 4hh + (i&3)
#pragma unroll
                for (int i = 0; i < 16; ++i) {
                    const float *vp = &s_v[buf][v_lane_off + (kb * 32 + 8 * (i >> 2) + (i & 3)) * PF32_VSTRIDE];
                    ot[0] = __builtin_amdgcn_mfma_f32_32x32x2f32(vp[0], st[i], ot[0], 0, 0, 0);
                    ot[1] = __builtin_amdgcn_mfma_f32_32x32x2f32(vp[32], st[i], ot[1], 0, 0, 0);
                }
            }
        }
        if (tile + 1 < n_tiles) stash(buf ^ 1u);
        __syncthreads();
    };
    auto edge = [&](uint32_t tile) {
        const uint32_t kt0 = tile0 + tile * PF_BN;
        return kt0 + (PF_BN - 1) > pos_first || (windowed && kt0 + window < pos_first + PF32_BM);
    };
    uint32_t tile = first_tile;
    for (; tile < n_tiles && edge(tile); ++tile) step(std::true_type{}, tile);   // window edge
    for (; tile < n_tiles && !edge(tile); ++tile) step(std::false_type{}, tile); // interior
    for (; tile < n_tiles; ++tile) step(std::true_type{}, tile);                 // diagonal

    if (!wave_active || !row_ok) return;
    const float total = l + __shfl_xor(l, 32, 64);
    if (partial) { // (max, sum, unnormalised output) for lng_prefill_merge, which also adds the sink
        const uint64_t slot = (((uint64_t)my_row * a.kv_heads + g) * a.splits + split) * group + (head - g * group);
        float *po = a.partial_o + slot * 64u;
#pragma unroll
        for (int db = 0; db < 2; ++db) {
#pragma unroll
            for (int blk = 0; blk < 4; ++blk) {
                *(float4 *)(po + 32 * db + 8 * blk + 4 * hh) = make_float4(ot[db][4 * blk + 0], ot[db][4 * blk + 1],
                                                                           ot[db][4 * blk + 2], ot[db][4 * blk + 3]);
            }
        }
        if (hh == 0) *(float2 *)(a.partial_ml + slot * 2u) = make_float2(m, total);
        return;
    }
    const float inv = total > 0.0f ? 1.0f / total : 0.0f;
    float *op = (float *)a.out + ((uint64_t)my_row * a.heads + head) * 64u;
#pragma unroll
    for (int db = 0; db < 2; ++db) {
#pragma unroll
        for (int blk = 0; blk < 4; ++blk) {
            *(float4 *)(op + 32 * db + 8 * blk + 4 * hh) = make_float4(ot[db][4 * blk + 0] * inv, ot[db][4 * blk + 1] * inv,
                                                                       ot[db][4 * blk + 2] * inv, ot[db][4 * blk + 3] * inv);
        }
    }
}

// One workgroup per compute unit (146 registers): passes with few workgroups, which then go to the compute units
// longest first, one at a time, and stay balanced.
extern "C" __global__ __launch_bounds__(PF_THREADS) void lng_prefill_f32_d64(lng_k_prefill a) { prefill_f32_body(a); }

// Two workgroups per compute unit (128 registers, 4 of them spilled): one's softmax and LDS traffic under the
// other's matrix instructions. For passes with many workgroups (the long causal pass +3-6 %, the windowed one +19 %);
// with two rounds of workgroups or fewer, co-resident pairs of unequal length leave units idle (2,048 positions -25 %).
extern "C" __global__ __launch_bounds__(PF_THREADS, 4) void lng_prefill_f32_d64_w4(lng_k_prefill a) { prefill_f32_body(a); }

// Combines the splits of a prompt pass; the sink joins here. Up to eight splits (the usual case: one
// workgroup per compute unit needs few): a thread per (row, head, four dims) requests its splits' partial
// outputs at once, works out the weights from the (max, sum) pairs itself - the 16 threads of a head all
// do, it is a handful of exponentials - and writes four outputs: no LDS, no barrier, one wait for memory.
// Grid x = ceil(t * heads / 16) workgroups of 256. More splits: one workgroup per (row, kv head), the
// decode path's merge (the layouts of the partials agree), grid y = t * kv_heads.
extern "C" __global__ __launch_bounds__(256) void lng_prefill_merge(lng_k_prefill p) {
    const uint32_t group = p.heads / p.kv_heads;
    if (p.splits <= 8u) {
        // dim / 4 threads per (row, head): 16 at head width 64, so 16 (row, head) pairs per workgroup; 2 at width 512
        const uint32_t per_pair = p.dim >> 2, pairs_per_wg = 256u / per_pair;
        const uint64_t pair = (uint64_t)blockIdx.x * pairs_per_wg + threadIdx.x / per_pair; // row * heads + head
        if (pair >= p.t * p.heads) return;
        const uint32_t row = (uint32_t)(pair / p.heads), head = (uint32_t)(pair % p.heads);
        const uint32_t g = head / group, h = head % group, d4 = (threadIdx.x % per_pair) * 4u;
        const uint64_t slot0 = (((uint64_t)row * p.kv_heads + g) * p.splits) * group + h;
        float4 o[8];
        float2 ml[8];
#pragma unroll
        for (int c = 0; c < 8; ++c) {
            if ((uint32_t)c < p.splits) {
                o[c] = *(const float4 *)(p.partial_o + (slot0 + (uint64_t)c * group) * p.dim + d4);
                ml[c] = *(const float2 *)(p.partial_ml + (slot0 + (uint64_t)c * group) * 2u);
            }
        }
        const float sink2 = p.sinks ? p.sinks[head] * LNG_LOG2E : LNG_NEG_INF;
        float top = sink2;
#pragma unroll
        for (int c = 0; c < 8; ++c) {
            if ((uint32_t)c < p.splits) top = fmaxf(top, ml[c].x);
        }
        float z = sink2 == LNG_NEG_INF ? 0.0f : __builtin_amdgcn_exp2f(sink2 - top);
        float4 sum = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
#pragma unroll
        for (int c = 0; c < 8; ++c) {
            if ((uint32_t)c < p.splits) {
                const float w = ml[c].x == LNG_NEG_INF ? 0.0f : __builtin_amdgcn_exp2f(ml[c].x - top);
                z += ml[c].y * w;
                sum.x += o[c].x * w;
                sum.y += o[c].y * w;
                sum.z += o[c].z * w;
                sum.w += o[c].w * w;
            }
        }
        if (p.dtype == LNG_F32) {
            *(float4 *)((float *)p.out + pair * p.dim + d4) = make_float4(sum.x / z, sum.y / z, sum.z / z, sum.w / z);
            return;
        }
        ushort4 r;
        r.x = f32_to_bf16_bits(sum.x / z);
        r.y = f32_to_bf16_bits(sum.y / z);
        r.z = f32_to_bf16_bits(sum.z / z);
        r.w = f32_to_bf16_bits(sum.w / z);
        *(ushort4 *)((uint16_t *)p.out + pair * p.dim + d4) = r;
        return;
    }
    const uint32_t row = blockIdx.y / p.kv_heads;
    const uint32_t g = blockIdx.y % p.kv_heads;
    lng_k_attn a{};
    a.out = p.out;
    a.sinks = (const char *)p.sinks;
    a.partial_o = p.partial_o;
    a.partial_ml = p.partial_ml;
    a.n_chunks = p.splits;
    a.dtype = p.dtype;
    lng_k_row it{};
    it.out_offset = (uint64_t)row * p.heads * 64u * (p.dtype == LNG_F32 ? 4u : 2u);
    it.sinks_offset = p.sinks ? 0u : LNG_NO_SINKS;
    merge_chunks<false>(a, it, blockIdx.y, g, group, p.splits);
}

#include "lng_prefill_pair.h"
#include "lng_prefill_wide.h"
