// What the bfloat16 attention kernels on the matrix cores share (gfx950, v_mfma_f32_16x16x32_bf16):
// fragment loads from pages in operand order, packing, reductions over an MFMA result's column, the
// running softmax state of a wave and the steps of one page of 64 keys.
// Scores are computed transposed, S^T[key][column] = K . Q^T, so that the lane that holds the scores
// of a column for 16 keys is the lane that supplies them as the second operand of
// O^T[d][column] = V^T[d][key] . P^T[key][column].
#pragma once
#include "common.h"

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

constexpr int kAttnWaves = 4;

__device__ __forceinline__ bf16x8 ld_frag(const bf16_t* p) {
    return __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(p));
}

// A fragment of a page, read once: 64 lanes x 16 bytes of consecutive memory, past the caches'
// keeping (a step reads every page once and the next step comes after all other layers).
typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ bf16x8 ld_frag_once(const bf16_t* p) {
    return __builtin_bit_cast(bf16x8, __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p)));
}

__device__ __forceinline__ bf16x8 zero_frag() {
    return __builtin_bit_cast(bf16x8, make_uint4(0, 0, 0, 0));
}

typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float f32x2 __attribute__((ext_vector_type(2)));

// two floats to packed bfloat16, round to nearest even (one v_cvt_pk_bf16_f32)
__device__ __forceinline__ uint32_t pack_bf16(float lo, float hi) {
    const f32x2 v = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2));
}

constexpr float kLog2e = 1.4426950408889634f;

// Maximum and sum over the four lanes l, l ^ 16, l ^ 32, l ^ 48 (one column of an MFMA result),
// left in all four.  v_permlane16_swap exchanges the odd rows of 16 lanes of its first operand
// with the even rows of its second, v_permlane32_swap the upper half of the first with the
// lower half of the second: fed the same value twice, the two results hold a lane's own value
// and its partner's.  (A shuffle would go through the LDS pipeline and cost its latency.)
typedef unsigned u32x2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ float quad_max(float x) {
    u32x2 r = __builtin_amdgcn_permlane16_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    x = fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
    r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float quad_sum(float x) {
    u32x2 r = __builtin_amdgcn_permlane16_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    x = __uint_as_float(r[0]) + __uint_as_float(r[1]);
    r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}

// Keeps the first n (0..8) of a fragment's eight values and zeroes the rest.
__device__ __forceinline__ bf16x8 keep_first(bf16x8 f, int n) {
    uint4 u = __builtin_bit_cast(uint4, f);
    uint32_t* w = reinterpret_cast<uint32_t*>(&u);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const uint32_t mask = (2 * j + 1 < n) ? 0xffffffffu : ((2 * j < n) ? 0x0000ffffu : 0u);
        w[j] &= mask;
    }
    return __builtin_bit_cast(bf16x8, u);
}

// Running softmax state of one wave: per column (lane & 15) the maximum and the sum, and
// the output sums O^T[d][column] with d = 16 db + 4 g + r in acc[db][r].  The maximum is kept
// in units of log2: m = max(score * scale) * log2(e), so that exp(x - max) is one
// multiply-add and one v_exp_f32.
template <int HD>
struct WaveState {
    float m, l;
    f32x4 acc[HD / 16];
    __device__ void init() {
        m = -INFINITY;
        l = 0.f;
#pragma unroll
        for (int db = 0; db < HD / 16; ++db) acc[db] = f32x4{0.f, 0.f, 0.f, 0.f};
    }
};

// Softmax of one page for one block of 16 columns.  s[rb][r]: raw dot products of this lane's
// column with key key0 + g * GS + rb * RS + r.  Returns the probabilities as the two second
// operands of O^T += V^T . P^T (step t, slot e <-> s[2 t + e / 4][e % 4]) and the factor by
// which the running sums shrink.  MASKED = false when every key of the page is visible to
// every column of the wave.
template <bool MASKED, int GS, int RS, int HD>
__device__ __forceinline__ void softmax_page(f32x4 (&s)[4], WaveState<HD>& st, float scale_log2, int q_pos,
                                             int key0, int window, int sinks, bf16x8 (&pf)[2], float& corr) {
    const int g = (threadIdx.x & (kWave - 1)) >> 4;
    float tile_max = -INFINITY;
#pragma unroll
    for (int rb = 0; rb < 4; ++rb)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            if (MASKED) {
                const int key = key0 + g * GS + rb * RS + r;
                if (!(q_pos >= 0 && key_visible(q_pos, key, window, sinks))) s[rb][r] = -INFINITY;
            }
            tile_max = fmaxf(tile_max, s[rb][r]);
        }
    tile_max = quad_max(tile_max);
    const float m_new = fmaxf(st.m, tile_max * scale_log2);              // scale > 0: the maximum commutes
    // a column that has seen no key yet keeps m = -inf; exp2(-inf - (-inf)) must not be taken
    const float m_use = (m_new == -INFINITY) ? 0.f : m_new;
    corr = __builtin_amdgcn_exp2f(st.m - m_use);                          // exp2(-inf) = 0 for the first page
    float p[16], sum = 0.f;
#pragma unroll
    for (int rb = 0; rb < 4; ++rb)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const float e = __builtin_amdgcn_exp2f(fmaf(s[rb][r], scale_log2, -m_use));   // masked: exp2(-inf) = 0
            p[4 * rb + r] = e;
            sum += e;
        }
    sum = quad_sum(sum);
    st.l = st.l * corr + sum;
    st.m = m_new;
#pragma unroll
    for (int t = 0; t < 2; ++t) {
        uint4 u;
        u.x = pack_bf16(p[8 * t + 0], p[8 * t + 1]);
        u.y = pack_bf16(p[8 * t + 2], p[8 * t + 3]);
        u.z = pack_bf16(p[8 * t + 4], p[8 * t + 5]);
        u.w = pack_bf16(p[8 * t + 6], p[8 * t + 7]);
        pf[t] = __builtin_bit_cast(bf16x8, u);
    }
}

// Whether every key of the page [key0, key0 + 63] is visible to every query at first_pos .. last_pos.
__device__ __forceinline__ bool page_fully_visible(int first_pos, int last_pos, int key0, int window, int sinks) {
    if (key0 + kPageTokens - 1 > first_pos) return false;
    if (window <= 0) return true;
    return key0 + kPageTokens - 1 < sinks || key0 > last_pos - window;
}

// The parts of a page's work.  kpage, vpage: one kv head's part of a page, in fragment order
// (common.h): fragment f of either is the 512 elements from 512 f on, lane l's eight at 8 l.
template <int HD>
__device__ __forceinline__ void load_keys(bf16x8 (&kf)[4][HD / 32], const bf16_t* __restrict__ kpage) {
    const bf16_t* mine = kpage + 8 * (threadIdx.x & (kWave - 1));
#pragma unroll
    for (int rb = 0; rb < 4; ++rb)
#pragma unroll
        for (int sk = 0; sk < HD / 32; ++sk) kf[rb][sk] = ld_frag_once(mine + 512 * (rb * (HD / 32) + sk));
}

template <int HD>
__device__ __forceinline__ void load_values(bf16x8 (&vf)[HD / 16][2], const bf16_t* __restrict__ vpage) {
    const bf16_t* mine = vpage + 8 * (threadIdx.x & (kWave - 1));
#pragma unroll
    for (int db = 0; db < HD / 16; ++db) {
        vf[db][0] = ld_frag_once(mine + 512 * (2 * db));
        vf[db][1] = ld_frag_once(mine + 512 * (2 * db + 1));
    }
}

// S^T = K . Q^T, four blocks of 16 keys; this lane: column lane & 15, keys 16 g + 4 rb + r in s[rb][r]
template <int HD>
__device__ __forceinline__ void page_scores(f32x4 (&s)[4], const bf16x8 (&kf)[4][HD / 32], const bf16x8 (&qf)[HD / 32]) {
#pragma unroll
    for (int rb = 0; rb < 4; ++rb) {
        s[rb] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int sk = 0; sk < HD / 32; ++sk)
            s[rb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf[rb][sk], qf[sk], s[rb], 0, 0, 0);
    }
}

// O^T = O^T * corr + V^T . P^T; slot (g, e) of step t is key 16 g + 8 t + e.  Values of keys
// that have not been written (valid_keys and on) are zeroed: 0 * NaN is NaN.
template <int HD>
__device__ __forceinline__ void weigh_values(WaveState<HD>& st, const bf16x8 (&vf)[HD / 16][2], const bf16x8 (&pf)[2],
                                             float corr, int valid_keys) {
    const int g = (threadIdx.x & (kWave - 1)) >> 4;
    const bool rescale = __ballot(corr != 1.0f) != 0;
#pragma unroll
    for (int db = 0; db < HD / 16; ++db) {
        f32x4 a = st.acc[db];
        if (rescale) {
#pragma unroll
            for (int r = 0; r < 4; ++r) a[r] *= corr;
        }
        bf16x8 v0 = vf[db][0], v1 = vf[db][1];
        if (valid_keys < kPageTokens) {
            v0 = keep_first(v0, valid_keys - 16 * g);
            v1 = keep_first(v1, valid_keys - 16 * g - 8);
        }
        a = __builtin_amdgcn_mfma_f32_16x16x32_bf16(v0, pf[0], a, 0, 0, 0);
        a = __builtin_amdgcn_mfma_f32_16x16x32_bf16(v1, pf[1], a, 0, 0, 0);
        st.acc[db] = a;
    }
}

// One page of 64 keys.  qf: the columns' queries as second operands (lane (c, g) holds
// Q[c][32 s + 8 g ..]); kpage, vpage: one kv head's part of a page; q_pos: position of this lane's column
// (-1: the column is not in use); key0: position of the page's first key; valid_keys: how
// many of the page's keys have been written (the rest of the page holds whatever was there
// before: such scores are masked, and such values are zeroed because 0 * NaN is NaN).
template <int HD>
__device__ __forceinline__ void attend_page(WaveState<HD>& st, const bf16x8 (&qf)[HD / 32],
                                            const bf16_t* __restrict__ kpage, const bf16_t* __restrict__ vpage,
                                            int q_pos, int key0, int valid_keys, bool all_visible,
                                            float scale_log2, int window, int sinks) {
    // all of the page's loads are issued before the first product
    bf16x8 kf[4][HD / 32], vf[HD / 16][2];
    load_keys<HD>(kf, kpage);
    load_values<HD>(vf, vpage);
    f32x4 s[4];
    page_scores<HD>(s, kf, qf);
    bf16x8 pf[2];
    float corr;
    if (all_visible) softmax_page<false, 16, 4, HD>(s, st, scale_log2, q_pos, key0, window, sinks, pf, corr);
    else             softmax_page<true, 16, 4, HD>(s, st, scale_log2, q_pos, key0, window, sinks, pf, corr);
    weigh_values<HD>(st, vf, pf, corr, valid_keys);
}

// Whether any key of the page [key0, key0 + 63] can be visible to a query at q_pos.
__device__ __forceinline__ bool page_may_be_visible(int q_pos, int key0, int window, int sinks) {
    if (key0 > q_pos) return false;
    if (window <= 0) return true;
    return key0 < sinks || key0 + kPageTokens - 1 > q_pos - window;
}

// The same for queries at positions first_pos .. last_pos: the causal bound is loosest for the
// last of them, the window's for the first.
__device__ __forceinline__ bool page_may_be_visible_to_range(int first_pos, int last_pos, int key0,
                                                             int window, int sinks) {
    if (key0 > last_pos) return false;
    if (window <= 0) return true;
    return key0 < sinks || key0 + kPageTokens - 1 > first_pos - window;
}
