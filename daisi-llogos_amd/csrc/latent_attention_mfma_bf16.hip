// Attention over a latent cache on the matrix cores (bfloat16): every head of a token reads the
// same cached rows, so a token's heads are columns of one product.  Keys are rows
// [latent | rotated part | zeros] of `row` dimensions (a multiple of 16) in the key pool; the
// values are the latent again, in a value pool of the same page shape, in the matrix cores'
// operand order for O^T += V^T . P^T (common.h).  Softmax state and sums are 32-bit; a head's
// learned sink joins the denominator once.
//
// Work: the (token, head) pairs of a sequence's part of the step, token-major, in tiles of 16
// columns; a wave owns one tile, with its queries as second operands in registers, and takes
// the sequence's pages one after the other: S^T = K . Q^T (four blocks of 16 keys), softmax in
// the log2 domain, O^T += V^T . P^T.  Fragments stream from memory in the order they lie there
// (1 KB a wave and load).  With `splits` > 1 (single-token steps over long contexts) the pages
// of a sequence are shared out over blockIdx.y, partial results go to a workspace, and a second
// kernel merges them.
#include "common.h"

typedef __bf16 lbf16x8 __attribute__((ext_vector_type(8)));
typedef float lf32x4 __attribute__((ext_vector_type(4)));
typedef __bf16 lbf16x2 __attribute__((ext_vector_type(2)));
typedef float lf32x2 __attribute__((ext_vector_type(2)));

namespace {

constexpr float kLog2eL = 1.4426950408889634f;
constexpr int kLatentWaves = 4;

__device__ __forceinline__ lbf16x8 frag_load(const bf16_t* p) {
    return __builtin_bit_cast(lbf16x8, *reinterpret_cast<const uint4*>(p));
}
__device__ __forceinline__ lbf16x8 frag_zero() { return __builtin_bit_cast(lbf16x8, make_uint4(0, 0, 0, 0)); }
__device__ __forceinline__ uint32_t pack2(float lo, float hi) {
    const lf32x2 v = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, lbf16x2));
}
// over the four lanes l, l ^ 16, l ^ 32, l ^ 48: one column of a product's result
__device__ __forceinline__ float col_max(float x) {
    x = fmaxf(x, __shfl_xor(x, 16, kWave));
    return fmaxf(x, __shfl_xor(x, 32, kWave));
}
__device__ __forceinline__ float col_sum(float x) {
    x += __shfl_xor(x, 16, kWave);
    return x + __shfl_xor(x, 32, kWave);
}
__device__ __forceinline__ lbf16x8 first_n(lbf16x8 f, int n) {      // the first n (0..8) values, zeros behind them
    uint4 u = __builtin_bit_cast(uint4, f);
    uint32_t* w = reinterpret_cast<uint32_t*>(&u);
#pragma unroll
    for (int j = 0; j < 4; ++j) w[j] &= (2 * j + 1 < n) ? 0xffffffffu : ((2 * j < n) ? 0x0000ffffu : 0u);
    return __builtin_bit_cast(lbf16x8, u);
}

}  // namespace

// KS: most steps of 32 dimensions in a key row; DVT: most tiles of 16 value dimensions.
template <int KS, int DVT>
__global__ __launch_bounds__(kLatentWaves* kWave) void latent_attn_kernel(
        bf16_t* __restrict__ out, int dv, const bf16_t* __restrict__ q, const bf16_t* __restrict__ k_pool,
        const bf16_t* __restrict__ v_pool, const int* __restrict__ table, int table_stride,
        const int* __restrict__ cu, const int* __restrict__ tok_pos, int batch, int n_heads, int row,
        float scale, const float* __restrict__ head_sink, int splits, int pages_per_split,
        float* __restrict__ ws_ml, float* __restrict__ ws_acc, int total_cols, int n_tiles) {
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    const int c = lane & 15, g = lane >> 4;
    const int tile = blockIdx.x * kLatentWaves + wave;
    if (tile >= n_tiles) return;
    // the sequence of this tile: tiles are numbered sequence by sequence
    int seq = 0, first_tok = 0, n_tok = 1, tile_in_seq = tile;
    if (cu) {
        for (seq = 0; seq < batch; ++seq) {
            first_tok = cu[seq];
            n_tok = cu[seq + 1] - first_tok;
            const int tiles = (n_tok * n_heads + 15) / 16;
            if (tile_in_seq < tiles) break;
            tile_in_seq -= tiles;
        }
        if (seq >= batch) return;
    } else {
        const int tiles = (n_heads + 15) / 16;
        seq = tile / tiles;
        tile_in_seq = tile % tiles;
        first_tok = seq;
    }
    const int col = tile_in_seq * 16 + c;                    // this lane's column within the sequence
    const bool used = col < n_tok * n_heads;
    const int tok = first_tok + (used ? col / n_heads : 0), head = used ? col % n_heads : 0;
    const int q_pos = used ? tok_pos[tok] : -1;
    // the tile's last position decides how many pages it needs; its first, from where on keys need a mask
    const int last_col = min(tile_in_seq * 16 + 15, n_tok * n_heads - 1);
    const int pos_hi = tok_pos[first_tok + last_col / n_heads], pos_lo = tok_pos[first_tok + (tile_in_seq * 16) / n_heads];
    const int n_pages = pos_hi / kPageTokens + 1;
    const int split = blockIdx.y;
    const int page0 = split * pages_per_split, page1 = min(n_pages, page0 + pages_per_split);

    const int ksteps = (row + 31) / 32, dvt = (dv + 15) / 16, octs = row >> 3;
    lbf16x8 qf[KS];
    const bf16_t* qrow = q + ((size_t)tok * n_heads + head) * row;
#pragma unroll
    for (int sk = 0; sk < KS; ++sk)
        qf[sk] = (used && sk < ksteps && 32 * sk + 8 * g < row) ? frag_load(qrow + 32 * sk + 8 * g) : frag_zero();

    const float scale_log2 = scale * kLog2eL;
    float m = -INFINITY, l = 0.f;
    if (head_sink && split == 0 && used) { m = head_sink[head] * kLog2eL; l = 1.f; }
    lf32x4 acc[DVT];
#pragma unroll
    for (int db = 0; db < DVT; ++db) acc[db] = lf32x4{0.f, 0.f, 0.f, 0.f};

    const int* trow = table + (size_t)seq * table_stride;
    for (int pg = page0; pg < page1; ++pg) {
        const size_t base = (size_t)trow[pg] * kPageTokens * row;
        const bf16_t* kpage = k_pool + base + 8 * c + 128 * g;
        const bf16_t* vpage = v_pool + base + 8 * lane;
        const int key0 = pg * kPageTokens;
        lf32x4 s[4];
#pragma unroll
        for (int rb = 0; rb < 4; ++rb) s[rb] = lf32x4{0.f, 0.f, 0.f, 0.f};
        // (the four blocks of keys side by side: four loads in flight and four independent chains of products)
#pragma unroll
        for (int sk = 0; sk < KS; ++sk) {
            if (sk < ksteps) {
                lbf16x8 kf[4];
#pragma unroll
                for (int rb = 0; rb < 4; ++rb)      // block rb of the page, dimensions 32 sk + 8 g ..: beyond the row's end nothing is there
                    kf[rb] = (4 * sk + g < octs) ? frag_load(kpage + (size_t)(rb * octs + 4 * sk) * 128) : frag_zero();
#pragma unroll
                for (int rb = 0; rb < 4; ++rb) s[rb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf[rb], qf[sk], s[rb], 0, 0, 0);
            }
        }
        // softmax of the page: this lane holds, for its column, keys key0 + 16 g + 4 rb + r
        const bool masked = key0 + kPageTokens - 1 > pos_lo;
        float tile_max = -INFINITY;
#pragma unroll
        for (int rb = 0; rb < 4; ++rb)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                if (masked && key0 + 16 * g + 4 * rb + r > q_pos) s[rb][r] = -INFINITY;
                tile_max = fmaxf(tile_max, s[rb][r]);
            }
        tile_max = col_max(tile_max);
        const float m_new = fmaxf(m, tile_max * scale_log2);
        const float m_use = (m_new == -INFINITY) ? 0.f : m_new;
        const float corr = __builtin_amdgcn_exp2f(m - m_use);
        float p[16], sum = 0.f;
#pragma unroll
        for (int rb = 0; rb < 4; ++rb)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const float e = __builtin_amdgcn_exp2f(fmaf(s[rb][r], scale_log2, -m_use));
                p[4 * rb + r] = e;
                sum += e;
            }
        l = l * corr + col_sum(sum);
        m = m_new;
        lbf16x8 pf[2];
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            uint4 u;
            u.x = pack2(p[8 * t + 0], p[8 * t + 1]);
            u.y = pack2(p[8 * t + 2], p[8 * t + 3]);
            u.z = pack2(p[8 * t + 4], p[8 * t + 5]);
            u.w = pack2(p[8 * t + 6], p[8 * t + 7]);
            pf[t] = __builtin_bit_cast(lbf16x8, u);
        }
        // values of keys that are not written yet are zeroed (whatever the page held before times 0 must be 0)
        const int valid = pos_hi + 1 - key0;
        // (four tiles of value dimensions at a time: eight loads in flight before the first product)
#pragma unroll
        for (int d0 = 0; d0 < DVT; d0 += 4) {
            if (d0 < dvt) {
                lbf16x8 v0[4], v1[4];
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const bool on = d0 + e < DVT && d0 + e < dvt;
                    v0[e] = on ? frag_load(vpage + 512 * (2 * (d0 + e))) : frag_zero();
                    v1[e] = on ? frag_load(vpage + 512 * (2 * (d0 + e) + 1)) : frag_zero();
                    if (valid < kPageTokens) {
                        v0[e] = first_n(v0[e], valid - 16 * g);
                        v1[e] = first_n(v1[e], valid - 16 * g - 8);
                    }
                }
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    if (d0 + e < DVT) {
                        lf32x4 a = acc[d0 + e];
#pragma unroll
                        for (int r = 0; r < 4; ++r) a[r] *= corr;
                        a = __builtin_amdgcn_mfma_f32_16x16x32_bf16(v0[e], pf[0], a, 0, 0, 0);
                        a = __builtin_amdgcn_mfma_f32_16x16x32_bf16(v1[e], pf[1], a, 0, 0, 0);
                        acc[d0 + e] = a;
                    }
                }
            }
        }
    }
    if (!used) return;
    const size_t gcol = (size_t)first_tok * n_heads + col;    // the column among all of the step's (token, head) pairs
    if (splits == 1) {
        const float inv = l > 0.f ? 1.0f / l : 0.f;
        bf16_t* o = out + gcol * dv;
#pragma unroll
        for (int db = 0; db < DVT; ++db)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int d = 16 * db + 4 * g + r;
                if (db < dvt && d < dv) o[d] = f32_to_bf16(acc[db][r] * inv);
            }
        return;
    }
    const int dvp = dvt * 16;
    if (g == 0) {
        ws_ml[((size_t)split * total_cols + gcol) * 2] = m;
        ws_ml[((size_t)split * total_cols + gcol) * 2 + 1] = l;
    }
    float* wa = ws_acc + ((size_t)split * total_cols + gcol) * dvp;
#pragma unroll
    for (int db = 0; db < DVT; ++db)
#pragma unroll
        for (int r = 0; r < 4; ++r)
            if (db < dvt) wa[16 * db + 4 * g + r] = acc[db][r];
}

// out[col, d] = sum_s acc_s[d] 2^(m_s - M) / sum_s l_s 2^(m_s - M), M the largest m_s (splits that saw
// no key have m = -inf and l = 0 and count for nothing).
constexpr int kMergeSplits = 16;      // splits whose partial results a thread asks for at once (the wrapper makes no more)

__global__ void latent_merge_kernel(bf16_t* __restrict__ out, int dv, int dvp, const float* __restrict__ ws_ml,
                                    const float* __restrict__ ws_acc, int splits, int total_cols) {
    const int col = blockIdx.x;
    float ms[kMergeSplits], ls[kMergeSplits];
#pragma unroll
    for (int s = 0; s < kMergeSplits; ++s) {
        ms[s] = s < splits ? ws_ml[((size_t)s * total_cols + col) * 2] : -INFINITY;
        ls[s] = s < splits ? ws_ml[((size_t)s * total_cols + col) * 2 + 1] : 0.f;
    }
    float M = -INFINITY, L = 0.f;
#pragma unroll
    for (int s = 0; s < kMergeSplits; ++s) M = fmaxf(M, ms[s]);
#pragma unroll
    for (int s = 0; s < kMergeSplits; ++s) {
        ms[s] = ms[s] == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(ms[s] - M);       // the split's weight
        L = fmaf(ls[s], ms[s], L);
    }
    const float inv = L > 0.f ? 1.0f / L : 0.f;
    for (int d = threadIdx.x; d < dv; d += blockDim.x) {
        float part[kMergeSplits];
#pragma unroll
        for (int s = 0; s < kMergeSplits; ++s) part[s] = s < splits ? ws_acc[((size_t)s * total_cols + col) * dvp + d] : 0.f;
        float a = 0.f;
#pragma unroll
        for (int s = 0; s < kMergeSplits; ++s) a = fmaf(part[s], ms[s], a);
        out[(size_t)col * dv + d] = f32_to_bf16(a * inv);
    }
}

// floats of workspace for a step with `splits` > 1: per split and column 2 + 16 ceil(dv / 16)
LLOGOS_EXPORT long long llogos_latent_attn_workspace(int total_cols, int dv, int splits) {
    if (splits <= 1) return 0;
    return (long long)splits * total_cols * (2 + (dv + 15) / 16 * 16);
}

// out [T, heads, dv] bfloat16; q [T, heads, row] bfloat16; pools [pages, 1, 64 * row].  cu: token offsets of
// the step's sequences (null: one token a sequence); n_tiles: sum over the sequences of
// ceil(tokens * heads / 16).  Returns LLOGOS_UNSUPPORTED for rows of more than 576 dimensions.
LLOGOS_EXPORT int llogos_latent_attn_bf16(void* out, int dv, const void* q, const void* k_pool, const void* v_pool,
                                          const int* table, int table_stride, const int* cu, const int* tok_pos,
                                          int batch, int T, int n_heads, int row, float scale, const float* head_sink,
                                          int n_tiles, int splits, int pages_per_split, float* workspace,
                                          long long workspace_floats, hipStream_t stream) {
    if (T <= 0 || batch <= 0 || n_heads <= 0 || row <= 0 || row % 16 || dv <= 0 || dv > row || n_tiles <= 0) return LLOGOS_BAD_ARGUMENT;
    if (splits < 1 || splits > kMergeSplits || pages_per_split < 1 || (!cu && T != batch)) return LLOGOS_BAD_ARGUMENT;
    if (row > 576) return LLOGOS_UNSUPPORTED;
    const int total_cols = T * n_heads, dvp = (dv + 15) / 16 * 16;
    float *ws_ml = nullptr, *ws_acc = nullptr;
    if (splits > 1) {
        if (!workspace || workspace_floats < llogos_latent_attn_workspace(total_cols, dv, splits)) return LLOGOS_BAD_ARGUMENT;
        ws_ml = workspace;
        ws_acc = workspace + (size_t)splits * total_cols * 2;
    }
    dim3 grid((n_tiles + kLatentWaves - 1) / kLatentWaves, splits);
#define LAT(KS, DVT) latent_attn_kernel<KS, DVT><<<grid, kLatentWaves * kWave, 0, stream>>>((bf16_t*)out, dv, (const bf16_t*)q, \
        (const bf16_t*)k_pool, (const bf16_t*)v_pool, table, table_stride, cu, tok_pos, batch, n_heads, row, scale, head_sink, \
        splits, pages_per_split, ws_ml, ws_acc, total_cols, n_tiles)
    if (row <= 128) LAT(4, 8);
    else if (row <= 256) LAT(8, 16);
    else LAT(18, 36);
#undef LAT
    if (splits > 1) latent_merge_kernel<<<total_cols, 256, 0, stream>>>((bf16_t*)out, dv, dvp, ws_ml, ws_acc, splits, total_cols);
    return LLOGOS_LAUNCH_CHECK();
}
