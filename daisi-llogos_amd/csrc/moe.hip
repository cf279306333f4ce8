// A mixture of experts whose choice is a table over token ids: token t goes to the `top` experts
// table[ids[t]][0..top), each weighted alike.  Everything is decided on the device from the step's
// ids, so a captured step replays with other tokens.
//
//   moe_route    (token, choice) pairs sorted by expert: order[], the experts' segments seg[], and
//                where[pair] = the pair's place in that order
//   moe_product  a product of the sorted rows with their expert's matrix, tile by tile within a segment
//                (plain 32-bit FMAs, any storage type), optionally gathering its input rows by pair
//                and squaring relu in its epilogue
//   moe_combine  out[t] = mean over choices of the pair rows + sigmoid(gate[t]) * shared[t]
//
// A row's sums are taken in the order of k alone, in the blocks of gemm_generic.hip (16 products, 16 of
// those, then the total), so a token's result does not depend on where it falls in a segment or on
// what else is in the step.
#include "common.h"

constexpr int kMoeMaxExperts = 1024;

// One block.  seg has E + 1 entries.
__global__ __launch_bounds__(1024) void moe_route_kernel(const int* __restrict__ ids, const int* __restrict__ table, int T, int top,
                                                         int E, int* __restrict__ order, int* __restrict__ seg,
                                                         int* __restrict__ where) {
    __shared__ int count[kMoeMaxExperts];
    __shared__ int start[kMoeMaxExperts + 1];
    const int P = T * top;
    for (int e = threadIdx.x; e < E; e += blockDim.x) count[e] = 0;
    __syncthreads();
    for (int p = threadIdx.x; p < P; p += blockDim.x) {
        int e = table[(size_t)ids[p / top] * top + p % top];
        e = min(max(e, 0), E - 1);
        atomicAdd(&count[e], 1);
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        int run = 0;
        for (int e = 0; e < E; ++e) { start[e] = run; run += count[e]; }
        start[E] = run;
    }
    __syncthreads();
    for (int e = threadIdx.x; e <= E; e += blockDim.x) seg[e] = start[e];
    for (int e = threadIdx.x; e < E; e += blockDim.x) count[e] = 0;
    __syncthreads();
    for (int p = threadIdx.x; p < P; p += blockDim.x) {
        int e = table[(size_t)ids[p / top] * top + p % top];
        e = min(max(e, 0), E - 1);
        const int at = start[e] + atomicAdd(&count[e], 1);
        order[at] = p;
        where[p] = at;
    }
}

LLOGOS_EXPORT int llogos_moe_route(const int* ids, const int* table, int T, int top, int E, int* order, int* seg, int* where,
                                   hipStream_t stream) {
    if (T <= 0 || top <= 0 || E <= 0 || E > kMoeMaxExperts) return LLOGOS_BAD_ARGUMENT;
    moe_route_kernel<<<1, 1024, 0, stream>>>(ids, table, T, top, E, order, seg, where);
    return LLOGOS_LAUNCH_CHECK();
}

// out[r, :] = act(a_row(r) . w[e]^T) * scale for the sorted rows r of expert e's segment.
// a_row(r) = a[order[r] / top] when gather (the step's token rows), else a[r] (rows already sorted).
// w is [E][N][K].  Tiles of 64 rows x 64 columns; blockIdx.y counts row tiles over all segments.
constexpr int GM = 64, GN = 64, GK = 16;

template <typename TA, typename TW, typename TO>
__global__ __launch_bounds__(256) void moe_product_kernel(TO* __restrict__ out, const TA* __restrict__ a, const TW* __restrict__ w,
                                                          const int* __restrict__ order, const int* __restrict__ seg, int E,
                                                          int top, int gather, int N, int K, int lda, int act, float scale) {
    __shared__ float As[GK][GM + 4];
    __shared__ float Ws[GK][GN + 4];
    __shared__ int src_row[GM];
    __shared__ int s_expert, s_first, s_end;
    const int tid = threadIdx.x;
    if (tid == 0) {
        int tile = blockIdx.y, e = 0, found = -1, first = 0, end = 0;
        for (; e < E; ++e) {
            const int lo = seg[e], hi = seg[e + 1];
            const int tiles = (hi - lo + GM - 1) / GM;
            if (tile < tiles) { found = e; first = lo + tile * GM; end = hi; break; }
            tile -= tiles;
        }
        s_expert = found; s_first = first; s_end = end;
    }
    __syncthreads();
    const int e = s_expert;
    if (e < 0) return;                                     // beyond the last segment's tiles
    const int m0 = s_first, m_end = s_end, n0 = blockIdx.x * GN;
    if (tid < GM) {
        const int r = m0 + tid;
        src_row[tid] = r < m_end ? (gather ? order[r] / top : r) : -1;
    }
    __syncthreads();
    const TW* we = w + (size_t)e * N * K;
    const int ty = tid / 16, tx = tid % 16;
    const int lr = tid / 4, lk = (tid % 4) * 4;
    const int arow = src_row[lr];
    float acc[4][4] = {}, mid[4][4] = {};
    for (int k0 = 0; k0 < K; k0 += GK) {
        float part[4][4] = {};
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int k = k0 + lk + j;
            const int wn = n0 + lr;
            As[lk + j][lr] = (arow >= 0 && k < K) ? load_f32(a + (size_t)arow * lda + k) : 0.f;
            Ws[lk + j][lr] = (wn < N && k < K) ? load_f32(we + (size_t)wn * K + k) : 0.f;
        }
        __syncthreads();
#pragma unroll
        for (int k = 0; k < GK; ++k) {
            float av[4], wv[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) { av[i] = As[k][ty * 4 + i]; wv[i] = Ws[k][tx * 4 + i]; }
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) part[i][j] = fmaf(av[i], wv[j], part[i][j]);
        }
        const bool fold = ((k0 / GK) & 15) == 15;
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                mid[i][j] += part[i][j];
                if (fold) { acc[i][j] += mid[i][j]; mid[i][j] = 0.f; }
            }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int m = m0 + ty * 4 + i;
        if (m >= m_end) continue;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int n = n0 + tx * 4 + j;
            if (n >= N) continue;
            float v = acc[i][j] + mid[i][j];
            if (act == 1) { v = fmaxf(v, 0.f); v = v * v; }
            store_f32(out + (size_t)m * N + n, v * scale);
        }
    }
}

// P = T * top sorted rows at most; row_tiles bounds the tiles of all segments: ceil(P / 64) + E covers them.
LLOGOS_EXPORT int llogos_moe_product(void* out, int out_dtype, const void* a, int a_dtype, const void* w, int w_dtype,
                                     const int* order, const int* seg, int E, int top, int gather, int P, int N, int K,
                                     int lda, int act, float scale, hipStream_t stream) {
    if (P <= 0 || N <= 0 || K <= 0 || E <= 0 || top <= 0 || lda < K || act < 0 || act > 1) return LLOGOS_BAD_ARGUMENT;
    if (a_dtype != w_dtype && !(a_dtype == DT_F32)) return LLOGOS_BAD_ARGUMENT;
    const int row_tiles = (P + GM - 1) / GM + E;
    dim3 grid((N + GN - 1) / GN, row_tiles);
#define MP(TA, TW, TO) moe_product_kernel<TA, TW, TO><<<grid, 256, 0, stream>>>((TO*)out, (const TA*)a, (const TW*)w, order, seg, E, \
        top, gather, N, K, lda, act, scale)
    if (a_dtype == DT_F32 && w_dtype == DT_F32 && out_dtype == DT_F32) MP(float, float, float);
    else if (a_dtype == DT_BF16 && w_dtype == DT_BF16 && out_dtype == DT_BF16) MP(bf16_t, bf16_t, bf16_t);
    else if (a_dtype == DT_BF16 && w_dtype == DT_BF16 && out_dtype == DT_F32) MP(bf16_t, bf16_t, float);
    else return LLOGOS_BAD_ARGUMENT;
#undef MP
    return LLOGOS_LAUNCH_CHECK();
}

// out[t, :] = (sum_j y[where[t * top + j], :]) / top + sigmoid(gate[t * gate_stride]) * (sum of the parts of shared[t, :])
// y float32 [P, W]; shared float32 [(parts,) T, W] or null; gate float32 (one number a token, maybe in
// parts gate_part_stride apart) or null: then the shared rows are added as they are.
__global__ void moe_combine_kernel(float* __restrict__ out, const float* __restrict__ y, const int* __restrict__ where, int top,
                                   const float* __restrict__ shared_rows, int parts, size_t part_stride,
                                   const float* __restrict__ gate, int gate_stride, int gate_parts, size_t gate_part_stride,
                                   int T, int W) {
    const int t = blockIdx.x;
    float g = 1.f;
    if (gate) {
        float z = gate[(size_t)t * gate_stride];
        for (int p = 1; p < gate_parts; ++p) z += gate[p * gate_part_stride + (size_t)t * gate_stride];
        g = 1.0f / (1.0f + expf(-z));
    }
    const float inv_top = 1.0f / (float)top;
    for (int c = blockIdx.y * blockDim.x + threadIdx.x; c < W; c += gridDim.y * blockDim.x) {
        float v = 0.f;
        for (int j = 0; j < top; ++j) v += y[(size_t)where[t * top + j] * W + c];
        v *= inv_top;
        if (shared_rows) {
            float s = shared_rows[(size_t)t * W + c];
            for (int p = 1; p < parts; ++p) s += shared_rows[p * part_stride + (size_t)t * W + c];
            v = fmaf(g, s, v);
        }
        out[(size_t)t * W + c] = v;
    }
}

LLOGOS_EXPORT int llogos_moe_combine(float* out, const float* y, const int* where, int top, const float* shared_rows, int parts,
                                     long long part_stride, const float* gate, int gate_stride, int gate_parts,
                                     long long gate_part_stride, int T, int W, hipStream_t stream) {
    if (T <= 0 || W <= 0 || top <= 0 || parts < 1 || gate_parts < 1) return LLOGOS_BAD_ARGUMENT;
    const int threads = 256;
    dim3 grid(T, (W + threads - 1) / threads);
    moe_combine_kernel<<<grid, threads, 0, stream>>>(out, y, where, top, shared_rows, parts, (size_t)part_stride, gate, gate_stride,
                                                     gate_parts, (size_t)gate_part_stride, T, W);
    return LLOGOS_LAUNCH_CHECK();
}
