// Layer norm with a weight and no bias, with the residual sum fused in as in the RMS norm's kernel.
// For output row r (source row s = rows ? rows[r] : r):
//   v = x[s] + delta[s]        (delta optional, maybe in parts; written back to x when write_back)
//   out[r] = (v - mean(v)) / sqrt(mean((v - mean(v))^2) + eps) * w
// The mean is taken first and the squared deviations from it second (two sums over the row, not
// E[v^2] - E[v]^2), all in 32-bit.  A thread keeps its values of the row in registers between the
// passes: up to kLnItems values a thread; wider rows are read again from memory.
#include "common.h"

constexpr int kLnItems = 16;

template <typename TD>
__device__ __forceinline__ float ln_sum_parts(const TD* p, size_t i, int parts, size_t part_stride) {
    float v = load_f32(p + i);
    for (int q = 1; q < parts; ++q) v += load_f32(p + q * part_stride + i);
    return v;
}

template <typename TO, typename TD, bool CACHED>
__global__ __launch_bounds__(1024) void layernorm_kernel(TO* __restrict__ out, float* __restrict__ x, const TD* __restrict__ delta,
                                                         int parts, size_t part_stride, const int* __restrict__ rows,
                                                         const float* __restrict__ w, float eps, int H, int write_back) {
    __shared__ float red[16];
    const int r = blockIdx.x;
    const size_t s = rows ? (size_t)rows[r] : (size_t)r;
    float* xr = x + s * H;
    const TD* dr = delta ? delta + s * H : nullptr;
    float keep[CACHED ? kLnItems : 1];
    float sum = 0.f;
    if (CACHED) {
#pragma unroll
        for (int it = 0; it < kLnItems; ++it) {
            const int i = it * blockDim.x + threadIdx.x;
            float v = 0.f;
            if (i < H) {
                v = xr[i];
                if (dr) {
                    v += ln_sum_parts(dr, (size_t)i, parts, part_stride);
                    if (write_back) xr[i] = v;
                }
            }
            keep[it] = v;
            sum += v;
        }
    } else {
        for (int i = threadIdx.x; i < H; i += blockDim.x) {
            float v = xr[i];
            if (dr) {
                v += ln_sum_parts(dr, (size_t)i, parts, part_stride);
                if (write_back) xr[i] = v;
            }
            sum += v;
        }
    }
    const float mean = block_sum(sum, red) / (float)H;
    float sq = 0.f;
    if (CACHED) {
#pragma unroll
        for (int it = 0; it < kLnItems; ++it) {
            const int i = it * blockDim.x + threadIdx.x;
            if (i < H) { const float d = keep[it] - mean; sq = fmaf(d, d, sq); }
        }
    } else {
        for (int i = threadIdx.x; i < H; i += blockDim.x) {
            float v = xr[i];
            if (dr && !write_back) v += ln_sum_parts(dr, (size_t)i, parts, part_stride);
            const float d = v - mean;
            sq = fmaf(d, d, sq);
        }
    }
    const float var = block_sum(sq, red) / (float)H;
    const float inv = 1.0f / sqrtf(var + eps);
    TO* o = out + (size_t)r * H;
    if (CACHED) {
#pragma unroll
        for (int it = 0; it < kLnItems; ++it) {
            const int i = it * blockDim.x + threadIdx.x;
            if (i < H) store_f32(o + i, (keep[it] - mean) * inv * w[i]);
        }
    } else {
        for (int i = threadIdx.x; i < H; i += blockDim.x) {
            float v = xr[i];
            if (dr && !write_back) v += ln_sum_parts(dr, (size_t)i, parts, part_stride);
            store_f32(o + i, (v - mean) * inv * w[i]);
        }
    }
}

LLOGOS_EXPORT int llogos_layernorm(void* out, int out_dtype, float* x, const void* delta, int delta_dtype,
                                   int parts, long long part_stride, const int* rows, const float* w, float eps,
                                   int R, int H, int write_back, hipStream_t stream) {
    if (R <= 0 || H <= 0 || parts < 1) return LLOGOS_BAD_ARGUMENT;
    // as many threads as give each at most kLnItems values, in whole waves, 64 to 1024
    int threads = H <= 256 ? 64 : (H <= 1024 ? 128 : (H <= 4096 ? 256 : 1024));
    if (R <= 64) {                       // few rows: four values a thread, so that a row's loads are all in flight at once
        threads = ((H + 3) / 4 + kWave - 1) / kWave * kWave;
        threads = threads < 64 ? 64 : (threads > 1024 ? 1024 : threads);
    }
    const bool cached = (size_t)threads * kLnItems >= (size_t)H;
#define LN(TO, TD) do { \
        if (cached) layernorm_kernel<TO, TD, true><<<R, threads, 0, stream>>>((TO*)out, x, (const TD*)delta, parts, (size_t)part_stride, rows, w, eps, H, write_back); \
        else layernorm_kernel<TO, TD, false><<<R, threads, 0, stream>>>((TO*)out, x, (const TD*)delta, parts, (size_t)part_stride, rows, w, eps, H, write_back); \
    } while (0)
    if (out_dtype == DT_F32 && delta_dtype == DT_F32) LN(float, float);
    else if (out_dtype == DT_BF16 && delta_dtype == DT_BF16) LN(bf16_t, bf16_t);
    else if (out_dtype == DT_BF16 && delta_dtype == DT_F32) LN(bf16_t, float);
    else if (out_dtype == DT_F32 && delta_dtype == DT_BF16) LN(float, bf16_t);
    else return LLOGOS_BAD_ARGUMENT;
#undef LN
    return LLOGOS_LAUNCH_CHECK();
}
