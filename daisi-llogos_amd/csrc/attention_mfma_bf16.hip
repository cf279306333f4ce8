// bfloat16 attention over the paged cache on the matrix cores (gfx950,
// v_mfma_f32_16x16x32_bf16), for head sizes 64 and 128 and up to 16 query heads per
// key/value head.  Softmax statistics, scores and the output sums are float32.
//
// One wave works on 16 "columns" and one page of 64 keys at a time:
//   decode  (one token per sequence): the columns are the query heads of one kv head;
//           a block of 4 waves takes a run of pages of one (sequence, kv head), each wave
//           every fourth of them in turn; the waves' running (max, sum, output) are merged
//           through LDS, blocks along the context write partial results that a second small
//           kernel merges;
//   prefill (many tokens per sequence): the columns are 16 consecutive tokens of one
//           sequence for one query head; each wave walks the pages up to its last row.
// Scores are computed transposed, S^T[key][column] = K . Q^T, so that the lane that holds
// the scores of a column for 16 keys is the lane that must supply them as the second
// operand of O^T[d][column] = V^T[d][key] . P^T[key][column]; no shuffle or LDS pass sits
// between the two products.  Pages are stored in the order of these operands (common.h): a
// fragment is 1 KB of consecutive memory, a lane's eight values 16 bytes of it; a value
// fragment holds eight consecutive tokens of one dimension per lane, and the rows of a key
// fragment are the keys 16 * (i / 4) + 4 * rb + i % 4 (i = operand row, rb = block of 16),
// which makes lane group g own keys 16 g .. 16 g + 15.
// (reference: gated_attention / batched_gated_attention, Daisi.Llogos.Cuda/kernels/
//  composite_ops.cu:275-512: tiles of keys with running maximum and sum, kv head = head /
//  group, scale after the dot, query m of a prompt sees keys 0 .. start + m.)
#include "common.h"
#include "llogos_api.h"
#include <algorithm>
#include <mutex>

#include "attention_mfma.h"

// ---------------------------------------------------------------- decode
// grid (batch, kv heads, blocks along the context); a block of WAVES waves covers WAVES * ppw
// consecutive pages, wave w taking pages w, w + WAVES, ... of them one after the other.  (Asking
// for the next page's keys and values while a wave works on this one takes twice the registers
// and was slower: what hides the latency is the other waves.)  With one block
// along the context (gridDim.z == 1) the block writes the attention output itself; otherwise
// partial: [batch][heads][grid.z][HD + 2] floats (max, sum, unnormalised output) for the merge
// kernel.  Dynamic LDS: decode_lds_bytes(WAVES, group, HD).
__host__ __device__ constexpr size_t decode_lds_bytes(int waves, int group, int hd) {
    return (size_t)waves * (group * (hd + 1) + 32) * sizeof(float);
}

// The fused form (FUSED, head size 64 or 128 rotated whole with split-half pairing) starts from the
// projection itself: a block first makes its queries (sum of the projection's partial products,
// bias, per-head norm, rotation) into LDS, and the block whose pages hold the step's position
// also makes the step's key and value and writes them to their page, which the rotation kernel
// does otherwise.  One token a sequence: token b is sequence b.
struct QkvSource {
    const float* qkv;          // [parts][batch][row_stride]: partial sums of the fused rows [q | k | v]
    int parts;
    size_t part_stride;
    int row_stride;
    const float* bias;         // [(heads + 2 kv heads) * head size] or null
    const float* q_norm_w;     // [head size] or null
    const float* k_norm_w;
    float eps;
    const float2* cs;          // [batch][head size / 2] (cos, sin) of each sequence's position
    bf16_t* k_pool;            // the pools, writable
    bf16_t* v_pool;
};

template <int HD, int WAVES, bool FUSED>
__global__ __launch_bounds__(WAVES * kWave) void attn_decode_kernel(
        bf16_t* __restrict__ out, float* __restrict__ partial, const bf16_t* __restrict__ q, int q_stride,
        QkvSource src, const bf16_t* k_pool, const bf16_t* v_pool,
        const int* __restrict__ table, int table_stride, const int* __restrict__ tok_pos,
        int n_heads, int n_kv_heads, int group, float scale, int window, int sinks, int ppw) {
    extern __shared__ float lds[];
    float* lds_m = lds;                                   // [WAVES][16]
    float* lds_l = lds + WAVES * 16;                      // [WAVES][16]
    float* lds_o = lds + WAVES * 32;                      // [WAVES][group][HD + 1]
    __shared__ __attribute__((aligned(16))) bf16_t q_lds[FUSED ? 16 : 1][HD];
    const int b = blockIdx.x, kvh = blockIdx.y, z = blockIdx.z;
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    const int c = lane & 15, g = lane >> 4;
    const int pos = tok_pos[b];
    const int n_pages = pos / kPageTokens + 1;
    const int first_page = z * WAVES * ppw;
    if (first_page >= n_pages) return;                           // nothing of this sequence here
    const int* row = table + (size_t)b * table_stride;

    // this wave's pages: first_page + wave + WAVES j, j < ppw, as far as the sequence goes and a
    // query at pos can see any of their keys (a page outside the window may have been given back)
    auto page_at = [&](int j) { return first_page + wave + WAVES * j; };
    auto next_from = [&](int j) {
        while (j < ppw && page_at(j) < n_pages && !page_may_be_visible(pos, page_at(j) * kPageTokens, window, sinks)) ++j;
        return (j < ppw && page_at(j) < n_pages) ? j : -1;
    };
    auto page_base = [&](int j) { return ((size_t)row[page_at(j)] * n_kv_heads + kvh) * kPageTokens * HD; };
    int j = next_from(0);

    if (FUSED) {
        // items 0 .. group - 1: the kv head's query heads; then, in the block that holds the
        // step's position, its key and its value.  A wave takes an item; lane l holds
        // dimensions PER l .. PER l + PER - 1 (two for head size 128, one for 64), and the
        // rotation partner, HD / 2 dimensions away, is lane l ^ 32.
        constexpr int PER = HD / kWave;
        static_assert(PER == 1 || PER == 2, "head sizes 64 and 128");
        const bool writer = (n_pages - 1) / (WAVES * ppw) == z;
        const int items = group + (writer ? 2 : 0);
        const int d = PER * lane;
        const size_t wbase = writer ? ((size_t)row[n_pages - 1] * n_kv_heads + kvh) * kPageTokens * HD : 0;
        for (int item = wave; item < items; item += WAVES) {
            const bool is_q = item < group, is_k = item == group;
            const int head = is_q ? kvh * group + item : (is_k ? n_heads + kvh : n_heads + n_kv_heads + kvh);
            const size_t col = (size_t)head * HD + d;
            const float* p = src.qkv + (size_t)b * src.row_stride + col;
            float x[PER];
#pragma unroll
            for (int e = 0; e < PER; ++e) x[e] = p[e];
            for (int part0 = 1; part0 < src.parts; part0 += 8) {     // eight loads in flight, added in ascending order
                float y[8][PER];
#pragma unroll
                for (int jj = 0; jj < 8; ++jj)
#pragma unroll
                    for (int e = 0; e < PER; ++e)
                        y[jj][e] = part0 + jj < src.parts ? p[(part0 + jj) * src.part_stride + e] : 0.f;
#pragma unroll
                for (int jj = 0; jj < 8; ++jj)
                    if (part0 + jj < src.parts) {
#pragma unroll
                        for (int e = 0; e < PER; ++e) x[e] += y[jj][e];
                    }
            }
            if (src.bias) {
#pragma unroll
                for (int e = 0; e < PER; ++e) x[e] += src.bias[col + e];
            }
            if (!is_q && !is_k) {
                bf16_t* vdst = src.v_pool + wbase;
#pragma unroll
                for (int e = 0; e < PER; ++e) vdst[page_value_offset(pos % kPageTokens, d + e)] = f32_to_bf16(x[e]);
                continue;
            }
            const float* norm_w = is_q ? src.q_norm_w : src.k_norm_w;
            if (norm_w) {
                float sq = 0.f;
#pragma unroll
                for (int e = 0; e < PER; ++e) sq += x[e] * x[e];
                const float inv = 1.0f / sqrtf(wave_sum(sq) / (float)HD + src.eps);
#pragma unroll
                for (int e = 0; e < PER; ++e) x[e] = x[e] * inv * norm_w[d + e];
            }
            bf16_t y[PER];
#pragma unroll
            for (int e = 0; e < PER; ++e) {
                const float partner = __shfl_xor(x[e], 32, kWave);
                const float2 cs = src.cs[(size_t)b * (HD / 2) + ((d + e) & (HD / 2 - 1))];
                y[e] = f32_to_bf16(lane < 32 ? x[e] * cs.x - partner * cs.y : partner * cs.y + x[e] * cs.x);
            }
            // (a lane's one or two dimensions are neighbours in a key page too)
            bf16_t* dst = is_q ? &q_lds[item][d] : src.k_pool + wbase + page_key_offset(pos % kPageTokens, d, HD);
#pragma unroll
            for (int e = 0; e < PER; ++e) dst[e] = y[e];
        }
        __syncthreads();          // the queries in LDS, and the key and value in memory, for every wave of the block
    }

    WaveState<HD> st;
    st.init();
    if (j >= 0) {
        bf16x8 qf[HD / 32];
        const bool col_ok = c < group;
        const bf16_t* qrow = FUSED ? &q_lds[col_ok ? c : 0][8 * g]
                                   : q + (size_t)b * q_stride + (size_t)(kvh * group + (col_ok ? c : 0)) * HD + 8 * g;
#pragma unroll
        for (int sk = 0; sk < HD / 32; ++sk) qf[sk] = col_ok ? ld_frag(qrow + 32 * sk) : zero_frag();
        // unused columns (c >= group) have zero queries and are never stored: they may run unmasked
        for (; j >= 0; j = next_from(j + 1)) {
            const int key0 = page_at(j) * kPageTokens;
            const size_t base = page_base(j);
            attend_page<HD>(st, qf, k_pool + base, v_pool + base, col_ok ? pos : -1, key0,
                            min(kPageTokens, pos - key0 + 1), page_fully_visible(pos, pos, key0, window, sinks),
                            scale * kLog2e, window, sinks);
        }
    }
    // merge the waves
    if (g == 0) { lds_m[wave * 16 + c] = st.m; lds_l[wave * 16 + c] = st.l; }
    if (c < group) {
        float* dst = lds_o + ((size_t)wave * group + c) * (HD + 1);
#pragma unroll
        for (int db = 0; db < HD / 16; ++db)
#pragma unroll
            for (int r = 0; r < 4; ++r) dst[16 * db + 4 * g + r] = st.acc[db][r];
    }
    __syncthreads();
    const int n_z = gridDim.z;
    for (int idx = threadIdx.x; idx < group * HD; idx += blockDim.x) {
        const int col = idx / HD, d = idx % HD;
        float m = -INFINITY;
#pragma unroll
        for (int w = 0; w < WAVES; ++w) m = fmaxf(m, lds_m[w * 16 + col]);
        float l = 0.f, o = 0.f;
#pragma unroll
        for (int w = 0; w < WAVES; ++w) {
            const float mw = lds_m[w * 16 + col];
            const float f = (mw == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f(mw - m);
            l += lds_l[w * 16 + col] * f;
            o += lds_o[((size_t)w * group + col) * (HD + 1) + d] * f;
        }
        if (n_z == 1) {
            out[((size_t)b * n_heads + kvh * group + col) * HD + d] = f32_to_bf16(l > 0.f ? o / l : 0.f);
        } else {
            float* dst = partial + (((size_t)b * n_heads + kvh * group + col) * n_z + z) * (HD + 2);
            dst[2 + d] = o;
            if (d == 0) { dst[0] = m; dst[1] = l; }
        }
    }
}

// grid (batch, heads); kMergeLanes x HD threads.  Adds the partial results of the blocks along
// the context, each of which covered pages_per_block pages: thread (j, d) takes blocks j,
// j + kMergeLanes, ... of dimension d, and LDS adds the kMergeLanes sums in ascending j, so the
// order depends on the sequence's own length alone.  (One thread per dimension walking all
// blocks took 17 us at 33 blocks: a chain of dependent L2 latencies.  Letting the last block
// to finish add them, behind a device-wide fence and a ticket counter, was measured too: the
// fence writes back whatever earlier kernels left dirty in the L2 and cost 20 us a layer at
// batch 8; this kernel costs 4.6.)
constexpr int kMergeLanes = 4;

template <int HD>
__global__ __launch_bounds__(kMergeLanes * HD) void attn_decode_merge_kernel(
        bf16_t* __restrict__ out, const float* __restrict__ partial, const int* __restrict__ tok_pos,
        int n_heads, int n_z, int pages_per_block) {
    __shared__ float lds_m[kMergeLanes], lds_l[kMergeLanes], lds_o[kMergeLanes][HD];
    const int b = blockIdx.x, h = blockIdx.y, d = threadIdx.x % HD, j = threadIdx.x / HD;
    const int n_pages = tok_pos[b] / kPageTokens + 1;
    const int used = min(n_z, (n_pages + pages_per_block - 1) / pages_per_block);
    const float* src = partial + ((size_t)b * n_heads + h) * n_z * (HD + 2);
    float m = -INFINITY;
#pragma unroll 4
    for (int z = j; z < used; z += kMergeLanes) m = fmaxf(m, src[(size_t)z * (HD + 2)]);
    if (d == 0) lds_m[j] = m;
    __syncthreads();
#pragma unroll
    for (int i = 0; i < kMergeLanes; ++i) m = fmaxf(m, lds_m[i]);
    float l = 0.f, o = 0.f;
#pragma unroll 4
    for (int z = j; z < used; z += kMergeLanes) {
        const float* p = src + (size_t)z * (HD + 2);
        const float f = (p[0] == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f(p[0] - m);
        l += p[1] * f;
        o += p[2 + d] * f;
    }
    lds_o[j][d] = o;
    if (d == 0) lds_l[j] = l;
    __syncthreads();
    if (j != 0) return;
    l = lds_l[0]; o = lds_o[0][d];
#pragma unroll
    for (int i = 1; i < kMergeLanes; ++i) { l += lds_l[i]; o += lds_o[i][d]; }
    out[((size_t)b * n_heads + h) * HD + d] = f32_to_bf16(l > 0.f ? o / l : 0.f);
}

// ---------------------------------------------------------------- prefill
// grid (tiles of 64 tokens over all sequences, heads); wave w of a block takes rows
// 16 w .. 16 w + 15 of the tile.  cu: token offsets of the sequences [batch + 1];
// starts: position of each sequence's first token in this step.
template <int HD>
__global__ __launch_bounds__(kAttnWaves * kWave) void attn_prefill_kernel(
        bf16_t* __restrict__ out, const bf16_t* __restrict__ q, int q_stride,
        const bf16_t* __restrict__ k_pool, const bf16_t* __restrict__ v_pool,
        const int* __restrict__ table, int table_stride, const int* __restrict__ cu,
        const int* __restrict__ tok_pos, int batch, int n_heads, int n_kv_heads, int group,
        float scale, int window, int sinks) {
    // which sequence does this tile belong to?
    int tile = blockIdx.x, b = 0, first = 0;
    for (; b < batch; ++b) {
        const int len = cu[b + 1] - cu[b];
        const int tiles = (len + 63) / 64;
        if (tile < tiles) { first = cu[b] + tile * 64; break; }
        tile -= tiles;
    }
    if (b >= batch) return;
    const int h = blockIdx.y, kvh = h / group;
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    const int c = lane & 15, g = lane >> 4;
    const int row0 = first + 16 * wave;                          // this wave's first token row
    const int seq_end = cu[b + 1];
    if (row0 >= seq_end) return;
    const int rows = min(16, seq_end - row0);
    const bool col_ok = c < rows;
    const int my_row = row0 + (col_ok ? c : 0);
    const int q_pos = col_ok ? tok_pos[my_row] : -1;
    const int last_pos = tok_pos[row0 + rows - 1];
    const int first_pos = tok_pos[row0];
    const int written = tok_pos[seq_end - 1] + 1;                // positions of this sequence that hold keys

    bf16x8 qf[HD / 32];
    const bf16_t* qrow = q + (size_t)my_row * q_stride + (size_t)h * HD + 8 * g;
#pragma unroll
    for (int sk = 0; sk < HD / 32; ++sk) qf[sk] = col_ok ? ld_frag(qrow + 32 * sk) : zero_frag();

    WaveState<HD> st;
    st.init();
    const int n_pages = last_pos / kPageTokens + 1;
    for (int pi = 0; pi < n_pages; ++pi) {
        const int key0 = pi * kPageTokens;
        if (!page_may_be_visible_to_range(first_pos, last_pos, key0, window, sinks)) continue;
        const int page = table[(size_t)b * table_stride + pi];
        const size_t base = ((size_t)page * n_kv_heads + kvh) * kPageTokens * HD;
        attend_page<HD>(st, qf, k_pool + base, v_pool + base, q_pos, key0, min(kPageTokens, written - key0),
                        rows == 16 && page_fully_visible(first_pos, last_pos, key0, window, sinks),
                        scale * kLog2e, window, sinks);
    }
    if (!col_ok) return;
    const float inv = st.l > 0.f ? 1.0f / st.l : 0.f;
    bf16_t* orow = out + ((size_t)my_row * n_heads + h) * HD;
#pragma unroll
    for (int db = 0; db < HD / 16; ++db) {
        uint2 u;
        u.x = pack_bf16(st.acc[db][0] * inv, st.acc[db][1] * inv);
        u.y = pack_bf16(st.acc[db][2] * inv, st.acc[db][3] * inv);
        *reinterpret_cast<uint2*>(orow + 16 * db + 4 * g) = u;
    }
}

// ---------------------------------------------------------------- entry points
static bool mfma_shape_ok(int n_heads, int n_kv_heads, int head_dim) {
    if (n_kv_heads <= 0 || n_heads % n_kv_heads) return false;
    return (head_dim == 64 || head_dim == 128) && n_heads / n_kv_heads <= 16;
}

// The classes of batch sizes: the sizes at which single-token steps are captured (a batch in
// between runs padded to the next of them).  Whatever a kernel's shape takes from the batch it
// takes from the class, or a sequence's sums would come in another order alone than beside
// others of its class.
LLOGOS_EXPORT int llogos_batch_class(int batch) {
    static const int classes[] = {1, 2, 3, 4, 5, 6, 7, 8, 12, 16, 24, 32, 48, 64};
    for (int c : classes) if (batch <= c) return c;
    return (batch + 63) / 64 * 64;
}

// compute units of the current device, asked for once per device
static int compute_units() {
    static int cached[64];
    int device = 0;
    if (hipGetDevice(&device) != hipSuccess || device < 0 || device >= 64) return 256;
    if (cached[device] == 0) {
        int n = 0;
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, device) != hipSuccess || n <= 0) n = 256;
        cached[device] = n;
    }
    return cached[device];
}

constexpr int kDecodeWaves = 4;
constexpr int kMaxPagesPerWave = 16;

// Pages per wave.  A wave's pages come one after the other, a "step" each; a CU works on one
// block's waves at a time as far as timings show, so a launch takes about as many steps as the
// blocks that fall to the busiest CU have together: blocks of ppw steps go round by round over
// the CUs, the shorter last block of each sequence after them.  Every round of blocks costs a
// quarter of a step more (queries, merge through LDS), the merge kernel three quarters.  The
// count of steps is what 26 shapes measured at the 8B head shape (32 query heads, 8 kv heads of
// 128; batch 1 to 64, 640 to 131,000 positions) order by.  Against one page a wave in blocks of
// up to 16 waves: batch 64 at 640 positions 42.5 us from 46.2, at 8,192 361 from 417; batch 8
// at 32,768 192 from 211; batch 1 at 131,000 102 from 117; batch 32 at 640 25.1 from 23.6.
static int decode_pages_per_wave(int table_width, int batch, int n_kv_heads) {
    const long long pairs = (long long)llogos_batch_class(batch) * n_kv_heads;
    const long long units = compute_units();
    int best = 1;
    double best_cost = 0;
    for (int ppw = 1; ppw <= kMaxPagesPerWave; ++ppw) {
        const int chunk = kDecodeWaves * ppw;
        const long long full = table_width / chunk;                       // whole blocks of a sequence
        const int rest = table_width % chunk;                             // pages of its last, shorter block
        const long long full_rounds = (pairs * full + units - 1) / units;
        double steps = (double)full_rounds * ppw, rounds = (double)full_rounds;
        if (rest > 0) {
            const long long room = full_rounds * units - pairs * full;    // places the last round of whole blocks leaves
            const long long more = pairs > room ? (pairs - room + units - 1) / units : 0;
            // (blocks a quarter as long as the whole ones, or less, run beside the last of those: half a step each)
            const int rest_steps = (rest + kDecodeWaves - 1) / kDecodeWaves;
            steps += (double)more * rest_steps * (full > 0 && 4 * rest_steps <= ppw ? 0.5 : 1.0);
            rounds += (double)more;
        }
        const double cost = steps + 0.25 * rounds + (full + (rest > 0) > 1 ? 0.75 : 0.0);
        if (ppw == 1 || cost < best_cost - 1e-9) { best = ppw; best_cost = cost; }
    }
    return best;
}

// floats the decode workspace needs
LLOGOS_EXPORT long long llogos_attn_decode_workspace(int batch, int n_heads, int n_kv_heads, int head_dim,
                                                     int table_width) {
    if (n_kv_heads <= 0 || n_heads % n_kv_heads) return 0;
    const int ppw = decode_pages_per_wave(table_width, batch, n_kv_heads);
    const int n_z = (table_width + kDecodeWaves * ppw - 1) / (kDecodeWaves * ppw);
    return n_z == 1 ? 0 : (long long)batch * n_heads * n_z * (head_dim + 2);
}

static int launch_decode(void* out, const void* q, int q_stride, const QkvSource* src, const void* k_pool,
                         const void* v_pool, const int* table, int table_stride, int table_width,
                         const int* tok_pos, int batch, int n_heads, int n_kv_heads, int head_dim,
                         float scale, int window, int sinks, float* workspace, long long workspace_floats,
                         hipStream_t stream) {
    if (batch <= 0 || table_width <= 0 || window < 0 || sinks < 0) return LLOGOS_BAD_ARGUMENT;
    if (!mfma_shape_ok(n_heads, n_kv_heads, head_dim)) return LLOGOS_UNSUPPORTED;
    if (workspace_floats < llogos_attn_decode_workspace(batch, n_heads, n_kv_heads, head_dim, table_width))
        return LLOGOS_BAD_ARGUMENT;
    const int group = n_heads / n_kv_heads;
    const int waves = kDecodeWaves, ppw = decode_pages_per_wave(table_width, batch, n_kv_heads);
    const int n_z = (table_width + waves * ppw - 1) / (waves * ppw);
    if (n_z > 1 && workspace == nullptr) return LLOGOS_BAD_ARGUMENT;
    dim3 grid(batch, n_kv_heads, n_z), mgrid(batch, n_heads);
    const size_t smem = decode_lds_bytes(waves, group, head_dim);
    const QkvSource none{};
#define GO(HD, FUSED) do { \
    attn_decode_kernel<HD, kDecodeWaves, FUSED><<<grid, kDecodeWaves * kWave, smem, stream>>>( \
        (bf16_t*)out, workspace, (const bf16_t*)q, q_stride, FUSED ? *src : none, (const bf16_t*)k_pool, \
        (const bf16_t*)v_pool, table, table_stride, tok_pos, n_heads, n_kv_heads, group, scale, window, sinks, ppw); \
    if (n_z > 1) attn_decode_merge_kernel<HD><<<mgrid, kMergeLanes * HD, 0, stream>>>((bf16_t*)out, workspace, tok_pos, n_heads, \
                                                                        n_z, kDecodeWaves * ppw); } while (0)
    if (src != nullptr && head_dim == 64) GO(64, true);
    else if (src != nullptr) GO(128, true);
    else if (head_dim == 64) GO(64, false);
    else GO(128, false);
#undef GO
    return LLOGOS_LAUNCH_CHECK();
}

LLOGOS_EXPORT int llogos_attn_decode_bf16(void* out, const void* q, int q_stride, const void* k_pool,
                                          const void* v_pool, const int* table, int table_stride, int table_width,
                                          const int* tok_pos, int batch, int n_heads, int n_kv_heads, int head_dim,
                                          float scale, int window, int sinks, float* workspace,
                                          long long workspace_floats, hipStream_t stream) {
    if ((q_stride % 8) || ((uintptr_t)q % 16)) return LLOGOS_UNSUPPORTED;
    return launch_decode(out, q, q_stride, nullptr, k_pool, v_pool, table, table_stride, table_width, tok_pos, batch,
                         n_heads, n_kv_heads, head_dim, scale, window, sinks, workspace, workspace_floats, stream);
}

// ---------------------------------------------------------------- decode without allocation
// The decode attention for callers that cannot allocate (see llogos_api.h).  The partial
// results of the blocks along the context, which llogos_attn_decode_bf16 takes in a workspace
// from its caller, live in a file-scope device array here.  In host code the array's name is
// only a stand-in for the symbol: its device address is asked for once per device, with that
// device current, and that pointer is what the kernels, and anything else on the host, get.
constexpr long long kStaticScratchFloats = 4ll << 20;                  // 16 MiB on each GPU the library runs on
static __device__ __align__(256) float scratch[kStaticScratchFloats];
constexpr int kMaxDevices = 64;
static float* scratch_ptr[kMaxDevices];                                // per device; null until asked for
static std::mutex scratch_mutex;

// The current device's copy of the array, through *ptr.
static int static_scratch(float** ptr) {
    int device = -1;
    hipError_t e = hipGetDevice(&device);
    if (e != hipSuccess) return (int)e;
    if (device < 0 || device >= kMaxDevices) return LLOGOS_BAD_ARGUMENT;
    std::lock_guard<std::mutex> hold(scratch_mutex);
    if (scratch_ptr[device] == nullptr) {
        float* p = nullptr;
        e = hipGetSymbolAddress((void**)&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess) return (int)e;
        if (p == nullptr) return (int)hipErrorInvalidSymbol;
        scratch_ptr[device] = p;
    }
    *ptr = scratch_ptr[device];
    return 0;
}

LLOGOS_EXPORT long long llogos_attn_decode_static_capacity(void) { return kStaticScratchFloats; }

LLOGOS_EXPORT int llogos_attn_decode_static_init(void) {
    float* p = nullptr;
    return static_scratch(&p);
}

LLOGOS_EXPORT int llogos_attn_decode_static_bf16(void* out, const void* q, int q_stride, const void* k_pool,
                                                 const void* v_pool, const int* table, int table_stride,
                                                 int table_width, const int* tok_pos, int batch, int n_heads,
                                                 int n_kv_heads, int head_dim, float scale, int window, int sinks,
                                                 hipStream_t stream) {
    if ((q_stride % 8) || ((uintptr_t)q % 16)) return LLOGOS_UNSUPPORTED;
    if (batch <= 0 || table_width <= 0) return LLOGOS_BAD_ARGUMENT;
    if (!mfma_shape_ok(n_heads, n_kv_heads, head_dim)) return LLOGOS_UNSUPPORTED;
    // Nothing in the array has to start at zero: the merge kernel reads only the partial results
    // that this call's blocks have written (blocks z < ceil(pages / pages per block) of each
    // sequence), so what an earlier call left is never looked at.
    const long long need = llogos_attn_decode_workspace(batch, n_heads, n_kv_heads, head_dim, table_width);
    if (need > kStaticScratchFloats) return LLOGOS_TOO_LARGE;
    float* ws = nullptr;
    const int code = static_scratch(&ws);
    if (code != 0) return code;
    return launch_decode(out, q, q_stride, nullptr, k_pool, v_pool, table, table_stride, table_width, tok_pos, batch,
                         n_heads, n_kv_heads, head_dim, scale, window, sinks, ws, kStaticScratchFloats, stream);
}

// The same from the fused projection (see QkvSource): head sizes 64 and 128; also writes the
// step's keys and values to their pages.  cs: [batch][head size / 2][2] floats.
LLOGOS_EXPORT int llogos_attn_decode_fused_bf16(void* out, const float* qkv, int parts, long long part_stride,
                                                int row_stride, const float* bias, const float* q_norm_w,
                                                const float* k_norm_w, float eps, const void* cs, void* k_pool,
                                                void* v_pool, const int* table, int table_stride, int table_width,
                                                const int* tok_pos, int batch, int n_heads, int n_kv_heads,
                                                int head_dim, float scale, int window, int sinks, float* workspace,
                                                long long workspace_floats, hipStream_t stream) {
    if (head_dim != 128 && head_dim != 64) return LLOGOS_UNSUPPORTED;
    if (parts < 1 || (row_stride % 2) || (part_stride % 2) || ((uintptr_t)qkv % 8) ||
        row_stride < (n_heads + 2 * n_kv_heads) * head_dim)
        return LLOGOS_BAD_ARGUMENT;
    const QkvSource src{qkv, parts, (size_t)part_stride, row_stride, bias, q_norm_w, k_norm_w, eps,
                        (const float2*)cs, (bf16_t*)k_pool, (bf16_t*)v_pool};
    return launch_decode(out, nullptr, 0, &src, k_pool, v_pool, table, table_stride, table_width, tok_pos, batch,
                         n_heads, n_kv_heads, head_dim, scale, window, sinks, workspace, workspace_floats, stream);
}

// tile_rows: 64 for the kernel whose waves read pages from global memory, 128 for the kernel
// that shares pages through LDS (n_tiles counts tiles of that many tokens per sequence).
LLOGOS_EXPORT int llogos_attn_prefill_bf16(void* out, const void* q, int q_stride, const void* k_pool,
                                           const void* v_pool, const int* table, int table_stride,
                                           const int* cu, const int* tok_pos, int batch, int n_tiles, int tile_rows,
                                           int n_heads, int n_kv_heads, int head_dim,
                                           float scale, int window, int sinks, int halves, hipStream_t stream) {
    if (batch <= 0 || n_tiles <= 0 || window < 0 || sinks < 0 || (halves != 1 && halves != 2)) return LLOGOS_BAD_ARGUMENT;
    if (tile_rows != 64 && tile_rows != kTileRows) return LLOGOS_BAD_ARGUMENT;
    if (!mfma_shape_ok(n_heads, n_kv_heads, head_dim) || (q_stride % 8) || ((uintptr_t)q % 16)) return LLOGOS_UNSUPPORTED;
    const int group = n_heads / n_kv_heads;
    dim3 grid(n_tiles, n_heads);
    if (tile_rows == kTileRows) {
        const long long pairs = (long long)n_tiles * n_kv_heads;
        const dim3 lgrid((unsigned)((pairs + 7) / 8 * 8 * group));
#define GOD(HD, HALVES) do { \
        const size_t smem = HALVES * 2 * sizeof(DirectPageLds<HD>); \
        hipError_t e = hipFuncSetAttribute((const void*)attn_prefill_direct_kernel<HD, HALVES>, \
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem); \
        if (e != hipSuccess) return (int)e; \
        attn_prefill_direct_kernel<HD, HALVES><<<lgrid, HALVES * kAttnWaves * kWave, smem, stream>>>( \
            (bf16_t*)out, (const bf16_t*)q, q_stride, (const bf16_t*)k_pool, (const bf16_t*)v_pool, table, table_stride, \
            cu, tok_pos, batch, n_tiles, n_heads, n_kv_heads, group, scale, window, sinks); \
        return LLOGOS_LAUNCH_CHECK(); } while (0)
        if (halves == 2) { if (head_dim == 64) GOD(64, 2); else GOD(128, 2); }
        if (head_dim == 64) GOD(64, 1); else GOD(128, 1);
#undef GOD
    }
#define GO(HD) attn_prefill_kernel<HD><<<grid, kAttnWaves * kWave, 0, stream>>>( \
        (bf16_t*)out, (const bf16_t*)q, q_stride, (const bf16_t*)k_pool, (const bf16_t*)v_pool, table, table_stride, \
        cu, tok_pos, batch, n_heads, n_kv_heads, group, scale, window, sinks)
    if (head_dim == 64) { GO(64); } else { GO(128); }
#undef GO
    return LLOGOS_LAUNCH_CHECK();
}
