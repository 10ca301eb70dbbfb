// Differential attention in bfloat16 on the matrix cores: two softmax maps a head over the same values,
//   o = a_1 - lambda * a_2;   out = o / sqrt(mean(o^2) + eps) * out_scale.
// A kv head's key row in its page holds both maps' keys side by side (2 * KP values, KP = 32 KS a map); values are
// rows of VP = 16 VB.  Pages are in the matrix cores' operand order (common.h), and the page steps of
// attention_mfma.h serve.
//   prefill: a map is a head of its own in the prompt kernel whose pages go straight into LDS (attention_mfma.h,
//            MAPS = 2); the maps' rows come out as 32-bit floats, and a small kernel takes their difference and norms it.
//   decode:  the columns of a wave are the query heads of one kv head; a wave holds the running softmax of both
//            maps and reads a page's values once for both; a block of 4 waves takes a run of pages of one
//            (sequence, kv head); blocks along the context leave partial results (max, sum, output a map) for the
//            kernel that merges them, takes the difference and norms it.
#include "attention_mfma.h"

#include <algorithm>

// Keys of one map out of a row of MAPS maps: fragment (rb, sk) lies at rb * (MAPS * KS) + map * KS + sk.
template <int KS>
__device__ __forceinline__ void load_map_keys(bf16x8 (&kf)[4][KS], const bf16_t* __restrict__ kpage, int map) {
    const bf16_t* mine = kpage + 8 * (threadIdx.x & (kWave - 1));
#pragma unroll
    for (int rb = 0; rb < 4; ++rb)
#pragma unroll
        for (int sk = 0; sk < KS; ++sk) kf[rb][sk] = ld_frag_once(mine + 512 * (rb * (2 * KS) + map * KS + sk));
}

// ---------------------------------------------------------------- decode
// grid (batch, kv heads, blocks along the context); wave w of a block takes pages first + w, first + w + 4, ...
// (ppw of them).  partial: [batch][heads][2][grid.z][VP + 2] floats (max in units of log2, sum, unnormalised output).
// LDS: 4 * 2 * (group * (VP + 1) + 32) floats.
template <int KS, int VB>
__global__ __launch_bounds__(kAttnWaves * kWave) void diff_decode_kernel(
        float* __restrict__ partial, const bf16_t* __restrict__ q, int q_stride, const bf16_t* __restrict__ k_pool,
        const bf16_t* __restrict__ v_pool, const int* __restrict__ table, int table_stride, const int* __restrict__ tok_pos,
        int n_heads, int n_kv_heads, int group, float scale, int window, int sinks, int ppw) {
    constexpr int KP = 32 * KS, VP = 16 * VB, WAVES = kAttnWaves;
    extern __shared__ float lds[];
    const int b = blockIdx.x, kvh = blockIdx.y, z = blockIdx.z;
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    const int c = lane & 15, g = lane >> 4;
    const int pos = tok_pos[b];
    const int n_pages = pos / kPageTokens + 1;
    const int first_page = z * WAVES * ppw;
    if (first_page >= n_pages) return;
    const int* row = table + (size_t)b * table_stride;

    WaveState<VP> st[2];
    st[0].init();
    st[1].init();
    const bool col_ok = c < group;
    bf16x8 qf[2][KS];
    const bf16_t* qrow = q + (size_t)b * q_stride + (size_t)(kvh * group + (col_ok ? c : 0)) * (2 * KP) + 8 * g;
#pragma unroll
    for (int m = 0; m < 2; ++m)
#pragma unroll
        for (int sk = 0; sk < KS; ++sk) qf[m][sk] = col_ok ? ld_frag(qrow + m * KP + 32 * sk) : zero_frag();
    const float scale_log2 = scale * kLog2e;
    for (int j = 0; j < ppw; ++j) {
        const int pi = first_page + wave + WAVES * j;
        if (pi >= n_pages) break;
        const int key0 = pi * kPageTokens;
        if (!page_may_be_visible(pos, key0, window, sinks)) continue;     // (such a page may have been given back)
        const size_t page = ((size_t)row[pi] * n_kv_heads + kvh) * kPageTokens;
        const int valid_keys = min(kPageTokens, pos - key0 + 1);
        const bool all_visible = page_fully_visible(pos, pos, key0, window, sinks);
        bf16x8 vf[VB][2];
        load_values<VP>(vf, v_pool + page * VP);
#pragma unroll
        for (int m = 0; m < 2; ++m) {
            bf16x8 kf[4][KS];
            load_map_keys<KS>(kf, k_pool + page * (2 * KP), m);
            f32x4 s[4];
            page_scores<KP>(s, kf, qf[m]);
            bf16x8 pf[2];
            float corr;
            if (all_visible) softmax_page<false, 16, 4, VP>(s, st[m], scale_log2, col_ok ? pos : -1, key0, window, sinks, pf, corr);
            else             softmax_page<true, 16, 4, VP>(s, st[m], scale_log2, col_ok ? pos : -1, key0, window, sinks, pf, corr);
            weigh_values<VP>(st[m], vf, pf, corr, valid_keys);
        }
    }
    // merge the waves, a map at a time
    const int n_z = gridDim.z;
    constexpr int kMapFloats = WAVES * 32;                 // maxima and sums of a map
    float* lds_o = lds + 2 * kMapFloats;                   // [2][WAVES][group][VP + 1]
#pragma unroll
    for (int m = 0; m < 2; ++m) {
        if (g == 0) { lds[m * kMapFloats + wave * 16 + c] = st[m].m; lds[m * kMapFloats + WAVES * 16 + wave * 16 + c] = st[m].l; }
        if (col_ok) {
            float* dst = lds_o + (((size_t)m * WAVES + wave) * group + c) * (VP + 1);
#pragma unroll
            for (int db = 0; db < VB; ++db)
#pragma unroll
                for (int r = 0; r < 4; ++r) dst[16 * db + 4 * g + r] = st[m].acc[db][r];
        }
    }
    __syncthreads();
    for (int idx = threadIdx.x; idx < 2 * group * VP; idx += blockDim.x) {
        const int m = idx / (group * VP), col = idx / VP % group, d = idx % VP;
        const float* lm = lds + m * kMapFloats;
        const float* ll = lm + WAVES * 16;
        float mx = -INFINITY;
#pragma unroll
        for (int w = 0; w < WAVES; ++w) mx = fmaxf(mx, lm[w * 16 + col]);
        float l = 0.f, o = 0.f;
#pragma unroll
        for (int w = 0; w < WAVES; ++w) {
            const float mw = lm[w * 16 + col];
            const float f = (mw == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f(mw - mx);
            l += ll[w * 16 + col] * f;
            o += lds_o[(((size_t)m * WAVES + w) * group + col) * (VP + 1) + d] * f;
        }
        float* dst = partial + ((((size_t)b * n_heads + kvh * group + col) * 2 + m) * n_z + z) * (VP + 2);
        dst[2 + d] = o;
        if (d == 0) { dst[0] = mx; dst[1] = l; }
    }
}

// grid (batch, heads), VP threads: thread d adds dimension d of the blocks' partial results of either map in
// ascending order, takes the difference, and the block norms it.
template <int VB>
__global__ __launch_bounds__(16 * VB) void diff_merge_kernel(bf16_t* __restrict__ out, const float* __restrict__ partial,
                                                             const int* __restrict__ tok_pos, int n_heads, int n_z,
                                                             int pages_per_block, float lambda, float out_scale, float eps) {
    constexpr int VP = 16 * VB;
    __shared__ float red[16];
    const int b = blockIdx.x, h = blockIdx.y, d = threadIdx.x;
    const int n_pages = tok_pos[b] / kPageTokens + 1;
    const int used = min(n_z, (n_pages + pages_per_block - 1) / pages_per_block);
    float a[2];
#pragma unroll
    for (int m = 0; m < 2; ++m) {
        const float* src = partial + (((size_t)b * n_heads + h) * 2 + m) * n_z * (VP + 2);
        float mx = -INFINITY;
        for (int z = 0; z < used; ++z) mx = fmaxf(mx, src[(size_t)z * (VP + 2)]);
        float l = 0.f, o = 0.f;
        for (int z = 0; z < used; ++z) {
            const float* p = src + (size_t)z * (VP + 2);
            const float f = (p[0] == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f(p[0] - mx);
            l += p[1] * f;
            o += p[2 + d] * f;
        }
        a[m] = l > 0.f ? o / l : 0.f;
    }
    const float o = a[0] - lambda * a[1];
    const float total = block_sum(o * o, red);
    out[((size_t)b * n_heads + h) * VP + d] = f32_to_bf16(o * (out_scale / sqrtf(total / (float)VP + eps)));
}

// ---------------------------------------------------------------- prefill: the maps' difference
// maps: [tokens][heads][2][VP] floats, the two maps' normalised rows.  grid (tokens, heads), VP threads.
template <int VB>
__global__ __launch_bounds__(16 * VB) void diff_combine_kernel(bf16_t* __restrict__ out, const float* __restrict__ maps,
                                                               int n_heads, float lambda, float out_scale, float eps) {
    constexpr int VP = 16 * VB;
    __shared__ float red[16];
    const int t = blockIdx.x, h = blockIdx.y, d = threadIdx.x;
    const float* src = maps + ((size_t)t * n_heads + h) * 2 * VP;
    const float o = src[d] - lambda * src[VP + d];
    const float total = block_sum(o * o, red);
    out[((size_t)t * n_heads + h) * VP + d] = f32_to_bf16(o * (out_scale / sqrtf(total / (float)VP + eps)));
}

// ---------------------------------------------------------------- entry points
static int diff_units() {
    static int units = 0;
    if (units == 0) {
        int dev = 0;
        hipDeviceProp_t prop;
        if (hipGetDevice(&dev) == hipSuccess && hipGetDeviceProperties(&prop, dev) == hipSuccess) units = prop.multiProcessorCount;
        if (units <= 0) units = 256;
    }
    return units;
}

static bool diff_shape_ok(int n_heads, int n_kv_heads, int dim, int dv) {
    if (n_heads <= 0 || n_kv_heads <= 0 || n_heads % n_kv_heads || n_heads / n_kv_heads > 16) return false;
    return (dim == 32 || dim == 64 || dim == 128) && (dv == 64 || dv == 128);
}

// pages a wave takes in a decode step: as few as leave no more than two blocks a compute unit
static int diff_pages_per_wave(int batch, int n_kv_heads, int table_width) {
    const int room = 2 * diff_units();
    for (int ppw = 1; ppw < 16; ++ppw) {
        const int n_z = (table_width + kAttnWaves * ppw - 1) / (kAttnWaves * ppw);
        if ((long long)batch * n_kv_heads * n_z <= room) return ppw;
    }
    return 16;
}

#define DIFF_SHAPES(DO) \
    if (dim == 32 && dv == 64) DO(1, 4); else if (dim == 32 && dv == 128) DO(1, 8); else if (dim == 64 && dv == 64) DO(2, 4); \
    else if (dim == 64 && dv == 128) DO(2, 8); else if (dim == 128 && dv == 64) DO(4, 4); else DO(4, 8);

// What the prompt kernel needs for the maps' rows: tokens * heads * 2 * dv floats.
LLOGOS_EXPORT long long llogos_diff_attn_prefill_workspace(int tokens, int n_heads, int dv) {
    return tokens > 0 && n_heads > 0 && dv > 0 ? (long long)tokens * n_heads * 2 * dv : 0;
}

// -2: a shape these kernels do not take (the caller uses the kernel for any shape).  Tiles of 128 tokens; one or two
// sets of waves a block (`halves`); n_tiles counts the tiles of all sequences.
LLOGOS_EXPORT int llogos_diff_attn_prefill_bf16(void* out, const void* q, int q_stride, const void* k_pool, const void* v_pool,
                                                const int* table, int table_stride, const int* cu, const int* tok_pos,
                                                int batch, int tokens, int n_tiles, int n_heads, int n_kv_heads, int dim, int dv,
                                                float scale, int window, int sinks, float lambda, float out_scale, float eps,
                                                int halves, float* workspace, long long workspace_floats, hipStream_t stream) {
    if (batch <= 0 || tokens <= 0 || n_tiles <= 0 || window < 0 || sinks < 0 || (halves != 1 && halves != 2)) return LLOGOS_BAD_ARGUMENT;
    if (!diff_shape_ok(n_heads, n_kv_heads, dim, dv) || q_stride % 8) return LLOGOS_UNSUPPORTED;
    if (!workspace || workspace_floats < (long long)tokens * n_heads * 2 * dv) return LLOGOS_TOO_LARGE;
    const int group2 = 2 * (n_heads / n_kv_heads);             // a map is a head of its own
    const long long pairs = (long long)n_tiles * n_kv_heads;
    const dim3 lgrid((unsigned)((pairs + 7) / 8 * 8 * group2));
#define DIRECT(KS, VB, HALVES) do { \
    size_t smem = HALVES * 2 * sizeof(DirectPageLds<32 * KS, 16 * VB>); \
    if (HALVES == 2) smem = std::max(smem, (size_t)kAttnWaves * 2 * (2 + 4 * VB) * kWave * sizeof(float)); \
    hipError_t e = hipFuncSetAttribute((const void*)attn_prefill_direct_kernel<32 * KS, HALVES, 16 * VB, false, 2>, \
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem); \
    if (e != hipSuccess) return (int)e; \
    attn_prefill_direct_kernel<32 * KS, HALVES, 16 * VB, false, 2><<<lgrid, HALVES * kAttnWaves * kWave, smem, stream>>>( \
        (bf16_t*)workspace, (const bf16_t*)q, q_stride, (const bf16_t*)k_pool, (const bf16_t*)v_pool, table, table_stride, \
        cu, tok_pos, batch, n_tiles, 2 * n_heads, n_kv_heads, group2, scale, window, sinks); \
    } while (0)
#define DIRECT1(KS, VB) DIRECT(KS, VB, 1)
#define DIRECT2(KS, VB) DIRECT(KS, VB, 2)
    if (halves == 2) { DIFF_SHAPES(DIRECT2) } else { DIFF_SHAPES(DIRECT1) }
#undef DIRECT2
#undef DIRECT1
#undef DIRECT
    int code = LLOGOS_LAUNCH_CHECK();
    if (code) return code;
    dim3 cgrid(tokens, n_heads);
    if (dv == 64) diff_combine_kernel<4><<<cgrid, 64, 0, stream>>>((bf16_t*)out, workspace, n_heads, lambda, out_scale, eps);
    else          diff_combine_kernel<8><<<cgrid, 128, 0, stream>>>((bf16_t*)out, workspace, n_heads, lambda, out_scale, eps);
    return LLOGOS_LAUNCH_CHECK();
}

LLOGOS_EXPORT long long llogos_diff_attn_decode_workspace(int batch, int n_heads, int n_kv_heads, int dv, int table_width) {
    if (batch <= 0 || n_heads <= 0 || n_kv_heads <= 0 || dv <= 0 || table_width <= 0) return 0;
    const int ppw = diff_pages_per_wave(batch, n_kv_heads, table_width);
    const int n_z = (table_width + kAttnWaves * ppw - 1) / (kAttnWaves * ppw);
    return (long long)batch * n_heads * 2 * n_z * (dv + 2);
}

LLOGOS_EXPORT int llogos_diff_attn_decode_bf16(void* out, const void* q, int q_stride, const void* k_pool, const void* v_pool,
                                               const int* table, int table_stride, int table_width, const int* tok_pos,
                                               int batch, int n_heads, int n_kv_heads, int dim, int dv, float scale, int window,
                                               int sinks, float lambda, float out_scale, float eps, float* workspace,
                                               long long workspace_floats, hipStream_t stream) {
    if (batch <= 0 || table_width <= 0 || window < 0 || sinks < 0) return LLOGOS_BAD_ARGUMENT;
    if (!diff_shape_ok(n_heads, n_kv_heads, dim, dv) || q_stride % 8) return LLOGOS_UNSUPPORTED;
    const int group = n_heads / n_kv_heads;
    const int ppw = diff_pages_per_wave(batch, n_kv_heads, table_width);
    const int n_z = (table_width + kAttnWaves * ppw - 1) / (kAttnWaves * ppw);
    if (!workspace || workspace_floats < (long long)batch * n_heads * 2 * n_z * (dv + 2)) return LLOGOS_TOO_LARGE;
    dim3 grid(batch, n_kv_heads, n_z);
    const size_t lds = (size_t)kAttnWaves * 2 * (group * (dv + 1) + 32) * sizeof(float);
#define DEC(KS, VB) do { \
    if (lds > 48 * 1024) { \
        hipError_t e = hipFuncSetAttribute((const void*)diff_decode_kernel<KS, VB>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds); \
        if (e != hipSuccess) return (int)e; \
    } \
    diff_decode_kernel<KS, VB><<<grid, kAttnWaves * kWave, lds, stream>>>(workspace, (const bf16_t*)q, q_stride, \
        (const bf16_t*)k_pool, (const bf16_t*)v_pool, table, table_stride, tok_pos, n_heads, n_kv_heads, group, scale, window, sinks, ppw); \
    } while (0)
    DIFF_SHAPES(DEC)
#undef DEC
    int code = LLOGOS_LAUNCH_CHECK();
    if (code) return code;
    dim3 mgrid(batch, n_heads);
    if (dv == 64) diff_merge_kernel<4><<<mgrid, 64, 0, stream>>>((bf16_t*)out, workspace, tok_pos, n_heads, n_z, kAttnWaves * ppw, lambda, out_scale, eps);
    else          diff_merge_kernel<8><<<mgrid, 128, 0, stream>>>((bf16_t*)out, workspace, tok_pos, n_heads, n_z, kAttnWaves * ppw, lambda, out_scale, eps);
    return LLOGOS_LAUNCH_CHECK();
}
