// bfloat16 attention on the matrix cores for heads whose keys and values have different widths,
// whose scores may be bent through a tanh (s -> cap * tanh(s / cap)), whose softmax may carry a
// sink (a score a head without a key or a value: exp(sink) joins the denominator) and whose output may be gated head by head
// (sigmoid of a logit a token and head).  No window: a query sees every key up to its own.
//
// Keys are rows of KP = 32 KS dimensions in their pages, values rows of VP = 16 VB; the pages are
// in the matrix cores' operand order (common.h), so the page steps of attention_mfma.h serve:
// one wave works on 16 columns and one page of 64 keys at a time.
//   prefill: the columns are 16 consecutive tokens of a sequence for one query head; a block of 4
//            waves takes a tile of 64 tokens; every wave walks the pages up to its last row.
//   decode:  the columns are the query heads of one kv head; a block of 4 waves takes a run of
//            pages of one (sequence, kv head), each wave every fourth of them; the waves' results
//            are merged through LDS, and blocks along the context leave partial results
//            (max, sum, output) for a small merge kernel.
// The sink and the gate are applied where a row is finished (a block's own write, or the merge).
#include "attention_mfma.h"
#include <algorithm>

template <int KP, int VP>
__device__ __forceinline__ void attend_page_kv(WaveState<VP>& st, const bf16x8 (&qf)[KP / 32], const bf16_t* __restrict__ kpage,
                                               const bf16_t* __restrict__ vpage, int q_pos, int key0, int valid_keys,
                                               bool all_visible, float scale, float cap) {
    bf16x8 kf[4][KP / 32], vf[VP / 16][2];
    load_keys<KP>(kf, kpage);
    load_values<VP>(vf, vpage);
    f32x4 s[4];
    page_scores<KP>(s, kf, qf);
    bf16x8 pf[2];
    float corr;
    if (all_visible) softmax_page_bent<false, VP>(s, st, scale, cap, q_pos, key0, pf, corr);
    else             softmax_page_bent<true, VP>(s, st, scale, cap, q_pos, key0, pf, corr);
    weigh_values<VP>(st, vf, pf, corr, valid_keys);
}

// Fragment loads that may stay in the caches: a prompt's four waves of a block, and the blocks of the other
// heads of a kv head, ask for the same pages at about the same time.
template <int KP>
__device__ __forceinline__ void load_keys_kept(bf16x8 (&kf)[4][KP / 32], const bf16_t* __restrict__ kpage) {
    const bf16_t* mine = kpage + 8 * (threadIdx.x & (kWave - 1));
#pragma unroll
    for (int rb = 0; rb < 4; ++rb)
#pragma unroll
        for (int sk = 0; sk < KP / 32; ++sk) kf[rb][sk] = ld_frag(mine + 512 * (rb * (KP / 32) + sk));
}

template <int VP>
__device__ __forceinline__ void load_values_kept(bf16x8 (&vf)[VP / 16][2], const bf16_t* __restrict__ vpage) {
    const bf16_t* mine = vpage + 8 * (threadIdx.x & (kWave - 1));
#pragma unroll
    for (int db = 0; db < VP / 16; ++db) {
        vf[db][0] = ld_frag(mine + 512 * (2 * db));
        vf[db][1] = ld_frag(mine + 512 * (2 * db + 1));
    }
}

// ---------------------------------------------------------------- prefill
// grid (tiles of 64 tokens over all sequences, heads); wave w takes rows 16 w .. 16 w + 15 of the tile.
template <int KS, int VB>
__global__ __launch_bounds__(kAttnWaves * kWave) __attribute__((amdgpu_waves_per_eu(2, 2))) void capped_prefill_kernel(
        bf16_t* __restrict__ out, const bf16_t* __restrict__ q, int q_stride, const bf16_t* __restrict__ k_pool,
        const bf16_t* __restrict__ v_pool, const int* __restrict__ table, int table_stride, const int* __restrict__ cu,
        const int* __restrict__ tok_pos, int batch, int n_heads, int n_kv_heads, int group, float scale, float cap,
        const float* __restrict__ head_sink, const float* __restrict__ gate, int gate_stride) {
    constexpr int KP = 32 * KS, VP = 16 * VB;
    int tile = blockIdx.x, b = 0, first = 0;
    for (; b < batch; ++b) {
        const int tiles = (cu[b + 1] - cu[b] + 63) / 64;
        if (tile < tiles) { first = cu[b] + tile * 64; break; }
        tile -= tiles;
    }
    if (b >= batch) return;
    const int h = blockIdx.y, kvh = h / group;
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    const int c = lane & 15, g = lane >> 4;
    const int row0 = first + 16 * wave;
    const int seq_end = cu[b + 1];
    if (row0 >= seq_end) return;
    const int rows = min(16, seq_end - row0);
    const bool col_ok = c < rows;
    const int my_row = row0 + (col_ok ? c : 0);
    const int q_pos = col_ok ? tok_pos[my_row] : -1;
    const int last_pos = tok_pos[row0 + rows - 1];
    const int first_pos = tok_pos[row0];
    const int written = tok_pos[seq_end - 1] + 1;

    bf16x8 qf[KS];
    const bf16_t* qrow = q + (size_t)my_row * q_stride + (size_t)h * KP + 8 * g;
#pragma unroll
    for (int sk = 0; sk < KS; ++sk) qf[sk] = col_ok ? ld_frag(qrow + 32 * sk) : zero_frag();

    WaveState<VP> st;
    st.init();
    const int n_pages = last_pos / kPageTokens + 1;
    // The next page's keys are asked for as soon as this page's scores are taken (their registers are free then),
    // behind this page's values: the softmax and the second product cover their way.
    auto page_of = [&](int pi) { return ((size_t)table[(size_t)b * table_stride + pi] * n_kv_heads + kvh) * kPageTokens; };
    bf16x8 kf[4][KS];
    size_t page = page_of(0);
    load_keys_kept<KP>(kf, k_pool + page * KP);
    for (int pi = 0; pi < n_pages; ++pi) {
        const int key0 = pi * kPageTokens;
        f32x4 s[4];
        page_scores<KP>(s, kf, qf);
        bf16x8 vf[VB][2];
        load_values_kept<VP>(vf, v_pool + page * VP);
        if (pi + 1 < n_pages) {
            page = page_of(pi + 1);
            load_keys_kept<KP>(kf, k_pool + page * KP);
        }
        bf16x8 pf[2];
        float corr;
        if (rows == 16 && key0 + kPageTokens - 1 <= first_pos) softmax_page_bent<false, VP>(s, st, scale, cap, q_pos, key0, pf, corr);
        else                                                   softmax_page_bent<true, VP>(s, st, scale, cap, q_pos, key0, pf, corr);
        weigh_values<VP>(st, vf, pf, corr, min(kPageTokens, written - key0));
    }
    if (!col_ok) return;
    const float f = finish_factor(st.m, st.l, head_sink ? head_sink + h : nullptr, gate ? gate + (size_t)my_row * gate_stride + h : nullptr);
    bf16_t* orow = out + ((size_t)my_row * n_heads + h) * VP;
#pragma unroll
    for (int db = 0; db < VB; ++db) {
        uint2 u;
        u.x = pack_bf16(st.acc[db][0] * f, st.acc[db][1] * f);
        u.y = pack_bf16(st.acc[db][2] * f, st.acc[db][3] * f);
        *reinterpret_cast<uint2*>(orow + 16 * db + 4 * g) = u;
    }
}

// ---------------------------------------------------------------- decode
// grid (batch, kv heads, blocks along the context); wave w of a block takes pages first + w, first + w + 4, ...
// (ppw of them).  One block along the context: the block writes the output; else partial
// [batch][heads][grid.z][VP + 2] floats (max, sum, unnormalised output).  LDS: 4 * (group * (VP + 1) + 32) floats.
template <int KS, int VB>
__global__ __launch_bounds__(kAttnWaves * kWave) void capped_decode_kernel(
        bf16_t* __restrict__ out, float* __restrict__ partial, const bf16_t* __restrict__ q, int q_stride,
        const bf16_t* __restrict__ k_pool, const bf16_t* __restrict__ v_pool, const int* __restrict__ table, int table_stride,
        const int* __restrict__ tok_pos, int n_heads, int n_kv_heads, int group, float scale, float cap, int ppw,
        const float* __restrict__ head_sink, const float* __restrict__ gate, int gate_stride) {
    constexpr int KP = 32 * KS, VP = 16 * VB, WAVES = kAttnWaves;
    extern __shared__ float lds[];
    float* lds_m = lds;
    float* lds_l = lds + WAVES * 16;
    float* lds_o = lds + WAVES * 32;                      // [WAVES][group][VP + 1]
    const int b = blockIdx.x, kvh = blockIdx.y, z = blockIdx.z;
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    const int c = lane & 15, g = lane >> 4;
    const int pos = tok_pos[b];
    const int n_pages = pos / kPageTokens + 1;
    const int first_page = z * WAVES * ppw;
    if (first_page >= n_pages) return;
    const int* row = table + (size_t)b * table_stride;

    WaveState<VP> st;
    st.init();
    const bool col_ok = c < group;
    bf16x8 qf[KS];
    const bf16_t* qrow = q + (size_t)b * q_stride + (size_t)(kvh * group + (col_ok ? c : 0)) * KP + 8 * g;
#pragma unroll
    for (int sk = 0; sk < KS; ++sk) qf[sk] = col_ok ? ld_frag(qrow + 32 * sk) : zero_frag();
    for (int j = 0; j < ppw; ++j) {
        const int pi = first_page + wave + WAVES * j;
        if (pi >= n_pages) break;
        const int key0 = pi * kPageTokens;
        const size_t page = ((size_t)row[pi] * n_kv_heads + kvh) * kPageTokens;
        attend_page_kv<KP, VP>(st, qf, k_pool + page * KP, v_pool + page * VP, col_ok ? pos : -1, key0,
                               min(kPageTokens, pos - key0 + 1), key0 + kPageTokens - 1 <= pos, scale, cap);
    }
    if (g == 0) { lds_m[wave * 16 + c] = st.m; lds_l[wave * 16 + c] = st.l; }
    if (col_ok) {
        float* dst = lds_o + ((size_t)wave * group + c) * (VP + 1);
#pragma unroll
        for (int db = 0; db < VB; ++db)
#pragma unroll
            for (int r = 0; r < 4; ++r) dst[16 * db + 4 * g + r] = st.acc[db][r];
    }
    __syncthreads();
    const int n_z = gridDim.z;
    for (int idx = threadIdx.x; idx < group * VP; idx += blockDim.x) {
        const int col = idx / VP, d = idx % VP;
        float m = -INFINITY;
#pragma unroll
        for (int w = 0; w < WAVES; ++w) m = fmaxf(m, lds_m[w * 16 + col]);
        float l = 0.f, o = 0.f;
#pragma unroll
        for (int w = 0; w < WAVES; ++w) {
            const float mw = lds_m[w * 16 + col];
            const float f = (mw == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f(mw - m);
            l += lds_l[w * 16 + col] * f;
            o += lds_o[((size_t)w * group + col) * (VP + 1) + d] * f;
        }
        const int head = kvh * group + col;
        if (n_z == 1) {
            const float f = finish_factor(m, l, head_sink ? head_sink + head : nullptr, gate ? gate + (size_t)b * gate_stride + head : nullptr);
            out[((size_t)b * n_heads + head) * VP + d] = f32_to_bf16(o * f);
        } else {
            float* dst = partial + (((size_t)b * n_heads + head) * n_z + z) * (VP + 2);
            dst[2 + d] = o;
            if (d == 0) { dst[0] = m; dst[1] = l; }
        }
    }
}

// grid (batch, heads), VP threads: thread d adds dimension d of the blocks' partial results in ascending order.
template <int VB>
__global__ __launch_bounds__(16 * VB) void capped_merge_kernel(bf16_t* __restrict__ out, const float* __restrict__ partial,
                                                               const int* __restrict__ tok_pos, int n_heads, int n_z,
                                                               int pages_per_block, const float* __restrict__ head_sink,
                                                               const float* __restrict__ gate, int gate_stride) {
    constexpr int VP = 16 * VB;
    const int b = blockIdx.x, h = blockIdx.y, d = threadIdx.x;
    const int n_pages = tok_pos[b] / kPageTokens + 1;
    const int used = min(n_z, (n_pages + pages_per_block - 1) / pages_per_block);
    const float* src = partial + ((size_t)b * n_heads + h) * n_z * (VP + 2);
    float m = -INFINITY;
    for (int z = 0; z < used; ++z) m = fmaxf(m, src[(size_t)z * (VP + 2)]);
    float l = 0.f, o = 0.f;
    for (int z = 0; z < used; ++z) {
        const float* p = src + (size_t)z * (VP + 2);
        const float f = (p[0] == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f(p[0] - m);
        l += p[1] * f;
        o += p[2 + d] * f;
    }
    const float f = finish_factor(m, l, head_sink ? head_sink + h : nullptr, gate ? gate + (size_t)b * gate_stride + h : nullptr);
    out[((size_t)b * n_heads + h) * VP + d] = f32_to_bf16(o * f);
}

// ---------------------------------------------------------------- entry points
static int capped_units() {
    static int units = 0;
    if (units == 0) {
        int dev = 0;
        hipDeviceProp_t prop;
        if (hipGetDevice(&dev) == hipSuccess && hipGetDeviceProperties(&prop, dev) == hipSuccess) units = prop.multiProcessorCount;
        if (units <= 0) units = 256;
    }
    return units;
}

static bool capped_shape_ok(int n_heads, int n_kv_heads, int dk, int dv) {
    if (n_heads <= 0 || n_kv_heads <= 0 || n_heads % n_kv_heads || n_heads / n_kv_heads > 16) return false;
    const bool k_ok = dk == 64 || dk == 96 || dk == 128;
    const bool v_ok = dv == 64 || dv == 80 || dv == 96 || dv == 128;
    return k_ok && v_ok;
}

// pages a wave takes in a decode step: as few as leave no more than two blocks a compute unit
static int capped_pages_per_wave(int batch, int n_kv_heads, int table_width) {
    const int room = 2 * capped_units();
    for (int ppw = 1; ppw < 16; ++ppw) {
        const int n_z = (table_width + kAttnWaves * ppw - 1) / (kAttnWaves * ppw);
        if ((long long)batch * n_kv_heads * n_z <= room) return ppw;
    }
    return 16;
}

#define CAPPED_SHAPES(DO) \
    if (dk == 64 && dv == 64) DO(2, 4); else if (dk == 64 && dv == 80) DO(2, 5); else if (dk == 64 && dv == 96) DO(2, 6); \
    else if (dk == 64 && dv == 128) DO(2, 8); else if (dk == 96 && dv == 64) DO(3, 4); else if (dk == 96 && dv == 80) DO(3, 5); \
    else if (dk == 96 && dv == 96) DO(3, 6); else if (dk == 96 && dv == 128) DO(3, 8); else if (dk == 128 && dv == 64) DO(4, 4); \
    else if (dk == 128 && dv == 80) DO(4, 5); else if (dk == 128 && dv == 96) DO(4, 6); else DO(4, 8);

// -2: a shape these kernels do not take (the caller uses the kernel for any shape).  tile_rows 64: the simple form;
// 128: pages shared through LDS, with one or two sets of waves (`halves`); n_tiles counts tiles of that many rows.
LLOGOS_EXPORT int llogos_capped_attn_prefill_bf16(void* out, const void* q, int q_stride, const void* k_pool, const void* v_pool,
                                                  const int* table, int table_stride, const int* cu, const int* tok_pos,
                                                  int batch, int n_tiles, int n_heads, int n_kv_heads, int dk, int dv, float scale,
                                                  float softcap, const float* head_sink, const float* gate, int gate_stride,
                                                  int tile_rows, int halves, hipStream_t stream) {
    if (batch <= 0 || n_tiles <= 0 || softcap < 0.f || (gate && gate_stride < n_heads)) return LLOGOS_BAD_ARGUMENT;
    if ((tile_rows != 64 && tile_rows != kTileRows) || (halves != 1 && halves != 2)) return LLOGOS_BAD_ARGUMENT;
    if (!capped_shape_ok(n_heads, n_kv_heads, dk, dv) || q_stride % 8) return LLOGOS_UNSUPPORTED;
    dim3 grid(n_tiles, n_heads);
    const int group = n_heads / n_kv_heads;
    if (tile_rows == kTileRows) {
        // tiles of 128 tokens whose pages go straight into LDS, once for a block's waves (attention_mfma.h)
        const long long pairs = (long long)n_tiles * n_kv_heads;
        const dim3 lgrid((unsigned)((pairs + 7) / 8 * 8 * group));
#define DIRECT(KS, VB, HALVES) do { \
        size_t smem = HALVES * 2 * sizeof(DirectPageLds<32 * KS, 16 * VB>); \
        if (HALVES == 2) smem = std::max(smem, (size_t)kAttnWaves * 2 * (2 + 4 * VB) * kWave * sizeof(float)); \
        hipError_t e = hipFuncSetAttribute((const void*)attn_prefill_direct_kernel<32 * KS, HALVES, 16 * VB, true>, \
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem); \
        if (e != hipSuccess) return (int)e; \
        attn_prefill_direct_kernel<32 * KS, HALVES, 16 * VB, true><<<lgrid, HALVES * kAttnWaves * kWave, smem, stream>>>( \
            (bf16_t*)out, (const bf16_t*)q, q_stride, (const bf16_t*)k_pool, (const bf16_t*)v_pool, table, table_stride, \
            cu, tok_pos, batch, n_tiles, n_heads, n_kv_heads, group, scale, 0, 0, softcap, head_sink, gate, gate_stride); \
        return LLOGOS_LAUNCH_CHECK(); } while (0)
#define DIRECT1(KS, VB) DIRECT(KS, VB, 1)
#define DIRECT2(KS, VB) DIRECT(KS, VB, 2)
        if (halves == 2) { CAPPED_SHAPES(DIRECT2) } else { CAPPED_SHAPES(DIRECT1) }
#undef DIRECT2
#undef DIRECT1
#undef DIRECT
    }
#define PRE(KS, VB) capped_prefill_kernel<KS, VB><<<grid, kAttnWaves * kWave, 0, stream>>>((bf16_t*)out, (const bf16_t*)q, q_stride, \
        (const bf16_t*)k_pool, (const bf16_t*)v_pool, table, table_stride, cu, tok_pos, batch, n_heads, n_kv_heads, group, scale, \
        softcap, head_sink, gate, gate_stride)
    CAPPED_SHAPES(PRE)
#undef PRE
    return LLOGOS_LAUNCH_CHECK();
}

LLOGOS_EXPORT long long llogos_capped_attn_decode_workspace(int batch, int n_heads, int n_kv_heads, int dv, int table_width) {
    if (batch <= 0 || n_heads <= 0 || n_kv_heads <= 0 || dv <= 0 || table_width <= 0) return 0;
    const int ppw = capped_pages_per_wave(batch, n_kv_heads, table_width);
    const int n_z = (table_width + kAttnWaves * ppw - 1) / (kAttnWaves * ppw);
    return n_z > 1 ? (long long)batch * n_heads * n_z * (dv + 2) : 0;
}

LLOGOS_EXPORT int llogos_capped_attn_decode_bf16(void* out, const void* q, int q_stride, const void* k_pool, const void* v_pool,
                                                 const int* table, int table_stride, int table_width, const int* tok_pos,
                                                 int batch, int n_heads, int n_kv_heads, int dk, int dv, float scale,
                                                 float softcap, const float* head_sink, const float* gate, int gate_stride,
                                                 float* workspace, long long workspace_floats, hipStream_t stream) {
    if (batch <= 0 || table_width <= 0 || softcap < 0.f || (gate && gate_stride < n_heads)) return LLOGOS_BAD_ARGUMENT;
    if (!capped_shape_ok(n_heads, n_kv_heads, dk, dv) || q_stride % 8) return LLOGOS_UNSUPPORTED;
    const int group = n_heads / n_kv_heads;
    const int ppw = capped_pages_per_wave(batch, n_kv_heads, table_width);
    const int n_z = (table_width + kAttnWaves * ppw - 1) / (kAttnWaves * ppw);
    if (n_z > 1 && (!workspace || workspace_floats < (long long)batch * n_heads * n_z * (dv + 2))) return LLOGOS_TOO_LARGE;
    dim3 grid(batch, n_kv_heads, n_z);
    const size_t lds = (size_t)kAttnWaves * (group * (dv + 1) + 32) * sizeof(float);
#define DEC(KS, VB) capped_decode_kernel<KS, VB><<<grid, kAttnWaves * kWave, lds, stream>>>((bf16_t*)out, workspace, (const bf16_t*)q, \
        q_stride, (const bf16_t*)k_pool, (const bf16_t*)v_pool, table, table_stride, tok_pos, n_heads, n_kv_heads, group, scale, \
        softcap, ppw, head_sink, gate, gate_stride)
    CAPPED_SHAPES(DEC)
#undef DEC
    if (n_z > 1) {
        dim3 mgrid(batch, n_heads);
#define MRG(VB) capped_merge_kernel<VB><<<mgrid, 16 * VB, 0, stream>>>((bf16_t*)out, workspace, tok_pos, n_heads, n_z, kAttnWaves * ppw, \
        head_sink, gate, gate_stride)
        if (dv == 64) MRG(4); else if (dv == 80) MRG(5); else if (dv == 96) MRG(6); else MRG(8);
#undef MRG
    }
    return LLOGOS_LAUNCH_CHECK();
}
