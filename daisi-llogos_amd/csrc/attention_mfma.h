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

// Softmax of one page with the score's scale and bend applied first, in place of softmax_page
// (which folds a plain scale into its exponent).  y = bend(s * scale) * log2(e); the tanh is
// 1 - 2 / (exp(2 x) + 1), with the hardware's exp2 and reciprocal.
template <bool MASKED, int VP>
__device__ __forceinline__ void softmax_page_bent(f32x4 (&s)[4], WaveState<VP>& st, float scale, float cap, int q_pos,
                                                  int key0, bf16x8 (&pf)[2], float& corr) {
    const int g = (threadIdx.x & (kWave - 1)) >> 4;
    float y[16];
    if (cap > 0.f) {
        // cap * tanh(x / cap) * log2(e) = a - 2 a / (exp2(s * b) + 1) with a = cap * log2(e), b = 2 scale log2(e) / cap
        const float a = cap * kLog2e, b2 = 2.0f * scale * kLog2e / cap;
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            const float t = __builtin_amdgcn_exp2f(s[i >> 2][i & 3] * b2);
            y[i] = fmaf(-2.0f * a, __builtin_amdgcn_rcpf(t + 1.0f), a);
        }
    } else {
        const float b1 = scale * kLog2e;
#pragma unroll
        for (int i = 0; i < 16; ++i) y[i] = s[i >> 2][i & 3] * b1;
    }
    float tile_max = -INFINITY;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
        if (MASKED) {
            const int key = key0 + g * 16 + i;                 // (i = 4 rb + r: the lane's keys are 16 in a row)
            if (!(q_pos >= 0 && key <= q_pos)) y[i] = -INFINITY;
        }
        tile_max = fmaxf(tile_max, y[i]);
    }
    tile_max = quad_max(tile_max);
    const float m_new = fmaxf(st.m, tile_max);
    const float m_use = (m_new == -INFINITY) ? 0.f : m_new;
    corr = __builtin_amdgcn_exp2f(st.m - m_use);
    float sum = 0.f;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
        y[i] = __builtin_amdgcn_exp2f(y[i] - m_use);
        sum += y[i];
    }
    sum = quad_sum(sum);
    st.l = st.l * corr + sum;
    st.m = m_new;
#pragma unroll
    for (int t = 0; t < 2; ++t) {
        uint4 u;
        u.x = pack_bf16(y[8 * t + 0], y[8 * t + 1]);
        u.y = pack_bf16(y[8 * t + 2], y[8 * t + 3]);
        u.z = pack_bf16(y[8 * t + 4], y[8 * t + 5]);
        u.w = pack_bf16(y[8 * t + 6], y[8 * t + 7]);
        pf[t] = __builtin_bit_cast(bf16x8, u);
    }
}

// What finishes a row: the sink's share of the denominator (exp(sink - max): `sink` points at the head's sink
// score, the maximum is in units of log2) and the head's gate.  Returns the factor on the unnormalised output.
__device__ __forceinline__ float finish_factor(float m, float l, const float* sink, const float* gate_logit) {
    if (sink) l += __builtin_amdgcn_exp2f(*sink * kLog2e - m);
    float f = l > 0.f ? 1.0f / l : 0.f;
    if (gate_logit) f *= 1.0f / (1.0f + expf(-*gate_logit));
    return f;
}

constexpr int kTileRows = 128;

// ---------------------------------------------------------------- prefill, pages shared through LDS
// grid: one block per (tile of 128 tokens over all sequences, head), in the order given in the
// kernel; the 4 waves of a block take 32 rows each (two blocks of 16 columns) and walk the same
// pages: a page is copied to LDS once per block (two buffers, the copy of the next page is in
// flight while the current one is used), and every key and value fragment a wave reads serves
// both of its column blocks.  A page's keys and values go from global memory into LDS without
// passing through registers (16 bytes a lane, a wave's 64 lanes to 1 KB of consecutive LDS),
// which frees the 32 registers of the copy and the time of the stores.  Pages are in fragment
// order in memory, and so they are in LDS: a wave's read of a fragment is 64 x 16 consecutive
// bytes, which LDS serves without a bank conflict; no padding and no swizzle.
template <int HD, int VD = HD>
struct DirectPageLds {
    bf16_t k[HD / 8][512];               // fragment (rb, sk) at rb * (HD / 32) + sk
    bf16_t v[VD / 8][512];               // fragment (db, half) at 2 db + half
};

// HALVES = 2: a block of 8 waves, two sets of 4 with page buffers of their own, takes the same
// 128 rows; the sets take the tile's pages in turn and add their results through LDS at the end.
// One such block fills a compute unit (two waves a SIMD, as two blocks of 4 do), and a tile's
// pages take half as long: with HALVES = 1 a block left alone on its unit goes no faster (one
// wave a SIMD cannot overlap its matrix and its vector instructions), so a prompt of few tiles
// took as long as the pages of its last tile, one after the other.
// VD: the values' width where it is not the keys' (HD); BENT: the scores are scaled and bent through a tanh before
// the softmax (cap > 0), a row may end with a sink in its denominator (head_sink: a score a head) and with a gate on its
// head (gate [tokens, gate_stride] logits), and there is no window.
// MAPS = 2: every head has two score maps over the same values (differential attention).  A map is a head of its own
// here: the caller gives twice the heads and twice the group, head 2 h + m is map m of head h; a kv head's key row
// in its page holds the maps' keys side by side (MAPS * HD values), of which a block copies its own map's; and the
// rows come out as 32-bit floats [tokens][heads][maps][VD] for the kernel that takes the maps' difference.
template <int HD, int HALVES, int VD = HD, bool BENT = false, int MAPS = 1>
__global__ __launch_bounds__(HALVES * kAttnWaves * kWave) __attribute__((amdgpu_waves_per_eu(2, 2)))
void attn_prefill_direct_kernel(
        bf16_t* __restrict__ out, const bf16_t* __restrict__ q, int q_stride,
        const bf16_t* __restrict__ k_pool, const bf16_t* __restrict__ v_pool,
        const int* __restrict__ table, int table_stride, const int* __restrict__ cu,
        const int* __restrict__ tok_pos, int batch, int n_tiles, int n_heads, int n_kv_heads, int group,
        float scale, int window, int sinks, float cap = 0.f, const float* __restrict__ head_sink = nullptr, const float* __restrict__ gate = nullptr,
        int gate_stride = 0) {
    extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
    const int set = HALVES == 2 ? __builtin_amdgcn_readfirstlane(threadIdx.x / (kAttnWaves * kWave)) : 0;
    DirectPageLds<HD, VD>* lds = reinterpret_cast<DirectPageLds<HD, VD>*>(smem_raw) + 2 * set;   // two buffers a set
    // Blocks start in the order of their index, round-robin over the 8 XCDs.  Block L is the
    // m-th block of XCD x (L = 8 m + x); an XCD takes the `group` query heads of one (tile, kv
    // head) pair one after the other, so that the pair's pages stay in its L2, and the pairs go
    // from the last tile to the first: late tiles of a causal prompt see the most keys, and
    // starting with them keeps the compute units evenly busy to the end.
    // A grid of at most two blocks per compute unit starts all at once, and the m-th and the
    // (m + 32)-th block of an XCD share a compute unit: the second half runs in rising order
    // then, so that the longest block shares with the shortest.
    int m_xcd = blockIdx.x / 8;
    const int xcd = blockIdx.x % 8, per_xcd = gridDim.x / 8;
    if (HALVES == 1 && per_xcd > 32 && per_xcd <= 64 && m_xcd >= 32) m_xcd = per_xcd - 1 - (m_xcd - 32);
    const int pair = (m_xcd / group) * 8 + xcd;
    if (pair >= n_tiles * n_kv_heads) return;
    const int kvh = pair % n_kv_heads, h = kvh * group + m_xcd % group;
    int tile = n_tiles - 1 - pair / n_kv_heads, b = 0, first = 0;
    for (; b < batch; ++b) {
        const int len = cu[b + 1] - cu[b];
        const int tiles = (len + kTileRows - 1) / kTileRows;
        if (tile < tiles) { first = cu[b] + tile * kTileRows; break; }
        tile -= tiles;
    }
    if (b >= batch) return;
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave) % kAttnWaves;   // within its set
    const int c = lane & 15, g = lane >> 4;
    const int seq_end = cu[b + 1];
    const int tile_rows = min(kTileRows, seq_end - first);
    const int tile_last_pos = tok_pos[first + tile_rows - 1];
    const int tile_first_pos = tok_pos[first];
    const int written = tok_pos[seq_end - 1] + 1;
    const int row0 = first + 32 * wave;
    const int wave_rows = max(0, min(32, seq_end - row0));
    const bool ok0 = c < wave_rows, ok1 = 16 + c < wave_rows;
    const int q_pos0 = ok0 ? tok_pos[row0 + c] : -1, q_pos1 = ok1 ? tok_pos[row0 + 16 + c] : -1;
    bf16x8 qf0[HD / 32], qf1[HD / 32];
    {
        const bf16_t* qrow0 = q + (size_t)(row0 + (ok0 ? c : 0)) * q_stride + (size_t)h * HD + 8 * g;
        const bf16_t* qrow1 = q + (size_t)(row0 + (ok1 ? 16 + c : 0)) * q_stride + (size_t)h * HD + 8 * g;
#pragma unroll
        for (int sk = 0; sk < HD / 32; ++sk) {
            qf0[sk] = ok0 ? ld_frag(qrow0 + 32 * sk) : zero_frag();
            qf1[sk] = ok1 ? ld_frag(qrow1 + 32 * sk) : zero_frag();
        }
    }
    WaveState<VD> st0, st1;
    st0.init();
    st1.init();
    const int wave_first_pos = wave_rows > 0 ? tok_pos[row0] : 0;
    const int wave_last_pos = wave_rows > 0 ? tok_pos[row0 + wave_rows - 1] : -1;
    const float scale_log2 = scale * kLog2e;

    const int n_pages = tile_last_pos / kPageTokens + 1;
    auto page_needed = [&](int pi) {
        return page_may_be_visible_to_range(tile_first_pos, tile_last_pos, pi * kPageTokens, window, sinks);
    };
    auto next_needed = [&](int pi) {
        ++pi;
        while (pi < n_pages && !page_needed(pi)) ++pi;
        return pi;
    };
    auto page_id = [&](int pi) { return table[(size_t)b * table_stride + pi]; };
    auto page_base = [&](int id) { return ((size_t)id * n_kv_heads + kvh) * kPageTokens; };     // in tokens: times a row's width
    // This wave's share of a page's copy, in instructions of 1 KB (64 lanes x 16 bytes, a fragment):
    // the block's instructions go to its waves in turn.
    auto copy_page = [&](int id, DirectPageLds<HD, VD>& pg) {
        const bf16_t* kpage = k_pool + page_base(id) * (MAPS * HD);
        const bf16_t* vpage = v_pool + page_base(id) * VD;
#pragma unroll
        for (int j = 0; j < (HD / 8 + kAttnWaves - 1) / kAttnWaves; ++j) {
            const int f = kAttnWaves * j + wave;
            if ((HD / 8) % kAttnWaves != 0 && f >= HD / 8) break;        // (the same for a whole wave)
            // fragment (rb, sk) of this map within the row of all maps' keys
            const int src = MAPS == 1 ? f : (f / (HD / 32)) * (MAPS * HD / 32) + (h % MAPS) * (HD / 32) + f % (HD / 32);
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(kpage + 512 * src + 8 * lane),
                                             (__attribute__((address_space(3))) void*)&pg.k[f][0], 16, 0, 0);
        }
#pragma unroll
        for (int j = 0; j < (VD / 8 + kAttnWaves - 1) / kAttnWaves; ++j) {
            const int f = kAttnWaves * j + wave;
            if (f >= VD / 8) break;                                       // (the same for a whole wave)
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(vpage + 512 * f + 8 * lane),
                                             (__attribute__((address_space(3))) void*)&pg.v[f][0], 16, 0, 0);
        }
    };
    // The values of tokens that have not been written may be anything, also NaN, and 0 * NaN is
    // NaN: in the one page of a sequence that is not full they are zeroed in LDS after the copy.
    // Every lane does so with the pieces it copied itself, once they have arrived and before the
    // block's barrier (one barrier a page, whatever the page: the two sets of HALVES = 2 are at
    // different pages and must meet the same barriers).
    auto zero_unwritten = [&](DirectPageLds<HD, VD>& pg, int valid_keys) {
#pragma unroll
        for (int j = 0; j < (VD / 8 + kAttnWaves - 1) / kAttnWaves; ++j) {
            const int f = kAttnWaves * j + wave;
            if (f >= VD / 8) break;
            const int keep = valid_keys - 16 * (lane >> 4) - 8 * (f & 1);          // of the tokens this piece holds
            if (keep >= 8) continue;
            uint4* at = reinterpret_cast<uint4*>(&pg.v[f][8 * lane]);
            *at = __builtin_bit_cast(uint4, keep_first(__builtin_bit_cast(bf16x8, *at), keep));
        }
    };
    auto land = [&](int pi, DirectPageLds<HD, VD>& pg) {                        // the copy of page pi is complete and visible
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        const int valid_keys = written - pi * kPageTokens;
        if (pi < n_pages && valid_keys < kPageTokens) zero_unwritten(pg, valid_keys);
        __syncthreads();
    };
    // The pages that are needed go to the sets in turn.  `lead` is the first set's page: every
    // wave follows it, so that both sets go round the loop, and through its barriers, equally often.
    auto advance = [&](int pi) {
        pi = next_needed(pi);
        return HALVES == 2 ? next_needed(pi) : pi;
    };
    int lead = next_needed(-1);
    if (lead >= n_pages) return;                                         // cannot happen: a row sees itself
    int cur = set ? next_needed(lead) : lead;
    int nxt = advance(cur);
    int nxt_id = nxt < n_pages ? page_id(nxt) : 0;
    if (cur < n_pages) copy_page(page_id(cur), lds[0]);
    land(cur, lds[0]);
    int buf = 0;
    while (lead < n_pages) {
        const int nxt2 = advance(nxt);
        if (nxt < n_pages) copy_page(nxt_id, lds[buf ^ 1]);
        const int nxt2_id = nxt2 < n_pages ? page_id(nxt2) : 0;
        do {
        const int key0 = cur * kPageTokens;
        if (cur >= n_pages) break;                                        // the second set, after an odd number of pages
        if (wave_rows <= 0 || key0 > wave_last_pos) break;                // nothing of this page for this wave
        if (!page_may_be_visible_to_range(wave_first_pos, wave_last_pos, key0, window, sinks)) break;
        const DirectPageLds<HD, VD>& pg = lds[buf];
        f32x4 s0[4], s1[4];
#pragma unroll
        for (int rb = 0; rb < 4; ++rb) {
            s0[rb] = f32x4{0.f, 0.f, 0.f, 0.f};
            s1[rb] = f32x4{0.f, 0.f, 0.f, 0.f};
        }
#pragma unroll
        for (int sk = 0; sk < HD / 32; ++sk) {
#pragma unroll
            for (int rb = 0; rb < 4; ++rb) {
                const bf16x8 kf = __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(
                    &pg.k[rb * (HD / 32) + sk][8 * lane]));
                s0[rb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf, qf0[sk], s0[rb], 0, 0, 0);
                s1[rb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf, qf1[sk], s1[rb], 0, 0, 0);
            }
        }
        auto read_v = [&](int db, int t) {
            return __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(&pg.v[2 * db + t][8 * lane]));
        };
        constexpr int kEarly = 2;
        bf16x8 vf[VD / 16][2];
#pragma unroll
        for (int db = 0; db < kEarly; ++db) { vf[db][0] = read_v(db, 0); vf[db][1] = read_v(db, 1); }
        bf16x8 pf0[2], pf1[2];
        float corr0, corr1;
        const bool all_visible = wave_rows == 32 &&
                                 page_fully_visible(wave_first_pos, wave_last_pos, key0, window, sinks);
        if (BENT) {
            if (all_visible) {
                softmax_page_bent<false, VD>(s0, st0, scale, cap, q_pos0, key0, pf0, corr0);
                softmax_page_bent<false, VD>(s1, st1, scale, cap, q_pos1, key0, pf1, corr1);
            } else {
                softmax_page_bent<true, VD>(s0, st0, scale, cap, q_pos0, key0, pf0, corr0);
                softmax_page_bent<true, VD>(s1, st1, scale, cap, q_pos1, key0, pf1, corr1);
            }
        } else if (all_visible) {
            softmax_page<false, 16, 4, VD>(s0, st0, scale_log2, q_pos0, key0, window, sinks, pf0, corr0);
            softmax_page<false, 16, 4, VD>(s1, st1, scale_log2, q_pos1, key0, window, sinks, pf1, corr1);
        } else {
            softmax_page<true, 16, 4, VD>(s0, st0, scale_log2, q_pos0, key0, window, sinks, pf0, corr0);
            softmax_page<true, 16, 4, VD>(s1, st1, scale_log2, q_pos1, key0, window, sinks, pf1, corr1);
        }
        const bool rescale = __ballot(corr0 != 1.0f || corr1 != 1.0f) != 0;
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int db = 0; db < VD / 16; ++db) {
            if (db + kEarly < VD / 16) {
                vf[db + kEarly][0] = read_v(db + kEarly, 0);
                vf[db + kEarly][1] = read_v(db + kEarly, 1);
            }
            f32x4 a0 = st0.acc[db], a1 = st1.acc[db];
            if (rescale) {
#pragma unroll
                for (int r = 0; r < 4; ++r) { a0[r] *= corr0; a1[r] *= corr1; }
            }
#pragma unroll
            for (int t = 0; t < 2; ++t) {
                a0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf[db][t], pf0[t], a0, 0, 0, 0);
                a1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf[db][t], pf1[t], a1, 0, 0, 0);
            }
            st0.acc[db] = a0;
            st1.acc[db] = a1;
        }
        } while (0);
        land(nxt, lds[buf ^ 1]);
        cur = nxt;
        nxt = nxt2;
        nxt_id = nxt2_id;
        buf ^= 1;
        lead = advance(lead);
    }
    if (HALVES == 2) {
        // The second set's running maxima, sums and outputs go through LDS (lane by lane: the two
        // sets hold the same rows in the same lanes) and are added to the first set's.  The loop's
        // last barrier came after the last read of a page.
        constexpr int kStateFloats = 2 + VD / 4;
        float* state = reinterpret_cast<float*>(smem_raw) + (size_t)wave * (2 * kStateFloats * kWave) + lane;
        auto put = [&](const WaveState<VD>& st, float* at) {
            at[0] = st.m;
            at[kWave] = st.l;
#pragma unroll
            for (int db = 0; db < VD / 16; ++db)
#pragma unroll
                for (int r = 0; r < 4; ++r) at[(2 + 4 * db + r) * kWave] = st.acc[db][r];
        };
        auto add = [&](WaveState<VD>& st, const float* at) {
            const float m_other = at[0], l_other = at[kWave];
            const float m = fmaxf(st.m, m_other);
            const float mine = st.m == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(st.m - m);
            const float theirs = m_other == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(m_other - m);
            st.l = st.l * mine + l_other * theirs;
            st.m = m;
#pragma unroll
            for (int db = 0; db < VD / 16; ++db)
#pragma unroll
                for (int r = 0; r < 4; ++r) st.acc[db][r] = st.acc[db][r] * mine + at[(2 + 4 * db + r) * kWave] * theirs;
        };
        if (set == 1) {
            put(st0, state);
            put(st1, state + kStateFloats * kWave);
        }
        __syncthreads();
        if (set == 1) return;
        add(st0, state);
        add(st1, state + kStateFloats * kWave);
    }
    auto write_out = [&](const WaveState<VD>& st, int rr) {
        if (rr >= wave_rows) return;
        const float inv = BENT ? finish_factor(st.m, st.l, head_sink ? head_sink + h : nullptr, gate ? gate + (size_t)(row0 + rr) * gate_stride + h : nullptr)
                               : (st.l > 0.f ? 1.0f / st.l : 0.f);
        if (MAPS > 1) {
            float* frow = reinterpret_cast<float*>(out) + ((size_t)(row0 + rr) * n_heads + h) * VD;
#pragma unroll
            for (int db = 0; db < VD / 16; ++db)
                *reinterpret_cast<f32x4*>(frow + 16 * db + 4 * g) = f32x4{st.acc[db][0] * inv, st.acc[db][1] * inv,
                                                                          st.acc[db][2] * inv, st.acc[db][3] * inv};
            return;
        }
        bf16_t* orow = out + ((size_t)(row0 + rr) * n_heads + h) * VD;
#pragma unroll
        for (int db = 0; db < VD / 16; ++db) {
            uint2 u;
            u.x = pack_bf16(st.acc[db][0] * inv, st.acc[db][1] * inv);
            u.y = pack_bf16(st.acc[db][2] * inv, st.acc[db][3] * inv);
            *reinterpret_cast<uint2*>(orow + 16 * db + 4 * g) = u;
        }
    };
    write_out(st0, c);
    write_out(st1, 16 + c);
}

