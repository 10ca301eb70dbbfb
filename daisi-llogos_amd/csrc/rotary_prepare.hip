// From the projected rows [q units | k units | v heads] of a step to what an attention kernel reads:
// rotated queries in a row of their own, rotated keys and plain values in their cache pages.
//
// A *unit* is a run of `dim` values that is normed and rotated by itself: a head, or one of the `maps`
// score maps of a head (heads laid out one after the other, each [map 0 | map 1 | ...]).  Per q and k unit:
//   - optionally an RMS norm over the unit with a weight [dim] shared by all units (before the rotation);
//   - rotation of the first `rot` dimensions with the step's (cos, sin) table, pairing 0: (i, i + rot / 2),
//     1: (2i, 2i + 1);
//   - optionally (unit_after) division by the unit's root mean square, without a weight (after the rotation).
// A kv head's key row in its page is its `maps` units side by side (k_page_dim >= maps * dim values); a value
// row has v_dim values in pages of v_page_dim.  All arithmetic in 32-bit; 16, 32 or 64 lanes of a wave a (token, unit).
#include "common.h"

constexpr int kPrepUnitsPerBlock = 4;
constexpr int kPrepMaxDim = 1024;

template <typename TI>
__device__ __forceinline__ float rp_sum_parts(const TI* p, size_t i, int parts, size_t part_stride) {
    float v = load_f32(p + i);
    for (int q0 = 1; q0 < parts; q0 += 8) {          // eight loads in flight, added in ascending order
        float y[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) y[j] = q0 + j < parts ? load_f32(p + (size_t)(q0 + j) * part_stride + i) : 0.f;
#pragma unroll
        for (int j = 0; j < 8; ++j)
            if (q0 + j < parts) v += y[j];
    }
    return v;
}

// L lanes of a wave take a unit (a wave takes 64 / L units side by side: a unit of 64 values is a quarter of a
// wave's worth of work); R: values a lane holds of a unit (dim <= L R).
template <int L>
__device__ __forceinline__ float group_sum(float v) {
#pragma unroll
    for (int o = L / 2; o > 0; o >>= 1) v += __shfl_xor(v, o, kWave);
    return v;
}

template <typename TI, typename T, int R, int L>
__global__ void rotary_prepare_kernel(const TI* __restrict__ qkv, int parts, size_t part_stride, int row_stride,
                                      const float* __restrict__ bias, T* __restrict__ q_out, int n_q, int n_k, int n_v,
                                      int dim, int v_dim, int maps, int rot, int pairing,
                                      const float* __restrict__ q_norm_w, const float* __restrict__ k_norm_w, int unit_after,
                                      float eps, const float2* __restrict__ cs, T* __restrict__ k_pool, T* __restrict__ v_pool,
                                      PagedKV cache, int v_page_dim, const int* __restrict__ tok_seq,
                                      const int* __restrict__ tok_pos, int lds_row) {
    extern __shared__ float smem[];
    constexpr int kPerWave = kWave / L;
    const int t = blockIdx.x;
    const int sub = threadIdx.x / L, lane = threadIdx.x % L;
    const int unit = (blockIdx.y * kPrepUnitsPerBlock + threadIdx.y) * kPerWave + sub;
    const bool active = unit < n_q + n_k + n_v;
    float* buf = smem + (threadIdx.y * kPerWave + sub) * lds_row;
    const bool is_q = unit < n_q;
    const bool is_k = !is_q && unit < n_q + n_k;
    const int width = (is_q || is_k) ? dim : v_dim;
    const size_t col0 = !active ? 0 : (is_q ? (size_t)unit * dim
                                            : (is_k ? (size_t)n_q * dim + (size_t)(unit - n_q) * dim
                                                    : (size_t)(n_q + n_k) * dim + (size_t)(unit - n_q - n_k) * v_dim));
    const TI* src = qkv + (size_t)t * row_stride + col0;
    const float* norm_w = is_q ? q_norm_w : (is_k ? k_norm_w : nullptr);
    const int pos = tok_pos[t], in_page = pos % kPageTokens;

    float ss = 0.f;
    if (active) {
        for (int d = lane; d < width; d += L) {
            float v = rp_sum_parts(src, (size_t)d, parts, part_stride);
            if (bias) v += bias[col0 + d];
            buf[d] = v;
            ss += v * v;
        }
    }
    __syncthreads();
    ss = group_sum<L>(ss);                                   // (every lane of the wave takes part, whatever its unit)
    if (active && norm_w) {
        const float inv = 1.0f / sqrtf(ss / (float)dim + eps);
        for (int d = lane; d < dim; d += L) buf[d] = buf[d] * inv * norm_w[d];
    }
    __syncthreads();
    if (active && !is_q && !is_k) {
        const int vh = unit - n_q - n_k;
        T* vdst = v_pool + paged_base(cache, tok_seq[t], vh, pos) / cache.head_dim * v_page_dim;
        for (int d = lane; d < v_dim; d += L) store_f32(vdst + page_value_offset(in_page, d), buf[d]);
    }
    const bool turns = active && (is_q || is_k);
    const int half = rot / 2;
    const float2* c = cs + (size_t)t * half;
    // a lane's rotated values: dimensions lane, lane + L, ... (both partners are read before either is stored)
    float mine[R];
    float s2 = 0.f;
#pragma unroll
    for (int r = 0; r < R; ++r) {
        const int d = lane + r * L;
        float v = 0.f;
        if (turns && d < dim) {
            v = buf[d];
            if (d < rot) {
                if (pairing == 0) {
                    if (d < half) v = buf[d] * c[d].x - buf[d + half] * c[d].y;
                    else          v = buf[d] * c[d - half].x + buf[d - half] * c[d - half].y;
                } else {
                    const int i = d >> 1;
                    if ((d & 1) == 0) v = buf[d] * c[i].x - buf[d + 1] * c[i].y;
                    else              v = buf[d] * c[i].x + buf[d - 1] * c[i].y;
                }
            }
        }
        mine[r] = v;
        s2 += v * v;
    }
    float after = 1.f;
    if (unit_after) after = 1.0f / sqrtf(group_sum<L>(s2) / (float)dim + eps);
    if (!turns) return;
    if (is_q) {
        T* dst = q_out + ((size_t)t * n_q + unit) * dim;
#pragma unroll
        for (int r = 0; r < R; ++r) {
            const int d = lane + r * L;
            if (d < dim) store_f32(dst + d, mine[r] * after);
        }
    } else {
        const int ku = unit - n_q;
        T* dst = k_pool + paged_base(cache, tok_seq[t], ku / maps, pos);
        const int col = (ku % maps) * dim;
#pragma unroll
        for (int r = 0; r < R; ++r) {
            const int d = lane + r * L;
            if (d < dim) store_f32(dst + page_key_offset(in_page, col + d, cache.head_dim), mine[r] * after);
        }
    }
}

// qkv: [parts][T][row_stride] float32 or the cache's type (parts are summed, then `bias` added).  n_q query units,
// n_kv kv heads of `maps` key units and one value row each; n_kv = 0: only the queries are made.
LLOGOS_EXPORT int llogos_rotary_prepare(const void* qkv, int in_dtype, int parts, long long part_stride, int row_stride,
                                        const float* bias, void* q_out, int dtype, int n_q, int n_kv, int dim, int v_dim, int maps,
                                        int rot, int pairing, const float* q_norm_w, const float* k_norm_w, int unit_after,
                                        float eps, const void* cs, void* k_pool, void* v_pool, int k_page_dim, int v_page_dim,
                                        const int* table, int table_stride, const int* tok_seq, const int* tok_pos, int T,
                                        hipStream_t stream) {
    if (T <= 0 || n_q <= 0 || n_kv < 0 || dim <= 0 || dim > kPrepMaxDim || v_dim < 0 || v_dim > kPrepMaxDim || maps < 1) return LLOGOS_BAD_ARGUMENT;
    if (rot < 0 || rot > dim || (rot & 1) || parts < 1 || (rot > 0 && !cs)) return LLOGOS_BAD_ARGUMENT;
    if (n_kv > 0 && (!k_pool || !v_pool || !table || v_dim <= 0 || k_page_dim < maps * dim || v_page_dim < v_dim ||
                     (k_page_dim % 8) || (v_page_dim % 16))) return LLOGOS_BAD_ARGUMENT;
    const int n_k = n_kv * maps, n_v = n_kv;
    if (row_stride < (n_q + n_k) * dim + n_v * v_dim) return LLOGOS_BAD_ARGUMENT;
    PagedKV cache{table, table_stride, n_kv, k_page_dim > 0 ? k_page_dim : 1};
    const int units = n_q + n_k + n_v;
    const int lds_row = dim > v_dim ? dim : v_dim;
    // lanes a unit: 16 up to 64 values, 32 up to 128, else the wave
    int lanes = dim <= 64 ? 16 : (dim <= 128 ? 32 : kWave);
    while (lanes < kWave && (size_t)kPrepUnitsPerBlock * (kWave / lanes) * lds_row * sizeof(float) > 32 * 1024) lanes *= 2;   // (wide values beside narrow keys)
    const int per_block = kPrepUnitsPerBlock * (kWave / lanes);
    dim3 grid(T, (units + per_block - 1) / per_block), block(kWave, kPrepUnitsPerBlock);
    const size_t smem = (size_t)per_block * lds_row * sizeof(float);
    if (smem > 64 * 1024) return LLOGOS_TOO_LARGE;
#define LAUNCH_RL(TI, T_, R_, L_) rotary_prepare_kernel<TI, T_, R_, L_><<<grid, block, smem, stream>>>( \
        (const TI*)qkv, parts, (size_t)part_stride, row_stride, bias, (T_*)q_out, n_q, n_k, n_v, dim, v_dim, maps, rot, pairing, \
        q_norm_w, k_norm_w, unit_after, eps, (const float2*)cs, (T_*)k_pool, (T_*)v_pool, cache, v_page_dim, tok_seq, tok_pos, lds_row)
#define LAUNCH(TI, T_) do { if (lanes == 16) LAUNCH_RL(TI, T_, 4, 16); else if (lanes == 32) LAUNCH_RL(TI, T_, 4, 32); \
        else if (dim <= 4 * kWave) LAUNCH_RL(TI, T_, 4, kWave); else LAUNCH_RL(TI, T_, kPrepMaxDim / kWave, kWave); } while (0)
    if (dtype == DT_F32 && in_dtype == DT_F32) LAUNCH(float, float);
    else if (dtype == DT_BF16 && in_dtype == DT_BF16) LAUNCH(bf16_t, bf16_t);
    else if (dtype == DT_BF16 && in_dtype == DT_F32) LAUNCH(float, bf16_t);
    else return LLOGOS_BAD_ARGUMENT;
#undef LAUNCH
#undef LAUNCH_RL
    return LLOGOS_LAUNCH_CHECK();
}
