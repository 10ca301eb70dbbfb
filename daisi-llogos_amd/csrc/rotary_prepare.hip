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
// row has v_dim values in pages of v_page_dim.  All arithmetic in 32-bit; one wave a (token, unit).
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

// R: values a lane holds of a unit (dim <= 64 R).
template <typename TI, typename T, int R>
__global__ void rotary_prepare_kernel(const TI* __restrict__ qkv, int parts, size_t part_stride, int row_stride,
                                      const float* __restrict__ bias, T* __restrict__ q_out, int n_q, int n_k, int n_v,
                                      int dim, int v_dim, int maps, int rot, int pairing,
                                      const float* __restrict__ q_norm_w, const float* __restrict__ k_norm_w, int unit_after,
                                      float eps, const float2* __restrict__ cs, T* __restrict__ k_pool, T* __restrict__ v_pool,
                                      PagedKV cache, int v_page_dim, const int* __restrict__ tok_seq,
                                      const int* __restrict__ tok_pos, int lds_row) {
    extern __shared__ float smem[];
    const int t = blockIdx.x;
    const int unit = blockIdx.y * kPrepUnitsPerBlock + threadIdx.y;
    const int lane = threadIdx.x;
    const bool active = unit < n_q + n_k + n_v;
    float* buf = smem + threadIdx.y * lds_row;
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
        for (int d = lane; d < width; d += kWave) {
            float v = rp_sum_parts(src, (size_t)d, parts, part_stride);
            if (bias) v += bias[col0 + d];
            buf[d] = v;
            ss += v * v;
        }
    }
    __syncthreads();
    if (active && norm_w) {
        ss = wave_sum(ss);
        const float inv = 1.0f / sqrtf(ss / (float)dim + eps);
        for (int d = lane; d < dim; d += kWave) buf[d] = buf[d] * inv * norm_w[d];
    }
    __syncthreads();
    if (!active) return;
    if (!is_q && !is_k) {
        const int vh = unit - n_q - n_k;
        T* vdst = v_pool + paged_base(cache, tok_seq[t], vh, pos) / cache.head_dim * v_page_dim;
        for (int d = lane; d < v_dim; d += kWave) store_f32(vdst + page_value_offset(in_page, d), buf[d]);
        return;
    }
    const int half = rot / 2;
    const float2* c = cs + (size_t)t * half;
    // a lane's rotated values: dimensions lane, lane + 64, ... (both partners are read before either is stored)
    float mine[R];
    float s2 = 0.f;
#pragma unroll
    for (int r = 0; r < R; ++r) {
        const int d = lane + r * kWave;
        float v = 0.f;
        if (d < dim) {
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
    if (unit_after) after = 1.0f / sqrtf(wave_sum(s2) / (float)dim + eps);
    if (is_q) {
        T* dst = q_out + ((size_t)t * n_q + unit) * dim;
#pragma unroll
        for (int r = 0; r < R; ++r) {
            const int d = lane + r * kWave;
            if (d < dim) store_f32(dst + d, mine[r] * after);
        }
    } else {
        const int ku = unit - n_q;
        T* dst = k_pool + paged_base(cache, tok_seq[t], ku / maps, pos);
        const int col = (ku % maps) * dim;
#pragma unroll
        for (int r = 0; r < R; ++r) {
            const int d = lane + r * kWave;
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
    dim3 grid(T, (units + kPrepUnitsPerBlock - 1) / kPrepUnitsPerBlock), block(kWave, kPrepUnitsPerBlock);
    const size_t smem = (size_t)kPrepUnitsPerBlock * lds_row * sizeof(float);
#define LAUNCH_R(TI, T_, R_) rotary_prepare_kernel<TI, T_, R_><<<grid, block, smem, stream>>>( \
        (const TI*)qkv, parts, (size_t)part_stride, row_stride, bias, (T_*)q_out, n_q, n_k, n_v, dim, v_dim, maps, rot, pairing, \
        q_norm_w, k_norm_w, unit_after, eps, (const float2*)cs, (T_*)k_pool, (T_*)v_pool, cache, v_page_dim, tok_seq, tok_pos, lds_row)
#define LAUNCH(TI, T_) do { if (dim <= kWave) LAUNCH_R(TI, T_, 1); else if (dim <= 2 * kWave) LAUNCH_R(TI, T_, 2); \
        else if (dim <= 4 * kWave) LAUNCH_R(TI, T_, 4); else LAUNCH_R(TI, T_, kPrepMaxDim / kWave); } while (0)
    if (dtype == DT_F32 && in_dtype == DT_F32) LAUNCH(float, float);
    else if (dtype == DT_BF16 && in_dtype == DT_BF16) LAUNCH(bf16_t, bf16_t);
    else if (dtype == DT_BF16 && in_dtype == DT_F32) LAUNCH(float, bf16_t);
    else return LLOGOS_BAD_ARGUMENT;
#undef LAUNCH
#undef LAUNCH_R
    return LLOGOS_LAUNCH_CHECK();
}
