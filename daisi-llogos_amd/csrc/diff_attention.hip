// Differential attention over the paged cache: every head has two score maps over the same values,
//   a_m = softmax_j((q_m . k_m,j) * scale) V      m = 1, 2       (causal; optionally a window that keeps the first keys)
//   o   = a_1 - lambda * a_2;   out = o / sqrt(mean(o^2) + eps) * out_scale        (over the head's v_dim values)
// A kv head's key row in its page holds both maps' keys side by side ([map 1 | map 2], 2 * dim values of a
// row of k_page_dim); a query row holds, head by head, [map 1 | map 2] likewise.
// This file: the kernel for any shape and element type, all arithmetic in 32-bit.  One block a (token, head);
// keys in tiles of 256 from key 0 on with running maxima and sums, so the order of a query's additions
// depends on its position alone.
#include "common.h"

constexpr int kDiffTileKeys = 256;
constexpr int kDiffMaxDim = 1024;

template <typename T>
__global__ __launch_bounds__(256) void diff_attn_generic_kernel(
        T* __restrict__ out, const T* __restrict__ q, int q_stride, const T* __restrict__ k_pool, const T* __restrict__ v_pool,
        PagedKV cache, int v_page_dim, const int* __restrict__ tok_seq, const int* __restrict__ tok_pos, int n_heads, int group,
        int dim, int v_dim, float scale, int window, int sinks, float lambda, float out_scale, float eps) {
    extern __shared__ float smem[];
    float* qf = smem;                          // [2 * dim]
    float* p1 = smem + 2 * dim;                // [kDiffTileKeys]
    float* p2 = p1 + kDiffTileKeys;            // [kDiffTileKeys]
    float* red = p2 + kDiffTileKeys;           // [16]
    const int t = blockIdx.x, h = blockIdx.y, tid = threadIdx.x;
    const int seq = tok_seq[t], pos = tok_pos[t];
    const int kvh = h / group;
    const T* qrow = q + (size_t)t * q_stride + (size_t)h * 2 * dim;
    for (int d = tid; d < 2 * dim; d += blockDim.x) qf[d] = load_f32(qrow + d);
    __syncthreads();

    float m1 = -INFINITY, l1 = 0.f, m2 = -INFINITY, l2 = 0.f;
    float acc1[kDiffMaxDim / 256] = {}, acc2[kDiffMaxDim / 256] = {};
    for (int j0 = 0; j0 <= pos; j0 += kDiffTileKeys) {
        if (window > 0 && j0 >= sinks && j0 + kDiffTileKeys - 1 <= pos - window) continue;
        const int j = j0 + tid;
        const bool vis = key_visible(pos, j, window, sinks);
        float s1 = -INFINITY, s2 = -INFINITY;
        if (vis) {
            const T* kpage = k_pool + paged_base(cache, seq, kvh, j);
            const int tk = j % kPageTokens;
            float d1 = 0.f, d2 = 0.f;
            for (int d = 0; d < dim; ++d) {
                d1 = fmaf(qf[d], load_f32(kpage + page_key_offset(tk, d, cache.head_dim)), d1);
                d2 = fmaf(qf[dim + d], load_f32(kpage + page_key_offset(tk, dim + d, cache.head_dim)), d2);
            }
            s1 = d1 * scale;
            s2 = d2 * scale;
        }
        const float t1 = block_max(s1, red);
        const float t2 = block_max(s2, red);
        if (t1 == -INFINITY) continue;           // (a key is visible to both maps or to neither)
        const float n1 = fmaxf(m1, t1), n2 = fmaxf(m2, t2);
        const float e1 = vis ? expf(s1 - n1) : 0.f, e2 = vis ? expf(s2 - n2) : 0.f;
        __syncthreads();
        p1[tid] = e1;
        p2[tid] = e2;
        const float sum1 = block_sum(e1, red);   // (its barriers also publish p1 and p2)
        const float sum2 = block_sum(e2, red);
        const float c1 = (m1 == -INFINITY) ? 0.f : expf(m1 - n1), c2 = (m2 == -INFINITY) ? 0.f : expf(m2 - n2);
        const int n_keys = min(kDiffTileKeys, pos - j0 + 1);
#pragma unroll
        for (int r = 0; r < kDiffMaxDim / 256; ++r) {
            const int d = tid + r * 256;
            if (d < v_dim) {
                float a1 = acc1[r] * c1, a2 = acc2[r] * c2;
                for (int jj = 0; jj < n_keys; ++jj) {
                    const float w1 = p1[jj], w2 = p2[jj];
                    if (w1 != 0.f || w2 != 0.f) {
                        const size_t base = paged_base(cache, seq, kvh, j0 + jj) / cache.head_dim * v_page_dim;
                        const float v = load_f32(v_pool + base + page_value_offset((j0 + jj) % kPageTokens, d));
                        a1 = fmaf(w1, v, a1);
                        a2 = fmaf(w2, v, a2);
                    }
                }
                acc1[r] = a1;
                acc2[r] = a2;
            }
        }
        l1 = l1 * c1 + sum1;  m1 = n1;
        l2 = l2 * c2 + sum2;  m2 = n2;
    }
    const float i1 = l1 > 0.f ? 1.0f / l1 : 0.f, i2 = l2 > 0.f ? 1.0f / l2 : 0.f;
    float o[kDiffMaxDim / 256];
    float ss = 0.f;
#pragma unroll
    for (int r = 0; r < kDiffMaxDim / 256; ++r) {
        const int d = tid + r * 256;
        o[r] = d < v_dim ? acc1[r] * i1 - lambda * (acc2[r] * i2) : 0.f;
        ss += o[r] * o[r];
    }
    const float total = block_sum(ss, red);
    const float f = out_scale / sqrtf(total / (float)v_dim + eps);
    T* orow = out + ((size_t)t * n_heads + h) * v_dim;
#pragma unroll
    for (int r = 0; r < kDiffMaxDim / 256; ++r) {
        const int d = tid + r * 256;
        if (d < v_dim) store_f32(orow + d, o[r] * f);
    }
}

LLOGOS_EXPORT int llogos_diff_attention_generic(void* out, const void* q, int dtype, int q_stride, const void* k_pool,
                                                const void* v_pool, const int* table, int table_stride, const int* tok_seq,
                                                const int* tok_pos, int T, int n_heads, int n_kv_heads, int dim, int v_dim,
                                                int k_page_dim, int v_page_dim, float scale, int window, int sinks, float lambda,
                                                float out_scale, float eps, hipStream_t stream) {
    if (T <= 0 || n_heads <= 0 || n_kv_heads <= 0 || n_heads % n_kv_heads || !k_pool || !v_pool || !table) return LLOGOS_BAD_ARGUMENT;
    if (dim <= 0 || 2 * dim > kDiffMaxDim || v_dim <= 0 || v_dim > kDiffMaxDim || window < 0 || sinks < 0) return LLOGOS_BAD_ARGUMENT;
    if (k_page_dim < 2 * dim || (k_page_dim % 8) || v_page_dim < v_dim || (v_page_dim % 16) || q_stride < n_heads * 2 * dim) return LLOGOS_BAD_ARGUMENT;
    PagedKV cache{table, table_stride, n_kv_heads, k_page_dim};
    dim3 grid(T, n_heads);
    const size_t smem = (size_t)(2 * dim + 2 * kDiffTileKeys + 16) * sizeof(float);
    const int group = n_heads / n_kv_heads;
    if (dtype == DT_F32)
        diff_attn_generic_kernel<float><<<grid, 256, smem, stream>>>((float*)out, (const float*)q, q_stride, (const float*)k_pool,
            (const float*)v_pool, cache, v_page_dim, tok_seq, tok_pos, n_heads, group, dim, v_dim, scale, window, sinks, lambda, out_scale, eps);
    else if (dtype == DT_BF16)
        diff_attn_generic_kernel<bf16_t><<<grid, 256, smem, stream>>>((bf16_t*)out, (const bf16_t*)q, q_stride, (const bf16_t*)k_pool,
            (const bf16_t*)v_pool, cache, v_page_dim, tok_seq, tok_pos, n_heads, group, dim, v_dim, scale, window, sinks, lambda, out_scale, eps);
    else
        return LLOGOS_BAD_ARGUMENT;
    return LLOGOS_LAUNCH_CHECK();
}
