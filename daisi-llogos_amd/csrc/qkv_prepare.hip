// From a token's projected row [q | k | v] to the attention's inputs: optional biases, an optional
// RMS norm over the whole of q and over the whole of k (all heads at once, one weight a channel), an
// optional rotation of the first `rot` dimensions of every head of q and k by the step's (cos, sin)
// table, an optional factor on the query that grows with the logarithm of its position's block
// number, then q to a plain row and k and v to the cache's pages.
//
//   q' = rotate(rmsnorm_all(q + bq) * wq) * (1 + coef * ln(floor((pos + 1) / every) + 1))
//   k' = rotate(rmsnorm_all(k + bk) * wk)           -> key page of (sequence, position), head by head
//   v' = v + bv                                     -> value page
//
// rotate: pairing 0 pairs dimension i with i + rot / 2, pairing 1 dimension 2i with 2i + 1; the pair
// (u, v) becomes (u cos - v sin, v cos + u sin) with the pair's entry of cs [T, rot / 2] (cos, sin).
//
// Keys have head_dim dimensions a head and values v_dim; their pages hold rows of k_page_dim and
// v_page_dim (each the size rounded up to the pages' step).  The row comes as float32, maybe in
// parts of a product split along k; norms, logarithm and factor are 32-bit.  One block a token.
#include "common.h"

template <typename T>
__global__ __launch_bounds__(1024) void qkv_prepare_kernel(
        const float* __restrict__ qkv, int parts, size_t part_stride, int row_stride, const float* __restrict__ bias,
        T* __restrict__ q_out, int n_heads, int n_kv_heads, int head_dim, int v_dim, int k_page_dim, int v_page_dim,
        const float* __restrict__ q_norm_w, const float* __restrict__ k_norm_w, float eps, float temp_coef, int temp_every,
        const float2* __restrict__ cs, int rot, int pairing,
        T* __restrict__ k_pool, T* __restrict__ v_pool, const int* __restrict__ table, int table_stride,
        const int* __restrict__ tok_seq, const int* __restrict__ tok_pos, int staged_values,
        const float* __restrict__ kv_rows, int kv_stride) {
    __shared__ float red[16];
    const int t = blockIdx.x, tid = threadIdx.x;
    const int Wq = n_heads * head_dim, Wk = n_kv_heads * head_dim, Wv = n_kv_heads * v_dim;
    const float* row = qkv + (size_t)t * row_stride;
    auto value = [&](int c) {
        if (kv_rows && c >= Wq) {                            // keys and values that come in rows of their own
            const float v = kv_rows[(size_t)t * kv_stride + (c - Wq)];
            return bias ? v + bias[c] : v;
        }
        float v = row[c];
        for (int p0 = 1; p0 < parts; p0 += 8) {              // eight loads in flight, added in ascending order
            float y[8];
#pragma unroll
            for (int j = 0; j < 8; ++j) y[j] = p0 + j < parts ? row[(size_t)(p0 + j) * part_stride + c] : 0.f;
#pragma unroll
            for (int j = 0; j < 8; ++j)
                if (p0 + j < parts) v += y[j];
        }
        if (bias) v += bias[c];
        return v;
    };
    const int seq = tok_seq[t], pos = tok_pos[t];

    // the row's q and k values are summed from the product's parts once and kept in LDS where they fit (staged_values
    // = Wq + Wk), since the norm's sum, a channel's own value and its partner in the rotation all read them
    extern __shared__ float staged[];
    const bool in_lds = staged_values > 0;
    float q_scale = 1.f, k_scale = 1.f;
    if (q_norm_w || in_lds) {
        float ss = 0.f;
        for (int c = tid; c < Wq; c += blockDim.x) { const float v = value(c); if (in_lds) staged[c] = v; ss = fmaf(v, v, ss); }
        if (q_norm_w) q_scale = 1.0f / sqrtf(block_sum(ss, red) / (float)Wq + eps);
    }
    if ((k_norm_w || in_lds) && Wk > 0) {
        float ss = 0.f;
        for (int c = tid; c < Wk; c += blockDim.x) { const float v = value(Wq + c); if (in_lds) staged[Wq + c] = v; ss = fmaf(v, v, ss); }
        if (k_norm_w) k_scale = 1.0f / sqrtf(block_sum(ss, red) / (float)Wk + eps);
    }
    if (in_lds) __syncthreads();
    auto qk_value = [&](int c) { return in_lds ? staged[c] : value(c); };
    float temp = 1.f;
    if (temp_coef != 0.f) temp = 1.0f + temp_coef * logf((float)((pos + 1) / temp_every + 1));

    // channel c of q (base 0) or k (base Wq), normed and, within a head's first `rot` dimensions, rotated:
    // a thread works out its own channel and its partner's (the same arithmetic in both of a pair's threads)
    const int half = rot / 2;
    const float2* crow = cs ? cs + (size_t)t * half : nullptr;
    auto turned = [&](int base, int c, const float* w, float inv) {
        auto normed = [&](int cc) { const float v = qk_value(base + cc); return w ? v * inv * w[cc] : v; };
        const float mine = normed(c);
        const int d = c % head_dim;
        if (d >= rot) return mine;
        if (pairing == 0) {
            if (d < half) { const float2 a = crow[d]; return mine * a.x - normed(c + half) * a.y; }
            const float2 a = crow[d - half];
            return mine * a.x + normed(c - half) * a.y;
        }
        const float2 a = crow[d >> 1];
        return (d & 1) == 0 ? mine * a.x - normed(c + 1) * a.y : mine * a.x + normed(c - 1) * a.y;
    };

    T* qo = q_out + (size_t)t * Wq;
    for (int c = tid; c < Wq; c += blockDim.x) store_f32(qo + c, turned(0, c, q_norm_w, q_scale) * temp);
    if (n_kv_heads <= 0) return;
    const int page = table[(size_t)seq * table_stride + pos / kPageTokens];
    const int in_page = pos % kPageTokens;
    T* kp = k_pool + (size_t)page * n_kv_heads * kPageTokens * k_page_dim;
    for (int c = tid; c < Wk; c += blockDim.x) {
        const float v = turned(Wq, c, k_norm_w, k_scale);
        const int g = c / head_dim, d = c % head_dim;
        store_f32(kp + (size_t)g * kPageTokens * k_page_dim + page_key_offset(in_page, d, k_page_dim), v);
    }
    T* vp = v_pool + (size_t)page * n_kv_heads * kPageTokens * v_page_dim;
    for (int c = tid; c < Wv; c += blockDim.x) {
        const int g = c / v_dim, d = c % v_dim;
        store_f32(vp + (size_t)g * kPageTokens * v_page_dim + page_value_offset(in_page, d), value(Wq + Wk + c));
    }
}

// qkv: float32 rows [T, row_stride] (row_stride >= the three widths together), `parts` of them
// part_stride apart; bias float32 [Wq + Wk + Wv] or null; q_norm_w [Wq], k_norm_w [Wk] or null.
// cs: float32 [T, rot / 2, 2] (cos, sin) or null with rot 0.
// kv_rows (or null): float32 rows [T, kv_stride] that hold [k | v] in one part; qkv then holds q alone.
// n_kv_heads 0: the keys and values of these positions are another run's; only q is made.
LLOGOS_EXPORT int llogos_qkv_prepare(const float* qkv, int parts, long long part_stride, int row_stride, const float* bias,
                                     void* q_out, int dtype, int n_heads, int n_kv_heads, int head_dim, int v_dim,
                                     int k_page_dim, int v_page_dim, const float* q_norm_w, const float* k_norm_w, float eps,
                                     float temp_coef, int temp_every, const float* cs, int rot, int pairing,
                                     void* k_pool, void* v_pool, const int* table,
                                     int table_stride, const int* tok_seq, const int* tok_pos, const float* kv_rows, int kv_stride,
                                     int T, hipStream_t stream) {
    if (T <= 0 || n_heads <= 0 || n_kv_heads < 0 || head_dim <= 0 || v_dim <= 0 || parts < 1) return LLOGOS_BAD_ARGUMENT;
    if (temp_coef != 0.f && temp_every < 1) return LLOGOS_BAD_ARGUMENT;
    if (rot < 0 || rot > head_dim || (rot & 1) || (rot > 0 && !cs) || (pairing != 0 && pairing != 1)) return LLOGOS_BAD_ARGUMENT;
    if (n_kv_heads > 0) {
        if (!k_pool || !v_pool || !table) return LLOGOS_BAD_ARGUMENT;
        if (k_page_dim < head_dim || v_page_dim < v_dim || (k_page_dim % 8) || (v_page_dim % 16)) return LLOGOS_BAD_ARGUMENT;
    }
    if (kv_rows) {
        if (row_stride < n_heads * head_dim || kv_stride < n_kv_heads * (head_dim + v_dim)) return LLOGOS_BAD_ARGUMENT;
    } else if (row_stride < n_heads * head_dim + n_kv_heads * (head_dim + v_dim)) return LLOGOS_BAD_ARGUMENT;
    // few rows: many threads a row, so that a row's loads are all in flight at once
    const int threads = T <= 64 ? 1024 : 256;
    const int qk_values = n_heads * head_dim + n_kv_heads * head_dim;
    const int staged_values = (size_t)qk_values * sizeof(float) <= 48 * 1024 ? qk_values : 0;
#define PREP(T_) qkv_prepare_kernel<T_><<<T, threads, staged_values * sizeof(float), stream>>>(qkv, parts, (size_t)part_stride, row_stride, bias, (T_*)q_out, \
        n_heads, n_kv_heads, head_dim, v_dim, k_page_dim, v_page_dim, q_norm_w, k_norm_w, eps, temp_coef, temp_every, \
        (const float2*)cs, rot, pairing, (T_*)k_pool, (T_*)v_pool, table, table_stride, tok_seq, tok_pos, staged_values, kv_rows, kv_stride)
    if (dtype == DT_F32) PREP(float);
    else if (dtype == DT_BF16) PREP(bf16_t);
    else return LLOGOS_BAD_ARGUMENT;
#undef PREP
    return LLOGOS_LAUNCH_CHECK();
}
