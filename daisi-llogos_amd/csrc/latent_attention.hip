// Attention through a low-rank latent.  Each token leaves one vector in the cache,
//     key row = [ c (rank) | rotated shared key part (rot) | zeros up to the page's head size ],
// with c the normed latent; there is one such row for all heads and no value pool: a value
// is the first `rank` dimensions of the key row.  Queries are brought into the same space
// (q_h . W_uk,h for the unrotated part, the rotated part as it is), so a head's score is one
// dot product with the cached row, and a head's output is a weighted sum of latents that the
// value matrix W_uv,h is applied to afterwards.
#include "common.h"

// ---------------------------------------------------------------- latent norm, rotation, cache write
// One block per token.  kv [T, ldkv] float: the first `rank` values are RMS-normed with weight
// norm_w (as it is) and stored as dimensions 0..rank-1 of the token's key row; the next `rot`
// are the shared key part: its first rot_dims dimensions are rotated in neighbouring pairs
// (2i, 2i + 1) by the table cs [T, rot_dims / 2] of (cos, sin), the rest pass unchanged.
// qfull [T, ldq] float holds per head [dim | rot]; the head's rot part is rotated the same way
// and written to q_out[t, h, rank .. rank + rot), zeros behind it up to hd.
// With a value pool (the matrix cores' attention reads values in their own operand order) the
// latent is stored there too, as dimensions 0..rank-1 of the token's value row.  With c_out the normed latents are
// also left as plain rows [T, rank] (for a caller that multiplies them with the heads' key and value matrices).
template <typename T>
__global__ void latent_prepare_kernel(const float* __restrict__ kv, int ldkv, const float* __restrict__ qfull, int ldq,
                                      T* __restrict__ q_out, const float* __restrict__ norm_w, float eps,
                                      const float2* __restrict__ cs, T* __restrict__ k_pool, T* __restrict__ v_pool, PagedKV cache,
                                      const int* __restrict__ tok_seq, const int* __restrict__ tok_pos,
                                      int n_heads, int dim, int rot, int rot_dims, int rank, int hd, T* __restrict__ c_out) {
    __shared__ float red[16];
    const int t = blockIdx.x, tid = threadIdx.x;
    const int seq = tok_seq[t], pos = tok_pos[t];
    const float* row = kv + (size_t)t * ldkv;
    const int half = rot_dims / 2;
    const float2* tab = cs + (size_t)t * half;
    const size_t page_at = paged_base(cache, seq, 0, pos);
    T* page = k_pool + page_at;
    const int in_page = pos % kPageTokens;

    float ss = 0.f;
    for (int i = tid; i < rank; i += blockDim.x) ss = fmaf(row[i], row[i], ss);
    const float inv = 1.0f / sqrtf(block_sum(ss, red) / (float)rank + eps);
    for (int i = tid; i < rank; i += blockDim.x) {
        const float v = row[i] * inv * norm_w[i];
        store_f32(page + page_key_offset(in_page, i, hd), v);
        if (v_pool) store_f32(v_pool + page_at + page_value_offset(in_page, i), v);     // the latent again, as a value
        if (c_out) store_f32(c_out + (size_t)t * rank + i, v);
    }
    for (int i = tid; i < hd - rank; i += blockDim.x) {
        float v = 0.f;
        if (i < rot) {
            v = row[rank + i];
            if (i < rot_dims) {
                const float2 c = tab[i >> 1];
                const float other = row[rank + (i ^ 1)];
                v = (i & 1) ? fmaf(v, c.x, other * c.y) : fmaf(v, c.x, -other * c.y);
            }
        }
        store_f32(page + page_key_offset(in_page, rank + i, hd), v);
    }
    const int tail = hd - rank;
    for (int e = tid; e < n_heads * tail; e += blockDim.x) {
        const int h = e / tail, i = e % tail;
        float v = 0.f;
        if (i < rot) {
            const float* q = qfull + (size_t)t * ldq + (size_t)h * (dim + rot) + dim;
            v = q[i];
            if (i < rot_dims) {
                const float2 c = tab[i >> 1];
                const float other = q[i ^ 1];
                v = (i & 1) ? fmaf(v, c.x, other * c.y) : fmaf(v, c.x, -other * c.y);
            }
        }
        store_f32(q_out + ((size_t)t * n_heads + h) * hd + rank + i, v);
    }
}

LLOGOS_EXPORT int llogos_latent_prepare(const float* kv, int ldkv, const float* qfull, int ldq, void* q_out, int dtype,
                                        const float* norm_w, float eps, const void* cs, void* k_pool, void* v_pool,
                                        const int* table, int table_stride, const int* tok_seq, const int* tok_pos,
                                        int T, int n_heads, int dim, int rot, int rot_dims, int rank, int hd, void* c_out,
                                        hipStream_t stream) {
    if (T <= 0 || n_heads <= 0 || dim < 0 || rot < 0 || rank <= 0 || hd < rank + rot || hd % 16) return LLOGOS_BAD_ARGUMENT;
    if (rot_dims < 0 || rot_dims > rot || rot_dims % 2 || ldkv < rank + rot || ldq < n_heads * (dim + rot)) return LLOGOS_BAD_ARGUMENT;
    PagedKV cache{table, table_stride, 1, hd};
    if (dtype == DT_F32)
        latent_prepare_kernel<float><<<T, 256, 0, stream>>>(kv, ldkv, qfull, ldq, (float*)q_out, norm_w, eps, (const float2*)cs,
                                                            (float*)k_pool, (float*)v_pool, cache, tok_seq, tok_pos, n_heads, dim, rot, rot_dims, rank, hd, (float*)c_out);
    else if (dtype == DT_BF16)
        latent_prepare_kernel<bf16_t><<<T, 256, 0, stream>>>(kv, ldkv, qfull, ldq, (bf16_t*)q_out, norm_w, eps, (const float2*)cs,
                                                             (bf16_t*)k_pool, (bf16_t*)v_pool, cache, tok_seq, tok_pos, n_heads, dim, rot, rot_dims, rank, hd, (bf16_t*)c_out);
    else
        return LLOGOS_BAD_ARGUMENT;
    return LLOGOS_LAUNCH_CHECK();
}

// ---------------------------------------------------------------- one small product per head
// out[t, h, n] = sum_k a[t, h, k] * w[h, n, k]   for n < N, k < K, every head with its own matrix.
// a: row stride lda, head stride a_head; out: row stride ldo, head stride o_head; w [H, N, K] dense.
// Tiles of 64 tokens x 64 outputs, 16 values of k at a time through LDS, 4 x 4 outputs a thread,
// sums in 32-bit in ascending k: an output's sum does not depend on what else is in the step.
// gate (or null): float32 logits, gate[t * gate_stride + h]; head h's outputs of row t are multiplied by its sigmoid.
template <typename TA, typename TW, typename TO>
__global__ __launch_bounds__(256) void head_products_kernel(TO* __restrict__ out, int ldo, int o_head,
                                                            const TA* __restrict__ a, int lda, int a_head,
                                                            const TW* __restrict__ w, int M, int N, int K,
                                                            const float* __restrict__ gate, int gate_stride) {
    __shared__ float sa[16][64 + 4];
    __shared__ float sw[16][64 + 4];
    const int h = blockIdx.z, m0 = blockIdx.x * 64, n0 = blockIdx.y * 64;
    const int tid = threadIdx.x, tx = tid % 16, ty = tid / 16;
    const TA* ah = a + (size_t)h * a_head;
    const TW* wh = w + (size_t)h * N * K;
    float acc[4][4] = {};
    for (int k0 = 0; k0 < K; k0 += 16) {
        for (int e = tid; e < 64 * 16; e += 256) {
            const int r = e / 16, kk = e % 16;
            sa[kk][r] = (m0 + r < M && k0 + kk < K) ? load_f32(ah + (size_t)(m0 + r) * lda + k0 + kk) : 0.f;
            sw[kk][r] = (n0 + r < N && k0 + kk < K) ? load_f32(wh + (size_t)(n0 + r) * K + k0 + kk) : 0.f;
        }
        __syncthreads();
#pragma unroll
        for (int kk = 0; kk < 16; ++kk) {
            float av[4], wv[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) { av[i] = sa[kk][ty * 4 + i]; wv[i] = sw[kk][tx * 4 + i]; }
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int jn = 0; jn < 4; ++jn) acc[i][jn] = fmaf(av[i], wv[jn], acc[i][jn]);
        }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int m = m0 + ty * 4 + i;
        if (m >= M) continue;
        const float f = gate ? 1.0f / (1.0f + expf(-gate[(size_t)m * gate_stride + h])) : 1.0f;
#pragma unroll
        for (int jn = 0; jn < 4; ++jn) {
            const int n = n0 + tx * 4 + jn;
            if (n < N) store_f32(out + (size_t)m * ldo + (size_t)h * o_head + n, gate ? acc[i][jn] * f : acc[i][jn]);
        }
    }
}

// The same for steps of up to 16 rows, where the tiles above would be nearly empty: the rows of a head go to
// LDS once, a thread owns an output n and one of KG groups of k and streams its part of the head's matrix, which for
// this kernel is stored k-major, w_kn [H, K, N], so that neighbouring threads read neighbouring values; the
// groups' sums are added in a fixed order.  TMAX: the rows
// rounded up to 1, 2, 4, 8 or 16 (rows that are not there are zeros in LDS).
template <int TMAX, int KG, typename TA, typename TW, typename TO>
__global__ __launch_bounds__(64 * KG) void head_products_few_kernel(TO* __restrict__ out, int ldo, int o_head, const TA* __restrict__ a, int lda, int a_head,
                                         const TW* __restrict__ w_kn, int M, int N, int K,
                                         const float* __restrict__ gate, int gate_stride) {
    // LDS: the head's rows as [k][TMAX] (one or two 16-byte reads bring every row's value of a k), then the KG
    // k-groups' sums [KG][64][TMAX]
    extern __shared__ float rows_lds[];
    float* sums = rows_lds + (size_t)K * TMAX;
    const int h = blockIdx.y, nl = threadIdx.x & 63, kg = threadIdx.x >> 6, n = blockIdx.x * 64 + nl;
#pragma unroll 4
    for (int e = threadIdx.x; e < TMAX * K; e += blockDim.x) {      // (neighbouring threads read neighbouring k of a row)
        const int t = e / K, k = e % K;
        rows_lds[k * TMAX + t] = t < M ? load_f32(a + (size_t)t * lda + (size_t)h * a_head + k) : 0.f;
    }
    __syncthreads();
    float acc[TMAX];
#pragma unroll
    for (int t = 0; t < TMAX; ++t) acc[t] = 0.f;
    // this thread: output n, the k of its group: kg, kg + KG, ... (the groups' loads of w lie KG rows apart)
    if (n < N) {
        const TW* wp = w_kn + (size_t)h * K * N + n;
        // (sixteen loads in flight: a thread's loads are 2 or 4 bytes each, and their latency is what the kernel waits for;
        // sixteen groups of k give a compute unit's SIMDs four waves each to wait with)
        for (int k0 = kg; k0 < K; k0 += 16 * KG) {
            float wv[16];
#pragma unroll
            for (int kk = 0; kk < 16; ++kk) wv[kk] = k0 + KG * kk < K ? load_f32(wp + (size_t)(k0 + KG * kk) * N) : 0.f;
#pragma unroll
            for (int kk = 0; kk < 16; ++kk) {
                const int k = min(k0 + KG * kk, K - 1);                  // (beyond the end: wv is 0)
#pragma unroll
                for (int t = 0; t < TMAX; ++t) acc[t] = fmaf(rows_lds[k * TMAX + t], wv[kk], acc[t]);
            }
        }
    }
#pragma unroll
    for (int t = 0; t < TMAX; ++t) sums[(kg * 64 + nl) * TMAX + t] = acc[t];
    __syncthreads();
    if (kg == 0 && n < N) {
#pragma unroll
        for (int t = 0; t < TMAX; ++t) {
            float v = sums[nl * TMAX + t];
#pragma unroll
            for (int j = 1; j < KG; ++j) v += sums[(j * 64 + nl) * TMAX + t];          // in the groups' order
            if (t < M && gate) v *= 1.0f / (1.0f + expf(-gate[(size_t)t * gate_stride + h]));
            if (t < M) store_f32(out + (size_t)t * ldo + (size_t)h * o_head + n, v);
        }
    }
}

LLOGOS_EXPORT int llogos_head_products_few(void* out, int out_dtype, int ldo, int o_head, const void* a, int a_dtype, int lda,
                                           int a_head, const void* w_kn, int w_dtype, int M, int H, int N, int K,
                                           const float* gate, int gate_stride, hipStream_t stream) {
    if (M <= 0 || M > 16 || H <= 0 || N <= 0 || K <= 0 || (gate && gate_stride < H)) return LLOGOS_BAD_ARGUMENT;
    int tmax = 1;
    while (tmax < M) tmax <<= 1;
    // sixteen groups of k where their sums fit beside the rows and every group has k of its own, else four
    const bool wide = K >= 64 && (size_t)tmax * (K + 16 * 64) * sizeof(float) <= 65536;
    const size_t smem = (size_t)tmax * (K + (wide ? 16 : 4) * 64) * sizeof(float);
    if (smem > 65536) return LLOGOS_UNSUPPORTED;
    dim3 grid((N + 63) / 64, H);
#define HPF(TM, TA, TW, TO) do { \
        if (wide) { \
            if (smem > 48 * 1024) { \
                hipError_t e = hipFuncSetAttribute((const void*)head_products_few_kernel<TM, 16, TA, TW, TO>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem); \
                if (e != hipSuccess) return (int)e; \
            } \
            head_products_few_kernel<TM, 16, TA, TW, TO><<<grid, 1024, smem, stream>>>((TO*)out, ldo, o_head, (const TA*)a, lda, a_head, (const TW*)w_kn, M, N, K, gate, gate_stride); \
        } else { \
            if (smem > 48 * 1024) { \
                hipError_t e = hipFuncSetAttribute((const void*)head_products_few_kernel<TM, 4, TA, TW, TO>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem); \
                if (e != hipSuccess) return (int)e; \
            } \
            head_products_few_kernel<TM, 4, TA, TW, TO><<<grid, 256, smem, stream>>>((TO*)out, ldo, o_head, (const TA*)a, lda, a_head, (const TW*)w_kn, M, N, K, gate, gate_stride); \
        } } while (0)
#define HPT(TA, TW, TO) do { if (tmax == 1) HPF(1, TA, TW, TO); else if (tmax == 2) HPF(2, TA, TW, TO); else if (tmax == 4) HPF(4, TA, TW, TO); \
                             else if (tmax == 8) HPF(8, TA, TW, TO); else HPF(16, TA, TW, TO); } while (0)
    if (a_dtype == DT_F32 && w_dtype == DT_F32 && out_dtype == DT_F32) HPT(float, float, float);
    else if (a_dtype == DT_F32 && w_dtype == DT_BF16 && out_dtype == DT_F32) HPT(float, bf16_t, float);
    else if (a_dtype == DT_F32 && w_dtype == DT_BF16 && out_dtype == DT_BF16) HPT(float, bf16_t, bf16_t);
    else if (a_dtype == DT_BF16 && w_dtype == DT_BF16 && out_dtype == DT_BF16) HPT(bf16_t, bf16_t, bf16_t);
    else if (a_dtype == DT_BF16 && w_dtype == DT_BF16 && out_dtype == DT_F32) HPT(bf16_t, bf16_t, float);
    else return LLOGOS_BAD_ARGUMENT;
#undef HPT
#undef HPF
    return LLOGOS_LAUNCH_CHECK();
}

LLOGOS_EXPORT int llogos_head_products(void* out, int out_dtype, int ldo, int o_head, const void* a, int a_dtype, int lda,
                                       int a_head, const void* w, int w_dtype, int M, int H, int N, int K,
                                       const float* gate, int gate_stride, hipStream_t stream) {
    if (M <= 0 || H <= 0 || N <= 0 || K <= 0 || (gate && gate_stride < H)) return LLOGOS_BAD_ARGUMENT;
    dim3 grid((M + 63) / 64, (N + 63) / 64, H);
#define HP(TA, TW, TO) head_products_kernel<TA, TW, TO><<<grid, 256, 0, stream>>>((TO*)out, ldo, o_head, (const TA*)a, lda, a_head, \
        (const TW*)w, M, N, K, gate, gate_stride)
    if (a_dtype == DT_F32 && w_dtype == DT_F32 && out_dtype == DT_F32) HP(float, float, float);
    else if (a_dtype == DT_F32 && w_dtype == DT_BF16 && out_dtype == DT_F32) HP(float, bf16_t, float);
    else if (a_dtype == DT_F32 && w_dtype == DT_BF16 && out_dtype == DT_BF16) HP(float, bf16_t, bf16_t);
    else if (a_dtype == DT_BF16 && w_dtype == DT_BF16 && out_dtype == DT_BF16) HP(bf16_t, bf16_t, bf16_t);
    else if (a_dtype == DT_BF16 && w_dtype == DT_BF16 && out_dtype == DT_F32) HP(bf16_t, bf16_t, float);
    else return LLOGOS_BAD_ARGUMENT;
#undef HP
    return LLOGOS_LAUNCH_CHECK();
}
