// The closing step of a sublayer in a block whose norm comes after the residual sum:
//   v = alpha * x + delta;   x <- v * rsqrt(mean(v^2) + eps) * w
// The float32 stream x is replaced by its normed value, and the same rows are left in the matrix
// products' input type for the sublayer that reads the stream next (`rows`, optional).  `delta` may be
// `parts` partial sums of a k-split product, added in ascending order.  All arithmetic in 32-bit.
#include "common.h"

template <typename TD>
__device__ __forceinline__ float pn_sum_parts(const TD* p, size_t i, int parts, size_t part_stride) {
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

// One block a row; the row lives in registers between the two passes (ITEMS values a thread), so x is
// read once and written once.  For H <= ITEMS * blockDim.
template <typename TO, typename TD, int ITEMS>
__global__ __launch_bounds__(1024) void post_norm_kernel(float* __restrict__ x, const TD* __restrict__ delta, int parts,
                                                         size_t part_stride, float alpha, const float* __restrict__ w, float eps,
                                                         int H, TO* __restrict__ rows) {
    __shared__ float red[16];
    const size_t r = blockIdx.x;
    float* xr = x + r * H;
    const TD* dr = delta ? delta + r * H : nullptr;
    float v[ITEMS], wv[ITEMS], xv[ITEMS], sum[ITEMS];
    float ss = 0.f;
#pragma unroll
    for (int it = 0; it < ITEMS; ++it) {
        const int i = it * blockDim.x + threadIdx.x;
        wv[it] = i < H ? w[i] : 0.f;        // (asked for with the row, not behind the block's sum)
        xv[it] = i < H ? xr[i] : 0.f;
        sum[it] = (dr && i < H) ? load_f32(dr + i) : 0.f;
    }
    // the product's other parts, four at a time for all of the thread's values at once (their loads are in flight
    // together), added in ascending order
    if (dr) {
        for (int q0 = 1; q0 < parts; q0 += 4) {
            float y[4][ITEMS];
#pragma unroll
            for (int j = 0; j < 4; ++j)
#pragma unroll
                for (int it = 0; it < ITEMS; ++it) {
                    const int i = it * blockDim.x + threadIdx.x;
                    y[j][it] = (q0 + j < parts && i < H) ? load_f32(dr + (size_t)(q0 + j) * part_stride + i) : 0.f;
                }
#pragma unroll
            for (int j = 0; j < 4; ++j)
                if (q0 + j < parts) {
#pragma unroll
                    for (int it = 0; it < ITEMS; ++it) sum[it] += y[j][it];
                }
        }
    }
#pragma unroll
    for (int it = 0; it < ITEMS; ++it) {
        const float a = alpha * xv[it] + sum[it];
        v[it] = a;
        ss += a * a;
    }
    const float total = block_sum(ss, red);
    const float inv = 1.0f / sqrtf(total / (float)H + eps);
#pragma unroll
    for (int it = 0; it < ITEMS; ++it) {
        const int i = it * blockDim.x + threadIdx.x;
        if (i < H) {
            const float o = v[it] * inv * wv[it];
            xr[i] = o;
            if (rows) store_f32(rows + r * H + i, o);
        }
    }
}

// Any width: the summed row is parked in x between the passes.
template <typename TO, typename TD>
__global__ void post_norm_long_kernel(float* __restrict__ x, const TD* __restrict__ delta, int parts, size_t part_stride,
                                      float alpha, const float* __restrict__ w, float eps, int H, TO* __restrict__ rows) {
    __shared__ float red[16];
    const size_t r = blockIdx.x;
    float* xr = x + r * H;
    const TD* dr = delta ? delta + r * H : nullptr;
    float ss = 0.f;
    for (int i = threadIdx.x; i < H; i += blockDim.x) {
        float a = alpha * xr[i];
        if (dr) a += pn_sum_parts(dr, (size_t)i, parts, part_stride);
        xr[i] = a;
        ss += a * a;
    }
    const float total = block_sum(ss, red);
    const float inv = 1.0f / sqrtf(total / (float)H + eps);
    for (int i = threadIdx.x; i < H; i += blockDim.x) {
        const float o = xr[i] * inv * w[i];
        xr[i] = o;
        if (rows) store_f32(rows + r * H + i, o);
    }
}

// x [T, H] float32 (in place); delta [parts][T][H] float32 or bfloat16 (or null); rows [T, H] of rows_dtype or null.
LLOGOS_EXPORT int llogos_post_norm(float* x, const void* delta, int delta_dtype, int parts, long long part_stride, float alpha,
                                   const float* w, float eps, int T, int H, void* rows, int rows_dtype, hipStream_t stream) {
    if (T <= 0 || H <= 0 || parts < 1 || !x || !w) return LLOGOS_BAD_ARGUMENT;
    if (rows && rows_dtype != DT_F32 && rows_dtype != DT_BF16) return LLOGOS_BAD_ARGUMENT;
    if (delta && delta_dtype != DT_F32 && delta_dtype != DT_BF16) return LLOGOS_BAD_ARGUMENT;
    const bool rows_bf16 = rows && rows_dtype == DT_BF16, delta_bf16 = delta && delta_dtype == DT_BF16;
    int threads = 64;
    while (threads < 1024 && threads * 4 < H) threads <<= 1;
    const int items = (H + threads - 1) / threads;
#define PN(TO, TD) do { \
        if (items <= 1) post_norm_kernel<TO, TD, 1><<<T, threads, 0, stream>>>(x, (const TD*)delta, parts, (size_t)part_stride, alpha, w, eps, H, (TO*)rows); \
        else if (items <= 2) post_norm_kernel<TO, TD, 2><<<T, threads, 0, stream>>>(x, (const TD*)delta, parts, (size_t)part_stride, alpha, w, eps, H, (TO*)rows); \
        else if (items <= 4) post_norm_kernel<TO, TD, 4><<<T, threads, 0, stream>>>(x, (const TD*)delta, parts, (size_t)part_stride, alpha, w, eps, H, (TO*)rows); \
        else if (items <= 8) post_norm_kernel<TO, TD, 8><<<T, threads, 0, stream>>>(x, (const TD*)delta, parts, (size_t)part_stride, alpha, w, eps, H, (TO*)rows); \
        else post_norm_long_kernel<TO, TD><<<T, 1024, 0, stream>>>(x, (const TD*)delta, parts, (size_t)part_stride, alpha, w, eps, H, (TO*)rows); \
    } while (0)
    if (rows_bf16 && delta_bf16) PN(bf16_t, bf16_t);
    else if (rows_bf16) PN(bf16_t, float);
    else if (delta_bf16) PN(float, bf16_t);
    else PN(float, float);
#undef PN
    return LLOGOS_LAUNCH_CHECK();
}
