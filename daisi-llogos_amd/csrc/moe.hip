// Mixtures of experts.  The choice is either a table over token ids (token t goes to the `top` experts
// table[ids[t]][0..top), each weighted alike) or a router's (moe_router_logits, moe_router_choose: a
// softmax over the router's outputs, a correction added for the choice alone, the best groups of
// neighbouring experts, the `top` best of those, weights from the uncorrected scores).  Everything is
// decided on the device, so a captured step replays with other tokens.
//
//   moe_route    (token, choice) pairs sorted by expert: order[], the experts' segments seg[], and
//                where[pair] = the pair's place in that order
//   moe_product  a product of the sorted rows with their expert's matrix, tile by tile within a segment
//                (plain 32-bit FMAs, any storage type), optionally gathering its input rows by pair
//                and squaring relu in its epilogue
//   moe_combine  out[t] = mean over choices of the pair rows + sigmoid(gate[t]) * shared[t]
//   moe_combine_weighted  out[t] = sum over choices of weight * pair row (or weight * the token's own row for a
//                router output that stands for no expert matrix) + shared[t]
//
// A row's sums are taken in the order of k alone, in the blocks of gemm_generic.hip (16 products, 16 of
// those, then the total), so a token's result does not depend on where it falls in a segment or on
// what else is in the step.
#include "common.h"

constexpr int kMoeMaxExperts = 1024;

// One block.  seg has E + 1 entries.  ids null: row t of the table is token t's own (a router's choice [T, top]).
__global__ __launch_bounds__(1024) void moe_route_kernel(const int* __restrict__ ids, const int* __restrict__ table, int T, int top,
                                                         int E, int* __restrict__ order, int* __restrict__ seg,
                                                         int* __restrict__ where) {
    __shared__ int count[kMoeMaxExperts];
    __shared__ int start[kMoeMaxExperts + 1];
    const int P = T * top;
    for (int e = threadIdx.x; e < E; e += blockDim.x) count[e] = 0;
    __syncthreads();
    for (int p = threadIdx.x; p < P; p += blockDim.x) {
        int e = table[(size_t)(ids ? ids[p / top] : p / top) * top + p % top];
        e = min(max(e, 0), E - 1);
        atomicAdd(&count[e], 1);
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        int run = 0;
        for (int e = 0; e < E; ++e) { start[e] = run; run += count[e]; }
        start[E] = run;
    }
    __syncthreads();
    for (int e = threadIdx.x; e <= E; e += blockDim.x) seg[e] = start[e];
    for (int e = threadIdx.x; e < E; e += blockDim.x) count[e] = 0;
    __syncthreads();
    for (int p = threadIdx.x; p < P; p += blockDim.x) {
        int e = table[(size_t)(ids ? ids[p / top] : p / top) * top + p % top];
        e = min(max(e, 0), E - 1);
        const int at = start[e] + atomicAdd(&count[e], 1);
        order[at] = p;
        where[p] = at;
    }
}

LLOGOS_EXPORT int llogos_moe_route(const int* ids, const int* table, int T, int top, int E, int* order, int* seg, int* where,
                                   hipStream_t stream) {
    if (T <= 0 || top <= 0 || E <= 0 || E > kMoeMaxExperts) return LLOGOS_BAD_ARGUMENT;
    moe_route_kernel<<<1, 1024, 0, stream>>>(ids, table, T, top, E, order, seg, where);
    return LLOGOS_LAUNCH_CHECK();
}

__device__ __forceinline__ float moe_gated(float gate, float up) { return gate / (1.0f + expf(-gate)) * up; }

// out[r, :] = act(a_row(r) . w[e]^T) * scale for the sorted rows r of expert e's segment.
// act 0: none; 1: the square of relu; 2: the matrix's rows are gate and up rows in turn (gate 0, up 0, gate 1, ...)
// and the result has N / 2 columns silu(gate_i) * up_i.
// a_row(r) = a[order[r] / top] when gather (the step's token rows), else a[r] (rows already sorted).
// w is [E][N][K].  Tiles of 64 rows x 64 columns; blockIdx.y counts row tiles over all segments.
constexpr int GM = 64, GN = 64, GK = 16;

template <typename TA, typename TW, typename TO>
__global__ __launch_bounds__(256) void moe_product_kernel(TO* __restrict__ out, const TA* __restrict__ a, const TW* __restrict__ w,
                                                          const int* __restrict__ order, const int* __restrict__ seg, int E,
                                                          int top, int gather, int N, int K, int lda, int act, float scale) {
    __shared__ float As[GK][GM + 4];
    __shared__ float Ws[GK][GN + 4];
    __shared__ int src_row[GM];
    __shared__ int s_expert, s_first, s_end;
    const int tid = threadIdx.x;
    if (tid == 0) {
        int tile = blockIdx.y, e = 0, found = -1, first = 0, end = 0;
        for (; e < E; ++e) {
            const int lo = seg[e], hi = seg[e + 1];
            const int tiles = (hi - lo + GM - 1) / GM;
            if (tile < tiles) { found = e; first = lo + tile * GM; end = hi; break; }
            tile -= tiles;
        }
        s_expert = found; s_first = first; s_end = end;
    }
    __syncthreads();
    const int e = s_expert;
    if (e < 0) return;                                     // beyond the last segment's tiles
    const int m0 = s_first, m_end = s_end, n0 = blockIdx.x * GN;
    if (tid < GM) {
        const int r = m0 + tid;
        src_row[tid] = r < m_end ? (gather ? order[r] / top : r) : -1;
    }
    __syncthreads();
    const TW* we = w + (size_t)e * N * K;
    const int ty = tid / 16, tx = tid % 16;
    const int lr = tid / 4, lk = (tid % 4) * 4;
    const int arow = src_row[lr];
    float acc[4][4] = {}, mid[4][4] = {};
    for (int k0 = 0; k0 < K; k0 += GK) {
        float part[4][4] = {};
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int k = k0 + lk + j;
            const int wn = n0 + lr;
            As[lk + j][lr] = (arow >= 0 && k < K) ? load_f32(a + (size_t)arow * lda + k) : 0.f;
            Ws[lk + j][lr] = (wn < N && k < K) ? load_f32(we + (size_t)wn * K + k) : 0.f;
        }
        __syncthreads();
#pragma unroll
        for (int k = 0; k < GK; ++k) {
            float av[4], wv[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) { av[i] = As[k][ty * 4 + i]; wv[i] = Ws[k][tx * 4 + i]; }
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) part[i][j] = fmaf(av[i], wv[j], part[i][j]);
        }
        const bool fold = ((k0 / GK) & 15) == 15;
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                mid[i][j] += part[i][j];
                if (fold) { acc[i][j] += mid[i][j]; mid[i][j] = 0.f; }
            }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int m = m0 + ty * 4 + i;
        if (m >= m_end) continue;
        if (act == 2) {                                     // columns in pairs (gate, up): silu(gate) * up
#pragma unroll
            for (int j = 0; j < 4; j += 2) {
                const int n = n0 + tx * 4 + j;
                if (n + 1 >= N) continue;
                const float gt = acc[i][j] + mid[i][j], up = acc[i][j + 1] + mid[i][j + 1];
                store_f32(out + (size_t)m * (N / 2) + n / 2, moe_gated(gt, up) * scale);
            }
            continue;
        }
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int n = n0 + tx * 4 + j;
            if (n >= N) continue;
            float v = acc[i][j] + mid[i][j];
            if (act == 1) { v = fmaxf(v, 0.f); v = v * v; }
            store_f32(out + (size_t)m * N + n, v * scale);
        }
    }
}

// P = T * top sorted rows at most; row_tiles bounds the tiles of all segments: ceil(P / 64) + E covers them.
LLOGOS_EXPORT int llogos_moe_product(void* out, int out_dtype, const void* a, int a_dtype, const void* w, int w_dtype,
                                     const int* order, const int* seg, int E, int top, int gather, int P, int N, int K,
                                     int lda, int act, float scale, hipStream_t stream) {
    if (P <= 0 || N <= 0 || K <= 0 || E <= 0 || top <= 0 || lda < K || act < 0 || act > 2 || (act == 2 && (N & 1))) return LLOGOS_BAD_ARGUMENT;
    if (a_dtype != w_dtype && !(a_dtype == DT_F32)) return LLOGOS_BAD_ARGUMENT;
    const int row_tiles = (P + GM - 1) / GM + E;
    dim3 grid((N + GN - 1) / GN, row_tiles);
#define MP(TA, TW, TO) moe_product_kernel<TA, TW, TO><<<grid, 256, 0, stream>>>((TO*)out, (const TA*)a, (const TW*)w, order, seg, E, \
        top, gather, N, K, lda, act, scale)
    if (a_dtype == DT_F32 && w_dtype == DT_F32 && out_dtype == DT_F32) MP(float, float, float);
    else if (a_dtype == DT_BF16 && w_dtype == DT_BF16 && out_dtype == DT_BF16) MP(bf16_t, bf16_t, bf16_t);
    else if (a_dtype == DT_BF16 && w_dtype == DT_BF16 && out_dtype == DT_F32) MP(bf16_t, bf16_t, float);
    else return LLOGOS_BAD_ARGUMENT;
#undef MP
    return LLOGOS_LAUNCH_CHECK();
}

// out[t, :] = (sum_j y[where[t * top + j], :]) / top + sigmoid(gate[t * gate_stride]) * (sum of the parts of shared[t, :])
// y float32 [P, W]; shared float32 [(parts,) T, W] or null; gate float32 (one number a token, maybe in
// parts gate_part_stride apart) or null: then the shared rows are added as they are.
__global__ void moe_combine_kernel(float* __restrict__ out, const float* __restrict__ y, const int* __restrict__ where, int top,
                                   const float* __restrict__ shared_rows, int parts, size_t part_stride,
                                   const float* __restrict__ gate, int gate_stride, int gate_parts, size_t gate_part_stride,
                                   int T, int W) {
    const int t = blockIdx.x;
    float g = 1.f;
    if (gate) {
        float z = gate[(size_t)t * gate_stride];
        for (int p = 1; p < gate_parts; ++p) z += gate[p * gate_part_stride + (size_t)t * gate_stride];
        g = 1.0f / (1.0f + expf(-z));
    }
    const float inv_top = 1.0f / (float)top;
    for (int c = blockIdx.y * blockDim.x + threadIdx.x; c < W; c += gridDim.y * blockDim.x) {
        float v = 0.f;
        for (int j = 0; j < top; ++j) v += y[(size_t)where[t * top + j] * W + c];
        v *= inv_top;
        if (shared_rows) {
            float s = shared_rows[(size_t)t * W + c];
            for (int p = 1; p < parts; ++p) s += shared_rows[p * part_stride + (size_t)t * W + c];
            v = fmaf(g, s, v);
        }
        out[(size_t)t * W + c] = v;
    }
}

LLOGOS_EXPORT int llogos_moe_combine(float* out, const float* y, const int* where, int top, const float* shared_rows, int parts,
                                     long long part_stride, const float* gate, int gate_stride, int gate_parts,
                                     long long gate_part_stride, int T, int W, hipStream_t stream) {
    if (T <= 0 || W <= 0 || top <= 0 || parts < 1 || gate_parts < 1) return LLOGOS_BAD_ARGUMENT;
    const int threads = 256;
    dim3 grid(T, (W + threads - 1) / threads);
    moe_combine_kernel<<<grid, threads, 0, stream>>>(out, y, where, top, shared_rows, parts, (size_t)part_stride, gate, gate_stride,
                                                     gate_parts, (size_t)gate_part_stride, T, W);
    return LLOGOS_LAUNCH_CHECK();
}

// ---------------------------------------------------------------- a router
// z[t, e] = w[e, :] . a[t, :] in 32-bit.  A wave takes R token rows and G router outputs: its lanes go along k four
// values at a time (lane l takes k = 4 l .. 4 l + 3, then 256 further on), every value of a row serves the G outputs
// and every value of w the R rows; the lanes' sums are added by the wave's reduction at the end.  The order of an
// output's additions depends on k alone, so a row's logits are the same bits in a step of one row and of thousands.
// w float32 [E, K]; a [T, lda] of any storage type.  VEC: K, lda and the pointers allow 16-byte (8-byte) loads.
template <typename TA> struct RouterRow4;
template <> struct RouterRow4<float> {
    static __device__ __forceinline__ float4 load(const float* p) { return *reinterpret_cast<const float4*>(p); }
};
template <> struct RouterRow4<bf16_t> {
    static __device__ __forceinline__ float4 load(const bf16_t* p) {
        const uint2 u = *reinterpret_cast<const uint2*>(p);
        return make_float4(__uint_as_float(u.x << 16), __uint_as_float(u.x & 0xffff0000u), __uint_as_float(u.y << 16),
                           __uint_as_float(u.y & 0xffff0000u));
    }
};

template <typename TA, int R, int G, bool VEC>
__global__ __launch_bounds__(256) void moe_router_logits_kernel(float* __restrict__ z, const TA* __restrict__ a, int lda,
                                                                const float* __restrict__ w, int T, int E, int K) {
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    const int t0 = (blockIdx.x * 4 + wave) * R, e0 = blockIdx.y * G;
    if (t0 >= T) return;
    float acc[R][G];
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
        for (int g = 0; g < G; ++g) acc[r][g] = 0.f;
    for (int k = 4 * lane; k < K; k += 4 * kWave) {
        float4 av[R], wv[G];
#pragma unroll
        for (int r = 0; r < R; ++r) {
            const TA* p = a + (size_t)min(t0 + r, T - 1) * lda + k;
            if (VEC) av[r] = RouterRow4<TA>::load(p);
            else av[r] = make_float4(load_f32(p), k + 1 < K ? load_f32(p + 1) : 0.f, k + 2 < K ? load_f32(p + 2) : 0.f,
                                     k + 3 < K ? load_f32(p + 3) : 0.f);
        }
#pragma unroll
        for (int g = 0; g < G; ++g) {
            const float* p = w + (size_t)min(e0 + g, E - 1) * K + k;
            if (VEC) wv[g] = *reinterpret_cast<const float4*>(p);
            else wv[g] = make_float4(p[0], k + 1 < K ? p[1] : 0.f, k + 2 < K ? p[2] : 0.f, k + 3 < K ? p[3] : 0.f);
        }
#pragma unroll
        for (int r = 0; r < R; ++r)
#pragma unroll
            for (int g = 0; g < G; ++g) {
                float s = acc[r][g];
                s = fmaf(av[r].x, wv[g].x, s);
                s = fmaf(av[r].y, wv[g].y, s);
                s = fmaf(av[r].z, wv[g].z, s);
                s = fmaf(av[r].w, wv[g].w, s);
                acc[r][g] = s;
            }
    }
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
        for (int g = 0; g < G; ++g) {
            const float s = wave_sum(acc[r][g]);
            if (lane == 0 && t0 + r < T && e0 + g < E) z[(size_t)(t0 + r) * E + e0 + g] = s;
        }
}

LLOGOS_EXPORT int llogos_moe_router_logits(float* z, const void* a, int a_dtype, int lda, const float* w, int T, int E, int K,
                                           hipStream_t stream) {
    if (T <= 0 || E <= 0 || K <= 0 || lda < K || (a_dtype != DT_F32 && a_dtype != DT_BF16)) return LLOGOS_BAD_ARGUMENT;
    const int elt = a_dtype == DT_F32 ? 4 : 2;
    const bool vec = K % 4 == 0 && lda % 4 == 0 && (uintptr_t)a % (4 * elt) == 0 && (uintptr_t)w % 16 == 0;
    // few rows: a row a wave and four outputs, so that the step has waves enough; many: four rows a wave and eight outputs
    const bool few = T <= 64;
    const int R = few ? 1 : 4, G = few ? 4 : 8;
    dim3 grid((T + 4 * R - 1) / (4 * R), (E + G - 1) / G);
#define RL(TA, R_, G_, V) moe_router_logits_kernel<TA, R_, G_, V><<<grid, 256, 0, stream>>>(z, (const TA*)a, lda, w, T, E, K)
#define RLV(TA, R_, G_) do { if (vec) RL(TA, R_, G_, true); else RL(TA, R_, G_, false); } while (0)
    if (a_dtype == DT_F32) { if (few) RLV(float, 1, 4); else RLV(float, 4, 8); }
    else { if (few) RLV(bf16_t, 1, 4); else RLV(bf16_t, 4, 8); }
#undef RLV
#undef RL
    return LLOGOS_LAUNCH_CHECK();
}

// the wave's largest (value, lowest index among equals); every lane returns it
__device__ __forceinline__ void wave_argmax(float& v, int& i) {
#pragma unroll
    for (int o = kWave / 2; o > 0; o >>= 1) {
        const float ov = __shfl_xor(v, o, kWave);
        const int oi = __shfl_xor(i, o, kWave);
        if (ov > v || (ov == v && oi < i)) { v = ov; i = oi; }
    }
}

// the largest of v[0..n) among the entries with open[.] != 0 (the lowest index among equals; n when none is open)
__device__ __forceinline__ int wave_best_open(const float* v, const unsigned char* open, int n, int lane) {
    float bv = -INFINITY;
    int bi = n;
    for (int e = lane; e < n; e += kWave)
        if (open[e] && (bi == n || v[e] > bv)) { bv = v[e]; bi = e; }
    wave_argmax(bv, bi);
    return bi;
}

// One wave a token.  From the router's logits z [T, E] (float32):
//   s = softmax(z) over all E outputs;  c = s + correction  (the choice's scores; correction may be null)
//   the E outputs form n_groups equal groups of neighbours; a group's score is its largest c; outputs outside the
//   `keep` best groups cannot be chosen (n_groups <= 1 or keep >= n_groups: all can)
//   choice[t, j] = the j-th largest c that can be chosen (the lowest index among equals), j < top
//   weight[t, j] = s[choice] / (sum_j s[choice_j] + 1e-20) * scale
// The caller sees to it that the kept groups hold at least `top` outputs.
__global__ __launch_bounds__(kWave) void moe_router_choose_kernel(const float* __restrict__ z, const float* __restrict__ correction,
                                                                  int E, int n_groups, int keep, int top, float scale,
                                                                  int* __restrict__ choice, float* __restrict__ weight) {
    __shared__ float s[kMoeMaxExperts], c[kMoeMaxExperts], gbest[kMoeMaxExperts], picked_s[kMoeMaxExperts];
    __shared__ int picked[kMoeMaxExperts];
    __shared__ unsigned char open[kMoeMaxExperts], gopen[kMoeMaxExperts];
    const int t = blockIdx.x, lane = threadIdx.x;
    const float* zr = z + (size_t)t * E;
    float m = -INFINITY;
    for (int e = lane; e < E; e += kWave) { const float v = zr[e]; s[e] = v; m = fmaxf(m, v); }
    m = wave_max(m);
    float sum = 0.f;
    for (int e = lane; e < E; e += kWave) { const float v = expf(s[e] - m); s[e] = v; sum += v; }
    sum = wave_sum(sum);
    for (int e = lane; e < E; e += kWave) {
        const float v = s[e] / sum;
        s[e] = v;
        c[e] = correction ? v + correction[e] : v;
        open[e] = 1;
    }
    __syncthreads();
    if (n_groups > 1 && keep < n_groups) {
        const int size = E / n_groups;
        for (int g = lane; g < n_groups; g += kWave) {
            float b = c[g * size];
            for (int j = 1; j < size; ++j) b = fmaxf(b, c[g * size + j]);
            gbest[g] = b;
            gopen[g] = 1;
        }
        __syncthreads();
        for (int r = 0; r < keep; ++r) {                     // the best group that is still open is kept and closed
            const int g = wave_best_open(gbest, gopen, n_groups, lane);
            __syncthreads();
            if (lane == 0 && g < n_groups) gopen[g] = 0;
            __syncthreads();
        }
        for (int e = lane; e < E; e += kWave) open[e] = gopen[e / size] ? 0 : 1;     // (what is still open was not kept)
        __syncthreads();
    }
    float total = 0.f;
    for (int j = 0; j < top; ++j) {
        const int e = min(wave_best_open(c, open, E, lane), E - 1);
        __syncthreads();
        if (lane == 0) { open[e] = 0; picked[j] = e; picked_s[j] = s[e]; }
        __syncthreads();
        total += s[e];
    }
    const float f = scale / (total + 1e-20f);
    for (int j = lane; j < top; j += kWave) {
        choice[(size_t)t * top + j] = picked[j];
        weight[(size_t)t * top + j] = picked_s[j] * f;
    }
}

LLOGOS_EXPORT int llogos_moe_router_choose(const float* z, const float* correction, int T, int E, int n_groups, int keep, int top,
                                           float scale, int* choice, float* weight, hipStream_t stream) {
    if (T <= 0 || E <= 0 || E > kMoeMaxExperts || top <= 0 || top > E) return LLOGOS_BAD_ARGUMENT;
    if (n_groups > 1 && (E % n_groups || keep < 1 || (long long)min(keep, n_groups) * (E / n_groups) < top)) return LLOGOS_BAD_ARGUMENT;
    moe_router_choose_kernel<<<T, kWave, 0, stream>>>(z, correction, E, n_groups, keep, top, scale, choice, weight);
    return LLOGOS_LAUNCH_CHECK();
}

// out[t, :] = sum_j weight[t, j] * row_j + (sum of the parts of shared[t, :]), with row_j = y[where[t * top + j], :] when
// choice[t, j] < n_real and the token's own row a[t, :] otherwise (a router output without matrices returns its input).
// y float32 [P, W]; a [T, lda] of any storage type; shared float32 [(parts,) T, W] or null.
template <typename TA>
__global__ void moe_combine_weighted_kernel(float* __restrict__ out, const float* __restrict__ y, const int* __restrict__ where,
                                            const int* __restrict__ choice, const float* __restrict__ weight, int top, int n_real,
                                            const TA* __restrict__ a, int lda, const float* __restrict__ shared_rows, int parts,
                                            size_t part_stride, int T, int W) {
    const int t = blockIdx.x;
    for (int col = blockIdx.y * blockDim.x + threadIdx.x; col < W; col += gridDim.y * blockDim.x) {
        float v = 0.f;
        for (int j = 0; j < top; ++j) {
            const int p = t * top + j;
            const float row = choice[p] < n_real ? y[(size_t)where[p] * W + col] : load_f32(a + (size_t)t * lda + col);
            v = fmaf(weight[p], row, v);
        }
        if (shared_rows) {
            float sh = shared_rows[(size_t)t * W + col];
            for (int q = 1; q < parts; ++q) sh += shared_rows[q * part_stride + (size_t)t * W + col];
            v += sh;
        }
        out[(size_t)t * W + col] = v;
    }
}

LLOGOS_EXPORT int llogos_moe_combine_weighted(float* out, const float* y, const int* where, const int* choice, const float* weight,
                                              int top, int n_real, const void* a, int a_dtype, int lda, const float* shared_rows,
                                              int parts, long long part_stride, int T, int W, hipStream_t stream) {
    if (T <= 0 || W <= 0 || top <= 0 || parts < 1 || lda < W || n_real < 0) return LLOGOS_BAD_ARGUMENT;
    const int threads = 256;
    dim3 grid(T, (W + threads - 1) / threads);
    if (a_dtype == DT_F32)
        moe_combine_weighted_kernel<float><<<grid, threads, 0, stream>>>(out, y, where, choice, weight, top, n_real, (const float*)a, lda,
                                                                         shared_rows, parts, (size_t)part_stride, T, W);
    else if (a_dtype == DT_BF16)
        moe_combine_weighted_kernel<bf16_t><<<grid, threads, 0, stream>>>(out, y, where, choice, weight, top, n_real, (const bf16_t*)a, lda,
                                                                          shared_rows, parts, (size_t)part_stride, T, W);
    else return LLOGOS_BAD_ARGUMENT;
    return LLOGOS_LAUNCH_CHECK();
}

// ---------------------------------------------------------------- bfloat16 on the matrix cores
// The same product with v_mfma_f32_16x16x32_bf16: the first operand holds 16 rows of the expert's matrix, the
// second 16 sorted rows of activations, so that a lane ends with four neighbouring outputs of one row:
// D[n = 4 g + r][m = c] for lane (c = lane & 15, g = lane >> 4).  A lane's share of an operand is 8 values of k,
// 16 bytes.  Two forms:
//   few rows  tiles of 16 sorted rows; a block of four waves owns 16 rows of the matrix, its waves take the
//             steps of 32 k in turn (together whole cache lines), straight from memory into operands, and LDS
//             adds the four waves' sums in order;
//   tiles     64 or 128 sorted rows x 128 rows of the matrix with v_mfma_f32_32x32x16_bf16, stages of 64 k
//             through LDS (swizzled rows of 128 bytes), the next stage's loads in registers meanwhile.
// Sums depend on k's order alone, as above.  K must be a multiple of 8 and N of 4.
typedef __bf16 moe_bf16x8 __attribute__((ext_vector_type(8)));
typedef float moe_f32x4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ moe_bf16x8 moe_frag(const bf16_t* p) {
    return __builtin_bit_cast(moe_bf16x8, *reinterpret_cast<const uint4*>(p));
}
__device__ __forceinline__ moe_bf16x8 moe_zero() { return __builtin_bit_cast(moe_bf16x8, make_uint4(0, 0, 0, 0)); }

__device__ __forceinline__ void moe_store4(float* p, float a, float b, float c, float d) {
    *reinterpret_cast<float4*>(p) = make_float4(a, b, c, d);
}
__device__ __forceinline__ void moe_store4(bf16_t* p, float a, float b, float c, float d) {
    uint2 u;
    u.x = (uint32_t)f32_to_bf16(a) | ((uint32_t)f32_to_bf16(b) << 16);
    u.y = (uint32_t)f32_to_bf16(c) | ((uint32_t)f32_to_bf16(d) << 16);
    *reinterpret_cast<uint2*>(p) = u;
}

__device__ __forceinline__ void moe_store2(float* p, float a, float b) { *reinterpret_cast<float2*>(p) = make_float2(a, b); }
__device__ __forceinline__ void moe_store2(bf16_t* p, float a, float b) {
    *reinterpret_cast<uint32_t*>(p) = (uint32_t)f32_to_bf16(a) | ((uint32_t)f32_to_bf16(b) << 16);
}

// which tile of `rows` sorted rows is this block's: expert, first row, end of the expert's segment (expert -1: none)
__device__ __forceinline__ void moe_find_tile(const int* __restrict__ seg, int E, int rows, int tile, int& expert, int& first, int& end) {
    expert = -1; first = 0; end = 0;
    for (int e = 0; e < E; ++e) {
        const int lo = seg[e], hi = seg[e + 1];
        const int tiles = (hi - lo + rows - 1) / rows;
        if (tile < tiles) { expert = e; first = lo + tile * rows; end = hi; return; }
        tile -= tiles;
    }
}

template <typename TO>
__global__ __launch_bounds__(256) void moe_few_kernel(TO* __restrict__ out, const bf16_t* __restrict__ a, const bf16_t* __restrict__ w,
                                                      const int* __restrict__ order, const int* __restrict__ seg, int E, int top,
                                                      int gather, int N, int K, int lda, int act, float scale) {
    __shared__ float red[3][kWave][4];
    __shared__ int s_tile[3];
    if (threadIdx.x == 0) moe_find_tile(seg, E, 16, blockIdx.y, s_tile[0], s_tile[1], s_tile[2]);
    __syncthreads();
    const int e = s_tile[0], m0 = s_tile[1], m_end = s_tile[2];
    if (e < 0) return;
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    const int c = lane & 15, g = lane >> 4;
    const int n0 = blockIdx.x * 16;
    const int m = m0 + c;
    const bf16_t* arow = m < m_end ? a + (size_t)(gather ? order[m] / top : m) * lda + 8 * g : nullptr;
    const bf16_t* wrow = n0 + c < N ? w + ((size_t)e * N + n0 + c) * K + 8 * g : nullptr;
    moe_f32x4 acc = {0.f, 0.f, 0.f, 0.f};
    const int steps = (K + 31) / 32;
#pragma unroll 4
    for (int s = wave; s < steps; s += 4) {
        const int k = 32 * s;
        const bool in = k + 8 * g < K;
        const moe_bf16x8 wf = (wrow && in) ? moe_frag(wrow + k) : moe_zero();
        const moe_bf16x8 af = (arow && in) ? moe_frag(arow + k) : moe_zero();
        acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf, af, acc, 0, 0, 0);
    }
    if (wave > 0) {
#pragma unroll
        for (int r = 0; r < 4; ++r) red[wave - 1][lane][r] = acc[r];
    }
    __syncthreads();
    if (wave > 0) return;
    float v[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        v[r] = ((acc[r] + red[0][lane][r]) + red[1][lane][r]) + red[2][lane][r];
        if (act == 1) { v[r] = fmaxf(v[r], 0.f); v[r] *= v[r]; }
        if (act != 2) v[r] *= scale;
    }
    const int n = n0 + 4 * g;
    if (m < m_end && n < N) {
        if (act == 2) moe_store2(out + (size_t)m * (N / 2) + n / 2, moe_gated(v[0], v[1]) * scale, moe_gated(v[2], v[3]) * scale);
        else moe_store4(out + (size_t)m * N + n, v[0], v[1], v[2], v[3]);
    }
}

constexpr int kMoeBK = 64;      // LDS rows of 64 values of k: 128 bytes, eight pieces of 16
typedef float moe_f32x16 __attribute__((ext_vector_type(16)));

// where piece `oct` (8 values of k) of row `row` lies in an LDS tile: the eight pieces of a row are swizzled so
// that the 32 rows an operand read touches spread over all banks
__device__ __forceinline__ int moe_lds_at(int row, int oct) { return row * kMoeBK + ((oct ^ ((row >> 1) & 7)) << 3); }

// v_mfma_f32_32x32x16_bf16: an operand is 32 rows x 16 k, lane l holding row l & 31 and k 8 (l >> 5) .. + 7; the
// rows of the expert's matrix are the first operand and the sorted rows the second, so a lane ends with the sums
// of one sorted row (l & 31) for 4 x 4 neighbouring columns: entry 4 q + e is column 8 q + 4 (l >> 5) + e.
template <int BM, int BN, typename TO>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(3, 3))) void moe_tiles_kernel(
        TO* __restrict__ out, const bf16_t* __restrict__ a, const bf16_t* __restrict__ w, const int* __restrict__ order,
        const int* __restrict__ seg, int E, int top, int gather, int N, int K, int lda, int act, float scale) {
    constexpr int CA = BM * 8 / 256, CW = BN * 8 / 256;           // 16-byte pieces a thread copies a stage
    constexpr int WN = BM == 128 ? BN / 2 : BN / 4, NT = WN / 32, MT = 2;     // a wave's part: 64 rows x WN columns of the tile
    __shared__ __attribute__((aligned(16))) bf16_t As[BM * kMoeBK];
    __shared__ __attribute__((aligned(16))) bf16_t Ws[BN * kMoeBK];
    __shared__ int src_row[BM];
    __shared__ int s_tile[3];
    const int tid = threadIdx.x;
    if (tid == 0) moe_find_tile(seg, E, BM, blockIdx.y, s_tile[0], s_tile[1], s_tile[2]);
    __syncthreads();
    const int e = s_tile[0], m0 = s_tile[1], m_end = s_tile[2];
    if (e < 0) return;
    if (tid < BM) {
        const int r = m0 + tid;
        src_row[tid] = r < m_end ? (gather ? order[r] / top : r) : -1;
    }
    __syncthreads();
    const int lane = tid & (kWave - 1), wave = tid / kWave;
    const int r32 = lane & 31, h = lane >> 5;
    const int wm = BM == 128 ? wave >> 1 : 0, wn = BM == 128 ? wave & 1 : wave;
    const int n0 = blockIdx.x * BN;
    const bf16_t* we = w + (size_t)e * N * K;

    const bf16_t* pa[CA];
    const bf16_t* pw[CW];
    int ka[CA], kw[CW], la[CA], lw[CW];
#pragma unroll
    for (int j = 0; j < CA; ++j) {
        const int q = tid + 256 * j, row = q >> 3;
        ka[j] = (q & 7) * 8;
        la[j] = moe_lds_at(row, q & 7);
        pa[j] = src_row[row] >= 0 ? a + (size_t)src_row[row] * lda + ka[j] : nullptr;
    }
#pragma unroll
    for (int j = 0; j < CW; ++j) {
        const int q = tid + 256 * j, row = q >> 3;
        kw[j] = (q & 7) * 8;
        lw[j] = moe_lds_at(row, q & 7);
        pw[j] = n0 + row < N ? we + (size_t)(n0 + row) * K + kw[j] : nullptr;
    }
    uint4 ra[CA], rw[CW];
    auto fetch = [&](int k0) {
#pragma unroll
        for (int j = 0; j < CA; ++j)
            ra[j] = (pa[j] && k0 + ka[j] < K) ? *reinterpret_cast<const uint4*>(pa[j] + k0) : make_uint4(0, 0, 0, 0);
#pragma unroll
        for (int j = 0; j < CW; ++j)
            rw[j] = (pw[j] && k0 + kw[j] < K) ? *reinterpret_cast<const uint4*>(pw[j] + k0) : make_uint4(0, 0, 0, 0);
    };
    moe_f32x16 acc[NT][MT];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[nt][mt][v] = 0.f;

    fetch(0);
    for (int k0 = 0; k0 < K; k0 += kMoeBK) {
#pragma unroll
        for (int j = 0; j < CA; ++j) *reinterpret_cast<uint4*>(As + la[j]) = ra[j];
#pragma unroll
        for (int j = 0; j < CW; ++j) *reinterpret_cast<uint4*>(Ws + lw[j]) = rw[j];
        __syncthreads();
        if (k0 + kMoeBK < K) fetch(k0 + kMoeBK);
#pragma unroll
        for (int ks = 0; ks < kMoeBK / 16; ++ks) {
            moe_bf16x8 af[MT], wf[NT];
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) af[mt] = moe_frag(As + moe_lds_at(wm * 64 + mt * 32 + r32, 2 * ks + h));
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) wf[nt] = moe_frag(Ws + moe_lds_at(wn * WN + nt * 32 + r32, 2 * ks + h));
#pragma unroll
            for (int nt = 0; nt < NT; ++nt)
#pragma unroll
                for (int mt = 0; mt < MT; ++mt)
                    acc[nt][mt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(wf[nt], af[mt], acc[nt][mt], 0, 0, 0);
        }
        __syncthreads();
    }
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
        const int m = m0 + wm * 64 + mt * 32 + r32;
        if (m >= m_end) continue;
#pragma unroll
        for (int nt = 0; nt < NT; ++nt)
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const int n = n0 + wn * WN + nt * 32 + 8 * q + 4 * h;
                if (n >= N) continue;
                float v[4];
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    v[r] = acc[nt][mt][4 * q + r];
                    if (act == 1) { v[r] = fmaxf(v[r], 0.f); v[r] *= v[r]; }
                    if (act != 2) v[r] *= scale;
                }
                if (act == 2) moe_store2(out + (size_t)m * (N / 2) + n / 2, moe_gated(v[0], v[1]) * scale, moe_gated(v[2], v[3]) * scale);
                else moe_store4(out + (size_t)m * N + n, v[0], v[1], v[2], v[3]);
            }
    }
}

// form 0: few rows (tiles of 16); 1: tiles of 64 rows; 2: tiles of 128 rows.  -2 for shapes these do not take.
LLOGOS_EXPORT int llogos_moe_product_bf16(void* out, int out_dtype, const void* a, const void* w, const int* order, const int* seg,
                                          int E, int top, int gather, int P, int N, int K, int lda, int act, float scale, int form,
                                          hipStream_t stream) {
    if (P <= 0 || N <= 0 || K <= 0 || E <= 0 || top <= 0 || lda < K || act < 0 || act > 2 || form < 0 || form > 2) return LLOGOS_BAD_ARGUMENT;
    if ((K % 8) || (N % 4) || (lda % 8) || ((uintptr_t)a % 16) || ((uintptr_t)w % 16) || ((uintptr_t)out % 16)) return LLOGOS_UNSUPPORTED;
    if (out_dtype != DT_F32 && out_dtype != DT_BF16) return LLOGOS_BAD_ARGUMENT;
    const int rows = form == 0 ? 16 : (form == 1 ? 64 : 128);
    const int row_tiles = (P + rows - 1) / rows + E;
#define MOE_GO(KERNEL, NB, TO) KERNEL<<<dim3((N + NB - 1) / NB, row_tiles), 256, 0, stream>>>((TO*)out, (const bf16_t*)a, (const bf16_t*)w, \
        order, seg, E, top, gather, N, K, lda, act, scale)
    if (form == 0) { if (out_dtype == DT_F32) MOE_GO(moe_few_kernel<float>, 16, float); else MOE_GO(moe_few_kernel<bf16_t>, 16, bf16_t); }
    else if (form == 1) { if (out_dtype == DT_F32) MOE_GO((moe_tiles_kernel<64, 128, float>), 128, float); else MOE_GO((moe_tiles_kernel<64, 128, bf16_t>), 128, bf16_t); }
    else { if (out_dtype == DT_F32) MOE_GO((moe_tiles_kernel<128, 128, float>), 128, float); else MOE_GO((moe_tiles_kernel<128, 128, bf16_t>), 128, bf16_t); }
#undef MOE_GO
    return LLOGOS_LAUNCH_CHECK();
}
