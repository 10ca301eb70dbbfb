// Kernels for parts that keep a fixed-size state for each sequence: a short causal
// convolution over time, the mix of a token with the one before it, and a linear recurrence
// with a matrix state per head.  State rows are indexed by cache slot (slots[seq]); a row
// is zero when its slot is handed out.  All arithmetic is 32-bit; inputs and outputs may be
// stored as float or bfloat16.
#include "common.h"

// ---------------------------------------------------------------- short causal convolution
// out[t, c] = [h[t, c] +] sum_j w[c, j] * h_(t - taps + 1 + j)[c]   (w[c, taps - 1] multiplies token t;
// the input itself is added when add_input is set; rows of h lie ldh values apart)
// Rows before the step's first token of a sequence come from the sequence's state
// [taps - 1, W], whose row i holds the input at position (length - (taps - 1) + i); positions
// before 0 count as zero.  cu (token offset of each sequence in the step) may be null: then
// every sequence brings one token, and the thread that computes a channel also shifts the
// channel's state (update_state).  For longer steps conv_state_kernel runs afterwards.
constexpr int kMaxTaps = 16;

template <typename TO>
__global__ void causal_conv_kernel(TO* __restrict__ out, const float* __restrict__ h, const float* __restrict__ w,
                                   float* __restrict__ state, const int* __restrict__ slots,
                                   const int* __restrict__ tok_seq, const int* __restrict__ tok_pos,
                                   const int* __restrict__ cu, int W, int ldh, int taps, int update_state, int add_input,
                                   int T, int per_block, const float* __restrict__ bias, size_t state_stride) {
  // a block takes per_block tokens in turn (a long step's blocks are otherwise too short to hide their loads)
  for (int t = blockIdx.x * per_block; t < min(T, (int)(blockIdx.x + 1) * per_block); ++t) {
    const int seq = tok_seq[t], pos = tok_pos[t];
    const int before = cu ? t - cu[seq] : 0;                 // tokens of this sequence earlier in the step
    float* st = state + (size_t)slots[seq] * state_stride;
    for (int c = blockIdx.y * blockDim.x + threadIdx.x; c < W; c += gridDim.y * blockDim.x) {
        const float* wc = w + (size_t)c * taps;
        const float x0 = h[(size_t)t * ldh + c];
        float acc = x0 * wc[taps - 1];
        float old[kMaxTaps];
#pragma unroll
        for (int j = 1; j < kMaxTaps; ++j) {
            if (j < taps) {
                float v = 0.f;
                if (j <= before) v = h[(size_t)(t - j) * ldh + c];
                else if (pos - j >= 0) v = st[(size_t)(taps - 1 + before - j) * W + c];
                old[j] = v;
                acc = fmaf(wc[taps - 1 - j], v, acc);
            }
        }
        if (bias) acc += bias[c];
        store_f32(out + (size_t)t * W + c, add_input ? x0 + acc : acc);
        if (update_state) {                                  // one token a sequence: row i <- row i + 1, last <- this token
#pragma unroll
            for (int j = 1; j < kMaxTaps; ++j)
                if (j < taps) st[(size_t)(taps - 1 - j) * W + c] = (j == 1) ? x0 : old[j - 1];
        }
    }
  }
}

// The same for steps of many tokens, four neighbouring channels a thread with 16-byte loads and stores (a thread's
// loads are all asked for before the first sum): a long step is bound by how many requests its threads have in
// flight, not by bytes.  For W, ldh multiples of 4 and 16-byte aligned rows; the state is not written here.
__device__ __forceinline__ void conv_store4(float* p, float4 v) { *reinterpret_cast<float4*>(p) = v; }
__device__ __forceinline__ void conv_store4(bf16_t* p, float4 v) {
    uint2 u;
    u.x = (uint32_t)f32_to_bf16(v.x) | ((uint32_t)f32_to_bf16(v.y) << 16);
    u.y = (uint32_t)f32_to_bf16(v.z) | ((uint32_t)f32_to_bf16(v.w) << 16);
    *reinterpret_cast<uint2*>(p) = u;
}

constexpr int kConvWideTokens = 8;      // tokens a block of the wide kernel takes one after the other with its weights in LDS

template <typename TO>
__global__ void causal_conv_wide_kernel(TO* __restrict__ out, const float* __restrict__ h, const float* __restrict__ w,
                                        const float* __restrict__ state, const int* __restrict__ slots,
                                        const int* __restrict__ tok_seq, const int* __restrict__ tok_pos,
                                        const int* __restrict__ cu, int T, int W, int ldh, int taps, int add_input,
                                        const float* __restrict__ bias, size_t state_stride) {
    // the block's weights (4 * blockDim channels x taps, one run of memory) go through LDS: read channel by
    // channel from memory they would cost a cache line a lane and load
    extern __shared__ float wl[];
    const int c0 = 4 * blockIdx.y * blockDim.x;
    const int n_w = min(4 * (int)blockDim.x, W - c0) * taps;
    for (int i = threadIdx.x; i < n_w; i += blockDim.x) wl[i] = w[(size_t)c0 * taps + i];
    __syncthreads();
    const int c = c0 + 4 * threadIdx.x;
    if (c >= W) return;
    const float* wc = wl + 4 * threadIdx.x * taps;
    const int t_end = min(T, (int)(blockIdx.x + 1) * kConvWideTokens);
#pragma unroll 2
    for (int t = blockIdx.x * kConvWideTokens; t < t_end; ++t) {
        const int seq = tok_seq[t], pos = tok_pos[t];
        const int before = t - cu[seq];
        const float* st = state + (size_t)slots[seq] * state_stride;
        float4 x[kMaxTaps];
#pragma unroll
        for (int j = 0; j < kMaxTaps; ++j) {
            if (j < taps) {
                float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
                if (j <= before) v = *reinterpret_cast<const float4*>(h + (size_t)(t - j) * ldh + c);
                else if (pos - j >= 0) v = *reinterpret_cast<const float4*>(st + (size_t)(taps - 1 + before - j) * W + c);
                x[j] = v;
            }
        }
        // (the sums in the order of the one-channel kernel: the present token's product first, then the rows before it)
        float4 acc;
        acc.x = x[0].x * wc[0 * taps + taps - 1];
        acc.y = x[0].y * wc[1 * taps + taps - 1];
        acc.z = x[0].z * wc[2 * taps + taps - 1];
        acc.w = x[0].w * wc[3 * taps + taps - 1];
#pragma unroll
        for (int j = 1; j < kMaxTaps; ++j) {
            if (j < taps) {
                const int k = taps - 1 - j;
                acc.x = fmaf(wc[0 * taps + k], x[j].x, acc.x);
                acc.y = fmaf(wc[1 * taps + k], x[j].y, acc.y);
                acc.z = fmaf(wc[2 * taps + k], x[j].z, acc.z);
                acc.w = fmaf(wc[3 * taps + k], x[j].w, acc.w);
            }
        }
        if (bias) { acc.x += bias[c]; acc.y += bias[c + 1]; acc.z += bias[c + 2]; acc.w += bias[c + 3]; }
        if (add_input) { acc.x += x[0].x; acc.y += x[0].y; acc.z += x[0].z; acc.w += x[0].w; }
        conv_store4(out + (size_t)t * W + c, acc);
    }
}

// The state after a step of any length: row i <- the input at position new_len - (taps - 1) + i,
// from this step's rows or from the old state.  A thread owns a channel of a sequence and
// reads all it needs before it writes.
__global__ void conv_state_kernel(const float* __restrict__ h, float* __restrict__ state, const int* __restrict__ slots,
                                  const int* __restrict__ cu, int W, int ldh, int taps, size_t state_stride) {
    const int seq = blockIdx.x;
    const int first = cu[seq], count = cu[seq + 1] - first;
    float* st = state + (size_t)slots[seq] * state_stride;
    for (int c = blockIdx.y * blockDim.x + threadIdx.x; c < W; c += gridDim.y * blockDim.x) {
        float keep[kMaxTaps];
#pragma unroll
        for (int i = 0; i < kMaxTaps - 1; ++i) {
            if (i < taps - 1) {
                const int back = taps - 1 - i;               // this row is the input `back` tokens before the new end
                keep[i] = back <= count ? h[(size_t)(first + count - back) * ldh + c] : st[(size_t)(i + count) * W + c];
            }
        }
#pragma unroll
        for (int i = 0; i < kMaxTaps - 1; ++i)
            if (i < taps - 1) st[(size_t)i * W + c] = keep[i];
    }
}

LLOGOS_EXPORT int llogos_causal_conv(void* out, int out_dtype, const float* h, const float* w, float* state,
                                     const int* slots, const int* tok_seq, const int* tok_pos, const int* cu,
                                     int T, int B, int W, int ldh, int taps, int add_input, const float* bias,
                                     long long slot_stride, hipStream_t stream) {
    // bias [W] (or null) is added to every output; slot_stride: floats between two slots' state rows (0: taps - 1 rows of W)
    if (T <= 0 || B <= 0 || W <= 0 || ldh < W || taps < 1 || taps > kMaxTaps) return LLOGOS_BAD_ARGUMENT;
    if (slot_stride != 0 && slot_stride < (long long)(taps - 1) * W) return LLOGOS_BAD_ARGUMENT;
    const size_t state_stride = slot_stride ? (size_t)slot_stride : (size_t)(taps - 1) * W;
    if (!cu && T != B) return LLOGOS_BAD_ARGUMENT;
    const int threads = 256;
    const int by = (W + threads - 1) / threads;
    const int per_block = 1;
    dim3 grid((T + per_block - 1) / per_block, by);
    const int fused = cu ? 0 : 1;
    const bool wide = cu && T > 64 && (W % 4) == 0 && (ldh % 4) == 0 && ((uintptr_t)h % 16) == 0 && ((uintptr_t)out % 16) == 0 &&
                      ((uintptr_t)state % 16) == 0;
    if (wide) {
        const int wthreads = 128;
        dim3 wgrid((T + kConvWideTokens - 1) / kConvWideTokens, (W / 4 + wthreads - 1) / wthreads);
        const size_t wlds = (size_t)wthreads * 4 * taps * sizeof(float);
        if (out_dtype == DT_F32)
            causal_conv_wide_kernel<float><<<wgrid, wthreads, wlds, stream>>>((float*)out, h, w, state, slots, tok_seq, tok_pos, cu, T, W, ldh, taps, add_input, bias, state_stride);
        else if (out_dtype == DT_BF16)
            causal_conv_wide_kernel<bf16_t><<<wgrid, wthreads, wlds, stream>>>((bf16_t*)out, h, w, state, slots, tok_seq, tok_pos, cu, T, W, ldh, taps, add_input, bias, state_stride);
        else
            return LLOGOS_BAD_ARGUMENT;
        if (taps > 1) conv_state_kernel<<<dim3(B, by), threads, 0, stream>>>(h, state, slots, cu, W, ldh, taps, state_stride);
        return LLOGOS_LAUNCH_CHECK();
    }
    if (out_dtype == DT_F32)
        causal_conv_kernel<float><<<grid, threads, 0, stream>>>((float*)out, h, w, state, slots, tok_seq, tok_pos, cu, W, ldh, taps, fused, add_input, T, per_block, bias, state_stride);
    else if (out_dtype == DT_BF16)
        causal_conv_kernel<bf16_t><<<grid, threads, 0, stream>>>((bf16_t*)out, h, w, state, slots, tok_seq, tok_pos, cu, W, ldh, taps, fused, add_input, T, per_block, bias, state_stride);
    else
        return LLOGOS_BAD_ARGUMENT;
    if (cu && taps > 1) conv_state_kernel<<<dim3(B, by), threads, 0, stream>>>(h, state, slots, cu, W, ldh, taps, state_stride);
    return LLOGOS_LAUNCH_CHECK();
}

// ---------------------------------------------------------------- mix with the token before
// out[s][t, c] = h[t, c] + (h_prev[c] - h[t, c]) * mu[s][c] for s < n_mix, where h_prev is the
// row before in the step, or, for a sequence's first row of the step, the sequence's state row
// `prev` (zero at the start of a sequence).  The state is not written here: the recurrence
// kernel, which runs after every reader, stores the step's last row.
template <typename TO>
__global__ void token_shift_kernel(TO* __restrict__ out, const float* __restrict__ h, const float* __restrict__ mu,
                                   const float* __restrict__ state, size_t state_stride, const int* __restrict__ slots,
                                   const int* __restrict__ tok_seq, const int* __restrict__ cu, int T, int W, int n_mix) {
    const int t = blockIdx.x;
    const int seq = tok_seq[t];
    const bool first = cu ? (t == cu[seq]) : true;
    const float* prev = first ? state + (size_t)slots[seq] * state_stride : h + (size_t)(t - 1) * W;
    for (int c = blockIdx.y * blockDim.x + threadIdx.x; c < W; c += gridDim.y * blockDim.x) {
        const float x = h[(size_t)t * W + c];
        const float d = prev[c] - x;
        for (int s = 0; s < n_mix; ++s)
            store_f32(out + ((size_t)s * T + t) * W + c, fmaf(d, mu[(size_t)s * W + c], x));
    }
}

LLOGOS_EXPORT int llogos_token_shift(void* out, int out_dtype, const float* h, const float* mu, const float* state,
                                     long long state_stride, const int* slots, const int* tok_seq, const int* cu,
                                     int T, int W, int n_mix, hipStream_t stream) {
    if (T <= 0 || W <= 0 || n_mix <= 0) return LLOGOS_BAD_ARGUMENT;
    const int threads = 256;
    dim3 grid(T, (W + threads - 1) / threads);
    if (out_dtype == DT_F32)
        token_shift_kernel<float><<<grid, threads, 0, stream>>>((float*)out, h, mu, state, (size_t)state_stride, slots, tok_seq, cu, T, W, n_mix);
    else if (out_dtype == DT_BF16)
        token_shift_kernel<bf16_t><<<grid, threads, 0, stream>>>((bf16_t*)out, h, mu, state, (size_t)state_stride, slots, tok_seq, cu, T, W, n_mix);
    else
        return LLOGOS_BAD_ARGUMENT;
    return LLOGOS_LAUNCH_CHECK();
}

// ---------------------------------------------------------------- recurrence with a matrix state per head
// Per sequence and head, with S [key channel i, value channel j] carried from token to token:
//     o_t[j] = sum_i r_t[i] * (S[i, j] + u[i] * k_t[i] * v_t[j])
//     S[i, j] <- w_t[i] * S[i, j] + k_t[i] * v_t[j],      w_t[i] = exp(-exp(d_t[i] + w0[i]))
// then y_t = o_t / sqrt(mean_j(o_t^2) + eps) * g[j] * silu(gate_t[j]) over the head's D channels.
// r, k, v, d, gate are float [T, H * D] (row stride ld), r, k, v, gate maybe as `parts` partial sums
// (part_stride floats apart) and d as d_parts; y is [T, H * D] in the output type.
//
// One block per (sequence, head).  Thread (j, part) keeps rows [part * rpt, (part + 1) * rpt) of
// column j of S in registers; the P <= 16 parts of a column are neighbouring lanes of a row of 16 and add
// their sums with cross-lane moves inside the vector unit, so the token loop needs no barrier and
// no trip through LDS.  Few rows a thread (4 where a block of D * P threads allows) keep a token's
// chain of dependent operations short: a long prompt of one sequence is a loop of as many steps as
// it has tokens, on as many blocks as there are heads.  Tokens go through LDS in chunks: a chunk's
// r, k, v, d, gate are asked for (into registers) while the chunk before is worked on, stored to LDS
// (the decay made on the way), and the chunk's outputs are normed, gated and stored by all waves.
// The state is stored [H][j][i] (a thread's rows in a row).  After its last token the block with
// head 0 copies the step's last mixer input row to the sequence's `prev` state (the token-shift
// kernel has read the old one by then).
constexpr int kScanChunk = 16;
constexpr int kScanAhead = 4;          // values of each array a thread asks for ahead (chunk <= kScanAhead * P tokens)

__device__ __forceinline__ float dpp_add(float x, int ctrl_index) {
    const int v = __float_as_int(x);
    int o;
    switch (ctrl_index) {
        case 0: o = __builtin_amdgcn_update_dpp(0, v, 0xB1, 0xf, 0xf, false); break;     // lane ^ 1 within a quad
        case 1: o = __builtin_amdgcn_update_dpp(0, v, 0x4E, 0xf, 0xf, false); break;     // lane ^ 2 within a quad
        case 2: o = __builtin_amdgcn_update_dpp(0, v, 0x141, 0xf, 0xf, false); break;    // mirror within 8 lanes
        default: o = __builtin_amdgcn_update_dpp(0, v, 0x140, 0xf, 0xf, false); break;   // mirror within 16 lanes
    }
    return x + __int_as_float(o);
}

// PP: parts of a column (a power of two up to 16); EXACT: every thread has exactly RPT rows (D = PP * RPT), read
// as float4s without a bound check.  Both are template arguments so that a token's loop has no branch.
// MODE 0: a sequence's part of the step from the cached state to the cached state.  Long prompts of few
// sequences are cut into segments that run side by side: MODE 1 takes a segment from a zero state and leaves its
// end state and the product of its decays (no outputs); wkv_combine_kernel chains those into every segment's true
// initial state and the sequence's final state, S_init[s + 1] = diag(prod decay_s) S_init[s] + S_local[s]; MODE 2
// runs the segment again from its initial state for the outputs, token by token as MODE 0 would.
template <int RPT, int PP, bool EXACT, int MODE, typename TO>
__global__ void wkv_scan_kernel(TO* __restrict__ y, const float* __restrict__ r, const float* __restrict__ k,
                                const float* __restrict__ v, const float* __restrict__ d, const float* __restrict__ gate,
                                int ld, int parts, size_t part_stride, int d_parts, size_t d_part_stride,
                                const float* __restrict__ w0, const float* __restrict__ u,
                                const float* __restrict__ g, float eps,
                                float* __restrict__ state, size_t state_stride, size_t prev_offset,
                                const float* __restrict__ h_in, int W,
                                const int* __restrict__ slots, const int* __restrict__ cu,
                                int H, int D, int rpt, int chunk, int Dc, float* __restrict__ o_raw,
                                int col_blocks, int n_seg, int seg_len, float* __restrict__ seg_state,
                                float* __restrict__ seg_decay) {
    constexpr int P = PP;
    extern __shared__ float smem[];
    const int seq = blockIdx.x, head = blockIdx.y;
    const int cbi = blockIdx.z % col_blocks, seg = blockIdx.z / col_blocks;
    const int first0 = cu ? cu[seq] : seq, count0 = cu ? cu[seq + 1] - first0 : 1;
    const int first = first0 + (MODE ? seg * seg_len : 0);
    const int count = MODE ? min(seg_len, count0 - seg * seg_len) : count0;
    const int tid = threadIdx.x, nthreads = blockDim.x;
    // the block's columns of S: all D, or, with several blocks a head (long prompts of few sequences: a
    // compute unit issues a token's instructions for all of a block's waves), Dc of them from cbi * Dc on
    const int j = cbi * Dc + tid / P, part = tid % P;
    const bool active = tid / P < Dc && j < D;
    const int i0 = part * rpt;
    float* seg_S = MODE ? seg_state + ((((size_t)seq * n_seg + seg) * H + head) * D + (active ? j : 0)) * D + i0 : nullptr;
    float* seg_P = MODE ? seg_decay + (((size_t)seq * n_seg + seg) * H + head) * D + i0 : nullptr;
    const bool keeps_decay = MODE == 1 && cbi == 0 && tid / P == 0;      // one column's threads keep the decays' product
    if (MODE && count <= 0) {
        if (MODE == 1) {                                   // a segment beyond the sequence's end: nothing added, nothing decayed
#pragma unroll
            for (int m = 0; m < RPT; ++m)
                if (m < rpt && i0 + m < D) {
                    if (active) seg_S[m] = 0.f;
                    if (keeps_decay) seg_P[m] = 1.f;
                }
        }
        return;
    }
    float* s_r = smem;                          // [chunk][D]
    float* s_k = s_r + chunk * D;
    float* s_w = s_k + chunk * D;
    float* s_v = s_w + chunk * D;
    float* s_g = s_v + chunk * D;
    float* s_o = s_g + chunk * D;
    float* row = state + (size_t)slots[seq] * state_stride;
    float* S = row + ((size_t)head * D + (active ? j : 0)) * D + i0;
    const size_t col0 = (size_t)head * D;

    float s[RPT], ur[RPT], pw[RPT];
#pragma unroll
    for (int m = 0; m < RPT; ++m) {
        const bool ok = active && m < rpt && i0 + m < D;
        s[m] = !ok || MODE == 1 ? 0.f : (MODE == 2 ? seg_S[m] : S[m]);
        ur[m] = ok ? u[col0 + i0 + m] : 0.f;
        pw[m] = 1.f;
    }

    // a chunk's values on their way: element e = tid + a * nthreads of the chunk's [n][D]
    float pr[kScanAhead], pk[kScanAhead], pv[kScanAhead], pd[kScanAhead], pg[kScanAhead];
    auto ask = [&](int c0) {
        const int n = min(chunk, count - c0);
#pragma unroll
        for (int a = 0; a < kScanAhead; ++a) {
            const int e = tid + a * nthreads;
            if (e < n * D) {
                const size_t at = (size_t)(first + c0 + e / D) * ld + col0 + e % D;
                float xr = r[at], xk = k[at], xv = v[at], xd = d[at], xg = gate[at];
                for (int q = 1; q < parts; ++q) {            // products that come as partial sums of a split along k
                    xr += r[q * part_stride + at]; xk += k[q * part_stride + at];
                    xv += v[q * part_stride + at]; xg += gate[q * part_stride + at];
                }
                for (int q = 1; q < d_parts; ++q) xd += d[q * d_part_stride + at];
                pr[a] = xr; pk[a] = xk; pv[a] = xv; pd[a] = xd; pg[a] = xg;
            }
        }
    };
    ask(0);
    for (int c0 = 0; c0 < count; c0 += chunk) {
        const int n = min(chunk, count - c0);
        __syncthreads();                        // the chunk before has been normed and stored
#pragma unroll
        for (int a = 0; a < kScanAhead; ++a) {
            const int e = tid + a * nthreads;
            if (e < n * D) {
                s_r[e] = pr[a]; s_k[e] = pk[a]; s_v[e] = pv[a]; s_g[e] = pg[a];
                s_w[e] = expf(-expf(pd[a] + w0[col0 + e % D]));
            }
        }
        __syncthreads();
        if (c0 + chunk < count) ask(c0 + chunk);
        for (int c = 0; c < n; ++c) {
            // (indices into the one LDS array, so that every read is an LDS read whatever the optimizer infers)
            const int at = c * D + i0, o_k = chunk * D, o_w = 2 * chunk * D;
            const float* rr = smem + at;
            const float* kk = smem + o_k + at;
            const float* ww = smem + o_w + at;
            const float vj = active ? smem[3 * chunk * D + c * D + j] : 0.f;
            if (MODE == 1) {                               // the state alone
#pragma unroll
                for (int m = 0; m < RPT; ++m) {
                    if (EXACT || (m < rpt && i0 + m < D)) {
                        s[m] = fmaf(ww[m], s[m], kk[m] * vj);
                        pw[m] *= ww[m];
                    }
                }
                continue;
            }
            float acc = 0.f;
            if (EXACT) {
#pragma unroll
                for (int m = 0; m < RPT; m += 4) {
                    {
                        const float4 r4 = *reinterpret_cast<const float4*>(&smem[at + m]);
                        const float4 k4 = *reinterpret_cast<const float4*>(&smem[o_k + at + m]);
                        const float4 w4 = *reinterpret_cast<const float4*>(&smem[o_w + at + m]);
                        const float rv[4] = {r4.x, r4.y, r4.z, r4.w}, kv4[4] = {k4.x, k4.y, k4.z, k4.w}, wv[4] = {w4.x, w4.y, w4.z, w4.w};
#pragma unroll
                        for (int q = 0; q < 4; ++q) {
                            const float kv = kv4[q] * vj;
                            acc = fmaf(rv[q], fmaf(ur[m + q], kv, s[m + q]), acc);
                            s[m + q] = fmaf(wv[q], s[m + q], kv);
                        }
                    }
                }
            } else {
#pragma unroll
                for (int m = 0; m < RPT; ++m) {
                    if (m < rpt && i0 + m < D) {
                        const float kv = kk[m] * vj;
                        acc = fmaf(rr[m], fmaf(ur[m], kv, s[m]), acc);
                        s[m] = fmaf(ww[m], s[m], kv);
                    }
                }
            }
            if (P >= 2) acc = dpp_add(acc, 0);
            if (P >= 4) acc = dpp_add(acc, 1);
            if (P >= 8) acc = dpp_add(acc, 2);
            if (P >= 16) acc = dpp_add(acc, 3);
            if (active && part == 0) smem[5 * chunk * D + c * D + j] = acc;
        }
        if (MODE == 1) continue;
        __syncthreads();
        if (o_raw) {
            // several blocks a head: the raw outputs of this block's columns; head_norm_gate_kernel norms the head
            for (int e = tid; e < n * Dc; e += nthreads) {
                const int c = e / Dc, jj = cbi * Dc + e % Dc;
                if (jj < D) o_raw[(size_t)(first + c0 + c) * H * D + col0 + jj] = s_o[c * D + jj];
            }
            continue;
        }
        // norm over the head, weight, gate: a wave takes a token at a time
        const int wave = tid / kWave, lane = tid % kWave, nwaves = (nthreads + kWave - 1) / kWave;
        for (int c = wave; c < n; c += nwaves) {
            float ss = 0.f;
            for (int i = lane; i < D; i += kWave) { const float o = s_o[c * D + i]; ss = fmaf(o, o, ss); }
            ss = wave_sum(ss);
            const float inv = 1.0f / sqrtf(ss / (float)D + eps);
            const size_t base = (size_t)(first + c0 + c);
            for (int i = lane; i < D; i += kWave) {
                const float z = s_g[c * D + i];
                const float sg = z / (1.0f + expf(-z));
                store_f32(y + base * (size_t)H * D + col0 + i, s_o[c * D + i] * inv * g[col0 + i] * sg);
            }
        }
    }
#pragma unroll
    for (int m = 0; m < RPT; ++m)
        if (m < rpt && i0 + m < D) {
            if (active && MODE == 0) S[m] = s[m];
            if (active && MODE == 1) seg_S[m] = s[m];
            if (keeps_decay) seg_P[m] = pw[m];
        }
    if (MODE != 1 && head == 0 && blockIdx.z == 0 && h_in) {
        const float* last = h_in + (size_t)(first0 + count0 - 1) * W;
        for (int c = tid; c < W; c += nthreads) row[prev_offset + c] = last[c];
    }
}

// The segments' local end states chained: seg_state[seg] <- the state the segment starts from, and the cached state
// <- the state after the last segment.  One block a (sequence, head); a thread owns elements (j, i) of S.
__global__ void wkv_combine_kernel(float* __restrict__ state, size_t state_stride, const int* __restrict__ slots,
                                   float* __restrict__ seg_state, const float* __restrict__ seg_decay, int H, int D, int n_seg) {
    const int seq = blockIdx.x, head = blockIdx.y;
    float* S = state + (size_t)slots[seq] * state_stride + (size_t)head * D * D;
    for (int e = threadIdx.x; e < D * D; e += blockDim.x) {
        const int i = e % D;
        float cur = S[e];
        for (int sg = 0; sg < n_seg; ++sg) {
            const size_t at = ((size_t)seq * n_seg + sg) * H + head;
            const float local = seg_state[at * D * D + e];
            seg_state[at * D * D + e] = cur;
            cur = fmaf(seg_decay[at * D + i], cur, local);
        }
        S[e] = cur;
    }
}

// y[t, head, :] = o / sqrt(mean(o^2) + eps) * g * silu(gate) over each head's D channels; one wave a (token, head).
template <typename TO>
__global__ void head_norm_gate_kernel(TO* __restrict__ y, const float* __restrict__ o, const float* __restrict__ gate, int ld,
                                      int parts, size_t part_stride, const float* __restrict__ g, float eps, int H, int D, int n) {
    const int item = blockIdx.x * (blockDim.x / kWave) + threadIdx.x / kWave, lane = threadIdx.x % kWave;
    if (item >= n) return;
    const int t = item / H, head = item % H;
    const float* orow = o + (size_t)t * H * D + (size_t)head * D;
    float ss = 0.f;
    for (int i = lane; i < D; i += kWave) ss = fmaf(orow[i], orow[i], ss);
    ss = wave_sum(ss);
    const float inv = 1.0f / sqrtf(ss / (float)D + eps);
    for (int i = lane; i < D; i += kWave) {
        float z = gate[(size_t)t * ld + (size_t)head * D + i];
        for (int q = 1; q < parts; ++q) z += gate[q * part_stride + (size_t)t * ld + (size_t)head * D + i];
        store_f32(y + (size_t)t * H * D + (size_t)head * D + i, orow[i] * inv * g[head * D + i] * (z / (1.0f + expf(-z))));
    }
}

// col_blocks > 1 (with o_raw, float [T, H * D] scratch): a head's columns are shared out over that many blocks
// and the head norm runs as a second kernel.
LLOGOS_EXPORT int llogos_wkv_scan(void* y, int out_dtype, const float* r, const float* k, const float* v, const float* d,
                                  const float* gate, int ld, int parts, long long part_stride, int d_parts,
                                  long long d_part_stride, const float* w0, const float* u, const float* g, float eps,
                                  float* state, long long state_stride, long long prev_offset, const float* h_in, int W,
                                  const int* slots, const int* cu, int B, int H, int D, int T, int col_blocks, float* o_raw,
                                  int n_seg, int seg_len, float* seg_state, float* seg_decay, int rows_hint,
                                  hipStream_t stream) {
    if (n_seg < 1 || (n_seg > 1 && (!cu || seg_len < 1 || !seg_state || !seg_decay))) return LLOGOS_BAD_ARGUMENT;
    if (B <= 0 || H <= 0 || D <= 0 || ld < H * D || parts < 1 || d_parts < 1 || col_blocks < 1 || (col_blocks > 1 && !o_raw)) return LLOGOS_BAD_ARGUMENT;
    // rows a thread: the fewest of 4, 16, 64 with which a column's parts (a power of two, at most 16: one
    // row of lanes) make a block of at most 1024 threads
    // (rows_hint 16: the caller has enough blocks to fill the machine and wants the threads with more rows each,
    // which spend fewer of their instructions on fetching r, k and the decay and on adding up)
    int rpt_max = 0, P = 1;
    for (int cand : {4, 16, 64}) {
        if (cand < rows_hint) continue;
        P = 1;
        while (P * cand < D) P <<= 1;
        if (P <= 16 && (long long)((D * P + kWave - 1) / kWave * kWave) <= 1024) { rpt_max = cand; break; }
    }
    if (!rpt_max) return LLOGOS_UNSUPPORTED;
    const int rpt = (D + P - 1) / P;
    const int Dc = (D + col_blocks - 1) / col_blocks;
    const int threads = (Dc * P + kWave - 1) / kWave * kWave;
    // so that a thread asks for <= kScanAhead values of a chunk's [tokens][D]
    int chunk = kScanChunk;
    while (chunk > 1 && (long long)chunk * D > (long long)kScanAhead * threads) chunk >>= 1;
    if ((long long)chunk * D > (long long)kScanAhead * threads) return LLOGOS_UNSUPPORTED;
    while (chunk > 1 && (size_t)6 * chunk * D * sizeof(float) > 65536) chunk >>= 1;
    const size_t smem = (size_t)6 * chunk * D * sizeof(float);
    if (smem > 65536) return LLOGOS_UNSUPPORTED;
    if (col_blocks == 1) o_raw = nullptr;
    dim3 grid(B, H, col_blocks * n_seg);
#define ARGS(TO) ((TO*)y, r, k, v, d, gate, ld, parts, (size_t)part_stride, d_parts, (size_t)d_part_stride, w0, u, g, eps, \
        state, (size_t)state_stride, (size_t)prev_offset, h_in, W, slots, cu, H, D, rpt, chunk, Dc, o_raw, col_blocks, n_seg, \
        seg_len, seg_state, seg_decay)
    const bool exact = rpt == rpt_max && P * rpt == D;
#define SCAN1(RPT, PP, EX, TO) do { \
        if (n_seg == 1) wkv_scan_kernel<RPT, PP, EX, 0, TO><<<grid, threads, smem, stream>>> ARGS(TO); \
        else { \
            wkv_scan_kernel<RPT, PP, EX, 1, float><<<grid, threads, smem, stream>>> ARGS(float); \
            wkv_combine_kernel<<<dim3(B, H), 256, 0, stream>>>(state, (size_t)state_stride, slots, seg_state, seg_decay, H, D, n_seg); \
            wkv_scan_kernel<RPT, PP, EX, 2, TO><<<grid, threads, smem, stream>>> ARGS(TO); \
        } } while (0)
#define SCAN(RPT, PP, TO) do { if (exact) SCAN1(RPT, PP, true, TO); else SCAN1(RPT, PP, false, TO); } while (0)
#define SCANS(TO) do { \
        if (rpt_max == 4) { if (P == 1) SCAN(4, 1, TO); else if (P == 2) SCAN(4, 2, TO); else if (P == 4) SCAN(4, 4, TO); \
                            else if (P == 8) SCAN(4, 8, TO); else SCAN(4, 16, TO); } \
        else if (rpt_max == 16) { if (P == 1) SCAN(16, 1, TO); else if (P == 2) SCAN(16, 2, TO); else if (P == 4) SCAN(16, 4, TO); \
                                  else if (P == 8) SCAN(16, 8, TO); else SCAN(16, 16, TO); } \
        else { if (P == 4) SCAN(64, 4, TO); else return LLOGOS_UNSUPPORTED; } } while (0)
    if (out_dtype == DT_F32) SCANS(float);
    else if (out_dtype == DT_BF16) SCANS(bf16_t);
    else return LLOGOS_BAD_ARGUMENT;
#undef SCANS
#undef SCAN
#undef SCAN1
#undef ARGS
    if (o_raw) {
        const int n = T * H, waves = 4;
        if (out_dtype == DT_F32)
            head_norm_gate_kernel<float><<<(n + waves - 1) / waves, waves * kWave, 0, stream>>>((float*)y, o_raw, gate, ld, parts, (size_t)part_stride, g, eps, H, D, n);
        else
            head_norm_gate_kernel<bf16_t><<<(n + waves - 1) / waves, waves * kWave, 0, stream>>>((bf16_t*)y, o_raw, gate, ld, parts, (size_t)part_stride, g, eps, H, D, n);
    }
    return LLOGOS_LAUNCH_CHECK();
}

// ---------------------------------------------------------------- a norm after a sublayer, the sum, the next norm
// For a block with norms on both sides of its sublayers:  x += norm_b(a) and then h = norm_n(x), one
// block a row, the row in LDS between the two passes:
//     v = sum of the parts of a;   x <- x + v / sqrt(mean(v^2) + eps) * wb
//     h = x / sqrt(mean(x^2) + eps) * wn           (skipped without wn)
// x is the float residual stream (written back), a the sublayer's output (float or bfloat16,
// maybe in parts of a k-split product), h the rows the next sublayer reads.  A thread keeps its
// elements of the row in registers between the two passes.
// (A step of few rows has few blocks, and a block's time is the latency of its loads: every part of every
// element a thread owns is asked for before the first sum, ITEMS elements a thread and up to kSandwichParts
// parts, as rmsnorm_vec_kernel does; more parts are added by a loop behind them.)
constexpr int kSandwichParts = 8;

template <typename TA, typename TH, int ITEMS>
__global__ __launch_bounds__(1024) void sandwich_norm_kernel(float* __restrict__ x, const TA* __restrict__ a, int parts, size_t part_stride,
                                     const float* __restrict__ wb, const float* __restrict__ wn, TH* __restrict__ h,
                                     float eps, int H) {
    __shared__ float red[16];
    const size_t r = blockIdx.x;
    float* xr = x + r * H;
    const TA* ar = a + r * H;
    float v[ITEMS], xv[ITEMS], wbv[ITEMS], wnv[ITEMS], pv[ITEMS][kSandwichParts];
#pragma unroll
    for (int it = 0; it < ITEMS; ++it) {
        const int i = it * blockDim.x + threadIdx.x;
        const bool ok = i < H;
        xv[it] = ok ? xr[i] : 0.f;
        wbv[it] = ok ? wb[i] : 0.f;
        wnv[it] = (ok && wn) ? wn[i] : 0.f;
#pragma unroll
        for (int q = 0; q < kSandwichParts; ++q) pv[it][q] = (ok && q < parts) ? load_f32(ar + q * part_stride + i) : 0.f;
    }
    float ss = 0.f;
#pragma unroll
    for (int it = 0; it < ITEMS; ++it) {
        const int i = it * blockDim.x + threadIdx.x;
        float t = pv[it][0];
#pragma unroll
        for (int q = 1; q < kSandwichParts; ++q) t += pv[it][q];            // ascending order
        for (int q = kSandwichParts; q < parts; ++q) if (i < H) t += load_f32(ar + q * part_stride + i);
        v[it] = t;
        ss = fmaf(t, t, ss);
    }
    const float inv_a = 1.0f / sqrtf(block_sum(ss, red) / (float)H + eps);
    ss = 0.f;
#pragma unroll
    for (int it = 0; it < ITEMS; ++it) {
        const int i = it * blockDim.x + threadIdx.x;
        const float t = fmaf(v[it] * inv_a, wbv[it], xv[it]);
        if (i < H) xr[i] = t;
        v[it] = t;
        ss = fmaf(t, t, ss);
    }
    if (!h) return;
    TH* hr = h + r * H;
    if (!wn) {                       // the completed rows as they are, in the reader's type
#pragma unroll
        for (int it = 0; it < ITEMS; ++it) {
            const int i = it * blockDim.x + threadIdx.x;
            if (i < H) store_f32(hr + i, v[it]);
        }
        return;
    }
    const float inv_x = 1.0f / sqrtf(block_sum(ss, red) / (float)H + eps);
#pragma unroll
    for (int it = 0; it < ITEMS; ++it) {
        const int i = it * blockDim.x + threadIdx.x;
        if (i < H) store_f32(hr + i, v[it] * inv_x * wnv[it]);
    }
}

LLOGOS_EXPORT int llogos_sandwich_norm(float* x, const void* a, int a_dtype, int parts, long long part_stride, const float* wb,
                                       const float* wn, void* h, int h_dtype, float eps, int T, int H, hipStream_t stream) {
    if (T <= 0 || H <= 0 || parts < 1 || H > 16384) return LLOGOS_BAD_ARGUMENT;
    // elements a thread: 1 for few rows (all of a row's loads in flight at once), up to 4 for many; blocks of up to 1024
    int items = T >= 256 ? 4 : 1;
    while ((H + items - 1) / items > 1024) items *= 2;
    if (items > 16) return LLOGOS_BAD_ARGUMENT;
    int threads = (H + items - 1) / items;
    threads = (threads + kWave - 1) / kWave * kWave;
#define SN(TA, TH, IT) sandwich_norm_kernel<TA, TH, IT><<<T, threads, 0, stream>>>(x, (const TA*)a, parts, (size_t)part_stride, wb, wn, (TH*)h, eps, H)
#define SNI(TA, TH) do { if (items == 1) SN(TA, TH, 1); else if (items == 2) SN(TA, TH, 2); else if (items == 4) SN(TA, TH, 4); \
                         else if (items == 8) SN(TA, TH, 8); else SN(TA, TH, 16); } while (0)
    if (a_dtype == DT_F32 && h_dtype == DT_F32) SNI(float, float);
    else if (a_dtype == DT_F32 && h_dtype == DT_BF16) SNI(float, bf16_t);
    else if (a_dtype == DT_BF16 && h_dtype == DT_F32) SNI(bf16_t, float);
    else if (a_dtype == DT_BF16 && h_dtype == DT_BF16) SNI(bf16_t, bf16_t);
    else return LLOGOS_BAD_ARGUMENT;
#undef SNI
#undef SN
    return LLOGOS_LAUNCH_CHECK();
}

// ---------------------------------------------------------------- activations of a product
// out = act(sum of the parts of `in`) element by element.  kinds:
//   0 tanh;  1 silu;  2 gelu (tanh form);
//   3 the piecewise xIELU with a = softplus(p), b = 1/2 + softplus(q):
//       z > 0: a z^2 + z / 2;   z <= 0: b (exp(z) - 1 - z) + z / 2
//   4 the square of relu: max(z, 0)^2
enum { ACT_TANH = 0, ACT_SILU = 1, ACT_GELU_TANH = 2, ACT_XIELU = 3, ACT_RELU2 = 4 };

__device__ __forceinline__ float activate(float z, int kind, float a, float b) {
    switch (kind) {
        case ACT_TANH: return tanhf(z);
        case ACT_SILU: return z / (1.0f + expf(-z));
        case ACT_GELU_TANH: return 0.5f * z * (1.0f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
        case ACT_RELU2: { const float r = fmaxf(z, 0.f); return r * r; }
        default: return z > 0.f ? fmaf(a * z, z, 0.5f * z) : fmaf(b, expm1f(z) - z, 0.5f * z);
    }
}

template <typename TO, typename TI>
__global__ void activation_kernel(TO* __restrict__ out, const TI* __restrict__ in, int parts, size_t part_stride,
                                  size_t n, int kind, float a, float b, int cols, int ld_in) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    // cols > 0: the input's rows lie ld_in values apart and their first `cols` values are taken (out is dense)
    const size_t src = cols > 0 ? (i / cols) * (size_t)ld_in + i % cols : i;
    float z = load_f32(in + src);
    for (int q = 1; q < parts; ++q) z += load_f32(in + q * part_stride + src);
    store_f32(out + i, activate(z, kind, a, b));
}

LLOGOS_EXPORT int llogos_activation(void* out, int out_dtype, const void* in, int in_dtype, int parts, long long part_stride,
                                    long long n, int kind, float a, float b, int cols, int ld_in, hipStream_t stream) {
    if (n <= 0 || parts < 1 || kind < 0 || kind > ACT_RELU2 || cols < 0 || (cols > 0 && ld_in < cols)) return LLOGOS_BAD_ARGUMENT;
    const unsigned blocks = (unsigned)((n + 255) / 256);
#define ACT(TO, TI) activation_kernel<TO, TI><<<blocks, 256, 0, stream>>>((TO*)out, (const TI*)in, parts, (size_t)part_stride, (size_t)n, kind, a, b, cols, ld_in)
    if (out_dtype == DT_F32 && in_dtype == DT_F32) ACT(float, float);
    else if (out_dtype == DT_BF16 && in_dtype == DT_F32) ACT(bf16_t, float);
    else if (out_dtype == DT_BF16 && in_dtype == DT_BF16) ACT(bf16_t, bf16_t);
    else if (out_dtype == DT_F32 && in_dtype == DT_BF16) ACT(float, bf16_t);
    else return LLOGOS_BAD_ARGUMENT;
#undef ACT
    return LLOGOS_LAUNCH_CHECK();
}
