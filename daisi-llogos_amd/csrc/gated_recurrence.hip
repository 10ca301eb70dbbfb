// A gated linear recurrence with a real, diagonal state (one number a channel and sequence):
//   r = sigmoid(gr + br),  i = sigmoid(gi + bi)             the two gates, from their logits
//   log a = -decay * r,    a = exp(log a)                   decay >= 0 is a constant of the channel
//   S <- a S + sqrt(1 - a^2) * (i * u)                      S starts at the sequence's state row
//   out = S * gelu_tanh(y)                                  the second branch gates the output
// All of it in 32-bit; 1 - a^2 is taken as -expm1(2 log a), which keeps its digits where a is near 1.
// The state row of a sequence (its cache slot) is read where the step's first token of the sequence
// starts and written behind its last.
//
// Long steps are cut into segments: since S_t = A S_0 + L with A the product of the segment's a and L
// its end state from zero, a first pass makes (A, L) of every segment, a second chains them into the
// state at every segment's start, and a third runs the segments side by side from those states.
#include "common.h"

__device__ __forceinline__ float gr_sigmoid(float z) { return 1.0f / (1.0f + expf(-z)); }
__device__ __forceinline__ float gr_gelu_tanh(float z) {
    return 0.5f * z * (1.0f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
}

struct GatedStep { float a, b; };

// (a, b) of S <- a S + b for one token and channel
__device__ __forceinline__ GatedStep gated_step(float gr, float gi, float u, float br, float bi, float decay) {
    const float r = gr_sigmoid(gr + br), i = gr_sigmoid(gi + bi);
    const float log_a = -decay * r;
    GatedStep s;
    s.a = expf(log_a);
    s.b = sqrtf(-expm1f(2.0f * log_a)) * (i * u);
    return s;
}

// gates: rows of ldg floats; channel c's logits are at (c / bs) * 2 * bs + c % bs (r) and bs further (i).
// mode 0: whole sequences, one thread a (sequence, channel): reads the state, runs the tokens, writes the state.
// mode 1: segment summaries (A, L) into seg_a, seg_l [segments, C], no outputs.
// mode 2: outputs of a segment from seg_l (which by then holds the state at the segment's start); the
//         last segment of a sequence writes the state.
template <typename TO, int MODE>
__global__ __launch_bounds__(256) void gated_recurrence_kernel(
        TO* __restrict__ out, const float* __restrict__ u, int ldu, const float* __restrict__ gates, int ldg, int bs,
        const float* __restrict__ br, const float* __restrict__ bi, const float* __restrict__ decay,
        const float* __restrict__ y, int ldy, float* __restrict__ state, size_t state_stride, const int* __restrict__ slots,
        const int* __restrict__ cu, int C, int seg_len, const int* __restrict__ seg_first, float* __restrict__ seg_a,
        float* __restrict__ seg_l) {
    const int c = blockIdx.x * blockDim.x + threadIdx.x;
    if (c >= C) return;
    int seq, t0, t1;
    size_t seg = 0;
    bool last_seg = true;
    if (MODE == 0) {
        seq = blockIdx.y;
        t0 = cu ? cu[seq] : seq;
        t1 = cu ? cu[seq + 1] : seq + 1;
    } else {
        // blockIdx.y numbers the segments of all sequences; seg_first[s] is the first segment of sequence s
        seg = blockIdx.y;
        seq = 0;
        while (seg_first[seq + 1] <= (int)seg) ++seq;
        const int k = (int)seg - seg_first[seq];
        t0 = cu[seq] + k * seg_len;
        t1 = min(cu[seq + 1], t0 + seg_len);
        last_seg = (int)seg + 1 == seg_first[seq + 1];
    }
    const int g0 = (c / bs) * 2 * bs + c % bs;
    const float brc = br[c], bic = bi[c], dc = decay[c];
    float* st = state + (size_t)slots[seq] * state_stride + c;
    float S = 0.f, A = 1.f;
    if (MODE == 0) S = *st;
    if (MODE == 2) S = seg_l[seg * C + c];
#pragma unroll 4
    for (int t = t0; t < t1; ++t) {
        const GatedStep s = gated_step(gates[(size_t)t * ldg + g0], gates[(size_t)t * ldg + g0 + bs], u[(size_t)t * ldu + c], brc, bic, dc);
        S = fmaf(s.a, S, s.b);
        if (MODE == 1) A *= s.a;
        else store_f32(out + (size_t)t * C + c, S * gr_gelu_tanh(y[(size_t)t * ldy + c]));
    }
    if (MODE == 1) { seg_a[seg * C + c] = A; seg_l[seg * C + c] = S; }
    else if (last_seg) *st = S;
}

// seg_l[s] <- the state at the start of segment s: the sequence's state row for its first segment, then
// S_start(s + 1) = A(s) S_start(s) + L(s).  One thread a (sequence, channel).
__global__ void gated_recurrence_chain_kernel(const float* __restrict__ seg_a, float* __restrict__ seg_l, const int* __restrict__ seg_first,
                                              const float* __restrict__ state, size_t state_stride, const int* __restrict__ slots, int C) {
    const int c = blockIdx.x * blockDim.x + threadIdx.x;
    if (c >= C) return;
    const int seq = blockIdx.y;
    float S = state[(size_t)slots[seq] * state_stride + c];
    for (int s = seg_first[seq]; s < seg_first[seq + 1]; ++s) {
        const float a = seg_a[(size_t)s * C + c], l = seg_l[(size_t)s * C + c];
        seg_l[(size_t)s * C + c] = S;
        S = fmaf(a, S, l);
    }
}

// u [T, >= C] (row stride ldu), gates [T, ldg], y [T, >= C] (row stride ldy): float32.  out [T, C] of out_dtype.
// state: float32, row `slots[seq]` of stride state_stride holds S [C].  cu [B + 1] token offsets (null: one token a
// sequence).  seg_len > 0 with seg_first [B + 1] (device) and scratch seg_a, seg_l [n_segments, C]: the three passes.
LLOGOS_EXPORT int llogos_gated_recurrence(void* out, int out_dtype, const float* u, int ldu, const float* gates, int ldg, int bs,
                                          const float* br, const float* bi, const float* decay, const float* y, int ldy,
                                          float* state, long long state_stride, const int* slots, const int* cu, int T, int B, int C,
                                          int seg_len, int n_segments, const int* seg_first, float* seg_a, float* seg_l,
                                          hipStream_t stream) {
    if (T <= 0 || B <= 0 || C <= 0 || bs <= 0 || C % bs || ldu < C || ldy < C || ldg < 2 * C || state_stride < C) return LLOGOS_BAD_ARGUMENT;
    if (!cu && T != B) return LLOGOS_BAD_ARGUMENT;
    if (out_dtype != DT_F32 && out_dtype != DT_BF16) return LLOGOS_BAD_ARGUMENT;
    const int threads = C >= 256 ? 256 : 64;
    const int bx = (C + threads - 1) / threads;
#define GR(TO, MODE, GY) gated_recurrence_kernel<TO, MODE><<<dim3(bx, GY), threads, 0, stream>>>((TO*)out, u, ldu, gates, ldg, bs, br, bi, \
        decay, y, ldy, state, (size_t)state_stride, slots, cu, C, seg_len, seg_first, seg_a, seg_l)
    if (seg_len > 0) {
        if (!cu || !seg_first || !seg_a || !seg_l || n_segments < B) return LLOGOS_BAD_ARGUMENT;
        GR(float, 1, n_segments);
        gated_recurrence_chain_kernel<<<dim3(bx, B), threads, 0, stream>>>(seg_a, seg_l, seg_first, state, (size_t)state_stride, slots, C);
        if (out_dtype == DT_F32) GR(float, 2, n_segments); else GR(bf16_t, 2, n_segments);
    } else {
        if (out_dtype == DT_F32) GR(float, 0, B); else GR(bf16_t, 0, B);
    }
#undef GR
    return LLOGOS_LAUNCH_CHECK();
}
