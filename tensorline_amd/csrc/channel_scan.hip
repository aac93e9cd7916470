// Mixing along the sequence one channel at a time, with what has to be carried from step to step kept
// in the request's state slot:
//
//   tl_causal_conv   a short causal convolution per channel: out[t][c] = act(bias[c] + sum_j taps[c][j] *
//                    x[t - (K - 1) + j][c]), the last tap the current token's; inputs ahead of the step's
//                    first row come from the slot (zeros for a new request), and afterwards the slot keeps
//                    the sequence's last K - 1 inputs
//   tl_gated_scan    the real-gated linear recurrent unit: per channel r = sigmoid(gr + br), i = sigmoid(gi +
//                    bi), a = exp(-c r softplus(lam)), S <- a S + sqrt(1 - a^2) i u, out = S * gelu_tanh(y)
//
// Everything is float.  A token's result is computed by the same instructions whatever the step brings
// with it, tokens in the order of the sequence, so neither the cutting of a prompt nor the batch changes a
// bit of a result.
#include "common.h"

#include <math.h>

#define CS_MAX_TAPS 16

__device__ __forceinline__ float cs_sigmoid(float z) { return 1.0f / (1.0f + expf(-z)); }
__device__ __forceinline__ float cs_softplus(float z) { return fmaxf(z, 0.f) + log1pf(expf(-fabsf(z))); }
__device__ __forceinline__ float cs_gelu_tanh(float z) {
    return 0.5f * z * (1.0f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
}

// One thread per (token, channel).  kept: the slot's [K - 1][C] inputs, the oldest first.
template <typename O>
__global__ void causal_conv_kernel(const float* __restrict__ x, int ldx, const float* __restrict__ taps,
                                   const float* __restrict__ bias, const float* __restrict__ kept, long long state_stride,
                                   const int32_t* __restrict__ state_slots, const int32_t* __restrict__ seq_of_token,
                                   const int32_t* __restrict__ q_start, O* __restrict__ out, int ldo, int C, int K, int act) {
    const int t = blockIdx.x, c = blockIdx.y * blockDim.x + threadIdx.x;
    if (c >= C) return;
    const int s = seq_of_token[t];
    const int r0 = q_start[s];
    const float* old = kept + (size_t)state_slots[s] * state_stride;
    float acc = bias ? bias[c] : 0.f;
    for (int j = 0; j < K; ++j) {
        const int r = t - (K - 1) + j;
        const float v = r >= r0 ? x[(size_t)r * ldx + c] : old[(size_t)(r - r0 + K - 1) * C + c];
        acc += taps[(size_t)c * K + j] * v;
    }
    if (act == 1) acc = acc / (1.0f + expf(-acc));
    out[(size_t)t * ldo + c] = tl_from_float<O>(acc);
}

// One thread per (sequence, channel): the last K - 1 inputs of the sequence, taken from the step's rows
// and, where the step brings fewer, from what the slot kept; read first, then written.
__global__ void causal_conv_keep_kernel(const float* __restrict__ x, int ldx, float* __restrict__ kept, long long state_stride,
                                        const int32_t* __restrict__ state_slots, const int32_t* __restrict__ q_start,
                                        int C, int K) {
    const int s = blockIdx.y, c = blockIdx.x * blockDim.x + threadIdx.x;
    if (c >= C) return;
    const int r0 = q_start[s], r1 = q_start[s + 1];
    if (r1 <= r0) return;
    float* old = kept + (size_t)state_slots[s] * state_stride;
    float keep[CS_MAX_TAPS - 1];
#pragma unroll
    for (int j = 0; j < CS_MAX_TAPS - 1; ++j) {
        if (j < K - 1) {
            const int r = r1 - (K - 1) + j;
            keep[j] = r >= r0 ? x[(size_t)r * ldx + c] : old[(size_t)(r - r0 + K - 1) * C + c];
        }
    }
#pragma unroll
    for (int j = 0; j < CS_MAX_TAPS - 1; ++j)
        if (j < K - 1) old[(size_t)j * C + c] = keep[j];
}

// x float [T, >= C] (row stride ldx); taps float [C, K]; bias float [C] or null; kept: the slots' [K - 1, C]
// at kept + slot * state_stride; act 0: none, 1: SiLU.  out [T, >= C] float or bfloat16.  `update` != 0
// also renews what the slots keep (a second launch, after every token of the step has read the old rows).
extern "C" int tl_causal_conv(const float* x, int ldx, const float* taps, const float* bias, float* kept,
                              long long state_stride, const int32_t* state_slots, const int32_t* seq_of_token,
                              const int32_t* q_start, void* out, int out_dtype, int ldo, int T, int S, int C, int K, int act,
                              int update, hipStream_t stream) {
    TL_CHECK_ARG(T >= 0 && S >= 0 && C > 0 && K >= 1 && K <= CS_MAX_TAPS, "tl_causal_conv: bad sizes C=%d taps=%d (at most %d)", C, K, CS_MAX_TAPS);
    TL_CHECK_ARG(ldx >= C && ldo >= C && state_stride >= (long long)(K - 1) * C, "tl_causal_conv: rows or the kept inputs are too short");
    TL_CHECK_ARG(S <= 65535 && tl_ceil_div(C, 256) <= 65535, "tl_causal_conv: too many sequences or channels for one launch");
    if (T == 0 || S == 0) return 0;
    dim3 block(256), grid(T, tl_ceil_div(C, 256));
    if (out_dtype == TL_F32)
        hipLaunchKernelGGL(causal_conv_kernel<float>, grid, block, 0, stream, x, ldx, taps, bias, kept, state_stride, state_slots,
                           seq_of_token, q_start, (float*)out, ldo, C, K, act);
    else if (out_dtype == TL_BF16)
        hipLaunchKernelGGL(causal_conv_kernel<bf16_t>, grid, block, 0, stream, x, ldx, taps, bias, kept, state_stride, state_slots,
                           seq_of_token, q_start, (bf16_t*)out, ldo, C, K, act);
    else return tl_fail("tl_causal_conv: unknown dtype %d", out_dtype);
    TL_CHECK_LAUNCH("tl_causal_conv");
    if (update && K > 1) {
        hipLaunchKernelGGL(causal_conv_keep_kernel, dim3(tl_ceil_div(C, 256), S), block, 0, stream, x, ldx, kept, state_stride,
                           state_slots, q_start, C, K);
        TL_CHECK_LAUNCH("tl_causal_conv keep");
    }
    return 0;
}

// One thread per (sequence, channel) walks the sequence's rows; the operands of the next GS_AHEAD tokens
// are on their way in registers meanwhile.
#define GS_AHEAD 4
template <typename O>
__global__ __launch_bounds__(64) void gated_scan_kernel(
    const float* __restrict__ gr, const float* __restrict__ gi, int ldg, const float* __restrict__ br,
    const float* __restrict__ bi, const float* __restrict__ u, int ldu, const float* __restrict__ y, int ldy,
    const float* __restrict__ lam, float c, float* __restrict__ state, long long state_stride,
    const int32_t* __restrict__ state_slots, const int32_t* __restrict__ q_start, O* __restrict__ out, int ldo, int W,
    int bw, int bstride) {
    const int s = blockIdx.y, ch = blockIdx.x * blockDim.x + threadIdx.x;
    if (ch >= W) return;
    const int gcol = (ch / bw) * bstride + ch % bw;       // where the channel's gates lie in a row of gr and gi
    const int r0 = q_start[s], r1 = q_start[s + 1];
    if (r1 <= r0) return;
    float* st = state + (size_t)state_slots[s] * state_stride + ch;
    float S = *st;
    const float rate = c * cs_softplus(lam[ch]);
    const float b_r = br ? br[ch] : 0.f, b_i = bi ? bi[ch] : 0.f;
    float a_r[GS_AHEAD], a_i[GS_AHEAD], a_u[GS_AHEAD], a_y[GS_AHEAD];
    auto fetch = [&](int t0) {
#pragma unroll
        for (int k = 0; k < GS_AHEAD; ++k) {
            const int t = t0 + k < r1 ? t0 + k : r1 - 1;
            a_r[k] = gr[(size_t)t * ldg + gcol];
            a_i[k] = gi[(size_t)t * ldg + gcol];
            a_u[k] = u[(size_t)t * ldu + ch];
            a_y[k] = y[(size_t)t * ldy + ch];
        }
    };
    fetch(r0);
    for (int t0 = r0; t0 < r1; t0 += GS_AHEAD) {
        float c_r[GS_AHEAD], c_i[GS_AHEAD], c_u[GS_AHEAD], c_y[GS_AHEAD];
#pragma unroll
        for (int k = 0; k < GS_AHEAD; ++k) c_r[k] = a_r[k], c_i[k] = a_i[k], c_u[k] = a_u[k], c_y[k] = a_y[k];
        if (t0 + GS_AHEAD < r1) fetch(t0 + GS_AHEAD);
#pragma unroll
        for (int k = 0; k < GS_AHEAD; ++k) {
            if (t0 + k >= r1) break;
            const float r = cs_sigmoid(c_r[k] + b_r), i = cs_sigmoid(c_i[k] + b_i);
            const float a = expf(-rate * r);
            S = a * S + sqrtf(1.0f - a * a) * i * c_u[k];
            out[(size_t)(t0 + k) * ldo + ch] = tl_from_float<O>(S * cs_gelu_tanh(c_y[k]));
        }
    }
    *st = S;
}

// gr, gi float (row stride ldg): the gates before their bias and sigmoid, channel ch at column (ch / bw) *
// bstride + ch % bw (blocks of bw channels lie bstride apart; bw = W: side by side); br, bi float [W] or
// null; u, y float [T, >= W]; lam float [W]; c: the factor on r * softplus(lam) in -ln a.  state: a
// request's [W] at state + slot * state_stride.  out [T, >= W] float or bfloat16.
extern "C" int tl_gated_scan(const float* gr, const float* gi, int ldg, const float* br, const float* bi, const float* u,
                             int ldu, const float* y, int ldy, const float* lam, float c, float* state,
                             long long state_stride, const int32_t* state_slots, const int32_t* q_start, void* out,
                             int out_dtype, int ldo, int S, int W, int bw, int bstride, hipStream_t stream) {
    TL_CHECK_ARG(S >= 0 && W > 0 && ldu >= W && ldy >= W && ldo >= W && state_stride >= W, "tl_gated_scan: bad sizes W=%d", W);
    TL_CHECK_ARG(bw > 0 && W % bw == 0 && bstride >= bw && ldg >= (W / bw - 1) * bstride + bw,
                 "tl_gated_scan: gates in blocks of %d channels %d apart do not fit rows of %d", bw, bstride, ldg);
    TL_CHECK_ARG(S <= 65535, "tl_gated_scan: too many sequences for one launch");
    if (S == 0) return 0;
    dim3 grid(tl_ceil_div(W, 64), S), block(64);
    if (out_dtype == TL_F32)
        hipLaunchKernelGGL(gated_scan_kernel<float>, grid, block, 0, stream, gr, gi, ldg, br, bi, u, ldu, y, ldy, lam, c, state,
                           state_stride, state_slots, q_start, (float*)out, ldo, W, bw, bstride);
    else if (out_dtype == TL_BF16)
        hipLaunchKernelGGL(gated_scan_kernel<bf16_t>, grid, block, 0, stream, gr, gi, ldg, br, bi, u, ldu, y, ldy, lam, c, state,
                           state_stride, state_slots, q_start, (bf16_t*)out, ldo, W, bw, bstride);
    else return tl_fail("tl_gated_scan: unknown dtype %d", out_dtype);
    TL_CHECK_LAUNCH("tl_gated_scan");
    return 0;
}
