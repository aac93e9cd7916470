// Linear recurrences over a matrix state per head, kept per request between steps:
//
//     o_t[j] = sum_i q_t[i] * (a_t[i] * S[i][j] + b[i] * k_t[i] * v_t[j])
//     S[i][j] <- w_t[i] * S[i][j] + k_t[i] * v_t[j]
//
// with two forms of the coefficients:
//   * one decay per head (linear attention with decay): a = w = decay[h], b = 1, so the output reads
//     the state after the update;
//   * a decay per token and key channel with a bonus for the current token (time mixing):
//     w_t[i] = exp(-exp(wlog_t[i])), a = 1, b = bonus[h][i], the output reads the state before the update.
//
// Everything is float.  Tokens are taken one after another in the order of the sequence, every
// token by the same instructions whatever the step brings with it, so the state and the outputs of
// a position are the same bits however the sequence was cut into steps and whatever else is in the
// batch.
//
// A work-group of four waves owns 64 value columns of one head of one sequence.  Lane j of wave g
// keeps S[g R .. g R + R)[j] in registers (R = ceil(dk / 4) rounded up to a template size); queries,
// keys, decays and values of REC_TB tokens at a time go through LDS, the four waves' shares of an
// output are added in the order of the waves.
#include "common.h"

#include <math.h>

#define REC_TB 8
#define REC_MAX_DK 256

__device__ __forceinline__ float rec_silu(float z) { return z / (1.0f + expf(-z)); }

template <int R, bool PER_TOKEN>
__global__ __launch_bounds__(256) void linear_recurrence_kernel(
    const float* __restrict__ q, int ldq, const float* __restrict__ k, int ldk, const float* __restrict__ v, int ldv,
    const float* __restrict__ wlog, int ldw, const float* __restrict__ decay, const float* __restrict__ bonus,
    float* __restrict__ state, long long state_stride, const int32_t* __restrict__ state_slots,
    const int32_t* __restrict__ q_start, float* __restrict__ out, int ldo, int H, int dk, int dv, int silu_inputs) {
    __shared__ float qs[REC_TB][4 * R], ks[REC_TB][4 * R], ws[PER_TOKEN ? REC_TB : 1][4 * R], vs[REC_TB][64];
    __shared__ float part[4][REC_TB][64];
    const int tid = threadIdx.x, lane = tid & 63, g = tid >> 6;
    const int j0 = blockIdx.x * 64, h = blockIdx.y, s = blockIdx.z;
    const int r0 = q_start[s], r1 = q_start[s + 1];
    if (r1 <= r0) return;
    const int j = j0 + lane;
    const bool col_ok = j < dv;
    float* st = state + (size_t)state_slots[s] * state_stride + (size_t)h * dk * dv;

    float S[R], ur[R];
#pragma unroll
    for (int rr = 0; rr < R; ++rr) {
        const int i = g * R + rr;
        S[rr] = (i < dk && col_ok) ? st[(size_t)i * dv + j] : 0.f;
        ur[rr] = (PER_TOKEN && bonus && i < dk) ? bonus[h * dk + i] : 1.f;
    }
    const float dec = PER_TOKEN ? 1.f : decay[h];
    // rows of the LDS tiles beyond dk stay zero: they multiply state rows that are zero and stay zero
    for (int idx = tid; idx < REC_TB * 4 * R; idx += 256) {
        (&qs[0][0])[idx] = 0.f;
        (&ks[0][0])[idx] = 0.f;
        if (PER_TOKEN) (&ws[0][0])[idx] = 0.f;
    }

    for (int t0 = r0; t0 < r1; t0 += REC_TB) {
        const int n = min(REC_TB, r1 - t0);
        __syncthreads();
        for (int idx = tid; idx < n * dk; idx += 256) {
            const int tt = idx / dk, i = idx - tt * dk;
            float qv = q[(size_t)(t0 + tt) * ldq + h * dk + i], kv = k[(size_t)(t0 + tt) * ldk + h * dk + i];
            if (silu_inputs) {
                qv = rec_silu(qv);
                kv = rec_silu(kv);
            }
            qs[tt][i] = qv;
            ks[tt][i] = kv;
            if (PER_TOKEN) ws[tt][i] = expf(-expf(wlog[(size_t)(t0 + tt) * ldw + h * dk + i]));
        }
        for (int idx = tid; idx < n * 64; idx += 256) {
            const int tt = idx >> 6, jj = idx & 63;
            float vv = 0.f;
            if (j0 + jj < dv) {
                vv = v[(size_t)(t0 + tt) * ldv + h * dv + j0 + jj];
                if (silu_inputs) vv = rec_silu(vv);
            }
            vs[tt][jj] = vv;
        }
        __syncthreads();
        for (int tt = 0; tt < n; ++tt) {
            const float vj = vs[tt][lane];
            float acc = 0.f;
#pragma unroll
            for (int rr = 0; rr < R; ++rr) {
                const int i = g * R + rr;
                const float kv = ks[tt][i] * vj;
                if (PER_TOKEN) {
                    acc += qs[tt][i] * (S[rr] + ur[rr] * kv);
                    S[rr] = ws[tt][i] * S[rr] + kv;
                } else {
                    S[rr] = dec * S[rr] + kv;
                    acc += qs[tt][i] * S[rr];
                }
            }
            part[g][tt][lane] = acc;
        }
        __syncthreads();
        for (int idx = tid; idx < n * 64; idx += 256) {
            const int tt = idx >> 6, jj = idx & 63;
            if (j0 + jj < dv)
                out[(size_t)(t0 + tt) * ldo + h * dv + j0 + jj] = ((part[0][tt][jj] + part[1][tt][jj]) + part[2][tt][jj]) + part[3][tt][jj];
        }
    }
#pragma unroll
    for (int rr = 0; rr < R; ++rr) {
        const int i = g * R + rr;
        if (i < dk && col_ok) st[(size_t)i * dv + j] = S[rr];
    }
}

extern "C" int tl_linear_recurrence_takes(int dk) { return dk > 0 && dk <= REC_MAX_DK ? 1 : 0; }

// q, k [T, >= H*dk], v [T, >= H*dv] float with row strides; per_token 0: decay [H]; per_token 1: wlog
// [T, >= H*dk] with row stride ldw, bonus [H, dk] or null.  state: float, a request's [H, dk, dv] at
// state + slot * state_stride.  out float [T, >= H*dv].  S sequences, rows q_start[s] .. q_start[s+1].
extern "C" int tl_linear_recurrence(const float* q, int ldq, const float* k, int ldk, const float* v, int ldv,
                                    const float* wlog, int ldw, const float* decay, const float* bonus, int per_token,
                                    float* state, long long state_stride, const int32_t* state_slots,
                                    const int32_t* q_start, float* out, int ldo, int S, int H, int dk, int dv,
                                    int silu_inputs, hipStream_t stream) {
    TL_CHECK_ARG(S >= 0 && H > 0 && dv > 0, "tl_linear_recurrence: bad sizes S=%d H=%d dv=%d", S, H, dv);
    TL_CHECK_ARG(tl_linear_recurrence_takes(dk), "tl_linear_recurrence: a key size of %d is not served (at most %d)", dk, REC_MAX_DK);
    TL_CHECK_ARG(ldq >= H * dk && ldk >= H * dk && ldv >= H * dv && ldo >= H * dv, "tl_linear_recurrence: rows too short");
    TL_CHECK_ARG(state_stride >= (long long)H * dk * dv, "tl_linear_recurrence: the state of a request is too small");
    TL_CHECK_ARG(per_token ? (wlog != nullptr && ldw >= H * dk) : decay != nullptr, "tl_linear_recurrence: decays are missing");
    TL_CHECK_ARG(H <= 65535 && S <= 65535, "tl_linear_recurrence: too many heads or sequences for one launch");
    if (S == 0) return 0;
    dim3 grid(tl_ceil_div(dv, 64), H, S), block(256);
#define GO(R)                                                                                                            \
    do {                                                                                                                 \
        if (per_token)                                                                                                   \
            hipLaunchKernelGGL((linear_recurrence_kernel<R, true>), grid, block, 0, stream, q, ldq, k, ldk, v, ldv, wlog, ldw, \
                               decay, bonus, state, state_stride, state_slots, q_start, out, ldo, H, dk, dv, silu_inputs); \
        else                                                                                                             \
            hipLaunchKernelGGL((linear_recurrence_kernel<R, false>), grid, block, 0, stream, q, ldq, k, ldk, v, ldv, wlog, ldw, \
                               decay, bonus, state, state_stride, state_slots, q_start, out, ldo, H, dk, dv, silu_inputs); \
    } while (0)
    if (dk <= 16) GO(4);
    else if (dk <= 32) GO(8);
    else if (dk <= 64) GO(16);
    else if (dk <= 128) GO(32);
    else GO(64);
#undef GO
    TL_CHECK_LAUNCH("tl_linear_recurrence");
    return 0;
}
