// Linear recurrences over a matrix state per head, kept per request between steps:
//
//     o_t[j] = sum_i q_t[i] * (a_t[i] * S[i][j] + b[i] * k_t[i] * v_t[j])
//     S[i][j] <- w_t[i] * S[i][j] + k_t[i] * v_t[j]
//
// with two forms of the coefficients:
//   * one decay per head (linear attention with decay): a = w = decay[h], b = 1, so the output reads
//     the state after the update;
//   * a decay per token and key channel with a bonus for the current token (time mixing):
//     w_t[i] = exp(-exp(wlog_t[i])), a = 1, b = bonus[h][i], the output reads the state before the update;
//   * a step size per token and head (state-space duality): dt = softplus(step_t[h] + step_bias[h]),
//     S <- exp(-exp(rate_log[h]) dt) S + dt k_t v_t^T, o_t = S^T q_t + skip[h] v_t (the state after the
//     update); queries and keys are shared by the `share` consecutive heads of a group.
//
// Everything is float.  Tokens are taken one after another in the order of the sequence, every
// token by the same instructions whatever the step brings with it, so the state and the outputs of
// a position are the same bits however the sequence was cut into steps and whatever else is in the
// batch.
//
// A work-group of four waves owns 16 value columns of one head of one sequence: that gives a prompt
// of one sequence heads x value columns / 16 work-groups to spread over the GPU, and what a token
// costs is the length of one thread's chain of instructions, not arithmetic.  Lane 16 r + j of wave g
// keeps rows (4 g + r) R .. + R of column j of S in registers (R = ceil(dk / 16) rounded up to a
// template size); queries, keys, decays and values of 16 tokens at a time go through LDS, the next
// chunk's on their way in registers meanwhile; a column's sixteen shares of an output are left in
// LDS and added in ascending order of the rows once per chunk.
#include "common.h"

#include <math.h>

#define REC_MAX_DK 256
#define REC_COLS 16

__device__ __forceinline__ float rec_silu(float z) { return z / (1.0f + expf(-z)); }

// softplus without overflow: max(z, 0) + ln(1 + exp(-|z|))
__device__ __forceinline__ float rec_softplus(float z) { return fmaxf(z, 0.f) + log1pf(expf(-fabsf(z))); }

// MODE 0: a decay per head; 1: per token and key channel; 2: a step size per token and head.  In mode 2
// wlog is the step [T, >= H] (row stride ldw), decay is rate_log [H], bonus is step_bias [H], skip [H] or
// null, and head h reads queries and keys of group h / share.
template <int R, int MODE>
__global__ __launch_bounds__(256) void linear_recurrence_kernel(
    const float* __restrict__ q, int ldq, const float* __restrict__ k, int ldk, const float* __restrict__ v, int ldv,
    const float* __restrict__ wlog, int ldw, const float* __restrict__ decay, const float* __restrict__ bonus,
    const float* __restrict__ skip, int share,
    float* __restrict__ state, long long state_stride, const int32_t* __restrict__ state_slots,
    const int32_t* __restrict__ q_start, float* __restrict__ out, int ldo, int H, int dk, int dv, int silu_inputs) {
    constexpr bool PER_TOKEN = MODE == 1;
    constexpr bool STEPS = MODE == 2;
    constexpr int DKP = 16 * R;                       // rows the tile holds; those beyond dk stay zero
    constexpr int REC_TB = R == 16 ? 8 : 16;          // tokens per chunk (fewer for the largest tile: LDS)
    constexpr int PER = REC_TB * DKP / 256;           // elements of a [REC_TB][DKP] tile per thread
    __shared__ __attribute__((aligned(16))) float qs[REC_TB][DKP], ks[REC_TB][DKP], ws[PER_TOKEN ? REC_TB : 1][DKP];
    __shared__ float vs[REC_TB][REC_COLS];
    __shared__ float dts[REC_TB], decs[REC_TB];       // mode 2: a token's step size and its decay
    __shared__ float part[16][REC_TB][REC_COLS];      // a row group's share of every output of the chunk
    const int tid = threadIdx.x, lane = tid & 63, g = tid >> 6;
    const int col = lane & 15, rg = 4 * g + (lane >> 4);
    const int j0 = blockIdx.x * REC_COLS, h = blockIdx.y, s = blockIdx.z;
    const int r0 = q_start[s], r1 = q_start[s + 1];
    if (r1 <= r0) return;
    const int j = j0 + col;
    const bool col_ok = j < dv;
    float* st = state + (size_t)state_slots[s] * state_stride + (size_t)h * dk * dv;

    float S[R], ur[R];
#pragma unroll
    for (int rr = 0; rr < R; ++rr) {
        const int i = rg * R + rr;
        S[rr] = (i < dk && col_ok) ? st[(size_t)i * dv + j] : 0.f;
        ur[rr] = (PER_TOKEN && bonus && i < dk) ? bonus[h * dk + i] : 1.f;
    }
    const float dec = MODE == 0 ? decay[h] : 1.f;
    const int hq = STEPS ? h / share : h;             // the head whose queries and keys this head reads
    const float rate = STEPS ? expf(decay[h]) : 0.f, step_bias = (STEPS && bonus) ? bonus[h] : 0.f;
    const float skip_h = (STEPS && skip) ? skip[h] : 0.f;

    // The next REC_TB tokens' operands are read into registers while this chunk is computed (with one
    // work-group or less per CU nothing else would hide those reads), and go to LDS afterwards: element
    // tid + 256 it of the [REC_TB][DKP] tile, R to a thread; what lies outside the step or the head is zero.
    float qreg[PER], kreg[PER], wreg[PER_TOKEN ? PER : 1], vreg = 0.f, dtreg = 0.f;
    auto fetch = [&](int t0, int n) {
#pragma unroll
        for (int it = 0; it < PER; ++it) {
            const int idx = tid + it * 256, tt = idx / DKP, i = idx - tt * DKP;
            const bool ok = tt < n && i < dk;
            qreg[it] = ok ? q[(size_t)(t0 + tt) * ldq + hq * dk + i] : 0.f;
            kreg[it] = ok ? k[(size_t)(t0 + tt) * ldk + hq * dk + i] : 0.f;
            if (PER_TOKEN) wreg[it] = ok ? wlog[(size_t)(t0 + tt) * ldw + h * dk + i] : 0.f;
        }
        const int tt = tid / REC_COLS, jj = tid % REC_COLS;      // beyond the chunk for tid >= REC_TB * REC_COLS: tt >= n
        vreg = (tt < n && j0 + jj < dv) ? v[(size_t)(t0 + tt) * ldv + h * dv + j0 + jj] : 0.f;
        if (STEPS) dtreg = tid < n ? wlog[(size_t)(t0 + tid) * ldw + h] : 0.f;
    };
    auto stash = [&](int n) {
#pragma unroll
        for (int it = 0; it < PER; ++it) {
            const int idx = tid + it * 256, tt = idx / DKP, i = idx - tt * DKP;
            const bool ok = tt < n && i < dk;
            (&qs[0][0])[idx] = silu_inputs ? rec_silu(qreg[it]) : qreg[it];
            (&ks[0][0])[idx] = silu_inputs ? rec_silu(kreg[it]) : kreg[it];
            if (PER_TOKEN) (&ws[0][0])[idx] = ok ? expf(-expf(wreg[it])) : 0.f;
        }
        if (tid < REC_TB * REC_COLS) (&vs[0][0])[tid] = silu_inputs ? rec_silu(vreg) : vreg;
        if (STEPS && tid < REC_TB) {
            const float dt = rec_softplus(dtreg + step_bias);
            dts[tid] = dt;
            decs[tid] = expf(-rate * dt);
        }
    };

    fetch(r0, min(REC_TB, r1 - r0));
    stash(min(REC_TB, r1 - r0));
    __syncthreads();
    for (int t0 = r0; t0 < r1; t0 += REC_TB) {
        const int n = min(REC_TB, r1 - t0);
        const bool more = t0 + REC_TB < r1;
        if (more) fetch(t0 + REC_TB, min(REC_TB, r1 - t0 - REC_TB));
#pragma unroll 4
        for (int tt = 0; tt < n; ++tt) {
            const float vj = STEPS ? dts[tt] * vs[tt][col] : vs[tt][col];
            const float dect = STEPS ? decs[tt] : dec;
            float acc = 0.f;
#pragma unroll
            for (int rr = 0; rr < R; ++rr) {
                const int i = rg * R + rr;
                const float kv = ks[tt][i] * vj;
                if (PER_TOKEN) {
                    acc += qs[tt][i] * (S[rr] + ur[rr] * kv);
                    S[rr] = ws[tt][i] * S[rr] + kv;
                } else {
                    S[rr] = dect * S[rr] + kv;
                    acc += qs[tt][i] * S[rr];
                }
            }
            part[rg][tt][col] = acc;
        }
        __syncthreads();
        {
            const int tt = tid / REC_COLS, jj = tid % REC_COLS;
            if (tt < n && j0 + jj < dv) {
                float sum = part[0][tt][jj];
#pragma unroll
                for (int r = 1; r < 16; ++r) sum += part[r][tt][jj];       // the row groups in ascending order
                if (STEPS) sum += skip_h * vs[tt][jj];
                out[(size_t)(t0 + tt) * ldo + h * dv + j0 + jj] = sum;
            }
        }
        if (more) stash(min(REC_TB, r1 - t0 - REC_TB));
        __syncthreads();
    }
#pragma unroll
    for (int rr = 0; rr < R; ++rr) {
        const int i = rg * R + rr;
        if (i < dk && col_ok) st[(size_t)i * dv + j] = S[rr];
    }
}

extern "C" int tl_linear_recurrence_takes(int dk) { return dk > 0 && dk <= REC_MAX_DK ? 1 : 0; }

// q, k [T, >= H*dk], v [T, >= H*dv] float with row strides; per_token 0: decay [H]; per_token 1: wlog
// [T, >= H*dk] with row stride ldw, bonus [H, dk] or null; per_token 2: q, k [T, >= (H/share)*dk], wlog the
// steps [T, >= H], decay rate_log [H], bonus step_bias [H] or null, skip [H] or null.  state: float, a
// request's [H, dk, dv] at state + slot * state_stride.  out float [T, >= H*dv].  S sequences, rows
// q_start[s] .. q_start[s+1].
extern "C" int tl_linear_recurrence(const float* q, int ldq, const float* k, int ldk, const float* v, int ldv,
                                    const float* wlog, int ldw, const float* decay, const float* bonus, int per_token,
                                    const float* skip, int share,
                                    float* state, long long state_stride, const int32_t* state_slots,
                                    const int32_t* q_start, float* out, int ldo, int S, int H, int dk, int dv,
                                    int silu_inputs, hipStream_t stream) {
    TL_CHECK_ARG(S >= 0 && H > 0 && dv > 0, "tl_linear_recurrence: bad sizes S=%d H=%d dv=%d", S, H, dv);
    TL_CHECK_ARG(tl_linear_recurrence_takes(dk), "tl_linear_recurrence: a key size of %d is not served (at most %d)", dk, REC_MAX_DK);
    TL_CHECK_ARG(per_token >= 0 && per_token <= 2, "tl_linear_recurrence: unknown form %d", per_token);
    if (per_token != 2) share = 1;
    TL_CHECK_ARG(share >= 1 && H % share == 0, "tl_linear_recurrence: %d heads do not share queries and keys in groups of %d", H, share);
    const int HQ = H / share;
    TL_CHECK_ARG(ldq >= HQ * dk && ldk >= HQ * dk && ldv >= H * dv && ldo >= H * dv, "tl_linear_recurrence: rows too short");
    TL_CHECK_ARG(state_stride >= (long long)H * dk * dv, "tl_linear_recurrence: the state of a request is too small");
    TL_CHECK_ARG(per_token == 1 ? (wlog != nullptr && ldw >= H * dk)
                 : per_token == 2 ? (wlog != nullptr && ldw >= H && decay != nullptr) : decay != nullptr,
                 "tl_linear_recurrence: decays are missing");
    TL_CHECK_ARG(H <= 65535 && S <= 65535, "tl_linear_recurrence: too many heads or sequences for one launch");
    if (S == 0) return 0;
    dim3 grid(tl_ceil_div(dv, REC_COLS), H, S), block(256);
#define GO(R)                                                                                                            \
    do {                                                                                                                 \
        if (per_token == 1)                                                                                              \
            hipLaunchKernelGGL((linear_recurrence_kernel<R, 1>), grid, block, 0, stream, q, ldq, k, ldk, v, ldv, wlog, ldw, \
                               decay, bonus, skip, share, state, state_stride, state_slots, q_start, out, ldo, H, dk, dv, silu_inputs); \
        else if (per_token == 2)                                                                                         \
            hipLaunchKernelGGL((linear_recurrence_kernel<R, 2>), grid, block, 0, stream, q, ldq, k, ldk, v, ldv, wlog, ldw, \
                               decay, bonus, skip, share, state, state_stride, state_slots, q_start, out, ldo, H, dk, dv, silu_inputs); \
        else                                                                                                             \
            hipLaunchKernelGGL((linear_recurrence_kernel<R, 0>), grid, block, 0, stream, q, ldq, k, ldk, v, ldv, wlog, ldw, \
                               decay, bonus, skip, share, state, state_stride, state_slots, q_start, out, ldo, H, dk, dv, silu_inputs); \
    } while (0)
    if (dk <= 16) GO(1);
    else if (dk <= 32) GO(2);
    else if (dk <= 64) GO(4);
    else if (dk <= 128) GO(8);
    else GO(16);
#undef GO
    TL_CHECK_LAUNCH("tl_linear_recurrence");
    return 0;
}
