// The state-space recurrence of tl_linear_recurrence's third form for prompt portions, in chunks:
//
//     dt_t = softplus(step_t + bias),  la_t = -exp(rate_log) dt_t,
//     S_t = exp(la_t) S_(t-1) + dt_t B_t x_t^T,   y_t = S_t^T C_t + skip x_t
//
// A sequence's rows of the step are cut into chunks of SC_L tokens from its first row.  With cs_t the sum of
// la over the chunk's tokens up to t (all <= 0, so no exponential below overflows), and S_0 the state that
// enters the chunk,
//
//     y_t = exp(cs_t) S_0^T C_t + sum_(s <= t) exp(cs_t - cs_s) dt_s (C_t . B_s) x_s + skip x_t
//     S_L = exp(cs_L) S_0 + sum_s exp(cs_L - cs_s) dt_s B_s x_s^T
//
// which makes everything but the hand-over of the state from chunk to chunk independent work:
//   1. ssd_local_state_kernel: per chunk, head and block of 16 value columns, the second term of S_L and exp(cs_L);
//   2. ssd_scan_states_kernel: per state element, the chunks of a sequence in order: what enters each chunk is
//      left in the workspace in place of the chunk's own term, and the last state goes to the request's slot;
//   3. ssd_outputs_kernel: per chunk and head, the L x L matrix exp(cs_t - cs_s) dt_s (C_t . B_s) through LDS and
//      both products with it and with the entering state.
// A prompt of 2,048 tokens has 32 chunks per head to spread over the GPU, where the token-by-token walk has one
// chain of 2,048 dependent steps per head and block of columns.  The products run on the float matrix
// instruction (v_mfma_f32_16x16x4_f32: float in, float out), operands with their k contiguous in LDS (rows padded
// so that a quarter wave's 16-byte reads fall into different banks) or, for the entering state, straight from the
// workspace, which holds states transposed ([value column][key row]) for that reason.  A lane's 16-byte read
// gives one k to each of four instructions; both operands of a product are read the same way, so every instruction
// pairs equal k.  Sums run in a fixed order, so a result depends on where its chunk starts, which is where the
// step starts, and on nothing else: a position's values differ from the walk's, and between cuttings, by
// rounding only.
#include "common.h"

#include <math.h>

#define SC_L 64            // tokens per chunk
#define SC_MAXN 128        // largest key size (state rows) the kernels take; a multiple of 16
#define SC_MAXP 128        // largest value size per head
#define SC_LDN (SC_MAXN + 4)   // floats per LDS row of a [token][key row] tile: 16-byte reads of 16 rows hit 64 banks
#define SC_LDT (SC_L + 4)      // the same for tiles whose rows hold the chunk's 64 tokens
#define SC_THREADS 256

typedef float sc_f32x4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ float sc_softplus(float z) { return fmaxf(z, 0.f) + log1pf(expf(-fabsf(z))); }

// four products with the k a lane's two 16-byte reads hold: A row li and W row li at k0 + 4 lg .. + 3
__device__ __forceinline__ sc_f32x4 sc_mfma4(float4 a, float4 w, sc_f32x4 acc) {
    acc = __builtin_amdgcn_mfma_f32_16x16x4f32(a.x, w.x, acc, 0, 0, 0);
    acc = __builtin_amdgcn_mfma_f32_16x16x4f32(a.y, w.y, acc, 0, 0, 0);
    acc = __builtin_amdgcn_mfma_f32_16x16x4f32(a.z, w.z, acc, 0, 0, 0);
    acc = __builtin_amdgcn_mfma_f32_16x16x4f32(a.w, w.w, acc, 0, 0, 0);
    return acc;
}

// A tile from memory into LDS: element idx < total is load(idx), kept by store(idx, value).  Eight loads of a
// thread are in flight before the first is stored; a loop of load-then-store would wait out the memory's latency
// once per element, which is most of what such a kernel would then take.
#define SC_BATCH 8
template <typename Load, typename Store>
__device__ __forceinline__ void sc_fill(int total, Load load, Store store) {
    for (int base = threadIdx.x; base < total; base += SC_THREADS * SC_BATCH) {
        float r[SC_BATCH];
#pragma unroll
        for (int u = 0; u < SC_BATCH; ++u) {
            const int idx = base + u * SC_THREADS;
            r[u] = idx < total ? load(idx) : 0.f;
        }
#pragma unroll
        for (int u = 0; u < SC_BATCH; ++u) {
            const int idx = base + u * SC_THREADS;
            if (idx < total) store(idx, r[u]);
        }
    }
}

// dts[t] = dt_t and cs[t] = la_1 + .. + la_t for the chunk's n tokens, by the same instructions in both
// kernels that need them.  Ends with a barrier.
__device__ __forceinline__ void sc_steps(const float* __restrict__ steps, int ldw, int t0, int n, int h, float rate,
                                         float bias, float* dts, float* cs) {
    const int tid = threadIdx.x;
    if (tid < SC_L) {                                        // the first wave: a token per lane
        float dt = 0.f, run = 0.f;
        if (tid < n) {
            dt = sc_softplus(steps[(size_t)(t0 + tid) * ldw + h] + bias);
            run = -rate * dt;
        }
#pragma unroll
        for (int off = 1; off < SC_L; off <<= 1) {           // inclusive sums over the lanes, in a fixed order
            const float below = __shfl_up(run, off, TL_WAVE);
            if (tid >= off) run += below;
        }
        dts[tid] = dt;
        cs[tid] = run;
    }
    __syncthreads();
}

// The chunk's own term of the state, transposed: out[j][i] = sum_s x_s[j] * (exp(cs_L - cs_s) dt_s B_s[i]).
// A work-group per (chunk, head, sequence); wave w takes the blocks of 16 value columns w, w + 4, ...
__global__ __launch_bounds__(SC_THREADS) void ssd_local_state_kernel(
    const float* __restrict__ k, int ldk, const float* __restrict__ v, int ldv, const float* __restrict__ steps, int ldw,
    const float* __restrict__ rate_log, const float* __restrict__ step_bias, int share, const int32_t* __restrict__ q_start,
    float* __restrict__ ws_state, float* __restrict__ ws_decay, int NC, int H, int N, int P) {
    extern __shared__ __attribute__((aligned(16))) float sc_smem[];
    float* xT = sc_smem;                         // [SC_MAXP][SC_LDT]: x transposed, tokens contiguous
    float* bT = xT + SC_MAXP * SC_LDT;           // [SC_MAXN][SC_LDT]: weighted B transposed
    float* dts = bT + SC_MAXN * SC_LDT;          // [SC_L]
    float* cs = dts + SC_L;                      // [SC_L]
    const int c = blockIdx.x, h = blockIdx.y, s = blockIdx.z, tid = threadIdx.x;
    const int r0 = q_start[s], r1 = q_start[s + 1];
    const int t0 = r0 + c * SC_L;
    if (t0 >= r1) return;
    const int n = min(SC_L, r1 - t0);
    const float rate = expf(rate_log[h]), bias = step_bias ? step_bias[h] : 0.f;
    sc_steps(steps, ldw, t0, n, h, rate, bias, dts, cs);
    const float cs_end = cs[n - 1];
    __syncthreads();
    if (tid < SC_L) dts[tid] = tid < n ? expf(cs_end - cs[tid]) * dts[tid] : 0.f;      // a token's weight in the state
    __syncthreads();
    // tokens beyond the chunk's are zero, so that no product has to know n
    const int pcols = (P + 15) / 16 * 16;
    sc_fill(SC_L * pcols,
            [&](int idx) { const int tt = idx / pcols, j = idx - tt * pcols;
                           return (tt < n && j < P) ? v[(size_t)(t0 + tt) * ldv + h * P + j] : 0.f; },
            [&](int idx, float x) { const int tt = idx / pcols, j = idx - tt * pcols; xT[j * SC_LDT + tt] = x; });
    const int g = h / share;
    sc_fill(SC_L * N,
            [&](int idx) { const int tt = idx / N, i = idx - tt * N;
                           return tt < n ? k[(size_t)(t0 + tt) * ldk + g * N + i] : 0.f; },
            [&](int idx, float b) { const int tt = idx / N, i = idx - tt * N; bT[i * SC_LDT + tt] = dts[tt] * b; });
    __syncthreads();
    const int lane = tid & 63, wave = tid >> 6, li = lane & 15, lg = lane >> 4;
    float* dst = ws_state + (((size_t)s * NC + c) * H + h) * (size_t)N * P;
    for (int jt = wave; jt * 16 < P; jt += SC_THREADS / 64) {
        float4 af[SC_L / 16];
#pragma unroll
        for (int kk = 0; kk < SC_L / 16; ++kk)
            af[kk] = *reinterpret_cast<const float4*>(&xT[(jt * 16 + li) * SC_LDT + kk * 16 + 4 * lg]);
        for (int it = 0; it * 16 < N; ++it) {
            sc_f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int kk = 0; kk < SC_L / 16; ++kk)
                acc = sc_mfma4(af[kk], *reinterpret_cast<const float4*>(&bT[(it * 16 + li) * SC_LDT + kk * 16 + 4 * lg]), acc);
            // this lane holds value columns jt * 16 + 4 lg + e and key row it * 16 + li
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int j = jt * 16 + 4 * lg + e;
                if (j < P) dst[(size_t)j * N + it * 16 + li] = acc[e];
            }
        }
    }
    if (tid == 0) ws_decay[((size_t)s * NC + c) * H + h] = expf(cs_end);
}

// Per state element, the chunks of a sequence in order; the workspace holds states as [value column][key row].
__global__ void ssd_scan_states_kernel(float* __restrict__ ws_state, const float* __restrict__ ws_decay,
                                       float* __restrict__ state, long long state_stride,
                                       const int32_t* __restrict__ state_slots, const int32_t* __restrict__ q_start, int NC,
                                       int H, int N, int P) {
    const int e = blockIdx.x * blockDim.x + threadIdx.x, h = blockIdx.y, s = blockIdx.z;
    const int NP = N * P;
    if (e >= NP) return;
    const int r0 = q_start[s], r1 = q_start[s + 1];
    if (r1 <= r0) return;
    const int nc = (r1 - r0 + SC_L - 1) / SC_L;
    const int j = e / N, i = e - j * N;
    float* st = state + (size_t)state_slots[s] * state_stride + (size_t)h * NP + (size_t)i * P + j;
    float S = *st;
    for (int c = 0; c < nc; ++c) {
        const size_t at = ((size_t)s * NC + c) * H + h;
        float* w = ws_state + at * NP + e;
        const float local = *w;
        *w = S;                                  // what enters chunk c
        S = ws_decay[at] * S + local;
    }
    *st = S;
}

// y_t = sum_(s <= t) exp(cs_t - cs_s) dt_s (C_t . B_s) x_s + exp(cs_t) S_0^T C_t + skip x_t for a chunk's tokens.
// A work-group per (chunk, head, sequence); wave w owns tokens 16 w .. 16 w + 15 of the chunk.
__global__ __launch_bounds__(SC_THREADS) void ssd_outputs_kernel(
    const float* __restrict__ q, int ldq, const float* __restrict__ k, int ldk, const float* __restrict__ v, int ldv,
    const float* __restrict__ steps, int ldw, const float* __restrict__ rate_log, const float* __restrict__ step_bias,
    const float* __restrict__ skip, int share, const int32_t* __restrict__ q_start, const float* __restrict__ ws_state,
    float* __restrict__ out, int ldo, int NC, int H, int N, int P, int vec) {
    extern __shared__ __attribute__((aligned(16))) float sc_smem[];
    float* Cs = sc_smem;                         // [SC_L][SC_LDN]
    float* Bs = Cs + SC_L * SC_LDN;              // [SC_L][SC_LDN]
    float* Ms = Bs + SC_L * SC_LDN;              // [SC_L][SC_LDT]: exp(cs_t - cs_s) dt_s (C_t . B_s), s <= t
    float* xT = Ms + SC_L * SC_LDT;              // [SC_L value columns][SC_LDT]: a block of x transposed
    float* dts = xT + SC_L * SC_LDT;             // [SC_L]
    float* cs = dts + SC_L;                      // [SC_L]
    const int c = blockIdx.x, h = blockIdx.y, s = blockIdx.z, tid = threadIdx.x;
    const int r0 = q_start[s], r1 = q_start[s + 1];
    const int t0 = r0 + c * SC_L;
    if (t0 >= r1) return;
    const int n = min(SC_L, r1 - t0);
    const float rate = expf(rate_log[h]), bias = step_bias ? step_bias[h] : 0.f, skip_h = skip ? skip[h] : 0.f;
    const int g = h / share;
    sc_steps(steps, ldw, t0, n, h, rate, bias, dts, cs);
    // rows beyond the chunk's tokens are zero, so that no product has to know n (N is a multiple of 16: no column
    // beyond it is read)
    if (vec) {
        // rows that start at 16-byte borders: 16 bytes to a load, all of a thread's loads in flight at once
        const int n4 = N >> 2, total = SC_L * n4;
        constexpr int PER = SC_L * (SC_MAXN / 4) / SC_THREADS;
        float4 cr[PER], br[PER];
#pragma unroll
        for (int u = 0; u < PER; ++u) {
            const int idx = tid + u * SC_THREADS, tt = idx / n4, i4 = idx - tt * n4;
            const bool ok = idx < total && tt < n;
            cr[u] = ok ? *reinterpret_cast<const float4*>(&q[(size_t)(t0 + tt) * ldq + g * N + 4 * i4]) : make_float4(0.f, 0.f, 0.f, 0.f);
            br[u] = ok ? *reinterpret_cast<const float4*>(&k[(size_t)(t0 + tt) * ldk + g * N + 4 * i4]) : make_float4(0.f, 0.f, 0.f, 0.f);
        }
#pragma unroll
        for (int u = 0; u < PER; ++u) {
            const int idx = tid + u * SC_THREADS, tt = idx / n4, i4 = idx - tt * n4;
            if (idx < total) {
                *reinterpret_cast<float4*>(&Cs[tt * SC_LDN + 4 * i4]) = cr[u];
                *reinterpret_cast<float4*>(&Bs[tt * SC_LDN + 4 * i4]) = br[u];
            }
        }
    } else {
        sc_fill(SC_L * N,
                [&](int idx) { const int tt = idx / N, i = idx - tt * N;
                               return tt < n ? q[(size_t)(t0 + tt) * ldq + g * N + i] : 0.f; },
                [&](int idx, float x) { const int tt = idx / N, i = idx - tt * N; Cs[tt * SC_LDN + i] = x; });
        sc_fill(SC_L * N,
                [&](int idx) { const int tt = idx / N, i = idx - tt * N;
                               return tt < n ? k[(size_t)(t0 + tt) * ldk + g * N + i] : 0.f; },
                [&](int idx, float x) { const int tt = idx / N, i = idx - tt * N; Bs[tt * SC_LDN + i] = x; });
    }
    __syncthreads();
    const int lane = tid & 63, wave = tid >> 6, li = lane & 15, lg = lane >> 4;
    const int ksteps = (N + 15) / 16;
    // ---- the chunk's own matrix: this wave's 16 tokens against the tokens of the blocks up to its own ----
    {
        sc_f32x4 acc[SC_L / 16];
#pragma unroll
        for (int sb = 0; sb < SC_L / 16; ++sb) acc[sb] = sc_f32x4{0.f, 0.f, 0.f, 0.f};
        for (int kk = 0; kk < ksteps; ++kk) {
            const float4 af = *reinterpret_cast<const float4*>(&Cs[(wave * 16 + li) * SC_LDN + kk * 16 + 4 * lg]);
#pragma unroll
            for (int sb = 0; sb < SC_L / 16; ++sb)
                if (sb <= wave)
                    acc[sb] = sc_mfma4(af, *reinterpret_cast<const float4*>(&Bs[(sb * 16 + li) * SC_LDN + kk * 16 + 4 * lg]), acc[sb]);
        }
        // this lane holds tokens t = 16 wave + 4 lg + e and s = 16 sb + li
#pragma unroll
        for (int sb = 0; sb < SC_L / 16; ++sb)
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int t = wave * 16 + 4 * lg + e, ss = sb * 16 + li;
                Ms[t * SC_LDT + ss] = (sb <= wave && ss <= t && t < n) ? acc[sb][e] * expf(cs[t] - cs[ss]) * dts[ss] : 0.f;
            }
    }
    const float* S0T = ws_state + (((size_t)s * NC + c) * H + h) * (size_t)N * P;        // [P][N]
    const float into = expf(cs[wave * 16 + li]);             // the factor on the entering state, for this lane's A row
    for (int j0 = 0; j0 < P; j0 += SC_L) {
        __syncthreads();                         // Ms is written; the block of x before is done with
        sc_fill(SC_L * SC_L,
                [&](int idx) { const int tt = idx >> 6, jj = idx & 63;
                               return (tt < n && j0 + jj < P) ? v[(size_t)(t0 + tt) * ldv + h * P + j0 + jj] : 0.f; },
                [&](int idx, float x) { const int tt = idx >> 6, jj = idx & 63; xT[jj * SC_LDT + tt] = x; });
        __syncthreads();
        // the entering state's fragments are asked for now and used after the products within the chunk
        float4 sf[SC_MAXN / 16][SC_L / 16];
#pragma unroll
        for (int kk = 0; kk < SC_MAXN / 16; ++kk)
#pragma unroll
            for (int jt = 0; jt < SC_L / 16; ++jt) {
                const int j = j0 + jt * 16 + li;
                sf[kk][jt] = (kk < ksteps && j < P) ? *reinterpret_cast<const float4*>(&S0T[(size_t)j * N + kk * 16 + 4 * lg])
                                                    : make_float4(0.f, 0.f, 0.f, 0.f);
            }
        sc_f32x4 y[SC_L / 16];
#pragma unroll
        for (int jt = 0; jt < SC_L / 16; ++jt) y[jt] = sc_f32x4{0.f, 0.f, 0.f, 0.f};
        // within the chunk: k runs over the tokens s of the blocks up to this wave's own
        for (int sb = 0; sb <= wave; ++sb) {
            const float4 af = *reinterpret_cast<const float4*>(&Ms[(wave * 16 + li) * SC_LDT + sb * 16 + 4 * lg]);
#pragma unroll
            for (int jt = 0; jt < SC_L / 16; ++jt)
                y[jt] = sc_mfma4(af, *reinterpret_cast<const float4*>(&xT[(jt * 16 + li) * SC_LDT + sb * 16 + 4 * lg]), y[jt]);
        }
        // the entering state: k runs over the key rows; A rows carry exp(cs_t)
#pragma unroll
        for (int kk = 0; kk < SC_MAXN / 16; ++kk) {
            if (kk < ksteps) {
                float4 af = *reinterpret_cast<const float4*>(&Cs[(wave * 16 + li) * SC_LDN + kk * 16 + 4 * lg]);
                af.x *= into, af.y *= into, af.z *= into, af.w *= into;
#pragma unroll
                for (int jt = 0; jt < SC_L / 16; ++jt) y[jt] = sc_mfma4(af, sf[kk][jt], y[jt]);
            }
        }
        // this lane holds tokens t = 16 wave + 4 lg + e and value column j0 + 16 jt + li
#pragma unroll
        for (int jt = 0; jt < SC_L / 16; ++jt) {
            const int jj = jt * 16 + li, j = j0 + jj;
            if (j >= P) continue;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int t = wave * 16 + 4 * lg + e;
                if (t < n) out[(size_t)(t0 + t) * ldo + h * P + j] = y[jt][e] + skip_h * xT[jj * SC_LDT + t];
            }
        }
    }
}

extern "C" int tl_ssd_chunked_takes(int N, int P) { return N > 0 && N <= SC_MAXN && N % 16 == 0 && P > 0 && P <= SC_MAXP ? 1 : 0; }
extern "C" int tl_ssd_chunk_tokens() { return SC_L; }

// The operands of tl_linear_recurrence's third form (q = C and k = B [T, >= (H / share) * N], v = x [T, >= H * P],
// steps [T, >= H], rate_log, step_bias, skip [H]); NC: the most chunks of SC_L tokens one sequence brings;
// ws_state: S * NC * H * N * P floats (16-byte aligned), ws_decay: S * NC * H floats.  The request's state [H, N, P]
// at state + slot * state_stride is read and renewed.
extern "C" int tl_ssd_chunked(const float* q, int ldq, const float* k, int ldk, const float* v, int ldv, const float* steps,
                              int ldw, const float* rate_log, const float* step_bias, const float* skip, int share,
                              float* state, long long state_stride, const int32_t* state_slots, const int32_t* q_start,
                              float* out, int ldo, float* ws_state, float* ws_decay, int S, int NC, int H, int N, int P,
                              hipStream_t stream) {
    TL_CHECK_ARG(S >= 0 && NC > 0 && H > 0 && tl_ssd_chunked_takes(N, P), "tl_ssd_chunked: bad sizes H=%d N=%d P=%d chunks=%d", H, N, P, NC);
    TL_CHECK_ARG(share >= 1 && H % share == 0, "tl_ssd_chunked: %d heads do not share queries and keys in groups of %d", H, share);
    TL_CHECK_ARG(ldq >= H / share * N && ldk >= H / share * N && ldv >= H * P && ldo >= H * P && ldw >= H, "tl_ssd_chunked: rows too short");
    TL_CHECK_ARG(state_stride >= (long long)H * N * P, "tl_ssd_chunked: the state of a request is too small");
    TL_CHECK_ARG(rate_log && ws_state && ws_decay && ((uintptr_t)ws_state % 16) == 0, "tl_ssd_chunked: rates or the (16-byte aligned) workspace are missing");
    TL_CHECK_ARG(S <= 65535 && H <= 65535, "tl_ssd_chunked: too many sequences or heads for one launch");
    if (S == 0) return 0;
    // whether every row of q and k that a chunk reads starts at a 16-byte border
    const int vec = ((uintptr_t)q % 16 == 0 && (uintptr_t)k % 16 == 0 && ldq % 4 == 0 && ldk % 4 == 0) ? 1 : 0;
    const size_t lds_a = sizeof(float) * ((SC_MAXP + SC_MAXN) * SC_LDT + 2 * SC_L);
    const size_t lds_c = sizeof(float) * (2 * SC_L * SC_LDN + 2 * SC_L * SC_LDT + 2 * SC_L);
    hipLaunchKernelGGL(ssd_local_state_kernel, dim3(NC, H, S), dim3(SC_THREADS), lds_a, stream, k, ldk, v, ldv, steps, ldw,
                       rate_log, step_bias, share, q_start, ws_state, ws_decay, NC, H, N, P);
    TL_CHECK_LAUNCH("tl_ssd_chunked local states");
    hipLaunchKernelGGL(ssd_scan_states_kernel, dim3(tl_ceil_div(N * P, 256), H, S), dim3(256), 0, stream, ws_state, ws_decay, state,
                       state_stride, state_slots, q_start, NC, H, N, P);
    TL_CHECK_LAUNCH("tl_ssd_chunked scan");
    hipLaunchKernelGGL(ssd_outputs_kernel, dim3(NC, H, S), dim3(SC_THREADS), lds_c, stream, q, ldq, k, ldk, v, ldv, steps, ldw,
                       rate_log, step_bias, skip, share, q_start, ws_state, out, ldo, NC, H, N, P, vec);
    TL_CHECK_LAUNCH("tl_ssd_chunked outputs");
    return 0;
}
