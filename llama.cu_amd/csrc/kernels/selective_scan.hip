// The selective scan of a state-space mixer: per channel c and state index n a running value in 32-bit,
//   dt_c   = softplus(dt_raw[t, c] + dt_bias[c])                      the token's step size for the channel
//   S[c,n] <- exp(dt_c * A[c, n]) * S[c, n] + dt_c * x[t, c] * B[t, n]
//   y[t,c] = sum_n S[c, n] * C[t, n] + D[c] * x[t, c]
//   out[t, c] = y[t, c] * silu(z[t, c])
// with A = -exp(A_log) made once at load.  B and C are shared by all channels of a token; dt, x and z are per
// channel.  A request's tokens are one chain; channels and states are independent.  The states of a channel are
// shared out over L neighbouring lanes (L a power of two, at most four states a lane), so that a token costs a lane
// four exponentials and eight multiply-adds and a wave holds 64 / L channels; the sum over n crosses the lanes of a
// channel at the end of a token.  The values of the next tokens are loaded while the ones before are folded in.
// The state [channels, states] of a request lives in its slot, is taken as zero where the request's first token of
// the step stands at position 0, and is left as the step's last token makes it.
// A request that feeds SCAN_LONG tokens or more is cut into SCAN_RUNS runs that are walked side by side: every run is
// walked from zero, which gives what its tokens add to any state it starts from (the recurrence is linear, and a run's
// decay of a state is exp(A * the sum of its step sizes)); a small kernel chains the runs' starts; the runs are walked
// again from their true starts, now with outputs.  Twice the arithmetic on SCAN_RUNS times the lanes.  For shorter
// portions every token is folded in by the same operations in the same order however the request is cut.
#include "common.h"

constexpr int SCAN_PER_LANE = 4;         // states a lane keeps
constexpr int SCAN_TOKENS = 4;           // tokens whose values are loaded together
constexpr int SCAN_LONG = 512;           // a request that feeds so many tokens in a step is walked in runs
constexpr int SCAN_RUNS = 32;

enum { SCAN_PLAIN = 0, SCAN_RUN_SUMS = 1, SCAN_RUN_OUTPUTS = 2 };

// The index of request r among the step's long requests (those that are walked in runs).
__device__ __forceinline__ int long_index(const int *__restrict__ q_start, int r) {
    int k = 0;
    for (int i = 0; i < r; ++i) k += (q_start[i + 1] - q_start[i] >= SCAN_LONG) ? 1 : 0;
    return k;
}

__device__ __forceinline__ float softplus_f(float z) { return z > 20.f ? z : log1pf(expf(z)); }
__device__ __forceinline__ float silu_f(float z) { return z / (1.0f + expf(-z)); }

// MODE SCAN_PLAIN: one block walks all tokens of a request (grid.z == 1).  SCAN_RUN_SUMS: blockIdx.z is a run of a long
// request, walked from zero; what it leaves goes to runs[(long index * SCAN_RUNS + run)] as [channels, states + 1]: the
// states' sums and the sum of the step sizes; no outputs; short requests are skipped.  SCAN_RUN_OUTPUTS: a long request's
// run starts from what the chaining kernel left in `runs` and stores no state; a short request is walked by the block of
// run 0 as in SCAN_PLAIN.
template <class T, int MODE>
__global__ void __launch_bounds__(256)
selective_scan_kernel(const T *__restrict__ x, int x_stride, const float *__restrict__ dt_raw, int dt_stride,
                      const float *__restrict__ dt_bias, const float *__restrict__ bc, int bc_stride,
                      const float *__restrict__ A, const float *__restrict__ D, const float *__restrict__ z, int z_stride,
                      float *__restrict__ state, size_t slot_stride, T *__restrict__ out, int out_stride,
                      const int *__restrict__ q_start, const int *__restrict__ ctx_len, const int *__restrict__ state_slot,
                      int channels, int states, int lanes, float *__restrict__ runs) {
    const int r = blockIdx.y;
    const int per_block = blockDim.x / lanes;                    // channels of a block
    const int cl = threadIdx.x / lanes, part = threadIdx.x % lanes;
    const int c_true = blockIdx.x * per_block + cl;
    const bool live = c_true < channels;
    const int c = live ? c_true : channels - 1;                  // lanes beyond the last channel compute along and store nothing
    const int n0 = part * SCAN_PER_LANE;
    int t0 = q_start[r], t1 = q_start[r + 1];
    const bool is_long = MODE != SCAN_PLAIN && t1 - t0 >= SCAN_LONG;
    if (MODE == SCAN_RUN_SUMS && !is_long) return;
    if (MODE == SCAN_RUN_OUTPUTS && !is_long && blockIdx.z > 0) return;
    const bool fresh = ctx_len[r] - (t1 - t0) == 0;
    float *st = state + (size_t)state_slot[r] * slot_stride + (size_t)c * states;
    float *run_st = nullptr;
    if (is_long) {
        const int len = t1 - t0, run = blockIdx.z;
        const int first = t0;
        t0 = first + (int)((long long)len * run / SCAN_RUNS);
        t1 = first + (int)((long long)len * (run + 1) / SCAN_RUNS);
        run_st = runs + (((size_t)long_index(q_start, r) * SCAN_RUNS + run) * channels + c) * (states + 1);
    }
    float S[SCAN_PER_LANE], a[SCAN_PER_LANE];
#pragma unroll
    for (int i = 0; i < SCAN_PER_LANE; ++i) {
        const bool in = n0 + i < states;
        if (MODE == SCAN_RUN_SUMS) S[i] = 0.f;
        else if (is_long) S[i] = in ? run_st[n0 + i] : 0.f;
        else S[i] = (fresh || !in) ? 0.f : st[n0 + i];
        a[i] = in ? A[(size_t)c * states + n0 + i] : 0.f;
    }
    const float bias = dt_bias[c], d = D[c];
    float dt_sum = 0.f;
    for (int t = t0; t < t1; t += SCAN_TOKENS) {
        float dtv[SCAN_TOKENS], xv[SCAN_TOKENS], zv[SCAN_TOKENS], Bv[SCAN_TOKENS][SCAN_PER_LANE], Cv[SCAN_TOKENS][SCAN_PER_LANE];
#pragma unroll
        for (int b = 0; b < SCAN_TOKENS; ++b) {
            const int tt = t + b < t1 ? t + b : t1 - 1;          // (rows beyond the last are read again and not used)
            dtv[b] = dt_raw[(size_t)tt * dt_stride + c];
            xv[b] = to_f32(x[(size_t)tt * x_stride + c]);
            if (MODE != SCAN_RUN_SUMS) zv[b] = z[(size_t)tt * z_stride + c];
#pragma unroll
            for (int i = 0; i < SCAN_PER_LANE; ++i) {
                const bool in = n0 + i < states;
                Bv[b][i] = in ? bc[(size_t)tt * bc_stride + n0 + i] : 0.f;
                if (MODE != SCAN_RUN_SUMS) Cv[b][i] = in ? bc[(size_t)tt * bc_stride + states + n0 + i] : 0.f;
            }
        }
#pragma unroll
        for (int b = 0; b < SCAN_TOKENS; ++b) {
            if (t + b >= t1) break;
            const float dt = softplus_f(dtv[b] + bias);
            const float dx = dt * xv[b];
            if (MODE == SCAN_RUN_SUMS) {
                dt_sum += dt;
#pragma unroll
                for (int i = 0; i < SCAN_PER_LANE; ++i) S[i] = expf(dt * a[i]) * S[i] + dx * Bv[b][i];
                continue;
            }
            float y = 0.f;
#pragma unroll
            for (int i = 0; i < SCAN_PER_LANE; ++i) {
                S[i] = expf(dt * a[i]) * S[i] + dx * Bv[b][i];
                y += S[i] * Cv[b][i];
            }
            for (int off = lanes >> 1; off > 0; off >>= 1) y += __shfl_xor(y, off, WAVE);
            if (live && part == 0) out[(size_t)(t + b) * out_stride + c] = from_f32<T>((y + d * xv[b]) * silu_f(zv[b]));
        }
    }
    if (!live) return;
    if (MODE == SCAN_RUN_SUMS) {
#pragma unroll
        for (int i = 0; i < SCAN_PER_LANE; ++i)
            if (n0 + i < states) run_st[n0 + i] = S[i];
        if (part == 0) run_st[states] = dt_sum;
        return;
    }
    if (is_long) return;                                         // (the chaining kernel has left the request's state)
#pragma unroll
    for (int i = 0; i < SCAN_PER_LANE; ++i)
        if (n0 + i < states) st[n0 + i] = S[i];
}

// One thread per (long request, channel, state): the state each run starts from takes the place of the run's own sum, in
// the order of the runs, and the request's slot gets what the last run leaves.
__global__ void __launch_bounds__(256)
selective_scan_chain_kernel(const float *__restrict__ A, float *__restrict__ state, size_t slot_stride, const int *__restrict__ q_start,
                            const int *__restrict__ ctx_len, const int *__restrict__ state_slot, int channels, int states,
                            float *__restrict__ runs) {
    const int r = blockIdx.y;
    const int len = q_start[r + 1] - q_start[r];
    if (len < SCAN_LONG) return;
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= channels * states) return;
    const int c = i / states, n = i % states;
    const bool fresh = ctx_len[r] - len == 0;
    float *st = state + (size_t)state_slot[r] * slot_stride + (size_t)c * states + n;
    float *run_st = runs + ((size_t)long_index(q_start, r) * SCAN_RUNS * channels + c) * (states + 1);
    const float a = A[(size_t)c * states + n];
    float S = fresh ? 0.f : *st;
    for (int run = 0; run < SCAN_RUNS; ++run) {
        float *p = run_st + (size_t)run * channels * (states + 1);
        const float own = p[n], dt_sum = p[states];
        p[n] = S;
        S = expf(a * dt_sum) * S + own;
    }
    *st = S;
}

template <class T>
static int selective_scan_t(const T *x, int x_stride, const float *dt_raw, int dt_stride, const float *dt_bias, const float *bc,
                            int bc_stride, const float *A, const float *D, const float *z, int z_stride, float *state, size_t slot_stride,
                            T *out, int out_stride, const int *q_start, const int *ctx_len, const int *state_slot, int n_req,
                            int channels, int states, float *runs, hipStream_t stream) {
    int lanes = 1;
    while (lanes * SCAN_PER_LANE < states) lanes *= 2;
    const int per_block = 256 / lanes;
    const unsigned gx = (channels + per_block - 1) / per_block;
    const dim3 block(256);
#define ARGS x, x_stride, dt_raw, dt_stride, dt_bias, bc, bc_stride, A, D, z, z_stride, state, slot_stride, out, out_stride, q_start, ctx_len, \
             state_slot, channels, states, lanes, runs
    if (!runs) {
        selective_scan_kernel<T, SCAN_PLAIN><<<dim3(gx, n_req), block, 0, stream>>>(ARGS);
        LCU_LAUNCH_CHECK();
        return LCU_OK;
    }
    selective_scan_kernel<T, SCAN_RUN_SUMS><<<dim3(gx, n_req, SCAN_RUNS), block, 0, stream>>>(ARGS);
    LCU_LAUNCH_CHECK();
    selective_scan_chain_kernel<<<dim3((channels * states + 255) / 256, n_req), block, 0, stream>>>(A, state, slot_stride, q_start, ctx_len,
                                                                                                  state_slot, channels, states, runs);
    LCU_LAUNCH_CHECK();
    selective_scan_kernel<T, SCAN_RUN_OUTPUTS><<<dim3(gx, n_req, SCAN_RUNS), block, 0, stream>>>(ARGS);
    LCU_LAUNCH_CHECK();
#undef ARGS
    return LCU_OK;
}

LCU_API int lcu_selective_scan_long() { return SCAN_LONG; }
LCU_API int lcu_selective_scan_runs() { return SCAN_RUNS; }

// x: [n, x_stride] of `type` (the channels at its first columns); dt_raw: [n, dt_stride], bc: [n, bc_stride] holding B then C
// (states each), z: [n, z_stride], all 32-bit, the channels (or states) at their first columns; dt_bias, D: [channels],
// A: [channels, states] 32-bit.  state: slot s at state + s * slot_stride, [channels, states] 32-bit.  out: [n, out_stride]
// of `type`.  runs: null (no request of the step feeds lcu_selective_scan_long() tokens or more), or scratch of (number of
// such requests) * lcu_selective_scan_runs() * channels * (states + 1) floats.
LCU_API int lcu_selective_scan(const void *x, int type, int x_stride, const float *dt_raw, int dt_stride, const float *dt_bias,
                               const float *bc, int bc_stride, const float *A, const float *D, const float *z, int z_stride,
                               float *state, long long slot_stride, void *out, int out_stride, const int *q_start,
                               const int *ctx_len, const int *state_slot, int n, int n_req, int channels, int states,
                               float *runs, hipStream_t stream) {
    if (n <= 0 || n_req <= 0) return LCU_OK;
    if (channels <= 0 || states <= 0 || states > SCAN_PER_LANE * WAVE || n_req > 65535) return LCU_BAD_ARGUMENT;
    if (type == LCU_F32)
        return selective_scan_t<float>((const float *)x, x_stride, dt_raw, dt_stride, dt_bias, bc, bc_stride, A, D, z, z_stride, state,
                                       (size_t)slot_stride, (float *)out, out_stride, q_start, ctx_len, state_slot, n_req, channels, states,
                                       runs, stream);
    if (type == LCU_BF16)
        return selective_scan_t<bf16_t>((const bf16_t *)x, x_stride, dt_raw, dt_stride, dt_bias, bc, bc_stride, A, D, z, z_stride, state,
                                        (size_t)slot_stride, (bf16_t *)out, out_stride, q_start, ctx_len, state_slot, n_req, channels, states,
                                        runs, stream);
    return LCU_BAD_ARGUMENT;
}
