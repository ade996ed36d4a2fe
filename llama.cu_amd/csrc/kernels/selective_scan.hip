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
// the step stands at position 0, and is left as the step's last token makes it.  Nothing depends on how a request's
// tokens are cut into steps: every token is folded in by the same operations in the same order.
#include "common.h"

constexpr int SCAN_PER_LANE = 4;         // states a lane keeps
constexpr int SCAN_TOKENS = 4;           // tokens whose values are loaded together

__device__ __forceinline__ float softplus_f(float z) { return z > 20.f ? z : log1pf(expf(z)); }
__device__ __forceinline__ float silu_f(float z) { return z / (1.0f + expf(-z)); }

template <class T>
__global__ void __launch_bounds__(256)
selective_scan_kernel(const T *__restrict__ x, int x_stride, const float *__restrict__ dt_raw, int dt_stride,
                      const float *__restrict__ dt_bias, const float *__restrict__ bc, int bc_stride,
                      const float *__restrict__ A, const float *__restrict__ D, const float *__restrict__ z, int z_stride,
                      float *__restrict__ state, size_t slot_stride, T *__restrict__ out, int out_stride,
                      const int *__restrict__ q_start, const int *__restrict__ ctx_len, const int *__restrict__ state_slot,
                      int channels, int states, int lanes) {
    const int r = blockIdx.y;
    const int per_block = blockDim.x / lanes;                    // channels of a block
    const int cl = threadIdx.x / lanes, part = threadIdx.x % lanes;
    const int c_true = blockIdx.x * per_block + cl;
    const bool live = c_true < channels;
    const int c = live ? c_true : channels - 1;                  // lanes beyond the last channel compute along and store nothing
    const int n0 = part * SCAN_PER_LANE;
    const int t0 = q_start[r], t1 = q_start[r + 1];
    const bool fresh = ctx_len[r] - (t1 - t0) == 0;
    float *st = state + (size_t)state_slot[r] * slot_stride + (size_t)c * states;
    float S[SCAN_PER_LANE], a[SCAN_PER_LANE];
#pragma unroll
    for (int i = 0; i < SCAN_PER_LANE; ++i) {
        const bool in = n0 + i < states;
        S[i] = (fresh || !in) ? 0.f : st[n0 + i];
        a[i] = in ? A[(size_t)c * states + n0 + i] : 0.f;
    }
    const float bias = dt_bias[c], d = D[c];
    for (int t = t0; t < t1; t += SCAN_TOKENS) {
        float dtv[SCAN_TOKENS], xv[SCAN_TOKENS], zv[SCAN_TOKENS], Bv[SCAN_TOKENS][SCAN_PER_LANE], Cv[SCAN_TOKENS][SCAN_PER_LANE];
#pragma unroll
        for (int b = 0; b < SCAN_TOKENS; ++b) {
            const int tt = t + b < t1 ? t + b : t1 - 1;          // (rows beyond the request's last are read again and not used)
            dtv[b] = dt_raw[(size_t)tt * dt_stride + c];
            xv[b] = to_f32(x[(size_t)tt * x_stride + c]);
            zv[b] = z[(size_t)tt * z_stride + c];
#pragma unroll
            for (int i = 0; i < SCAN_PER_LANE; ++i) {
                const bool in = n0 + i < states;
                Bv[b][i] = in ? bc[(size_t)tt * bc_stride + n0 + i] : 0.f;
                Cv[b][i] = in ? bc[(size_t)tt * bc_stride + states + n0 + i] : 0.f;
            }
        }
#pragma unroll
        for (int b = 0; b < SCAN_TOKENS; ++b) {
            if (t + b >= t1) break;
            const float dt = softplus_f(dtv[b] + bias);
            const float dx = dt * xv[b];
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
    if (live) {
#pragma unroll
        for (int i = 0; i < SCAN_PER_LANE; ++i)
            if (n0 + i < states) st[n0 + i] = S[i];
    }
}

// x: [n, x_stride] of `type` (the channels at its first columns); dt_raw: [n, dt_stride], bc: [n, bc_stride] holding B then C
// (states each), z: [n, z_stride], all 32-bit, the channels (or states) at their first columns; dt_bias, D: [channels],
// A: [channels, states] 32-bit.  state: slot s at state + s * slot_stride, [channels, states] 32-bit.  out: [n, out_stride]
// of `type`.
LCU_API int lcu_selective_scan(const void *x, int type, int x_stride, const float *dt_raw, int dt_stride, const float *dt_bias,
                               const float *bc, int bc_stride, const float *A, const float *D, const float *z, int z_stride,
                               float *state, long long slot_stride, void *out, int out_stride, const int *q_start,
                               const int *ctx_len, const int *state_slot, int n, int n_req, int channels, int states,
                               hipStream_t stream) {
    if (n <= 0 || n_req <= 0) return LCU_OK;
    if (channels <= 0 || states <= 0 || states > SCAN_PER_LANE * WAVE || n_req > 65535) return LCU_BAD_ARGUMENT;
    int lanes = 1;
    while (lanes * SCAN_PER_LANE < states) lanes *= 2;
    const int per_block = 256 / lanes;
    const dim3 grid((channels + per_block - 1) / per_block, n_req), block(256);
    if (type == LCU_F32)
        selective_scan_kernel<float><<<grid, block, 0, stream>>>((const float *)x, x_stride, dt_raw, dt_stride, dt_bias, bc, bc_stride, A, D, z,
                                                                z_stride, state, (size_t)slot_stride, (float *)out, out_stride, q_start,
                                                                ctx_len, state_slot, channels, states, lanes);
    else if (type == LCU_BF16)
        selective_scan_kernel<bf16_t><<<grid, block, 0, stream>>>((const bf16_t *)x, x_stride, dt_raw, dt_stride, dt_bias, bc, bc_stride, A, D,
                                                                 z, z_stride, state, (size_t)slot_stride, (bf16_t *)out, out_stride, q_start,
                                                                 ctx_len, state_slot, channels, states, lanes);
    else
        return LCU_BAD_ARGUMENT;
    LCU_LAUNCH_CHECK();
    return LCU_OK;
}
