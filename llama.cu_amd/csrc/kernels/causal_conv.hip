// A short causal convolution over time on each channel of a step's rows, with the inputs that a request fed in
// earlier steps kept as state:
//   y[t, c] = act(bias[c] + sum_j w[c, j] * x[t - taps + 1 + j, c])        j = 0 .. taps - 1, the last column is the
//                                                                          current token's
// x at places before a request's position 0 counts as zero.  x are `channels` neighbouring columns of rows that a
// matrix product left (32-bit or bfloat16); weights, bias and state are 32-bit; the sums are 32-bit.  The state of a
// request, [taps - 1, channels] in its slot, holds its last taps - 1 inputs, oldest first; it is taken as zeros where
// the request's first token of the step stands at position 0.  Two kernels: the convolution reads the state, the
// update (behind it on the stream) moves the state on: a portion shorter than taps - 1 tokens keeps some of the old
// rows, so the two cannot be one pass over the same memory.  For a step in which every request feeds one token
// one kernel does both: a thread owns a channel of a request and reads what it overwrites before it does.
#include "common.h"

constexpr int CONV_MAX_TAPS = 16;

enum { CONV_ACT_NONE = 0, CONV_ACT_SILU = 1 };

__device__ __forceinline__ float conv_act(float z, int act) { return act == CONV_ACT_SILU ? z / (1.0f + expf(-z)) : z; }

template <class TI, class TO>
__global__ void __launch_bounds__(256)
causal_conv_kernel(const TI *__restrict__ x, int x_stride, int x_off, const float *__restrict__ w,
                   const float *__restrict__ bias, const float *__restrict__ state, size_t slot_stride,
                   TO *__restrict__ out, int out_stride, const int *__restrict__ req_of_token,
                   const int *__restrict__ q_start, const int *__restrict__ ctx_len, const int *__restrict__ state_slot,
                   int channels, int taps, int act) {
    const int c = blockIdx.x * blockDim.x + threadIdx.x;
    if (c >= channels) return;
    const int t = blockIdx.y;
    const int r = req_of_token[t];
    const int t0 = q_start[r];
    const bool fresh = ctx_len[r] - (q_start[r + 1] - t0) == 0;
    const float *st = state + (size_t)state_slot[r] * slot_stride + c;
    float acc = bias ? bias[c] : 0.f;
    for (int j = 0; j < taps; ++j) {
        const int s = t - (taps - 1) + j;                // the row that tap j reads
        float v;
        if (s >= t0) v = to_f32(x[(size_t)s * x_stride + x_off + c]);
        else v = fresh ? 0.f : st[(size_t)(taps - 1 + s - t0) * channels];
        acc += w[(size_t)c * taps + j] * v;
    }
    out[(size_t)t * out_stride + c] = from_f32<TO>(conv_act(acc, act));
}

// One thread per (request, channel): the state's rows move up by the number of tokens fed, oldest first, so that a
// row is read before it is written.
template <class TI>
__global__ void __launch_bounds__(256)
causal_conv_update_kernel(const TI *__restrict__ x, int x_stride, int x_off, float *__restrict__ state, size_t slot_stride,
                          const int *__restrict__ q_start, const int *__restrict__ ctx_len,
                          const int *__restrict__ state_slot, int channels, int taps) {
    const int c = blockIdx.x * blockDim.x + threadIdx.x;
    if (c >= channels) return;
    const int r = blockIdx.y;
    const int t0 = q_start[r], len = q_start[r + 1] - t0;
    if (len <= 0) return;
    const bool fresh = ctx_len[r] - len == 0;
    float *st = state + (size_t)state_slot[r] * slot_stride + c;
    for (int i = 0; i < taps - 1; ++i) {
        const int rel = len + i - (taps - 1);            // the step's row that becomes the state's row i (negative: an old row)
        float v;
        if (rel >= 0) v = to_f32(x[(size_t)(t0 + rel) * x_stride + x_off + c]);
        else v = fresh ? 0.f : st[(size_t)(i + len) * channels];
        st[(size_t)i * channels] = v;
    }
}

// Every request feeds one token: row r is request r's.  Convolution and update in one pass.
template <class TI, class TO>
__global__ void __launch_bounds__(256)
causal_conv_single_kernel(const TI *__restrict__ x, int x_stride, int x_off, const float *__restrict__ w,
                          const float *__restrict__ bias, float *__restrict__ state, size_t slot_stride,
                          TO *__restrict__ out, int out_stride, const int *__restrict__ ctx_len,
                          const int *__restrict__ state_slot, int channels, int taps, int act) {
    const int c = blockIdx.x * blockDim.x + threadIdx.x;
    if (c >= channels) return;
    const int r = blockIdx.y;
    const bool fresh = ctx_len[r] == 1;
    float *st = state + (size_t)state_slot[r] * slot_stride + c;
    const float cur = to_f32(x[(size_t)r * x_stride + x_off + c]);
    float acc = bias ? bias[c] : 0.f;
    for (int i = 0; i < taps - 1; ++i) {                 // (the taps in the order of the kernel for portions: the same bits)
        const float v = fresh ? 0.f : st[(size_t)i * channels];
        acc += w[(size_t)c * taps + i] * v;
        if (i > 0) st[(size_t)(i - 1) * channels] = v;
    }
    acc += w[(size_t)c * taps + taps - 1] * cur;
    if (taps > 1) st[(size_t)(taps - 2) * channels] = cur;
    out[(size_t)r * out_stride + c] = from_f32<TO>(conv_act(acc, act));
}

template <class TI, class TO>
static int causal_conv_t(const TI *x, int x_stride, int x_off, const float *w, const float *bias, float *state, size_t slot_stride,
                         TO *out, int out_stride, const int *req_of_token, const int *q_start, const int *ctx_len,
                         const int *state_slot, int n, int n_req, int channels, int taps, int act, int single, hipStream_t stream) {
    const dim3 block(256);
    const int gx = (channels + 255) / 256;
    if (single) {
        causal_conv_single_kernel<TI, TO><<<dim3(gx, n_req), block, 0, stream>>>(x, x_stride, x_off, w, bias, state, slot_stride, out,
                                                                              out_stride, ctx_len, state_slot, channels, taps, act);
        LCU_LAUNCH_CHECK();
        return LCU_OK;
    }
    causal_conv_kernel<TI, TO><<<dim3(gx, n), block, 0, stream>>>(x, x_stride, x_off, w, bias, state, slot_stride, out, out_stride,
                                                              req_of_token, q_start, ctx_len, state_slot, channels, taps, act);
    LCU_LAUNCH_CHECK();
    if (taps > 1) {
        causal_conv_update_kernel<TI><<<dim3(gx, n_req), block, 0, stream>>>(x, x_stride, x_off, state, slot_stride, q_start, ctx_len,
                                                                          state_slot, channels, taps);
        LCU_LAUNCH_CHECK();
    }
    return LCU_OK;
}

// x: [n, x_stride] of x_type, the channels at columns x_off ..; w: [channels, taps], bias: null or [channels], 32-bit.
// state: the slots' [taps - 1, channels] 32-bit rows, slot s at state + s * slot_stride (not read or written with one tap).
// out: [n, out_stride] of out_type, the channels at its first columns.  single: every request feeds one token (n == n_req).
LCU_API int lcu_causal_conv(const void *x, int x_type, int x_stride, int x_off, const float *w, const float *bias, float *state,
                            long long slot_stride, void *out, int out_type, int out_stride, const int *req_of_token,
                            const int *q_start, const int *ctx_len, const int *state_slot, int n, int n_req, int channels,
                            int taps, int act, int single, hipStream_t stream) {
    if (n <= 0 || n_req <= 0) return LCU_OK;
    if (channels <= 0 || taps < 1 || taps > CONV_MAX_TAPS || n > 65535 * 1024 || (single && n != n_req) || (taps > 1 && !state) ||
        (act != CONV_ACT_NONE && act != CONV_ACT_SILU))
        return LCU_BAD_ARGUMENT;
    if (n > 65535) return LCU_UNSUPPORTED;
#define GO(TI, TO) return causal_conv_t<TI, TO>((const TI *)x, x_stride, x_off, w, bias, state, (size_t)slot_stride, (TO *)out, out_stride, \
                                                req_of_token, q_start, ctx_len, state_slot, n, n_req, channels, taps, act, single, stream)
    if (x_type == LCU_F32 && out_type == LCU_F32) GO(float, float);
    if (x_type == LCU_F32 && out_type == LCU_BF16) GO(float, bf16_t);
    if (x_type == LCU_BF16 && out_type == LCU_F32) GO(bf16_t, float);
    if (x_type == LCU_BF16 && out_type == LCU_BF16) GO(bf16_t, bf16_t);
#undef GO
    return LCU_BAD_ARGUMENT;
}
