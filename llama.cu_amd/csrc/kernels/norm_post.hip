// A norm BEHIND a sublayer, the residual sum, and the norm in front of the next sublayer, in one pass:
//
//   x <- x + a * rsqrt(mean(a^2) + eps_post) * w_post          (a: the sublayer's output; x: the 32-bit residual stream)
//   h  = x * rsqrt(mean(x^2) + eps_pre) * w_pre                (only if w_pre is given; with out but no w_pre: h = x, the
//                                                              stream itself rounded to out's type, for a sublayer that reads it so)
//
// One block per row; sums, factors and the stream are 32-bit, one rounding where h is stored.  The weights are the
// factors themselves (a model that stores them around zero adds the one when it loads them).  The order of the sums
// depends on the width and the block size only.
#include "common.h"

constexpr int NP_KEEP = 8;          // elements of a row that a thread keeps in registers: rows up to 8 x the block's threads are read once

// THREADS: 256, or 1024 where a step has few rows (what counts then is how many loads a row has in flight).  All loads of
// the kept elements go out before anything waits for one.
template <class TA, class TO, int THREADS>
__global__ void __launch_bounds__(THREADS)
norm_post_kernel(float *__restrict__ x, const TA *__restrict__ a, const float *__restrict__ a_bias, const float *__restrict__ w_post, float eps_post,
                 const float *__restrict__ w_pre, float eps_pre, TO *__restrict__ out, int d) {
    __shared__ float scratch[16];
    float *xr = x + (size_t)blockIdx.x * d;
    const TA *ar = a + (size_t)blockIdx.x * d;
    float keep[NP_KEEP], xs[NP_KEEP], wp[NP_KEEP], wq[NP_KEEP];
    float acc = 0.f;
#pragma unroll
    for (int e = 0; e < NP_KEEP; ++e) {
        const int c = threadIdx.x + e * THREADS;
        const bool in = c < d;
        keep[e] = in ? to_f32(ar[c]) + (a_bias ? a_bias[c] : 0.f) : 0.f;
        xs[e] = in ? xr[c] : 0.f;
        wp[e] = in ? w_post[c] : 0.f;
        wq[e] = (in && w_pre) ? w_pre[c] : 0.f;
    }
#pragma unroll
    for (int e = 0; e < NP_KEEP; ++e) acc += keep[e] * keep[e];
    for (int c = threadIdx.x + NP_KEEP * THREADS; c < d; c += THREADS) {
        const float v = to_f32(ar[c]) + (a_bias ? a_bias[c] : 0.f);
        acc += v * v;
    }
    const float f_post = rsqrtf(block_sum(acc, scratch) / (float)d + eps_post);
    acc = 0.f;
#pragma unroll
    for (int e = 0; e < NP_KEEP; ++e) {
        const int c = threadIdx.x + e * THREADS;
        if (c < d) {
            keep[e] = xs[e] + keep[e] * f_post * wp[e];
            xr[c] = keep[e];
            acc += keep[e] * keep[e];
        }
    }
    for (int c = threadIdx.x + NP_KEEP * THREADS; c < d; c += THREADS) {
        const float v = xr[c] + (to_f32(ar[c]) + (a_bias ? a_bias[c] : 0.f)) * f_post * w_post[c];
        xr[c] = v;
        acc += v * v;
    }
    if (!out) return;
    TO *o = out + (size_t)blockIdx.x * d;
    if (!w_pre) {                            // the stream itself, rounded once
#pragma unroll
        for (int e = 0; e < NP_KEEP; ++e) {
            const int c = threadIdx.x + e * THREADS;
            if (c < d) o[c] = from_f32<TO>(keep[e]);
        }
        for (int c = threadIdx.x + NP_KEEP * THREADS; c < d; c += THREADS) o[c] = from_f32<TO>(xr[c]);
        return;
    }
    const float f_pre = rsqrtf(block_sum(acc, scratch) / (float)d + eps_pre);
#pragma unroll
    for (int e = 0; e < NP_KEEP; ++e) {
        const int c = threadIdx.x + e * THREADS;
        if (c < d) o[c] = from_f32<TO>(keep[e] * f_pre * wq[e]);
    }
    for (int c = threadIdx.x + NP_KEEP * THREADS; c < d; c += THREADS)      // (a thread reads what it wrote itself)
        o[c] = from_f32<TO>(xr[c] * f_pre * w_pre[c]);
}

// x: [n, d] float32, updated in place.  a: [n, d] of a_type.  w_post, w_pre: float32 [d]; w_pre and out may be null.
// a_bias: null, or float32 [d] that the sublayer's output still lacks (a bias of its last product): a + a_bias is normed.
LCU_API int lcu_norm_post(float *x, const void *a, int a_type, const float *a_bias, const float *w_post, float eps_post, const float *w_pre,
                          float eps_pre, void *out, int out_type, int n, int d, hipStream_t stream) {
    if (n <= 0) return LCU_OK;
    if (d <= 0 || !x || !a || !w_post || (w_pre && !out)) return LCU_BAD_ARGUMENT;
    // few rows of some width: 1024 threads a row (a row's sums are then added in another order than with 256: a
    // difference of rounding between steps of few and of many rows)
    const bool wide = n <= 64 && d >= 1024;
    dim3 grid(n);
#define GO(TA, TO) do { if (wide) norm_post_kernel<TA, TO, 1024><<<grid, dim3(1024), 0, stream>>>(x, (const TA *)a, a_bias, w_post, eps_post, w_pre, eps_pre, (TO *)out, d); \
                        else norm_post_kernel<TA, TO, 256><<<grid, dim3(256), 0, stream>>>(x, (const TA *)a, a_bias, w_post, eps_post, w_pre, eps_pre, (TO *)out, d); } while (0)
    if (a_type == LCU_F32 && out_type == LCU_F32) GO(float, float);
    else if (a_type == LCU_F32 && out_type == LCU_BF16) GO(float, bf16_t);
    else if (a_type == LCU_BF16 && out_type == LCU_BF16) GO(bf16_t, bf16_t);
    else if (a_type == LCU_BF16 && out_type == LCU_F32) GO(bf16_t, float);
    else return LCU_BAD_ARGUMENT;
#undef GO
    LCU_LAUNCH_CHECK();
    return LCU_OK;
}

// acc = (first ? 0 : acc) + scale * x over `count` floats: the 32-bit sum of several branches' outputs.
template <class TX>
__global__ void scaled_sum_kernel(float *__restrict__ acc, const TX *__restrict__ x, float scale, long long count, int first) {
    const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < count) acc[i] = (first ? 0.f : acc[i]) + scale * to_f32(x[i]);
}

LCU_API int lcu_scaled_sum(float *acc, const void *x, int x_type, float scale, long long count, int first, hipStream_t stream) {
    if (count <= 0) return LCU_OK;
    if (!acc || !x) return LCU_BAD_ARGUMENT;
    dim3 grid((unsigned)((count + 255) / 256)), block(256);
    if (x_type == LCU_F32) scaled_sum_kernel<float><<<grid, block, 0, stream>>>(acc, (const float *)x, scale, count, first);
    else if (x_type == LCU_BF16) scaled_sum_kernel<bf16_t><<<grid, block, 0, stream>>>(acc, (const bf16_t *)x, scale, count, first);
    else return LCU_BAD_ARGUMENT;
    LCU_LAUNCH_CHECK();
    return LCU_OK;
}

// rows[t, c] += bias[c] in place (rows: [n, d] of `type`, the sum in 32-bit, one rounding): the bias of a product whose
// kernel adds none.
template <class T>
__global__ void row_bias_kernel(T *__restrict__ rows, const float *__restrict__ bias, long long count, int d) {
    const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < count) rows[i] = from_f32<T>(to_f32(rows[i]) + bias[i % d]);
}

LCU_API int lcu_row_bias(void *rows, int type, const float *bias, int n, int d, hipStream_t stream) {
    if (n <= 0) return LCU_OK;
    if (d <= 0 || !rows || !bias) return LCU_BAD_ARGUMENT;
    const long long count = (long long)n * d;
    dim3 grid((unsigned)((count + 255) / 256)), block(256);
    if (type == LCU_F32) row_bias_kernel<float><<<grid, block, 0, stream>>>((float *)rows, bias, count, d);
    else if (type == LCU_BF16) row_bias_kernel<bf16_t><<<grid, block, 0, stream>>>((bf16_t *)rows, bias, count, d);
    else return LCU_BAD_ARGUMENT;
    LCU_LAUNCH_CHECK();
    return LCU_OK;
}
