// The generalised delta rule: a recurrent mixer whose state per head is a matrix S [dk, dv]
// (key channel, value channel) in 32-bit.  For every token, with per key channel a decay w, a
// removal rate a, the key k, its unit vector u = k / sqrt(sum(k^2) + 1e-6), the query r, and
// per value channel v:
//   S <- diag(w) S - (a * u) (u^T S) + k v^T        (decay and removal act on S as the token found it)
//   o  = S^T r
// Everything that enters the recurrence is 32-bit.  Three kernels:
//   prep  (parallel over tokens and heads): w, a * u, u, k, r as 32-bit vectors;
//           w = exp(-exp(-1/2) * sigmoid(w0 + W2 tanh(l))), l the row's low-rank projection,
//           a = sigmoid(a_lin + a_bias);
//   scan  (sequential over a request's tokens, parallel over requests, heads and value
//           channels: column j of S depends on column j alone, so a column stays in the registers
//           of its lanes from the request's first token of the step to its last);
//   out   (parallel): o of each head divided by its root mean square, times a weight, times
//           sigmoid(gate).
// A token's result depends on the tokens before it in its request only, in an order of
// operations that does not depend on how the request was cut into steps.
#include "common.h"

constexpr int MAX_RANK = 512;
constexpr float DECAY_SCALE = 0.6065306597126334f;      // exp(-1/2)

__device__ __forceinline__ float sigmoidf_(float z) { return 1.0f / (1.0f + expf(-z)); }

// proj: [n, row_stride] rows that hold r, k, a_lin (dk per head each) and the low-rank
// projection l (rank) at the given column offsets.  w2t: [rank, heads * dk], the decay's second matrix
// transposed.  prep: [n, heads, 5, dk] 32-bit.
template <class T>
__global__ void delta_prep_kernel(const T *__restrict__ proj, int row_stride, int off_r, int off_k, int off_a, int off_l,
                                  const float *__restrict__ w2t, const float *__restrict__ w0,
                                  const float *__restrict__ a_bias, float *__restrict__ prep, int heads, int dk, int rank) {
    __shared__ float th[MAX_RANK];
    __shared__ float scratch[16];
    const int t = blockIdx.x, h = blockIdx.y;
    const T *row = proj + (size_t)t * row_stride;
    for (int i = threadIdx.x; i < rank; i += blockDim.x) th[i] = tanhf(to_f32(row[off_l + i]));
    float ss = 0.f;
    for (int i = threadIdx.x; i < dk; i += blockDim.x) {
        const float kk = to_f32(row[off_k + h * dk + i]);
        ss += kk * kk;
    }
    ss = block_sum(ss, scratch);                 // (its barriers also make th visible)
    const float inv = 1.0f / sqrtf(ss + 1e-6f);
    float *out = prep + ((size_t)t * heads + h) * 5 * dk;
    for (int i = threadIdx.x; i < dk; i += blockDim.x) {
        const int c = h * dk + i;
        float z = w0[c];
#pragma unroll 8
        for (int j = 0; j < rank; ++j) z += w2t[(size_t)j * heads * dk + c] * th[j];      // (neighbouring lanes, neighbouring addresses)
        const float w = expf(-DECAY_SCALE * sigmoidf_(z));
        const float a = sigmoidf_(to_f32(row[off_a + c]) + a_bias[c]);
        const float kk = to_f32(row[off_k + c]);
        const float u = kk * inv;
        out[i] = w;
        out[dk + i] = a * u;
        out[2 * dk + i] = u;
        out[3 * dk + i] = kk;
        out[4 * dk + i] = to_f32(row[off_r + c]);
    }
}

// DK > 0 (a multiple of 16): one wave per (request, head, 16 or 8 value channels).  The wave's lanes are four groups of
// 16 (eight of 8 where DK is a multiple of 32): lane (g, j) keeps the part g of column j of S (key channels
// g * DK/groups .. + DK/groups - 1) in registers, so a token costs a lane DK/groups of each pass, and the two sums over
// key channels (u^T S and S^T r) cross the groups in the vector unit.  A request's tokens are one chain, so what a
// token costs a wave is what counts: more lanes a column make it shorter.  The tokens' five vectors go through LDS, eight tokens at a time (all lanes copy, each reads its
// quarter), the next eight tokens' are on their way meanwhile.
// DK == 0: any dk, one wave per (request, head, 64 value channels), the column stays in the state's memory.
// state: [slots, heads, dk, dv]; o: [n, heads * dv] 32-bit.

// The sum of the values that the lanes l, l + 16, l + 32 and l + 48 hold (and l + 8 of each, with eight groups), in all
// of them, always added in the same order.  The rows of 16 lanes are swapped in the vector unit (v_permlane16_swap,
// v_permlane32_swap): a shuffle through LDS takes far longer, and the recurrence waits for this value twice a token.
template <int GROUPS>
__device__ __forceinline__ float sum_over_groups(float x) {
    if (GROUPS == 8)            // eight groups of 8 lanes: first the two groups of a row of 16 (the row rotated by 8, in the vector unit too)
        x += __uint_as_float((unsigned)__builtin_amdgcn_update_dpp(0, (int)__float_as_uint(x), 0x128, 0xf, 0xf, false));
    const unsigned u = __float_as_uint(x);
    const auto a = __builtin_amdgcn_permlane16_swap(u, u, false, false);     // (rows 0 0 2 2, rows 1 1 3 3)
    const unsigned v = __float_as_uint(__uint_as_float(a[0]) + __uint_as_float(a[1]));
    const auto b = __builtin_amdgcn_permlane32_swap(v, v, false, false);     // (lower half twice, upper half twice)
    return __uint_as_float(b[0]) + __uint_as_float(b[1]);
}

template <class T, int DK>
constexpr int scan_groups() { return DK > 0 && DK % 32 == 0 ? 8 : 4; }

// GATED: the gated rule, whose decay g and rate beta are one number each per token and head and whose key is its unit
// key: S <- g S + u (v - (beta g) (u^T S)) with v the value times beta already.  A token then brings two vectors (u, r) and
// two numbers (g, beta g) instead of five vectors: prep rows are [u | r | g, beta g, 0, 0], 2 dk + 4 floats.
template <class T, int DK, bool GATED>
__global__ void __launch_bounds__(64)
delta_scan_kernel(const T *__restrict__ proj, int row_stride, int off_v, const float *__restrict__ vf, const float *__restrict__ prep,
                  float *__restrict__ state, size_t slot_stride, float *__restrict__ o, const int *__restrict__ q_start,
                  const int *__restrict__ ctx_len, const int *__restrict__ state_slot, int heads, int dk_rt, int dv) {
    const int r = blockIdx.x, h = blockIdx.y;
    const int t0 = q_start[r], t1 = q_start[r + 1];
    const bool fresh = ctx_len[r] - (t1 - t0) == 0;          // the request's first token: the state starts at zero
    if constexpr (DK > 0) {
        constexpr int SCAN_GROUPS = scan_groups<T, DK>(), SCAN_COLS = WAVE / SCAN_GROUPS;
        constexpr int SL = DK / SCAN_GROUPS;                  // key channels of a lane
        constexpr int NV = GATED ? 2 : 5;                     // vectors of a token
        constexpr int ROW = NV * DK + (GATED ? 4 : 0);        // floats of a token's prep row
        constexpr int PER_LANE = (ROW + 63) / 64;
        constexpr int TB = DK <= 128 ? 8 : 4;                 // tokens whose vectors are brought in together
        const int g = threadIdx.x / SCAN_COLS, j = blockIdx.z * SCAN_COLS + threadIdx.x % SCAN_COLS;
        const bool live = j < dv;
        const int jj = live ? j : dv - 1;                     // lanes beyond dv compute along and store nothing
        float *col = state + (size_t)state_slot[r] * slot_stride + ((size_t)h * DK + g * SL) * dv + jj;   // S[g * SL + i][j] at col[i * dv]
        // a vector in LDS: the four groups' quarters, each followed by four floats of padding, so that the groups' reads of
        // their quarters (the same offset in each) fall into different banks
        constexpr int SLP = SL + 4, VEC = SCAN_GROUPS * SLP;
        __shared__ __attribute__((aligned(16))) float vec[2][TB][NV * VEC + (GATED ? 4 : 0)];
        float S[SL];
#pragma unroll
        for (int i = 0; i < SL; ++i) S[i] = fresh ? 0.f : col[(size_t)i * dv];
        // the vectors and values of the next TB tokens, on their way while the TB before them are folded in: a
        // token's own arithmetic is far shorter than a trip to memory
        float next[TB][PER_LANE], v_next[TB];
        const T *vp = proj + off_v + h * dv + jj;
        const float *vfp = vf ? vf + h * dv + jj : nullptr;         // the values as 32-bit rows [n, heads * dv] of their own
        auto fetch = [&](int t) {
#pragma unroll
            for (int b = 0; b < TB; ++b) {
                if (t + b >= t1) break;                       // (a step of one token brings in one token)
                const float *p = prep + ((size_t)(t + b) * heads + h) * ROW;
#pragma unroll
                for (int e = 0; e < PER_LANE; ++e) {
                    const int idx = e * 64 + threadIdx.x;
                    next[b][e] = idx < ROW ? p[idx] : 0.f;
                }
                v_next[b] = vfp ? vfp[(size_t)(t + b) * heads * dv] : to_f32(vp[(size_t)(t + b) * row_stride]);
            }
        };
        if (t0 < t1) fetch(t0);
        int turn = 0;
        for (int t = t0; t < t1; t += TB, turn ^= 1) {
            float v[TB];
#pragma unroll
            for (int b = 0; b < TB; ++b) {
                if (t + b >= t1) break;
                v[b] = v_next[b];
#pragma unroll
                for (int e = 0; e < PER_LANE; ++e) {
                    const int idx = e * 64 + threadIdx.x;
                    if (idx < NV * DK) vec[turn][b][idx / DK * VEC + idx % DK / SL * SLP + idx % SL] = next[b][e];
                    else if (GATED && idx < ROW) vec[turn][b][NV * VEC + idx - NV * DK] = next[b][e];
                }
            }
            __syncthreads();                                  // (the buffer of two turns ago was last read before the barrier of the turn between)
            if (t + TB < t1) fetch(t + TB);
#pragma unroll
            for (int b = 0; b < TB; ++b) {
                if (t + b >= t1) break;
                const float *W = vec[turn][b] + g * SLP, *AU = W + VEC, *U = GATED ? W : W + 2 * VEC, *K = W + 3 * VEC,
                            *R = GATED ? W + VEC : W + 4 * VEC;
                // four sums side by side in each pass (added in a fixed order): one chain of SL dependent additions
                // would be most of a token's time
                float us4[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int i = 0; i < SL; ++i) us4[i & 3] += U[i] * S[i];
                const float us = sum_over_groups<SCAN_GROUPS>((us4[0] + us4[1]) + (us4[2] + us4[3]));
                float acc4[4] = {0.f, 0.f, 0.f, 0.f};
                if constexpr (GATED) {
                    const float gd = vec[turn][b][NV * VEC], c = v[b] - vec[turn][b][NV * VEC + 1] * us;
#pragma unroll
                    for (int i = 0; i < SL; ++i) {
                        S[i] = gd * S[i] + U[i] * c;
                        acc4[i & 3] += S[i] * R[i];
                    }
                } else {
#pragma unroll
                    for (int i = 0; i < SL; ++i) {
                        S[i] = W[i] * S[i] - AU[i] * us + K[i] * v[b];
                        acc4[i & 3] += S[i] * R[i];
                    }
                }
                const float acc = sum_over_groups<SCAN_GROUPS>((acc4[0] + acc4[1]) + (acc4[2] + acc4[3]));
                if (live && g == 0) o[(size_t)(t + b) * heads * dv + h * dv + j] = acc;
            }
        }
        if (live) {
#pragma unroll
            for (int i = 0; i < SL; ++i) col[(size_t)i * dv] = S[i];
        }
    } else {
        const int dk = dk_rt, j = blockIdx.z * 64 + threadIdx.x;
        const bool live = j < dv;
        const int jj = live ? j : dv - 1;
        float *col = state + (size_t)state_slot[r] * slot_stride + ((size_t)h * dk) * dv + jj;     // S[i][j] at col[i * dv]
        if (fresh && live)
            for (int i = 0; i < dk; ++i) col[(size_t)i * dv] = 0.f;
        for (int t = t0; t < t1; ++t) {
            const float v = vf ? vf[(size_t)t * heads * dv + h * dv + jj] : to_f32(proj[(size_t)t * row_stride + off_v + h * dv + jj]);
            const float *p = prep + ((size_t)t * heads + h) * (GATED ? 2 * dk + 4 : 5 * dk);
            float us = 0.f, acc = 0.f;
            if constexpr (GATED) {
                for (int i = 0; i < dk; ++i) us += p[i] * col[(size_t)i * dv];
                const float gd = p[2 * dk], c = v - p[2 * dk + 1] * us;
                for (int i = 0; i < dk; ++i) {
                    const float s = gd * col[(size_t)i * dv] + p[i] * c;
                    if (live) col[(size_t)i * dv] = s;
                    acc += s * p[dk + i];
                }
            } else {
                for (int i = 0; i < dk; ++i) us += p[2 * dk + i] * col[(size_t)i * dv];
                for (int i = 0; i < dk; ++i) {
                    const float s = p[i] * col[(size_t)i * dv] - p[dk + i] * us + p[3 * dk + i] * v;
                    if (live) col[(size_t)i * dv] = s;
                    acc += s * p[4 * dk + i];
                }
            }
            if (live) o[(size_t)t * heads * dv + h * dv + j] = acc;
        }
    }
}

// One wave per (token, head): out = o / rms(o) * weight * sigmoid(gate).
template <class T>
__global__ void __launch_bounds__(64)
delta_out_kernel(const float *__restrict__ o, const T *__restrict__ proj, int row_stride, int off_g,
                 const float *__restrict__ weight, T *__restrict__ out, int heads, int dv, float eps) {
    const int t = blockIdx.x, h = blockIdx.y;
    const float *oh = o + (size_t)t * heads * dv + h * dv;
    float ss = 0.f;
    for (int j = threadIdx.x; j < dv; j += 64) ss += oh[j] * oh[j];
    const float f = rsqrtf(wave_sum(ss) / (float)dv + eps);
    for (int j = threadIdx.x; j < dv; j += 64) {
        const int c = h * dv + j;
        const float g = sigmoidf_(to_f32(proj[(size_t)t * row_stride + off_g + c]));
        out[(size_t)t * heads * dv + c] = from_f32<T>(oh[j] * f * weight[c] * g);
    }
}

// The scan over the step's tokens for every head size it is compiled for.  vf: null, or the values as 32-bit rows.
template <class T, bool GATED = false>
static int delta_scan_launch(const T *proj, int row_stride, int off_v, const float *vf, const float *prep, float *state,
                             size_t slot_stride, float *o, const int *q_start, const int *ctx_len, const int *state_slot,
                             int n_req, int heads, int dk, int dv, hipStream_t stream) {
#define SCAN(DK) delta_scan_kernel<T, DK, GATED><<<dim3(n_req, heads, (dv + (DK ? 64 / scan_groups<T, DK>() : 64) - 1) / (DK ? 64 / scan_groups<T, DK>() : 64)), dim3(64), 0, stream>>>(proj, row_stride, off_v, vf, prep, state, slot_stride, o, q_start, ctx_len, state_slot, heads, dk, dv)
    switch (dk) {
    case 16: SCAN(16); break;
    case 32: SCAN(32); break;
    case 48: SCAN(48); break;
    case 64: SCAN(64); break;
    case 80: SCAN(80); break;
    case 96: SCAN(96); break;
    case 112: SCAN(112); break;
    case 128: SCAN(128); break;
    case 192: SCAN(192); break;
    case 256: SCAN(256); break;
    default: SCAN(0); break;
    }
#undef SCAN
    LCU_LAUNCH_CHECK();
    return LCU_OK;
}

template <class T>
static int delta_rule_t(const T *proj, int row_stride, int off_r, int off_k, int off_v, int off_g, int off_a, int off_l,
                        const float *w2, const float *w0, const float *a_bias, const float *weight, float *prep,
                        float *o, float *state, T *out, const int *q_start, const int *ctx_len, const int *state_slot,
                        int n, int n_req, int heads, int dk, int dv, int rank, float eps, hipStream_t stream) {
    int threads = ((dk > rank ? dk : rank) + 63) / 64 * 64;
    if (threads > 256) threads = 256;
    delta_prep_kernel<T><<<dim3(n, heads), dim3(threads), 0, stream>>>(proj, row_stride, off_r, off_k, off_a, off_l, w2, w0, a_bias, prep, heads, dk, rank);
    LCU_LAUNCH_CHECK();
    const int rc = delta_scan_launch<T>(proj, row_stride, off_v, nullptr, prep, state, (size_t)heads * dk * dv, o, q_start, ctx_len,
                                        state_slot, n_req, heads, dk, dv, stream);
    if (rc != LCU_OK) return rc;
    delta_out_kernel<T><<<dim3(n, heads), dim3(64), 0, stream>>>(o, proj, row_stride, off_g, weight, out, heads, dv, eps);
    LCU_LAUNCH_CHECK();
    return LCU_OK;
}

// proj: [n, row_stride] of `type`; the offsets are columns.  w2: [rank, heads * dk] (transposed), w0, a_bias: [heads * dk],
// weight: [heads * dv], all 32-bit.  prep: scratch [n, heads, 5, dk], o: scratch [n, heads * dv], both 32-bit.
// state: [slots, heads, dk, dv] 32-bit.  out: [n, heads * dv] of `type`.
LCU_API int lcu_delta_rule(const void *proj, int type, int row_stride, int off_r, int off_k, int off_v, int off_g,
                           int off_a, int off_l, const float *w2, const float *w0, const float *a_bias,
                           const float *weight, float *prep, float *o, float *state, void *out, const int *q_start,
                           const int *ctx_len, const int *state_slot, int n, int n_req, int heads, int dk, int dv,
                           int rank, float eps, hipStream_t stream) {
    if (n <= 0 || n_req <= 0) return LCU_OK;
    if (heads <= 0 || heads > 65535 || dk <= 0 || dv <= 0 || rank <= 0 || rank > MAX_RANK || dv > 8 * 65535) return LCU_BAD_ARGUMENT;
    if (type == LCU_F32)
        return delta_rule_t<float>((const float *)proj, row_stride, off_r, off_k, off_v, off_g, off_a, off_l, w2, w0, a_bias, weight, prep, o, state, (float *)out, q_start, ctx_len, state_slot, n, n_req, heads, dk, dv, rank, eps, stream);
    if (type == LCU_BF16)
        return delta_rule_t<bf16_t>((const bf16_t *)proj, row_stride, off_r, off_k, off_v, off_g, off_a, off_l, w2, w0, a_bias, weight, prep, o, state, (bf16_t *)out, q_start, ctx_len, state_slot, n, n_req, heads, dk, dv, rank, eps, stream);
    return LCU_BAD_ARGUMENT;
}

// ---------------------------------------------------------------- the gated delta rule
// One decay and one rate per head and token:  S <- g S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q,  with q and k
// unit vectors per head (q also times dk^-1/2).  Written out, S <- g S - (beta g k)(k^T S) + k (beta v)^T with S as the
// token found it, or S <- g S + k (beta v - (beta g)(k^T S)): the scan above in its gated form, which takes per token
// the unit key, the query, the two numbers g and beta g, and the values beta v.  Several value heads may share one
// query/key head (`group` of them).
//   prep (parallel over tokens and value heads): the scan's two vectors and two numbers, and the values times beta;
//   out  (parallel): o of each head divided by its root mean square, times a weight, times silu(gate).
// qkv: [n, qk_heads * dk (q) | qk_heads * dk (k) | heads * dv (v)] 32-bit, the projections behind their convolutions
// and activations.  rows: [n, row_stride] 32-bit holding per head the decay's and the rate's projections at columns
// off_a and off_b, and the gate's heads * dv columns at off_g.
__device__ __forceinline__ float softplus_(float z) { return z > 20.f ? z : log1pf(expf(z)); }

__global__ void gated_delta_prep_kernel(const float *__restrict__ qkv, const float *__restrict__ rows, int row_stride, int off_a,
                                        int off_b, const float *__restrict__ a_log, const float *__restrict__ dt_bias,
                                        float *__restrict__ prep, float *__restrict__ vb, int heads, int group, int dk, int dv) {
    __shared__ float scratch[16];
    const int t = blockIdx.x, h = blockIdx.y, qh = h / group, qk_heads = heads / group;
    const int width = 2 * qk_heads * dk + heads * dv;
    const float *q = qkv + (size_t)t * width + qh * dk, *k = q + qk_heads * dk;
    const float *v = qkv + (size_t)t * width + 2 * qk_heads * dk + h * dv;
    float sq = 0.f, sk = 0.f;
    for (int i = threadIdx.x; i < dk; i += blockDim.x) {
        sq += q[i] * q[i];
        sk += k[i] * k[i];
    }
    sq = block_sum(sq, scratch);
    sk = block_sum(sk, scratch);
    const float qf = 1.0f / sqrtf(sq + 1e-6f) / sqrtf((float)dk), kf = 1.0f / sqrtf(sk + 1e-6f);
    const float *row = rows + (size_t)t * row_stride;
    const float beta = sigmoidf_(row[off_b + h]);
    const float g = expf(-expf(a_log[h]) * softplus_(row[off_a + h] + dt_bias[h]));
    float *out = prep + ((size_t)t * heads + h) * (2 * dk + 4);
    for (int i = threadIdx.x; i < dk; i += blockDim.x) {
        out[i] = k[i] * kf;
        out[dk + i] = q[i] * qf;
    }
    if (threadIdx.x < 4) out[2 * dk + threadIdx.x] = threadIdx.x == 0 ? g : (threadIdx.x == 1 ? beta * g : 0.f);
    for (int j = threadIdx.x; j < dv; j += blockDim.x) vb[((size_t)t * heads + h) * dv + j] = beta * v[j];
}

// One wave per (token, head): out = o / rms(o) * weight * silu(gate); weight: [dv], shared by the heads.
template <class T>
__global__ void __launch_bounds__(64)
gated_delta_out_kernel(const float *__restrict__ o, const float *__restrict__ rows, int row_stride, int off_g,
                       const float *__restrict__ weight, T *__restrict__ out, int heads, int dv, float eps) {
    const int t = blockIdx.x, h = blockIdx.y;
    const float *oh = o + (size_t)t * heads * dv + h * dv;
    float ss = 0.f;
    for (int j = threadIdx.x; j < dv; j += 64) ss += oh[j] * oh[j];
    const float f = 1.0f / sqrtf(wave_sum(ss) / (float)dv + eps);
    for (int j = threadIdx.x; j < dv; j += 64) {
        const float z = rows[(size_t)t * row_stride + off_g + h * dv + j];
        out[(size_t)t * heads * dv + h * dv + j] = from_f32<T>(oh[j] * f * weight[j] * (z / (1.0f + expf(-z))));
    }
}

// a_log, dt_bias: [heads]; weight: [dv], 32-bit.  prep: scratch [n, heads, 2 * dk + 4]; vb, o: scratch [n, heads * dv], 32-bit.
// state: slot s at state + s * slot_stride, [heads, dk, dv] 32-bit.  out: [n, heads * dv] of out_type.
LCU_API int lcu_gated_delta_rule(const float *qkv, const float *rows, int row_stride, int off_a, int off_b, int off_g,
                                 const float *a_log, const float *dt_bias, const float *weight, float *prep, float *vb, float *o,
                                 float *state, long long slot_stride, void *out, int out_type, const int *q_start,
                                 const int *ctx_len, const int *state_slot, int n, int n_req, int heads, int qk_heads, int dk,
                                 int dv, float eps, hipStream_t stream) {
    if (n <= 0 || n_req <= 0) return LCU_OK;
    if (heads <= 0 || heads > 65535 || qk_heads <= 0 || heads % qk_heads || dk <= 0 || dv <= 0 || dv > 8 * 65535 ||
        (out_type != LCU_F32 && out_type != LCU_BF16))
        return LCU_BAD_ARGUMENT;
    int threads = ((dk > dv ? dk : dv) + 63) / 64 * 64;
    if (threads > 256) threads = 256;
    gated_delta_prep_kernel<<<dim3(n, heads), dim3(threads), 0, stream>>>(qkv, rows, row_stride, off_a, off_b, a_log, dt_bias, prep, vb,
                                                                           heads, heads / qk_heads, dk, dv);
    LCU_LAUNCH_CHECK();
    const int rc = delta_scan_launch<float, true>(nullptr, 0, 0, vb, prep, state, (size_t)slot_stride, o, q_start, ctx_len, state_slot, n_req,
                                            heads, dk, dv, stream);
    if (rc != LCU_OK) return rc;
    if (out_type == LCU_F32)
        gated_delta_out_kernel<float><<<dim3(n, heads), dim3(64), 0, stream>>>(o, rows, row_stride, off_g, weight, (float *)out, heads, dv, eps);
    else
        gated_delta_out_kernel<bf16_t><<<dim3(n, heads), dim3(64), 0, stream>>>(o, rows, row_stride, off_g, weight, (bf16_t *)out, heads, dv, eps);
    LCU_LAUNCH_CHECK();
    return LCU_OK;
}
