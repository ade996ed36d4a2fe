// A feed-forward of many small experts of which each token uses a few.
//
//   route:   z = W_router h (+ bias) (32-bit), the `top` experts with the largest z (ties: the lower
//            index), each with the weight sigmoid(z) (a token's weights are not made to add up to one) or,
//            in the other mode, with the softmax over the chosen logits alone; or, in a third, with scores s = softmax(z)
//            over all experts, the choice by s + a correction per expert, and the chosen scores divided by their sum as
//            weights; rows of the router's matrix behind the experts' are gates: sigmoid of their logit goes out per
//            token; the last experts may be identity experts, which have no matrices and return their input;
//   group:   the (token, choice) pairs sorted by expert and cut into tiles of up to 16 or 64 rows of
//            one expert, on the device (nothing comes back to the host);
//   up:      act = gelu(W_up[e] (weight * h))    the weight scales what goes INTO the expert; or, gated:
//            act = silu(W_gate[e] h) * (W_up[e] h), and the weight scales what comes OUT of the expert
//   down:    y = W_down[e] act, added to the token's output row (32-bit), in the gated form times the weight
//            and beside a shared expert's row times its gate.
// The products run on the matrix cores: bfloat16 operands with v_mfma_f32_16x16x32_bf16, or
// true 32-bit with v_mfma_f32_16x16x4_f32; sums are 32-bit.  A row's result depends on that
// row and its expert alone (never on which rows share its tile), so it does not depend on
// the batch.
#include "common.h"

constexpr int MOE_MAX_EXPERTS = 1024;
constexpr int MOE_TILE_ROWS = 64;        // rows of a tile of the kernel for many rows; the kernel for few rows takes 16

typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;

// ---------------------------------------------------------------- route
// One block per token (256 threads; 1024 where a step has few tokens, so that more of a token's experts are
// multiplied side by side).  h: [n, d] of T; router: [experts, d] 32-bit.  ids, wts: [n, top].  A wave takes
// the experts e = wave, wave + waves, ...; with d a multiple of 8 a lane keeps its share of the row (eight
// neighbouring elements of every 512) in registers for all of them.
template <class T> struct alignas(8 * sizeof(T)) Row8 { T v[8]; };
constexpr int ROUTE_CHUNKS = 8;                  // rows of up to 8 * 512 elements stay in registers

// bias: null or [experts], added to the logits.  mode 0: the weight of a chosen expert is sigmoid(z); 1: the softmax over
// the chosen logits; 2: s = softmax(z) over all experts, the choice goes by s + bias (the bias is not added to the
// logits), the weights are the chosen s divided by their sum + 1e-20.  extra: rows of `router` behind the experts' (at most MOE_MAX_EXTRA); gates [n, extra] takes sigmoid
// of their logits (they are no experts and are never chosen).
constexpr int MOE_MAX_EXTRA = 8;
template <class T, int THREADS>
__global__ void __launch_bounds__(THREADS)
moe_route_kernel(const T *__restrict__ h, const float *__restrict__ router, const float *__restrict__ bias, int *__restrict__ ids,
                 float *__restrict__ wts, float *__restrict__ gates, int d, int n_experts, int top, int mode, int extra) {
    __shared__ float z[MOE_MAX_EXPERTS + MOE_MAX_EXTRA];
    __shared__ float zc[MOE_MAX_EXPERTS];
    __shared__ float sc[MOE_MAX_EXPERTS];
    const float *logit_bias = mode == 2 ? nullptr : bias;
    const int experts = n_experts + extra;          // rows of the router's matrix
    const int t = blockIdx.x, wave = threadIdx.x / WAVE, lane = threadIdx.x % WAVE;
    const T *row = h + (size_t)t * d;
    if (d % 8 == 0 && d <= ROUTE_CHUNKS * 512) {
        float x[ROUTE_CHUNKS][8];
#pragma unroll
        for (int k = 0; k < ROUTE_CHUNKS; ++k) {
            const int c = k * 512 + lane * 8;
            if (c < d) {
                const Row8<T> in = *(const Row8<T> *)(row + c);
#pragma unroll
                for (int e = 0; e < 8; ++e) x[k][e] = to_f32(in.v[e]);
            }
        }
        for (int e = wave; e < experts; e += THREADS / WAVE) {
            const float *w = router + (size_t)e * d;
            float acc = 0.f;
#pragma unroll
            for (int k = 0; k < ROUTE_CHUNKS; ++k) {
                const int c = k * 512 + lane * 8;
                if (c < d) {
                    const f32x4 w0 = *(const f32x4 *)(w + c), w1 = *(const f32x4 *)(w + c + 4);
#pragma unroll
                    for (int i = 0; i < 4; ++i) acc += x[k][i] * w0[i];
#pragma unroll
                    for (int i = 0; i < 4; ++i) acc += x[k][4 + i] * w1[i];
                }
            }
            acc = wave_sum(acc);
            if (lane == 0) z[e] = acc + (logit_bias && e < n_experts ? logit_bias[e] : 0.f);
        }
    } else {
        for (int e = wave; e < experts; e += THREADS / WAVE) {
            const float *w = router + (size_t)e * d;
            float acc = 0.f;
            for (int c = lane; c < d; c += WAVE) acc += to_f32(row[c]) * w[c];
            acc = wave_sum(acc);
            if (lane == 0) z[e] = acc + (logit_bias && e < n_experts ? logit_bias[e] : 0.f);
        }
    }
    __syncthreads();
    for (int e = threadIdx.x; e < extra; e += THREADS) gates[(size_t)t * extra + e] = 1.0f / (1.0f + expf(-z[n_experts + e]));
    if (mode == 2) {                                 // scores over all experts; z becomes what the choice goes by
        if (wave == 0) {
            float m = -INFINITY;
            for (int e = lane; e < n_experts; e += WAVE) m = fmaxf(m, z[e]);
            m = wave_max(m);
            float part = 0.f;
            for (int e = lane; e < n_experts; e += WAVE) part += expf(z[e] - m);
            const float sum = wave_sum(part);
            for (int e = lane; e < n_experts; e += WAVE) {
                const float s = expf(z[e] - m) / sum;
                sc[e] = s;
                z[e] = s + (bias ? bias[e] : 0.f);
            }
        }
        __syncthreads();
    }
    for (int k = 0; k < top; ++k) {                  // the first wave chooses; the others only keep the barriers
        if (wave == 0) {
            float best = -INFINITY;
            int arg = 0x7fffffff;
            for (int e = lane; e < n_experts; e += WAVE) {
                const float v = z[e];
                if (v > best || (v == best && e < arg)) { best = v; arg = e; }
            }
#pragma unroll
            for (int off = 32; off > 0; off >>= 1) {
                const float ob = __shfl_xor(best, off, WAVE);
                const int oa = __shfl_xor(arg, off, WAVE);
                if (ob > best || (ob == best && oa < arg)) { best = ob; arg = oa; }
            }
            if (arg >= n_experts) arg = 0;               // every logit NaN: any expert
            if (lane == 0) {
                ids[(size_t)t * top + k] = arg;
                zc[k] = mode == 2 ? sc[arg] : z[arg];
                if (mode == 0) wts[(size_t)t * top + k] = 1.0f / (1.0f + expf(-z[arg]));
                z[arg] = -INFINITY;
            }
        }
        __syncthreads();
    }
    if (mode == 2 && wave == 0) {                    // the chosen scores, made to add up to one
        float part = 0.f;
        for (int k = lane; k < top; k += WAVE) part += zc[k];
        const float sum = wave_sum(part) + 1e-20f;
        for (int k = lane; k < top; k += WAVE) wts[(size_t)t * top + k] = zc[k] / sum;
    }
    if (mode == 1 && wave == 0) {                    // the softmax over the chosen logits (the first is the largest)
        const float z0 = zc[0];
        float part = 0.f;
        for (int k = lane; k < top; k += WAVE) part += expf(zc[k] - z0);
        const float sum = wave_sum(part);
        for (int k = lane; k < top; k += WAVE) wts[(size_t)t * top + k] = expf(zc[k] - z0) / sum;
    }
}

// ---------------------------------------------------------------- group
// One block.  ids: [total] experts of the (token, choice) pairs in flat order.  Writes
// sorted_to_flat [total] (the pairs sorted by expert), and the tiles of up to rows_per_tile rows:
// tile_expert, tile_begin (first sorted row), tile_rows, each [max_tiles], and n_tiles [1].  Only the first `tiled`
// experts get tiles: the ones behind them have no matrices (identity experts), and their pairs are only sorted.
__global__ void __launch_bounds__(1024)
moe_group_kernel(const int *__restrict__ ids, int total, int experts, int *__restrict__ sorted_to_flat,
                 int *__restrict__ tile_expert, int *__restrict__ tile_begin, int *__restrict__ tile_rows,
                 int *__restrict__ n_tiles, int max_tiles, int rows_per_tile, int tiled) {
    __shared__ int count[MOE_MAX_EXPERTS];
    __shared__ int cursor[MOE_MAX_EXPERTS];
    for (int e = threadIdx.x; e < experts; e += blockDim.x) count[e] = 0;
    __syncthreads();
    for (int i = threadIdx.x; i < total; i += blockDim.x) atomicAdd(&count[ids[i]], 1);
    __syncthreads();
    if (threadIdx.x == 0) {
        int at = 0, tiles = 0;
        for (int e = 0; e < experts; ++e) {
            cursor[e] = at;
            for (int r = 0; e < tiled && r < count[e] && tiles < max_tiles; r += rows_per_tile) {
                tile_expert[tiles] = e;
                tile_begin[tiles] = at + r;
                tile_rows[tiles] = count[e] - r < rows_per_tile ? count[e] - r : rows_per_tile;
                ++tiles;
            }
            at += count[e];
        }
        n_tiles[0] = tiles;
    }
    __syncthreads();
    for (int i = threadIdx.x; i < total; i += blockDim.x) sorted_to_flat[atomicAdd(&cursor[ids[i]], 1)] = i;
}

// ---------------------------------------------------------------- the experts' products
template <class T> struct Mma;
template <> struct Mma<bf16_t> {
    static constexpr int PER_LANE = 8, KSTEP = 32;       // elements of k a lane loads (16 bytes), and a step covers
    typedef u32x4 frag;
    static __device__ __forceinline__ frag zero() { return frag{0u, 0u, 0u, 0u}; }
    static __device__ __forceinline__ frag load(const bf16_t *p) { return *(const frag *)p; }
    static __device__ __forceinline__ frag scaled(frag v, float s) {
        frag o;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const float lo = __uint_as_float(v[i] << 16) * s, hi = __uint_as_float(v[i] & 0xffff0000u) * s;
            o[i] = pack2_bf16(lo, hi);
        }
        return o;
    }
    static __device__ __forceinline__ f32x4 mma(frag a, frag b, f32x4 c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
    }
};
template <> struct Mma<float> {
    static constexpr int PER_LANE = 4, KSTEP = 16;
    typedef f32x4 frag;
    static __device__ __forceinline__ frag zero() { return frag{0.f, 0.f, 0.f, 0.f}; }
    static __device__ __forceinline__ frag load(const float *p) { return *(const frag *)p; }
    static __device__ __forceinline__ frag scaled(frag v, float s) { return v * s; }
    // four instructions of k = 4: instruction e takes element e of every lane's four, so the sixteen k of a step are
    // shared out the same way on both operands
    static __device__ __forceinline__ f32x4 mma(frag a, frag b, f32x4 c) {
#pragma unroll
        for (int e = 0; e < 4; ++e) c = __builtin_amdgcn_mfma_f32_16x16x4f32(a[e], b[e], c, 0, 0, 0);
        return c;
    }
};

__device__ __forceinline__ float gelu_erf(float z) { return 0.5f * z * (1.0f + erff(z * 0.70710678118654752f)); }

enum { MOE_UP = 0, MOE_DOWN = 1, MOE_UP_GATED = 2 };
__device__ __forceinline__ float silu_f(float z) { return z / (1.0f + expf(-z)); }

// Both kernels below multiply the rows of a tile (sorted rows of one expert) with that expert's matrix
// w[e] ([N, K], row-major) on the matrix cores.  The weight is the instruction's first operand (16
// features x k), the rows the second (k x 16 rows): a lane then holds four neighbouring features of
// one row.  Rows and features beyond the tile's or the matrix's end are computed from clamped
// addresses and never stored.  K is a multiple of the elements in 16 bytes.
//   MOE_UP:   x = h [n, K], a row is the token of its pair, scaled by the pair's weight; out_t = act
//             [total, N] at the sorted row, gelu applied.
//   MOE_DOWN: x = act [total, K] at the sorted row; out_f [total or n, N] 32-bit at the flat pair
//             (add == 0: stored) or at the pair's token (add == 1: added; only with top == 1).
//   MOE_UP_GATED: x = h [n, K], not scaled; w[e] holds N = 2 * features rows, in turns 16 rows of the gate matrix and the
//             16 rows of the up matrix that meet them; out_t = act [total, N / 2] at the sorted row,
//             silu(gate) * up.
template <class T, int MODE>
__device__ __forceinline__ void moe_store(const f32x4 &acc, int dst, int col0, int N, T *__restrict__ out_t,
                                          float *__restrict__ out_f, int out_stride, int add) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int col = col0 + i;
        if (col >= N) continue;
        if (MODE == MOE_UP) {
            out_t[(size_t)dst * out_stride + col] = from_f32<T>(gelu_erf(acc[i]));
        } else {
            float *o = out_f + (size_t)dst * out_stride + col;
            *o = add ? *o + acc[i] : acc[i];
        }
    }
}

// Few rows an expert (decoding): tiles of up to 16 rows; a block of four waves takes a tile and 64
// features, a wave 16 of them, and streams its 16 rows of the weight once, eight steps of loads in flight.
template <class T, int MODE>
__global__ void __launch_bounds__(256)
moe_gemm_few_kernel(const T *__restrict__ x, int x_stride, const T *__restrict__ w, size_t w_expert_stride, int N, int K,
                    const int *__restrict__ sorted_to_flat, const float *__restrict__ wts,
                    const int *__restrict__ tile_expert, const int *__restrict__ tile_begin,
                    const int *__restrict__ tile_rows, const int *__restrict__ n_tiles, int /* max_tiles */, T *__restrict__ out_t,
                    float *__restrict__ out_f, int out_stride, int top, int add) {
    typedef Mma<T> M;
    typedef typename M::frag frag;
    const int tile = blockIdx.x;
    if (tile >= n_tiles[0]) return;
    const int wave = threadIdx.x / WAVE, lane = threadIdx.x % WAVE, g = lane / 16, l16 = lane % 16;
    constexpr bool GATED = MODE == MOE_UP_GATED, UP = MODE != MOE_DOWN;
    const int NF = GATED ? N / 2 : N;                // output features
    const int f0 = blockIdx.y * 64 + wave * 16;
    if (f0 >= NF) return;
    const int e = tile_expert[tile], row0 = tile_begin[tile], rows = tile_rows[tile];
    const int f = f0 + l16 < NF ? f0 + l16 : NF - 1;
    const int wr = GATED ? (f / 16) * 32 + f % 16 : f;       // the gate's row; the up row that meets it lies 16 further
    const T *wrow = w + (size_t)e * w_expert_stride + (size_t)wr * K + g * M::PER_LANE;
    const bool valid = l16 < rows;
    const int srow = row0 + (valid ? l16 : 0);
    const int flat = sorted_to_flat[srow];
    const T *xrow = (UP ? x + (size_t)(flat / top) * x_stride : x + (size_t)srow * x_stride) + g * M::PER_LANE;
    const float sc = MODE == MOE_UP ? wts[flat] : 1.f;
    const int dst = UP ? srow : (add ? flat / top : flat);
    f32x4 acc = f32x4{0.f, 0.f, 0.f, 0.f}, acc2 = f32x4{0.f, 0.f, 0.f, 0.f};
    const int kfull = K / M::KSTEP * M::KSTEP;
    int k0 = 0;
    constexpr int AHEAD = 8;                         // steps of loads in flight: a wave's own arithmetic is short
    for (; k0 + AHEAD * M::KSTEP <= kfull; k0 += AHEAD * M::KSTEP) {
        frag a[AHEAD], b[AHEAD], a2[GATED ? AHEAD : 1];
#pragma unroll
        for (int u = 0; u < AHEAD; ++u) a[u] = M::load(wrow + k0 + u * M::KSTEP);    // (through the caches: a load takes half of each line, the next one the other half)
        if (GATED) {
#pragma unroll
            for (int u = 0; u < AHEAD; ++u) a2[GATED ? u : 0] = M::load(wrow + (size_t)16 * K + k0 + u * M::KSTEP);
        }
#pragma unroll
        for (int u = 0; u < AHEAD; ++u) b[u] = M::load(xrow + k0 + u * M::KSTEP);
#pragma unroll
        for (int u = 0; u < AHEAD; ++u) {
            acc = M::mma(a[u], MODE == MOE_UP ? M::scaled(b[u], sc) : b[u], acc);
            if (GATED) acc2 = M::mma(a2[GATED ? u : 0], b[u], acc2);
        }
    }
    for (; k0 < K; k0 += M::KSTEP) {                 // the steps that are left, the last one perhaps in part
        const bool in = k0 + g * M::PER_LANE < K;
        const frag a = in ? M::load(wrow + k0) : M::zero();
        const frag b = in ? M::load(xrow + k0) : M::zero();
        acc = M::mma(a, MODE == MOE_UP ? M::scaled(b, sc) : b, acc);
        if (GATED) acc2 = M::mma(in ? M::load(wrow + (size_t)16 * K + k0) : M::zero(), b, acc2);
    }
    if (!valid) return;
    if (GATED) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int col = f0 + 4 * g + i;
            if (col < NF) out_t[(size_t)dst * out_stride + col] = from_f32<T>(silu_f(acc[i]) * acc2[i]);
        }
    } else {
        moe_store<T, MODE>(acc, dst, f0 + 4 * g, N, out_t, out_f, out_stride, add);
    }
}

// Many rows an expert (prompts): tiles of up to 64 rows; a block of four waves takes a tile and 128
// features.  Rows and weights go through LDS in steps of 128 bytes of k, the next step's loads on their
// way while one is multiplied; a wave multiplies 32 features with all 64 rows (eight sums).
template <class T, int MODE>
__global__ void __launch_bounds__(256)
moe_gemm_many_kernel(const T *__restrict__ x, int x_stride, const T *__restrict__ w, size_t w_expert_stride, int N, int K,
                     const int *__restrict__ sorted_to_flat, const float *__restrict__ wts,
                     const int *__restrict__ tile_expert, const int *__restrict__ tile_begin,
                     const int *__restrict__ tile_rows, const int *__restrict__ n_tiles, int max_tiles, T *__restrict__ out_t,
                     float *__restrict__ out_f, int out_stride, int top, int add) {
    typedef Mma<T> M;
    typedef typename M::frag frag;
    constexpr int PL = M::PER_LANE;                 // elements in 16 bytes
    constexpr int KS = 128 / sizeof(T);             // elements of k a step
    constexpr int CH = KS / PL;                     // 16-byte pieces of a row a step: 8
    constexpr int LD = KS + PL;                     // a row in LDS, with a piece of padding against bank conflicts
    __shared__ __attribute__((aligned(16))) T xs[64 * LD];
    __shared__ __attribute__((aligned(16))) T ws[128 * LD];
    // Workgroups go to the chip's eight dies in turn (workgroup i to die i % 8), and each die has an L2 of its own.  The
    // tiles of one expert want the same block of its matrix: a die takes the feature blocks die, die + 8, ... and walks
    // the tiles of each in turn, so that a block of a matrix comes from memory to one die only.
    const int n_fb = (N + 127) / 128, die = blockIdx.x % 8, at = blockIdx.x / 8;
    const int fb = die + 8 * (at / max_tiles), tile = at % max_tiles;
    if (fb >= n_fb || tile >= n_tiles[0]) return;
    const int n0 = fb * 128;
    const int e = tile_expert[tile], row0 = tile_begin[tile], rows = tile_rows[tile];
    const int tid = threadIdx.x, wave = tid / WAVE, lane = tid % WAVE, g = lane / 16, l16 = lane % 16;
    const int ch = tid % CH;                        // this thread's piece of k in every row it copies
    const T *xptr[2];
    float xsc[2];
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const int r = tid / CH + 32 * i;
        const int srow = row0 + (r < rows ? r : 0);
        if (MODE != MOE_DOWN) {
            const int flat = sorted_to_flat[srow];
            xptr[i] = x + (size_t)(flat / top) * x_stride + ch * PL;
            xsc[i] = MODE == MOE_UP ? wts[flat] : 1.f;
        } else {
            xptr[i] = x + (size_t)srow * x_stride + ch * PL;
            xsc[i] = 1.f;
        }
    }
    const T *wptr[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int fr = n0 + tid / CH + 32 * i;
        wptr[i] = w + (size_t)e * w_expert_stride + (size_t)(fr < N ? fr : N - 1) * K + ch * PL;
    }
    frag xreg[2], wreg[4];
    auto from_memory = [&](int k0) {
        const bool in = k0 + ch * PL < K;
#pragma unroll
        for (int i = 0; i < 4; ++i) wreg[i] = in ? M::load(wptr[i] + k0) : M::zero();
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            xreg[i] = in ? M::load(xptr[i] + k0) : M::zero();
            if (MODE == MOE_UP) xreg[i] = M::scaled(xreg[i], xsc[i]);
        }
    };
    f32x4 acc[2][4];
#pragma unroll
    for (int ft = 0; ft < 2; ++ft)
#pragma unroll
        for (int m = 0; m < 4; ++m) acc[ft][m] = f32x4{0.f, 0.f, 0.f, 0.f};
    from_memory(0);
    // (one buffer and two barriers a step: with two buffers in turn and one barrier the kernel was a quarter slower, its
    // workgroups being fewer on a compute unit)
    for (int k0 = 0; k0 < K; k0 += KS) {
        __syncthreads();                            // the step before has been read
#pragma unroll
        for (int i = 0; i < 2; ++i) *(frag *)(xs + (tid / CH + 32 * i) * LD + ch * PL) = xreg[i];
#pragma unroll
        for (int i = 0; i < 4; ++i) *(frag *)(ws + (tid / CH + 32 * i) * LD + ch * PL) = wreg[i];
        __syncthreads();
        if (k0 + KS < K) from_memory(k0 + KS);
#pragma unroll
        for (int ks = 0; ks < KS / M::KSTEP; ++ks) {
            frag a[2], b[4];
#pragma unroll
            for (int ft = 0; ft < 2; ++ft) a[ft] = *(const frag *)(ws + (32 * wave + 16 * ft + l16) * LD + ks * M::KSTEP + g * PL);
#pragma unroll
            for (int m = 0; m < 4; ++m) b[m] = *(const frag *)(xs + (16 * m + l16) * LD + ks * M::KSTEP + g * PL);
#pragma unroll
            for (int m = 0; m < 4; ++m) {
                if (16 * m < rows) {
#pragma unroll
                    for (int ft = 0; ft < 2; ++ft) acc[ft][m] = M::mma(a[ft], b[m], acc[ft][m]);
                }
            }
        }
    }
#pragma unroll
    for (int m = 0; m < 4; ++m) {
        const int r = 16 * m + l16;
        if (r >= rows) continue;
        const int srow = row0 + r;
        int dst = srow;
        if (MODE == MOE_DOWN) {
            const int flat = sorted_to_flat[srow];
            dst = add ? flat / top : flat;
        }
        if (MODE == MOE_UP_GATED) {                 // the wave's first 16 rows are a gate block, its second the up block that meets it
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int col = (n0 + 32 * wave) / 2 + 4 * g + i;
                if (col < N / 2) out_t[(size_t)dst * out_stride + col] = from_f32<T>(silu_f(acc[0][m][i]) * acc[1][m][i]);
            }
            continue;
        }
#pragma unroll
        for (int ft = 0; ft < 2; ++ft)
            moe_store<T, MODE == MOE_UP_GATED ? MOE_UP : MODE>(acc[ft][m], dst, n0 + 32 * wave + 16 * ft + 4 * g, N, out_t, out_f, out_stride, add);
    }
}

// out[t, c] (+)= sum_k wts[t, k] * y[t * top + k, c]  (in the order of k; wts null: ones)  + gate[t] * shared[t, c]  (shared null: nothing)
// fresh: out is written, not added to (what it held is not read).  ids (null: none), real, h: a pair whose expert is
// `real` or beyond is an identity expert, whose output is the token's input row h[t] itself.
template <class T>
__global__ void moe_combine_kernel(float *__restrict__ out, const float *__restrict__ y, const float *__restrict__ wts,
                                   const T *__restrict__ shared, const float *__restrict__ gate, int n, int d, int top, int fresh,
                                   const int *__restrict__ ids, int real, const T *__restrict__ h) {
    const int c = blockIdx.x * blockDim.x + threadIdx.x;
    if (c >= d) return;
    for (size_t t = blockIdx.y; t < (size_t)n; t += gridDim.y) {
        float acc = fresh ? 0.f : out[t * d + c];
        for (int k = 0; k < top; ++k) {
            const float w = wts ? wts[t * top + k] : 1.f;
            if (ids && ids[t * top + k] >= real) acc += w * to_f32(h[t * d + c]);
            else acc += w * y[(t * top + k) * d + c];
        }
        if (shared) acc += (gate ? gate[t] : 1.f) * to_f32(shared[t * d + c]);
        out[t * d + c] = acc;
    }
}

// Rows of a tile for n * top pairs over so many experts: 16 (the kernel for few rows) while an expert has 16 rows
// or fewer on average, else 64.  The caller sizes its scratch with it: max_tiles = min(total, total / rows + experts).
LCU_API int lcu_moe_tile_rows(int total, int experts) { return (long long)total <= 16ll * experts ? 16 : MOE_TILE_ROWS; }

// h: [n, d] of `type`; router: [experts, d] 32-bit; ids, wts: [n * top].
// bias: null or [experts] 32-bit; mode 0: sigmoid weights, 1: softmax over the chosen; extra, gates: see the kernel
// (router then has experts + extra rows).
LCU_API int lcu_moe_route(const void *h, int type, const float *router, const float *bias, int *ids, float *wts, float *gates,
                          int n, int d, int experts, int top, int mode, int extra, hipStream_t stream) {
    if (n <= 0) return LCU_OK;
    if (d <= 0 || experts <= 0 || experts > MOE_MAX_EXPERTS || top <= 0 || top > experts || mode < 0 || mode > 2 ||
        extra < 0 || extra > MOE_MAX_EXTRA || (extra && !gates))
        return LCU_BAD_ARGUMENT;
    const bool few = n <= 256 && experts > 4;
#define GO(T, TH) moe_route_kernel<T, TH><<<dim3(n), dim3(TH), 0, stream>>>((const T *)h, router, bias, ids, wts, gates, d, experts, top, mode, extra)
    if (type == LCU_F32) { if (few) GO(float, 1024); else GO(float, 256); }
    else if (type == LCU_BF16) { if (few) GO(bf16_t, 1024); else GO(bf16_t, 256); }
    else return LCU_BAD_ARGUMENT;
#undef GO
    LCU_LAUNCH_CHECK();
    return LCU_OK;
}

// ints: scratch of total + 3 * max_tiles + 1 entries, laid out as sorted_to_flat, tile_expert, tile_begin,
// tile_rows, n_tiles.
// w_up: [experts, ff, d], w_down: [experts, d, ff] of `type`.  act: scratch [total, ff] of `type`; y: scratch
// [total, d] 32-bit (only read and written when top > 1 or gated).  out: [n, d] 32-bit, added to.
// gated: w_up is [experts, 2 * ff, d], in turns 16 rows of the gate matrix and the 16 rows of the up matrix that meet
// them (ff a multiple of 16); act = silu(gate h) * (up h), and the weight scales what comes out; fresh: out is written
// and not added to.  identity: ids may name experts + identity experts; the last `identity` have no matrices and return the
// token's input.  shared (null or
// [n, d] of `type`) with shared_gate (null or [n] 32-bit): rows that are added beside the experts', times the gate.
LCU_API int lcu_moe_experts(const void *h, int type, const int *ids, const float *wts, int *ints, int max_tiles,
                            const void *w_up, const void *w_down, void *act, float *y, float *out, int n, int d, int ff,
                            int experts, int top, int gated, const void *shared, const float *shared_gate, int fresh,
                            int identity, hipStream_t stream) {
    if (n <= 0) return LCU_OK;
    const int per = type == LCU_BF16 ? 8 : 4;
    if (d <= 0 || ff <= 0 || d % per || ff % per || experts <= 0 || experts > MOE_MAX_EXPERTS || top <= 0 || max_tiles <= 0 ||
        (type != LCU_F32 && type != LCU_BF16) || (gated && ff % 16) || (shared && !gated) || (fresh && !gated) || identity < 0 ||
        (identity && !gated) || experts + identity > MOE_MAX_EXPERTS)
        return LCU_BAD_ARGUMENT;
    const int total = n * top;
    const int tile_rows = lcu_moe_tile_rows(total, experts);
    int *sorted = ints, *t_exp = ints + total, *t_beg = t_exp + max_tiles, *t_rows = t_beg + max_tiles, *n_tiles = t_rows + max_tiles;
    moe_group_kernel<<<dim3(1), dim3(1024), 0, stream>>>(ids, total, experts + identity, sorted, t_exp, t_beg, t_rows, n_tiles, max_tiles, tile_rows, experts);
    LCU_LAUNCH_CHECK();
    const int add = top == 1 && !gated;
    float *down_to = add ? out : y;
    if (!add && !y) return LCU_BAD_ARGUMENT;
    const int per_block = tile_rows == 16 ? 64 : 128;         // features a block takes
    dim3 block(256), gu(max_tiles, (ff + per_block - 1) / per_block), gd(max_tiles, (d + per_block - 1) / per_block);
    const int up_rows = gated ? 2 * ff : ff;                  // rows of an expert's first matrix
    if (tile_rows != 16) {                                    // a flat grid: the kernel shares it out over the dies itself
        gu = dim3(8 * max_tiles * (((up_rows + 127) / 128 + 7) / 8));
        gd = dim3(8 * max_tiles * (((d + 127) / 128 + 7) / 8));
    }
#define GO(KERNEL, T)                                                                                                              \
    if (gated)                                                                                                                     \
        KERNEL<T, MOE_UP_GATED><<<gu, block, 0, stream>>>((const T *)h, d, (const T *)w_up, (size_t)up_rows * d, up_rows, d, sorted, wts, \
                                                      t_exp, t_beg, t_rows, n_tiles, max_tiles, (T *)act, nullptr, ff, top, 0);       \
    else                                                                                                                           \
        KERNEL<T, MOE_UP><<<gu, block, 0, stream>>>((const T *)h, d, (const T *)w_up, (size_t)ff * d, ff, d, sorted, wts, t_exp, t_beg, \
                                                t_rows, n_tiles, max_tiles, (T *)act, nullptr, ff, top, 0);                         \
    KERNEL<T, MOE_DOWN><<<gd, block, 0, stream>>>((const T *)act, ff, (const T *)w_down, (size_t)ff * d, d, ff, sorted, wts, t_exp, \
                                                  t_beg, t_rows, n_tiles, max_tiles, nullptr, down_to, d, top, add)
    if (type == LCU_BF16) {
        if (tile_rows == 16) { GO(moe_gemm_few_kernel, bf16_t); } else { GO(moe_gemm_many_kernel, bf16_t); }
    } else {
        if (tile_rows == 16) { GO(moe_gemm_few_kernel, float); } else { GO(moe_gemm_many_kernel, float); }
    }
#undef GO
    LCU_LAUNCH_CHECK();
    if (!add) {
        const dim3 gc((d + 255) / 256, n < 65535 ? n : 65535);
        const int *idp = identity ? ids : nullptr;
        if (type == LCU_BF16) moe_combine_kernel<bf16_t><<<gc, dim3(256), 0, stream>>>(out, y, gated ? wts : nullptr, (const bf16_t *)shared, shared_gate, n, d, top, fresh, idp, experts, (const bf16_t *)h);
        else moe_combine_kernel<float><<<gc, dim3(256), 0, stream>>>(out, y, gated ? wts : nullptr, (const float *)shared, shared_gate, n, d, top, fresh, idp, experts, (const float *)h);
        LCU_LAUNCH_CHECK();
    }
    return LCU_OK;
}
