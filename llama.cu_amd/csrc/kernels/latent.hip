// Latent attention: what stands between the input product and the attention over the cache.
//
// A token's keys and values of all heads are functions of one latent vector c [rank] and one turned key part r [rot]
// that all heads share:  k_h = [W_uk_h c, r],  v_h = W_uv_h c.  The score of a query q_h = [q_plain, q_turned] is then
//   q_plain . (W_uk_h c) + q_turned . r  =  (W_uk_h^T q_plain) . c + q_turned . r,
// a dot product of the folded query [W_uk_h^T q_plain, q_turned] with the cached row [c, r]: attention of all heads over ONE
// key/value head whose key is [c, r] and whose value is c; W_uv_h is applied to the attention's output.  The cache holds
// c and r only.
//
// This kernel, one wave per (token, head) and one more per token for the cache:
//   query head h:  the turned part of the product's row is rotated by the token's position and written behind the
//                  folded plain part (which a matrix product has written into q_out already); dims beyond the true
//                  ones are zeros;
//   cache:         c = x * rsqrt(mean(x^2) + eps) * w over the first `rank` columns of the token's latent product,
//                  r = the last `rot` columns rotated; key = [c, r, zeros], value = [c, zeros] at the token's place.
// The rotation pairs dim i with dim i + rot / 2 (tables [max_pos, rot / 2] of the 32-bit angle's cosine and sine).
// All arithmetic is 32-bit, one rounding at each store.
#include "common.h"
#include "kv_layout.h"

constexpr int LP_MAX_DIM = 640;

template <class TI, class T>
__global__ void __launch_bounds__(WAVE)
latent_prepare_kernel(const TI *__restrict__ rows, int row_stride, int q_head_stride, int q_rot_off, int kv_off,
                      const float *__restrict__ c_norm, float eps, const int *__restrict__ positions,
                      const float *__restrict__ cos_t, const float *__restrict__ sin_t, int max_pos, T *__restrict__ q_out,
                      const int *__restrict__ slots, T *__restrict__ cache, int nh, int rank, int rot, int dhp, int dvp,
                      int page) {
    const int t = blockIdx.x, head = blockIdx.y, lane = threadIdx.x;
    const TI *row = rows + (size_t)t * row_stride;
    const int pos = positions[t], half = rot / 2;
    const bool in_table = pos >= 0 && pos < max_pos;
    const float nan = __uint_as_float(0x7fc00000u);          // a position outside the table gives NaN, not a wrong value
    __shared__ float xs[LP_MAX_DIM];
    if (head < nh) {
        const TI *qr = row + (size_t)head * q_head_stride + q_rot_off;
        T *o = q_out + ((size_t)t * nh + head) * dhp;
        for (int i = lane; i < half; i += WAVE) {
            float ra = nan, rb = nan;
            if (in_table) rotate_pair(to_f32(qr[i]), to_f32(qr[i + half]), cos_t[(size_t)pos * half + i], sin_t[(size_t)pos * half + i], ra, rb);
            o[rank + i] = from_f32<T>(ra);
            o[rank + half + i] = from_f32<T>(rb);
        }
        for (int c = rank + rot + lane; c < dhp; c += WAVE) o[c] = from_f32<T>(0.f);
        return;
    }
    const int slot = slots[t];
    if (slot < 0) return;
    T *pg = cache + (size_t)(slot / page) * kv_page_elems(1, dhp, dvp, page);
    const int tok = slot % page;
    const TI *kv = row + kv_off;
    float sq = 0.f;
    for (int c = lane; c < rank; c += WAVE) {
        const float v = to_f32(kv[c]);
        xs[c] = v;
        sq += v * v;
    }
    const float f = rsqrtf(wave_sum(sq) / (float)rank + eps);
    for (int c = lane; c < rank; c += WAVE) {
        const T v = from_f32<T>(xs[c] * f * c_norm[c]);
        pg[kv_key_offset(0, tok, c, dhp, page)] = v;
        pg[kv_value_offset(1, 0, tok, c, dhp, dvp, page)] = v;
    }
    for (int i = lane; i < half; i += WAVE) {
        float ra = nan, rb = nan;
        if (in_table) rotate_pair(to_f32(kv[rank + i]), to_f32(kv[rank + half + i]), cos_t[(size_t)pos * half + i], sin_t[(size_t)pos * half + i], ra, rb);
        pg[kv_key_offset(0, tok, rank + i, dhp, page)] = from_f32<T>(ra);
        pg[kv_key_offset(0, tok, rank + half + i, dhp, page)] = from_f32<T>(rb);
    }
    for (int c = rank + rot + lane; c < dhp; c += WAVE) pg[kv_key_offset(0, tok, c, dhp, page)] = from_f32<T>(0.f);
    for (int c = rank + lane; c < dvp; c += WAVE) pg[kv_value_offset(1, 0, tok, c, dhp, dvp, page)] = from_f32<T>(0.f);
}

// rows: [n, row_stride] of in_type; query head h's turned part at column h * q_head_stride + q_rot_off (rot columns); the
// latent product at column kv_off (rank + rot columns).  c_norm: float32 [rank].  q_out: [n, nh * dhp] of type, a head's
// first `rank` columns filled already.  cache: pages of one key/value head, keys of dhp and values of dvp dims
// (kv_page_elems(1, dhp, dvp, page) each); slots[t] = page * page_size + place, or -1; store_kv 0: queries only.
LCU_API int lcu_latent_prepare(const void *rows, int in_type, int n, int row_stride, int q_head_stride, int q_rot_off, int kv_off,
                               const float *c_norm, float eps, const int *positions, const float *cos_t, const float *sin_t,
                               int max_pos, void *q_out, int type, const int *slots, void *cache, int nh, int rank, int rot,
                               int dhp, int dvp, int page, int store_kv, hipStream_t stream) {
    if (n <= 0) return LCU_OK;
    if (nh <= 0 || nh >= 65535 || rank <= 0 || rot <= 0 || rot % 2 || rank + rot > dhp || dhp % 8 || dhp > LP_MAX_DIM || dvp < rank ||
        dvp > LP_MAX_DIM || page <= 0 || page % 8 || !rows || !q_out || !positions || !cos_t || !sin_t || max_pos <= 0)
        return LCU_BAD_ARGUMENT;
    if (store_kv && (!cache || !slots || !c_norm)) return LCU_BAD_ARGUMENT;
    dim3 grid(n, store_kv ? nh + 1 : nh), block(WAVE);
#define GO(TI, T) latent_prepare_kernel<TI, T><<<grid, block, 0, stream>>>((const TI *)rows, row_stride, q_head_stride, q_rot_off, kv_off, c_norm, eps, positions, cos_t, sin_t, max_pos, (T *)q_out, slots, (T *)cache, nh, rank, rot, dhp, dvp, page)
    if (in_type == LCU_F32 && type == LCU_F32) GO(float, float);
    else if (in_type == LCU_F32 && type == LCU_BF16) GO(float, bf16_t);
    else if (in_type == LCU_BF16 && type == LCU_BF16) GO(bf16_t, bf16_t);
    else return LCU_BAD_ARGUMENT;
#undef GO
    LCU_LAUNCH_CHECK();
    return LCU_OK;
}
