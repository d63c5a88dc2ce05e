// What stands between the q, k, v product and an attention that has no rotation: a norm
// over the whole query projection and over the whole key projection (all heads at once, a
// weight per column), a factor on the queries that grows with the logarithm of the position,
// and the write of keys and values into their pages.  Each piece is optional.
//
//   q <- q * rsqrt(mean(q^2) + eps) * qw          (mean over all nh * dh columns, or over q_count of them where heads
//                                                   were filled up with columns of zeros; qw null: no norm)
//   q <- q * (1 + coef * ln(floor((p + 1) / every) + 1))      (p the row's position; coef 0: none)
//   k <- k * rsqrt(mean(k^2) + eps) * kw          (over all nkvh * dh columns), into the cache
//   v into the cache as it is (head size dv)
// Sums, norms and factors are 32-bit; one rounding where q is written back and where k
// is stored.
#include "common.h"
#include "kv_layout.h"

constexpr int QK_THREADS = 256;

// One block per row of qkv = [q (nh*dh) | k (nkvh*dh) | v (nkvh*dv)] (only q if !store_kv).
template <class T>
__global__ void __launch_bounds__(QK_THREADS)
qk_norm_store_kernel(T *__restrict__ qkv, int row_stride, const int *__restrict__ positions,
                     const int *__restrict__ slots, const float *__restrict__ qw, const float *__restrict__ kw,
                     T *__restrict__ cache, int nh, int nkvh, int dh, int dv, int page, float eps, float coef,
                     int every, int store_kv, int q_count, int k_count) {
    __shared__ float scratch[16];
    const int t = blockIdx.x;
    T *row = qkv + (size_t)t * row_stride;
    const int nq = nh * dh, nk = nkvh * dh, nv = nkvh * dv;
    float fq = 1.f, fk = 1.f;
    if (qw) {
        float acc = 0.f;
        for (int c = threadIdx.x; c < nq; c += QK_THREADS) {
            const float v = to_f32(row[c]);
            acc += v * v;
        }
        fq = rsqrtf(block_sum(acc, scratch) / (float)q_count + eps);
    }
    if (coef != 0.f) {
        const int p = positions[t];
        fq *= 1.0f + coef * logf((float)((p + 1) / every) + 1.0f);
    }
    if (qw || coef != 0.f)
        for (int c = threadIdx.x; c < nq; c += QK_THREADS)
            row[c] = from_f32<T>(to_f32(row[c]) * fq * (qw ? qw[c] : 1.f));
    if (!store_kv) return;
    const int slot = slots[t];
    if (slot < 0) return;
    if (kw) {
        float acc = 0.f;
        for (int c = threadIdx.x; c < nk; c += QK_THREADS) {
            const float v = to_f32(row[nq + c]);
            acc += v * v;
        }
        fk = rsqrtf(block_sum(acc, scratch) / (float)k_count + eps);
    }
    T *pg = cache + (size_t)(slot / page) * kv_page_elems(nkvh, dh, dv, page);
    const int tok = slot % page;
    for (int c = threadIdx.x; c < nk; c += QK_THREADS)
        pg[kv_key_offset(c / dh, tok, c % dh, dh, page)] = from_f32<T>(to_f32(row[nq + c]) * fk * (kw ? kw[c] : 1.f));
    for (int c = threadIdx.x; c < nv; c += QK_THREADS)
        pg[kv_value_offset(nkvh, c / dv, tok, c % dv, dh, dv, page)] = row[nq + nk + c];
}

LCU_API int lcu_qk_norm_store(void *qkv, int type, int n, int row_stride, const int *positions, const int *slots,
                              const float *qw, const float *kw, void *cache, int nh, int nkvh, int dh, int dv, int page,
                              float eps, float coef, int every, int store_kv, int q_count, int k_count, hipStream_t stream) {
    if (n <= 0) return LCU_OK;
    if (nh <= 0 || nkvh <= 0 || dh <= 0 || dh % 8 || dv <= 0 || page <= 0 || (coef != 0.f && (every <= 0 || !positions)) ||
        (store_kv && (!cache || !slots)))
        return LCU_BAD_ARGUMENT;
    // the columns that a mean runs over: fewer than the rows hold where heads were filled up with columns of zeros
    if (q_count <= 0) q_count = nh * dh;
    if (k_count <= 0) k_count = nkvh * dh;
    dim3 grid(n), block(QK_THREADS);
    if (type == LCU_F32)
        qk_norm_store_kernel<float><<<grid, block, 0, stream>>>((float *)qkv, row_stride, positions, slots, qw, kw, (float *)cache, nh, nkvh, dh, dv, page, eps, coef, every, store_kv, q_count, k_count);
    else if (type == LCU_BF16)
        qk_norm_store_kernel<bf16_t><<<grid, block, 0, stream>>>((bf16_t *)qkv, row_stride, positions, slots, qw, kw, (bf16_t *)cache, nh, nkvh, dh, dv, page, eps, coef, every, store_kv, q_count, k_count);
    else
        return LCU_BAD_ARGUMENT;
    LCU_LAUNCH_CHECK();
    return LCU_OK;
}
