// Everything between the q, k, v product and the attention, for attention whose queries, keys and values take more
// than a rotation of whole heads: each step is optional and a parameter.
//
//   q, k, v <- product + bias                                           (bias: one vector over the row's columns)
//   q, k    <- x * rsqrt(mean over the head's dims of x^2 + eps) * w     (w [dh], shared by all heads; one for q, one for k)
//   q, k    <- the first rot_dim dims of every head turned by the angle of the token's position (tables
//              [max_pos, rot_dim / 2]; pairing 0: (i, i + rot_dim/2), 1: (2i, 2i + 1)); the other dims pass
//   q -> q_out [n, nh * dhp]; k, v -> the token's place in its page
//
// The head sizes of the rows (dh, dv) may be any; what is stored has dhp >= dh and dvp >= dv dims per head, the
// dims beyond the true ones zeros (dhp a multiple of 8, as the pages' layout wants; zeros change no score and no
// output).  All arithmetic is 32-bit, one rounding at each store.  One wave per (token, head).
#include "common.h"
#include "kv_layout.h"

constexpr int QP_MAX_DIM = 256;

template <class TI, class T>
__global__ void __launch_bounds__(WAVE)
qkv_prepare_kernel(const TI *__restrict__ rows, int row_stride, int q_off, int k_off, int v_off,
                   const float *__restrict__ bias, const float *__restrict__ q_norm, const float *__restrict__ k_norm,
                   float eps, const int *__restrict__ positions, const float *__restrict__ cos_t,
                   const float *__restrict__ sin_t, int max_pos, int rot_dim, int pairing, T *__restrict__ q_out,
                   const int *__restrict__ slots, T *__restrict__ cache, int nh, int nkvh, int dh, int dhp, int dv,
                   int dvp, int page, int store_kv) {
    const int t = blockIdx.x, head = blockIdx.y, lane = threadIdx.x;
    const TI *row = rows + (size_t)t * row_stride;
    __shared__ float xs[QP_MAX_DIM];
    int slot = -1;
    T *pg = nullptr;
    int tok = 0;
    if (head >= nh) {
        slot = store_kv ? slots[t] : -1;
        if (slot < 0) return;
        pg = cache + (size_t)(slot / page) * kv_page_elems(nkvh, dhp, dvp, page);
        tok = slot % page;
    }
    if (head >= nh + nkvh) {                                  // a value head: product + bias, as it is
        const int kvh = head - nh - nkvh, col0 = v_off + kvh * dv;
        for (int c = lane; c < dvp; c += WAVE) {
            float v = 0.f;
            if (c < dv) v = to_f32(row[col0 + c]) + (bias ? bias[col0 + c] : 0.f);
            pg[kv_value_offset(nkvh, kvh, tok, c, dhp, dvp, page)] = from_f32<T>(v);
        }
        return;
    }
    const bool is_key = head >= nh;
    const int col0 = is_key ? k_off + (head - nh) * dh : q_off + head * dh;
    const float *nw = is_key ? k_norm : q_norm;
    float sq = 0.f;
    for (int c = lane; c < dh; c += WAVE) {
        const float v = to_f32(row[col0 + c]) + (bias ? bias[col0 + c] : 0.f);
        xs[c] = v;
        sq += v * v;
    }
    if (nw) {
        const float f = rsqrtf(wave_sum(sq) / (float)dh + eps);
        for (int c = lane; c < dh; c += WAVE) xs[c] = xs[c] * f * nw[c];
    }
    __syncthreads();
    if (cos_t) {
        const int pos = positions[t], half = rot_dim / 2;
        const bool in_table = pos >= 0 && pos < max_pos;
        for (int i = lane; i < half; i += WAVE) {
            const int ia = pairing == 0 ? i : 2 * i, ib = pairing == 0 ? i + half : 2 * i + 1;
            float ra = __uint_as_float(0x7fc00000u), rb = ra;      // a position outside the table gives NaN, not a wrong value
            if (in_table) rotate_pair(xs[ia], xs[ib], cos_t[(size_t)pos * half + i], sin_t[(size_t)pos * half + i], ra, rb);
            xs[ia] = ra;
            xs[ib] = rb;
        }
        __syncthreads();
    }
    if (!is_key) {
        T *o = q_out + (size_t)t * nh * dhp + (size_t)head * dhp;
        for (int c = lane; c < dhp; c += WAVE) o[c] = from_f32<T>(c < dh ? xs[c] : 0.f);
    } else {
        const int kvh = head - nh;
        for (int c = lane; c < dhp; c += WAVE) pg[kv_key_offset(kvh, tok, c, dhp, page)] = from_f32<T>(c < dh ? xs[c] : 0.f);
    }
}

// rows: [n, row_stride] of in_type, a token's q heads at column q_off (nh * dh), k heads at k_off (nkvh * dh), v heads
// at v_off (nkvh * dv); bias: null or float32 over the row's columns; q_norm, k_norm: null or float32 [dh].
// q_out: [n, nh * dhp] of type; cache: this layer's pages of type, kv_page_elems(nkvh, dhp, dvp, page) each;
// slots[t] = page * page_size + place, or -1 to store nothing for token t.  store_kv 0: queries only.
LCU_API int lcu_qkv_prepare(const void *rows, int in_type, int n, int row_stride, int q_off, int k_off, int v_off,
                            const float *bias, const float *q_norm, const float *k_norm, float eps, const int *positions,
                            const float *cos_t, const float *sin_t, int max_pos, int rot_dim, int pairing, void *q_out,
                            int type, const int *slots, void *cache, int nh, int nkvh, int dh, int dhp, int dv, int dvp,
                            int page, int store_kv, hipStream_t stream) {
    if (n <= 0) return LCU_OK;
    if (nh <= 0 || nkvh < 0 || dh <= 0 || dh > QP_MAX_DIM || dhp < dh || dhp % 8 || dhp > QP_MAX_DIM || dv <= 0 || dvp < dv ||
        dvp > QP_MAX_DIM || page <= 0 || page % 8 || rot_dim < 0 || rot_dim % 2 || rot_dim > dh || (pairing != 0 && pairing != 1) ||
        !rows || !q_out || (cos_t && (!sin_t || !positions || rot_dim == 0)) || nh + 2 * nkvh > 65535)
        return LCU_BAD_ARGUMENT;
    if (store_kv && (!cache || !slots || nkvh <= 0)) return LCU_BAD_ARGUMENT;
    dim3 grid(n, store_kv ? nh + 2 * nkvh : nh), block(WAVE);
#define GO(TI, T) qkv_prepare_kernel<TI, T><<<grid, block, 0, stream>>>((const TI *)rows, row_stride, q_off, k_off, v_off, bias, q_norm, k_norm, eps, positions, cos_t, sin_t, max_pos, rot_dim, pairing, (T *)q_out, slots, (T *)cache, nh, nkvh, dh, dhp, dv, dvp, page, store_kv)
    if (in_type == LCU_F32 && type == LCU_F32) GO(float, float);
    else if (in_type == LCU_F32 && type == LCU_BF16) GO(float, bf16_t);
    else if (in_type == LCU_BF16 && type == LCU_BF16) GO(bf16_t, bf16_t);
    else return LCU_BAD_ARGUMENT;
#undef GO
    LCU_LAUNCH_CHECK();
    return LCU_OK;
}

// The output of every head times sigmoid of the head's gate: out[t, h, :] *= sigmoid(gate[t, h]), the gate's rows
// [n, gate_stride] with the heads' numbers from column g_off.  The factor is 32-bit.
template <class TG, class T>
__global__ void head_gate_kernel(T *__restrict__ out, const TG *__restrict__ gate, int gate_stride, int g_off, int nh, int dv) {
    const int t = blockIdx.x;
    for (int c = threadIdx.x; c < nh * dv; c += blockDim.x) {
        const float g = to_f32(gate[(size_t)t * gate_stride + g_off + c / dv]);
        T *o = out + (size_t)t * nh * dv + c;
        *o = from_f32<T>(to_f32(*o) / (1.0f + expf(-g)));
    }
}

LCU_API int lcu_head_gate(void *out, int type, const void *gate, int gate_type, int gate_stride, int g_off, int n, int nh,
                          int dv, hipStream_t stream) {
    if (n <= 0) return LCU_OK;
    if (nh <= 0 || dv <= 0 || !out || !gate) return LCU_BAD_ARGUMENT;
    dim3 grid(n), block(256);
#define GO(TG, T) head_gate_kernel<TG, T><<<grid, block, 0, stream>>>((T *)out, (const TG *)gate, gate_stride, g_off, nh, dv)
    if (gate_type == LCU_F32 && type == LCU_F32) GO(float, float);
    else if (gate_type == LCU_F32 && type == LCU_BF16) GO(float, bf16_t);
    else if (gate_type == LCU_BF16 && type == LCU_BF16) GO(bf16_t, bf16_t);
    else return LCU_BAD_ARGUMENT;
#undef GO
    LCU_LAUNCH_CHECK();
    return LCU_OK;
}
