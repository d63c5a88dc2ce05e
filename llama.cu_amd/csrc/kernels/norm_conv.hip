// Layer norm (mean and variance, weight and bias) fused with the residual sum that precedes
// it, for one or two norms of the same row; and the short causal convolution over time that
// a sublayer may put in front of what it reads, with its per-request state.
//
// Layer norm of a row x of width d, all in 32-bit:
//   m = mean(x), var = mean((x - m)^2) (the deviations are taken from the mean that was
//   computed first), y = (x - m) * rsqrt(var + eps) * w + b.
// Short convolution of taps T on every channel c of rows h that belong to requests:
//   out[t] = h[t] + sum_{j < T} cw[c][j] * h[t - (T - 1) + j]
// where rows before the request's first row of this step come from the request's state (the
// last T - 1 rows of earlier steps) and rows before position 0 are zeros.
#include "common.h"

constexpr int NC_THREADS = 256;
constexpr int MAX_TAPS = 16;

// x (32-bit residual stream, [n, d]) takes in `planes` planes of delta (type TD, plane_stride
// apart), is written back, and is normed with (w1, b1) into out1 and, if w2 is not null, with
// (w2, b2) into out2.  One block per row.
template <class TD, class TO>
__global__ void __launch_bounds__(NC_THREADS)
layernorm_kernel(float *__restrict__ x, const TD *__restrict__ delta, int planes, size_t plane_stride,
                 const float *__restrict__ w1, const float *__restrict__ b1, TO *__restrict__ out1,
                 const float *__restrict__ w2, const float *__restrict__ b2, TO *__restrict__ out2, int d, float eps) {
    __shared__ float scratch[16];
    float *xr = x + (size_t)blockIdx.x * d;
    float sum = 0.f;
    for (int c = threadIdx.x; c < d; c += NC_THREADS) {
        float v = xr[c];
        if (delta) {
            for (int p = 0; p < planes; ++p) v += to_f32(delta[p * plane_stride + (size_t)blockIdx.x * d + c]);
            xr[c] = v;
        }
        sum += v;
    }
    const float mean = block_sum(sum, scratch) / (float)d;
    float sq = 0.f;
    for (int c = threadIdx.x; c < d; c += NC_THREADS) {     // each thread reads back what it wrote itself
        const float dev = xr[c] - mean;
        sq += dev * dev;
    }
    const float rstd = rsqrtf(block_sum(sq, scratch) / (float)d + eps);
    for (int c = threadIdx.x; c < d; c += NC_THREADS) {
        const float z = (xr[c] - mean) * rstd;
        out1[(size_t)blockIdx.x * d + c] = from_f32<TO>(z * w1[c] + b1[c]);
        if (w2) out2[(size_t)blockIdx.x * d + c] = from_f32<TO>(z * w2[c] + b2[c]);
    }
}

// The same for rows of up to NC_THREADS * PT elements: the row stays in registers between its one read and
// its writes (a step of few rows is a chain of dependent trips to memory, and this kernel has one, not three).
template <class TD, class TO, int PT>
__global__ void __launch_bounds__(NC_THREADS)
layernorm_row_kernel(float *__restrict__ x, const TD *__restrict__ delta, int planes, size_t plane_stride,
                     const float *__restrict__ w1, const float *__restrict__ b1, TO *__restrict__ out1,
                     const float *__restrict__ w2, const float *__restrict__ b2, TO *__restrict__ out2, int d, float eps) {
    __shared__ float scratch[16];
    float *xr = x + (size_t)blockIdx.x * d;
    float v[PT], sum = 0.f;
#pragma unroll
    for (int i = 0; i < PT; ++i) {
        const int c = threadIdx.x + NC_THREADS * i;
        v[i] = 0.f;
        if (c < d) {
            v[i] = xr[c];
            if (delta) {
                for (int p = 0; p < planes; ++p) v[i] += to_f32(delta[p * plane_stride + (size_t)blockIdx.x * d + c]);
                xr[c] = v[i];
            }
            sum += v[i];
        }
    }
    const float mean = block_sum(sum, scratch) / (float)d;
    float sq = 0.f;
#pragma unroll
    for (int i = 0; i < PT; ++i) {
        const float dev = v[i] - mean;
        if (threadIdx.x + NC_THREADS * i < d) sq += dev * dev;
    }
    const float rstd = rsqrtf(block_sum(sq, scratch) / (float)d + eps);
#pragma unroll
    for (int i = 0; i < PT; ++i) {
        const int c = threadIdx.x + NC_THREADS * i;
        if (c < d) {
            const float z = (v[i] - mean) * rstd;
            out1[(size_t)blockIdx.x * d + c] = from_f32<TO>(z * w1[c] + b1[c]);
            if (w2) out2[(size_t)blockIdx.x * d + c] = from_f32<TO>(z * w2[c] + b2[c]);
        }
    }
}

// delta_type: -1 none, LCU_F32 or LCU_BF16.  out_type: LCU_F32 or LCU_BF16.
LCU_API int lcu_layernorm(float *x, const void *delta, int delta_type, int planes, const float *w1, const float *b1,
                          void *out1, const float *w2, const float *b2, void *out2, int out_type, int n, int d,
                          float eps, hipStream_t stream) {
    if (n <= 0) return LCU_OK;
    if (d <= 0 || !w1 || !b1 || !out1 || (w2 && (!b2 || !out2)) || (delta && planes <= 0)) return LCU_BAD_ARGUMENT;
    const size_t stride = (size_t)n * d;
    dim3 grid(n), block(NC_THREADS);
#define ROW(TD, TO, PT) layernorm_row_kernel<TD, TO, PT><<<grid, block, 0, stream>>>(x, (const TD *)delta, planes, stride, w1, b1, (TO *)out1, w2, b2, (TO *)out2, d, eps)
#define GO(TD, TO)                                                                                                           \
    do {                                                                                                                     \
        if (d <= 4 * NC_THREADS) ROW(TD, TO, 4);                                                                             \
        else if (d <= 16 * NC_THREADS) ROW(TD, TO, 16);                                                                      \
        else layernorm_kernel<TD, TO><<<grid, block, 0, stream>>>(x, (const TD *)delta, planes, stride, w1, b1, (TO *)out1,  \
                                                                  w2, b2, (TO *)out2, d, eps);                               \
    } while (0)
    const int dt = delta ? delta_type : LCU_F32;
    if (dt == LCU_F32 && out_type == LCU_F32) GO(float, float);
    else if (dt == LCU_F32 && out_type == LCU_BF16) GO(float, bf16_t);
    else if (dt == LCU_BF16 && out_type == LCU_F32) GO(bf16_t, float);
    else if (dt == LCU_BF16 && out_type == LCU_BF16) GO(bf16_t, bf16_t);
    else return LCU_BAD_ARGUMENT;
#undef ROW
#undef GO
    LCU_LAUNCH_CHECK();
    return LCU_OK;
}

// ---------------------------------------------------------------- short convolution
// `sets` independent convolutions at once (blockIdx.y): set s reads h + s * set_stride_h, the
// weights cw + s * d * taps ([d, taps]), its part of the state and writes
// out + s * set_stride_out.  state: [slots, sets, taps - 1, d] 32-bit, row i of a request's state is
// the row at position P0 - (taps - 1) + i, P0 the position of the request's first row of this
// step.  The state is only read here.
template <class TI, class TW, class TO>
__global__ void __launch_bounds__(NC_THREADS)
short_conv_kernel(const TI *__restrict__ h, size_t set_stride_h, const TW *__restrict__ cw, const float *__restrict__ st, TO *__restrict__ out, size_t set_stride_out, const int *__restrict__ q_start,
                  const int *__restrict__ ctx_len, const int *__restrict__ req_of_token,
                  const int *__restrict__ state_slot, int d, int taps) {
    const int t = blockIdx.x, s = blockIdx.y;
    const int r = req_of_token[t];
    const int first = q_start[r];
    const int pos = ctx_len[r] - (q_start[r + 1] - t);          // this row's position
    const TI *hs = h + s * set_stride_h;
    const TW *w = cw + (size_t)s * d * taps;
    const float *state = st + ((size_t)state_slot[r] * gridDim.y + s) * (taps - 1) * d;
    for (int c = threadIdx.x; c < d; c += NC_THREADS) {
        float acc = to_f32(hs[(size_t)t * d + c]);
        for (int j = 0; j < taps; ++j) {
            const int back = taps - 1 - j;                      // the row `back` positions earlier
            if (pos - back < 0) continue;                       // no such row: the request starts later
            float v;
            if (t - back >= first) v = to_f32(hs[(size_t)(t - back) * d + c]);
            else v = state[(size_t)(taps - 1 - (first - (t - back))) * d + c];
            acc += to_f32(w[(size_t)c * taps + j]) * v;
        }
        out[s * set_stride_out + (size_t)t * d + c] = from_f32<TO>(acc);
    }
}

// After the convolution has run: every request's state becomes the last taps - 1 rows up to
// the end of this step (rows of this step, or of the old state, or zeros before position 0).
// A thread owns a channel: it reads all it needs, then writes.
template <class TI>
__global__ void __launch_bounds__(NC_THREADS)
short_conv_update_kernel(const TI *__restrict__ h, size_t set_stride_h, float *__restrict__ st,
                         const int *__restrict__ q_start, const int *__restrict__ ctx_len,
                         const int *__restrict__ state_slot, int d, int taps) {
    const int r = blockIdx.x, s = blockIdx.y;
    const int first = q_start[r], n_new = q_start[r + 1] - first;
    const int p0 = ctx_len[r] - n_new;                          // position of the first row of this step
    const TI *hs = h + s * set_stride_h;
    float *state = st + ((size_t)state_slot[r] * gridDim.y + s) * (taps - 1) * d;
    for (int c = blockIdx.z * NC_THREADS + threadIdx.x; c < d; c += gridDim.z * NC_THREADS) {
        float keep[MAX_TAPS];
#pragma unroll
        for (int i = 0; i < MAX_TAPS; ++i) {
            if (i < taps - 1) {
                const int back = taps - 1 - i;                  // the new row i lies `back` rows before the step's end
                const int row = n_new - back;                   // among this step's rows, if >= 0
                float v = 0.f;
                if (row >= 0) v = to_f32(hs[(size_t)(first + row) * d + c]);
                else if (p0 + row >= 0) v = state[(size_t)(taps - 1 + row) * d + c];
                keep[i] = v;
            }
        }
#pragma unroll
        for (int i = 0; i < MAX_TAPS; ++i)
            if (i < taps - 1) state[(size_t)i * d + c] = keep[i];
    }
}

// h: [sets][n, d] (sets set_stride_h elements apart), cw: [sets][d, taps], state: [slots, sets, taps - 1, d],
// out: [sets][n, d] (set_stride_out apart).  update: 0 only the convolution,
// 1 the convolution and then the state.
LCU_API int lcu_short_conv(const void *h, int h_type, long long set_stride_h, const void *cw, int w_type, float *state,
                           void *out, int out_type, long long set_stride_out, const int *q_start,
                           const int *ctx_len, const int *req_of_token, const int *state_slot, int n, int n_req, int d,
                           int taps, int sets, int update, hipStream_t stream) {
    if (n <= 0 || n_req <= 0) return LCU_OK;
    if (d <= 0 || taps < 1 || taps > MAX_TAPS || sets < 1 || sets > 8 || h_type != LCU_F32 && h_type != LCU_BF16) return LCU_BAD_ARGUMENT;
    if (w_type != h_type && !(w_type == LCU_F32) && !(h_type == LCU_F32 && w_type == LCU_BF16)) return LCU_BAD_ARGUMENT;
    dim3 grid(n, sets), block(NC_THREADS);
#define GO(TI, TW, TO) short_conv_kernel<TI, TW, TO><<<grid, block, 0, stream>>>((const TI *)h, (size_t)set_stride_h, (const TW *)cw, state, (TO *)out, (size_t)set_stride_out, q_start, ctx_len, req_of_token, state_slot, d, taps)
    if (h_type == LCU_F32 && w_type == LCU_F32 && out_type == LCU_F32) GO(float, float, float);
    else if (h_type == LCU_F32 && w_type == LCU_F32 && out_type == LCU_BF16) GO(float, float, bf16_t);
    else if (h_type == LCU_F32 && w_type == LCU_BF16 && out_type == LCU_BF16) GO(float, bf16_t, bf16_t);
    else if (h_type == LCU_F32 && w_type == LCU_BF16 && out_type == LCU_F32) GO(float, bf16_t, float);
    else if (h_type == LCU_BF16 && w_type == LCU_BF16 && out_type == LCU_BF16) GO(bf16_t, bf16_t, bf16_t);
    else if (h_type == LCU_BF16 && w_type == LCU_F32 && out_type == LCU_BF16) GO(bf16_t, float, bf16_t);
    else return LCU_BAD_ARGUMENT;
#undef GO
    LCU_LAUNCH_CHECK();
    if (update && taps > 1) {
        dim3 ugrid(n_req, sets, (d + NC_THREADS - 1) / NC_THREADS);
        if (h_type == LCU_F32)
            short_conv_update_kernel<float><<<ugrid, block, 0, stream>>>((const float *)h, (size_t)set_stride_h, state, q_start, ctx_len, state_slot, d, taps);
        else
            short_conv_update_kernel<bf16_t><<<ugrid, block, 0, stream>>>((const bf16_t *)h, (size_t)set_stride_h, state, q_start, ctx_len, state_slot, d, taps);
        LCU_LAUNCH_CHECK();
    }
    return LCU_OK;
}

// ---------------------------------------------------------------- a step of single tokens: all of the above in one kernel
// Every request feeds one token (row r is request r's): the residual sum, one or two layer norms, their short
// convolutions from the requests' states, and the states' update, with the row in registers throughout.  A block
// is the only reader and writer of its request's state, and a thread of its channels'.
// out: [sets][n, d] of TO; state: [slots, sets, taps - 1, d]; cw: [sets][d, taps] 32-bit.
template <class TD, class TO, int PT>
__global__ void __launch_bounds__(NC_THREADS)
norm_conv_single_kernel(float *__restrict__ x, const TD *__restrict__ delta, int planes, size_t plane_stride,
                        const float *__restrict__ w1, const float *__restrict__ b1, const float *__restrict__ w2,
                        const float *__restrict__ b2, const float *__restrict__ cw, float *__restrict__ st,
                        TO *__restrict__ out, size_t set_stride_out, const int *__restrict__ ctx_len,
                        const int *__restrict__ state_slot, int d, int taps, int sets, float eps) {
    __shared__ float scratch[16];
    const int r = blockIdx.x;
    const int pos = ctx_len[r] - 1;                  // the token's position
    float *xr = x + (size_t)r * d;
    float v[PT], sum = 0.f;
#pragma unroll
    for (int i = 0; i < PT; ++i) {
        const int c = threadIdx.x + NC_THREADS * i;
        v[i] = 0.f;
        if (c < d) {
            v[i] = xr[c];
            if (delta) {
                for (int p = 0; p < planes; ++p) v[i] += to_f32(delta[p * plane_stride + (size_t)r * d + c]);
                xr[c] = v[i];
            }
            sum += v[i];
        }
    }
    const float mean = block_sum(sum, scratch) / (float)d;
    float sq = 0.f;
#pragma unroll
    for (int i = 0; i < PT; ++i) {
        const float dev = v[i] - mean;
        if (threadIdx.x + NC_THREADS * i < d) sq += dev * dev;
    }
    const float rstd = rsqrtf(block_sum(sq, scratch) / (float)d + eps);
    constexpr int FUSED_TAPS = 8;                    // the most taps this kernel takes
    for (int s = 0; s < sets; ++s) {
        const float *w = s ? w2 : w1, *b = s ? b2 : b1;
        float *state = st + ((size_t)state_slot[r] * sets + s) * (taps - 1) * d;
        // everything is read before anything is written: the state's new rows are its old ones, and loads that had to
        // wait for the stores before them would be a chain of trips to memory
        float old[PT][FUSED_TAPS - 1], k[PT][FUSED_TAPS], wv[PT], bv[PT];
#pragma unroll
        for (int i = 0; i < PT; ++i) {
            const int c = threadIdx.x + NC_THREADS * i;
            if (c >= d) continue;
            wv[i] = w[c];
            bv[i] = b[c];
#pragma unroll
            for (int j = 0; j < FUSED_TAPS; ++j)
                if (j < taps) k[i][j] = cw[((size_t)s * d + c) * taps + j];
#pragma unroll
            for (int j = 0; j < FUSED_TAPS - 1; ++j)      // row j of the state lies taps - 1 - j positions before the token
                if (j < taps - 1) old[i][j] = pos - (taps - 1 - j) >= 0 ? state[(size_t)j * d + c] : 0.f;
        }
#pragma unroll
        for (int i = 0; i < PT; ++i) {
            const int c = threadIdx.x + NC_THREADS * i;
            if (c >= d) continue;
            const float h = (v[i] - mean) * rstd * wv[i] + bv[i];
            float acc = h;                            // (the order of short_conv_kernel's additions)
#pragma unroll
            for (int j = 0; j < FUSED_TAPS - 1; ++j)
                if (j < taps - 1) {
                    acc += k[i][j] * old[i][j];
                    if (j > 0) state[(size_t)(j - 1) * d + c] = old[i][j];     // row j becomes row j - 1
                }
#pragma unroll
            for (int j = 0; j < FUSED_TAPS; ++j)
                if (j == taps - 1) acc += k[i][j] * h;
            if (taps > 1) state[(size_t)(taps - 2) * d + c] = h;
            out[s * set_stride_out + (size_t)r * d + c] = from_f32<TO>(acc);
        }
    }
}

LCU_API int lcu_norm_conv_single(float *x, const void *delta, int delta_type, int planes, const float *w1, const float *b1,
                                 const float *w2, const float *b2, const float *cw, float *state, void *out, int out_type,
                                 const int *ctx_len, const int *state_slot, int n, int d, int taps, int sets, float eps,
                                 hipStream_t stream) {
    if (n <= 0) return LCU_OK;
    if (d <= 0 || d > 8 * NC_THREADS || taps < 1 || taps > 8 || sets < 1 || sets > 2 || !w1 || !b1 || (sets == 2 && (!w2 || !b2)) ||
        !cw || (taps > 1 && !state) || (delta && planes <= 0))
        return LCU_BAD_ARGUMENT;
    const size_t stride = (size_t)n * d;
    dim3 grid(n), block(NC_THREADS);
#define ROW(TD, TO, PT) norm_conv_single_kernel<TD, TO, PT><<<grid, block, 0, stream>>>(x, (const TD *)delta, planes, stride, w1, b1, w2, b2, cw, state, (TO *)out, stride, ctx_len, state_slot, d, taps, sets, eps)
#define GO(TD, TO)                                   \
    do {                                             \
        if (d <= 4 * NC_THREADS) ROW(TD, TO, 4);     \
        else ROW(TD, TO, 8);                         \
    } while (0)
    const int dt = delta ? delta_type : LCU_F32;
    if (dt == LCU_F32 && out_type == LCU_F32) GO(float, float);
    else if (dt == LCU_F32 && out_type == LCU_BF16) GO(float, bf16_t);
    else if (dt == LCU_BF16 && out_type == LCU_F32) GO(bf16_t, float);
    else if (dt == LCU_BF16 && out_type == LCU_BF16) GO(bf16_t, bf16_t);
    else return LCU_BAD_ARGUMENT;
#undef ROW
#undef GO
    LCU_LAUNCH_CHECK();
    return LCU_OK;
}

