// The recurrent block with a real-gated linear recurrent unit.  The mixer's product gives, per token, two branches
// of `width` channels, yin and xin (bias added here).  Then, per channel c and in 32-bit:
//
//   u   = conv_b + sum_j conv[c, j] * xin[t - taps + 1 + j]              (causal; rows before the request's start are zeros)
//   r   = sigmoid(Wa[b] u_b + ba),  i = sigmoid(Wi[b] u_b + bi)          (the channels in `blocks` equal parts, a square matrix each)
//   a   = exp(-c_exp * r * softplus(lam)),   S <- a * S + sqrt(1 - a^2) * i * u
//   out = S * gelu_tanh(yin)
//
// Per request the state is [taps, width] floats: rows 0 .. taps-2 the last taps-1 rows of xin (oldest first), row
// taps-1 the recurrence's S.  It is taken as zero where the request's first token of the step stands at position 0.
// Two kernels: the convolution with the gates (a workgroup per tile of tokens, block of channels and tile of outputs; the
// block's two matrices are given transposed, [block][in][out], so that the lanes read neighbours), and the scan (a
// thread per request and channel walks the request's tokens in their order, then leaves the state; the state is read by
// the first kernel and written by the second alone).  Everything that does not depend on the token before (the gelu of
// the y branch too) is made in the first kernel, so that the chain carries one multiply-add and one product a token.  sqrt(1 - a^2) is
// taken as sqrt(-expm1(2 log a)): no cancellation where a is close to 1.
#include "common.h"

// Where (token t, channel c) stands in the scratch arrays a, gx and y: tiles of 64 channels, each tile's tokens one after
// the other, so that the scan's wave, which owns a tile, streams one contiguous run of memory (with rows of `width`
// floats all waves would walk the same few rows at the same time, and those rows lie in few memory channels).
__device__ __forceinline__ size_t tile_index(int t, int c, int n) {
    return ((size_t)(c >> 6) * n + t) * 64 + (c & 63);
}

__device__ __forceinline__ float gelu_tanh(float z) {
    return 0.5f * z * (1.0f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
}

// xin of channel c at token t (a row of the step), or what stood `m` tokens before the step's first token of the
// request (from the state: its row taps - 1 - m; zero before the request's start).
template <class TI>
__device__ __forceinline__ float conv_at(const TI *__restrict__ rows, int row_stride, int x_off, const float *__restrict__ bias,
                                         const float *__restrict__ conv_w, const float *__restrict__ conv_b,
                                         const float *__restrict__ st, int t, int t0, int first_pos, int c, int width, int taps) {
    float acc = conv_b ? conv_b[c] : 0.f;
    const float bx = bias ? bias[x_off + c] : 0.f;
    // no branch around a load: both places are read (at indices that exist) and one value is chosen, so that the loads of
    // all taps, and of the elements that a thread makes one after the other, are in flight together
    for (int j = 0; j < taps; ++j) {
        const int back = taps - 1 - j;                       // how many tokens before t
        const bool in_step = t - back >= t0;
        const int m = in_step ? 1 : t0 - (t - back);         // else: so many tokens before the step
        const bool in_state = !in_step && first_pos - m >= 0;
        const float here = to_f32(rows[(size_t)(in_step ? t - back : t) * row_stride + x_off + c]) + bx;
        const float before = st[(size_t)(in_state ? taps - 1 - m : 0) * width + c];
        acc += conv_w[(size_t)c * taps + j] * (in_step ? here : in_state ? before : 0.f);
    }
    return acc;
}

constexpr int RG_TOK = 8;          // tokens a workgroup of the gates kernel takes
constexpr int RG_OUT = 32;         // output channels a workgroup takes
constexpr int RG_SLICES = 8;       // parts into which the sum over a block's input channels is cut (one per 32 threads)
constexpr int RG_MAX_BS = 1024;    // channels of a block (LDS holds RG_TOK rows of them)

// The convolution and the gates.  A workgroup takes RG_TOK tokens, one block of channels and RG_OUT of its outputs: it
// makes u for all the block's channels of its tokens (in LDS; workgroups of the same block make the same u), then each
// of its eight groups of 32 threads sums over an eighth of the input channels, and the eight partial sums are added in
// a fixed order.  So a decoding step, with few tokens, still has blocks x (bs / 32) workgroups.
template <class TI>
__global__ void __launch_bounds__(RG_OUT * RG_SLICES)
rglru_gates_kernel(const TI *__restrict__ rows, int row_stride, int x_off, const float *__restrict__ bias,
                   const float *__restrict__ conv_w, const float *__restrict__ conv_b, const float *__restrict__ state,
                   const float *__restrict__ wa_t, const float *__restrict__ wi_t,
                   const float *__restrict__ ba, const float *__restrict__ bi, const float *__restrict__ lam, float c_exp,
                   float *__restrict__ a_out, float *__restrict__ gx_out, float *__restrict__ y_out, int y_off,
                   const int *__restrict__ q_start,
                   const int *__restrict__ ctx_len, const int *__restrict__ req_of_token, const int *__restrict__ state_slot,
                   int n, int width, int bs, int taps) {
    __shared__ __attribute__((aligned(16))) float us[RG_TOK][RG_MAX_BS];
    __shared__ float part[RG_SLICES][RG_TOK][2][RG_OUT];
    const int b = blockIdx.y, tok0 = blockIdx.x * RG_TOK, o0 = blockIdx.z * RG_OUT;
    const int nt = min(RG_TOK, n - tok0);
#pragma unroll 4
    for (int w = threadIdx.x; w < RG_TOK * bs; w += blockDim.x) {
        const int tt = w / bs, i = w % bs;
        float u = 0.f;
        if (tt < nt) {
            const int t = tok0 + tt, r = req_of_token[t], t0 = q_start[r];
            const int first_pos = ctx_len[r] - (q_start[r + 1] - t0);
            u = conv_at(rows, row_stride, x_off, bias, conv_w, conv_b, state + (size_t)state_slot[r] * taps * width, t, t0,
                        first_pos, b * bs + i, width, taps);
        }
        us[tt][i] = u;
    }
    __syncthreads();
    const int og = threadIdx.x % RG_OUT, slice = threadIdx.x / RG_OUT, o = o0 + og;
    const int per = (bs + RG_SLICES - 1) / RG_SLICES;
    const int i0 = slice * per, i1 = min(bs, i0 + per);
    float ra[RG_TOK], ri[RG_TOK];
#pragma unroll
    for (int tt = 0; tt < RG_TOK; ++tt) ra[tt] = ri[tt] = 0.f;
    if (o < bs) {
        const float *wa = wa_t + (size_t)b * bs * bs + o, *wi = wi_t + (size_t)b * bs * bs + o;
        int i = i0;
        if (per % 4 == 0 && bs % 4 == 0) {
            for (; i + 4 <= i1; i += 4) {
                float a[4], g[4];
#pragma unroll
                for (int e = 0; e < 4; ++e) { a[e] = wa[(size_t)(i + e) * bs]; g[e] = wi[(size_t)(i + e) * bs]; }
#pragma unroll
                for (int tt = 0; tt < RG_TOK; ++tt) {
                    const float4 u = *(const float4 *)&us[tt][i];
                    ra[tt] += a[0] * u.x; ra[tt] += a[1] * u.y; ra[tt] += a[2] * u.z; ra[tt] += a[3] * u.w;
                    ri[tt] += g[0] * u.x; ri[tt] += g[1] * u.y; ri[tt] += g[2] * u.z; ri[tt] += g[3] * u.w;
                }
            }
        }
        for (; i < i1; ++i) {
            const float a = wa[(size_t)i * bs], g = wi[(size_t)i * bs];
#pragma unroll
            for (int tt = 0; tt < RG_TOK; ++tt) {
                ra[tt] += a * us[tt][i];
                ri[tt] += g * us[tt][i];
            }
        }
    }
#pragma unroll
    for (int tt = 0; tt < RG_TOK; ++tt) {
        part[slice][tt][0][og] = ra[tt];
        part[slice][tt][1][og] = ri[tt];
    }
    __syncthreads();
    const int tt = slice;                                     // eight slices, eight tokens: a thread finishes one token's channel
    if (o >= bs || tt >= nt) return;
    float sa = 0.f, si = 0.f;
#pragma unroll
    for (int k = 0; k < RG_SLICES; ++k) {
        sa += part[k][tt][0][og];
        si += part[k][tt][1][og];
    }
    const int c = b * bs + o;
    const float l = lam[c];
    const float sp = l > 20.f ? l : log1pf(expf(l));          // softplus
    const float r = 1.0f / (1.0f + expf(-(sa + ba[c])));
    const float gate = 1.0f / (1.0f + expf(-(si + bi[c])));
    const float log_a = -c_exp * r * sp;
    const float mult = sqrtf(-expm1f(2.0f * log_a));
    a_out[tile_index(tok0 + tt, c, n)] = expf(log_a);
    gx_out[tile_index(tok0 + tt, c, n)] = mult * gate * us[tt][o];
    y_out[tile_index(tok0 + tt, c, n)] = gelu_tanh(to_f32(rows[(size_t)(tok0 + tt) * row_stride + y_off + c]) + (bias ? bias[y_off + c] : 0.f));
}

constexpr int RG_BATCH = 16;       // tokens whose loads the scan has in flight at a time
constexpr int RG_RUNS = 16;        // runs into which the scan cuts a request that feeds many tokens
constexpr int RG_LONG = 512;       // from so many tokens on

// The same for many tokens: a workgroup takes RG_ROWS tokens and one block of channels, makes u once, and every thread
// sums over all input channels for its outputs, in one run (the sliced kernel adds eight partial sums: a token's gates
// differ between the two by rounding).
constexpr int RG_ROWS = 16;
constexpr int RG_FEW_ROWS = 64;    // up to so many tokens a step the sliced kernel runs (more workgroups), beyond it this one

template <class TI>
__global__ void __launch_bounds__(256)
rglru_gates_rows_kernel(const TI *__restrict__ rows, int row_stride, int x_off, const float *__restrict__ bias,
                        const float *__restrict__ conv_w, const float *__restrict__ conv_b, const float *__restrict__ state,
                        const float *__restrict__ wa_t, const float *__restrict__ wi_t,
                        const float *__restrict__ ba, const float *__restrict__ bi, const float *__restrict__ lam, float c_exp,
                        float *__restrict__ a_out, float *__restrict__ gx_out, float *__restrict__ y_out, int y_off,
                        const int *__restrict__ q_start,
                        const int *__restrict__ ctx_len, const int *__restrict__ req_of_token, const int *__restrict__ state_slot,
                        int n, int width, int bs, int taps) {
    extern __shared__ __attribute__((aligned(16))) float us_rows[];       // [RG_ROWS][bs4], bs4 = bs rounded up to 4
    const int bs4 = (bs + 3) / 4 * 4;
    const int b = blockIdx.y, tok0 = blockIdx.x * RG_ROWS;
    const int nt = min(RG_ROWS, n - tok0);
#pragma unroll 4
    for (int w = threadIdx.x; w < RG_ROWS * bs4; w += blockDim.x) {
        const int tt = w / bs4, i = w % bs4;
        float u = 0.f;
        if (tt < nt && i < bs) {
            const int t = tok0 + tt, r = req_of_token[t], t0 = q_start[r];
            const int first_pos = ctx_len[r] - (q_start[r + 1] - t0);
            u = conv_at(rows, row_stride, x_off, bias, conv_w, conv_b, state + (size_t)state_slot[r] * taps * width, t, t0,
                        first_pos, b * bs + i, width, taps);
        }
        us_rows[w] = u;
    }
    __syncthreads();
    for (int o = threadIdx.x; o < bs; o += blockDim.x) {
        const float *wa = wa_t + (size_t)b * bs * bs + o, *wi = wi_t + (size_t)b * bs * bs + o;
        float ra[RG_ROWS], ri[RG_ROWS];
#pragma unroll
        for (int tt = 0; tt < RG_ROWS; ++tt) ra[tt] = ri[tt] = 0.f;
        int i = 0;
        for (; i + 4 <= bs; i += 4) {
            float a[4], g[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) { a[e] = wa[(size_t)(i + e) * bs]; g[e] = wi[(size_t)(i + e) * bs]; }
#pragma unroll
            for (int tt = 0; tt < RG_ROWS; ++tt) {
                const float4 u = *(const float4 *)&us_rows[tt * bs4 + i];
                ra[tt] += a[0] * u.x; ra[tt] += a[1] * u.y; ra[tt] += a[2] * u.z; ra[tt] += a[3] * u.w;
                ri[tt] += g[0] * u.x; ri[tt] += g[1] * u.y; ri[tt] += g[2] * u.z; ri[tt] += g[3] * u.w;
            }
        }
        for (; i < bs; ++i) {
            const float a = wa[(size_t)i * bs], g = wi[(size_t)i * bs];
#pragma unroll
            for (int tt = 0; tt < RG_ROWS; ++tt) {
                ra[tt] += a * us_rows[tt * bs4 + i];
                ri[tt] += g * us_rows[tt * bs4 + i];
            }
        }
        const int c = b * bs + o;
        const float l = lam[c];
        const float sp = l > 20.f ? l : log1pf(expf(l));          // softplus
        const float bias_a = ba[c], bias_i = bi[c];
#pragma unroll
        for (int tt = 0; tt < RG_ROWS; ++tt) {
            if (tt < nt) {
                const float r = 1.0f / (1.0f + expf(-(ra[tt] + bias_a)));
                const float gate = 1.0f / (1.0f + expf(-(ri[tt] + bias_i)));
                const float log_a = -c_exp * r * sp;
                const float mult = sqrtf(-expm1f(2.0f * log_a));
                a_out[tile_index(tok0 + tt, c, n)] = expf(log_a);
                gx_out[tile_index(tok0 + tt, c, n)] = mult * gate * us_rows[tt * bs4 + o];
                y_out[tile_index(tok0 + tt, c, n)] = gelu_tanh(to_f32(rows[(size_t)(tok0 + tt) * row_stride + y_off + c]) + (bias ? bias[y_off + c] : 0.f));
            }
        }
    }
}

// The recurrence over [s0, s1) from S, in the tokens' order; with WRITE the outputs too.  RG_BATCH tokens at a time: their
// loads go out together.  prod (if not null) receives the product of the decays.
template <class T, bool WRITE>
__device__ __forceinline__ float scan_run(const float *__restrict__ a, const float *__restrict__ gx, const float *__restrict__ y,
                                          T *__restrict__ out, int s0, int s1, int c, int n, int width, float S, float *prod) {
    float P = 1.f;
    int t = s0;
    for (; t + RG_BATCH <= s1; t += RG_BATCH) {
        float av[RG_BATCH], gv[RG_BATCH], yv[RG_BATCH];
#pragma unroll
        for (int e = 0; e < RG_BATCH; ++e) {
            av[e] = a[tile_index(t + e, c, n)];
            gv[e] = gx[tile_index(t + e, c, n)];
            if (WRITE) yv[e] = y[tile_index(t + e, c, n)];
        }
#pragma unroll
        for (int e = 0; e < RG_BATCH; ++e) {
            S = av[e] * S + gv[e];
            if (WRITE) out[(size_t)(t + e) * width + c] = from_f32<T>(S * yv[e]);
            else P *= av[e];
        }
    }
    for (; t < s1; ++t) {
        const float av = a[tile_index(t, c, n)];
        S = av * S + gx[tile_index(t, c, n)];
        if (WRITE) out[(size_t)t * width + c] = from_f32<T>(S * y[tile_index(t, c, n)]);
        else P *= av;
    }
    if (prod) *prod = P;
    return S;
}

// NSEG 1: a wave per 64 channels walks the request's tokens in their order.  NSEG > 1, for a request that feeds many
// tokens: the tokens are cut into NSEG runs, a wave each; every wave first walks its run from zero, which gives the run's
// effect on whatever state it starts from (S_end = P * S_start + B); then the runs' effects are chained, in order; then
// every wave walks its run again from its true start and writes.  (The recurrence is the same; the sums are made in
// another order, so the results differ from NSEG = 1 by rounding.)
template <class TI, class T, int NSEG>
__global__ void __launch_bounds__(64 * NSEG)
rglru_scan_kernel(const TI *__restrict__ rows, int row_stride, int y_off, int x_off, const float *__restrict__ bias,
                  const float *__restrict__ a, const float *__restrict__ gx, const float *__restrict__ y, float *__restrict__ state,
                  T *__restrict__ out, const int *__restrict__ q_start, const int *__restrict__ ctx_len,
                  const int *__restrict__ state_slot, int n, int width, int taps, int min_tokens) {
    __shared__ float eff[NSEG][2][64];
    const int r = blockIdx.y, lane = threadIdx.x % 64, seg = threadIdx.x / 64;
    const int c = blockIdx.x * 64 + lane;
    const int t0 = q_start[r], t1 = q_start[r + 1];
    // (a kernel of several runs leaves requests with few tokens to the kernel of one, and the other way round)
    if (t1 <= t0 || (NSEG > 1) != (t1 - t0 >= min_tokens)) return;
    const bool live = c < width;
    const int first_pos = ctx_len[r] - (t1 - t0);
    float *st = state + (size_t)state_slot[r] * taps * width;
    float S = (live && first_pos > 0) ? st[(size_t)(taps - 1) * width + c] : 0.f;
    if (NSEG == 1) {
        if (!live) return;
        S = scan_run<T, true>(a, gx, y, out, t0, t1, c, n, width, S, nullptr);
    } else {
        const int len = (t1 - t0 + NSEG - 1) / NSEG;
        const int s0 = min(t1, t0 + seg * len), s1 = min(t1, s0 + len);
        float P = 1.f, B = 0.f;
        if (live) B = scan_run<T, false>(a, gx, y, out, s0, s1, c, n, width, 0.f, &P);
        eff[seg][0][lane] = P;
        eff[seg][1][lane] = B;
        __syncthreads();
        for (int k = 0; k < seg; ++k) S = eff[k][0][lane] * S + eff[k][1][lane];
        if (!live) return;
        S = scan_run<T, true>(a, gx, y, out, s0, s1, c, n, width, S, nullptr);
        if (seg != NSEG - 1) return;                          // the last run's end is the request's
    }
    st[(size_t)(taps - 1) * width + c] = S;
    // the convolution's state: the last taps - 1 rows of xin, oldest first; where the step brought fewer, older rows move up
    const int q = t1 - t0;
    const float bx = bias ? bias[x_off + c] : 0.f;
    float keep[16];
    for (int k = 0; k < taps - 1; ++k) {
        const int back = taps - 1 - k;                           // row k is the one `back` tokens before the request's end
        float x = 0.f;
        if (back <= q) x = to_f32(rows[(size_t)(t1 - back) * row_stride + x_off + c]) + bx;
        else if (first_pos > 0) {
            const int old = k + q;                               // where that row stands in the state as the step found it
            if (old < taps - 1 && first_pos - (back - q) >= 0) x = st[(size_t)old * width + c];
        }
        keep[k] = x;
    }
    for (int k = 0; k < taps - 1; ++k) st[(size_t)k * width + c] = keep[k];
}

// rows: [n, row_stride] of in_type, yin at y_off and xin at x_off (width each); bias: null or float32 over the row's
// columns.  conv_w [width, taps], conv_b [width] (may be null), wa_t / wi_t [blocks, bs, bs] transposed ([in][out]),
// ba / bi / lam [width], all float32.  state: float32 [slots, taps, width].  a, gx, y: float32 scratch of n * (width rounded up to 64) floats each.
// out: [n, width] of out_type.
LCU_API int lcu_rglru(const void *rows, int in_type, int row_stride, int y_off, int x_off, const float *bias,
                      const float *conv_w, const float *conv_b, const float *wa_t, const float *wi_t, const float *ba,
                      const float *bi, const float *lam, float c_exp, float *state, float *a, float *gx, float *y, void *out,
                      int out_type, const int *q_start, const int *ctx_len, const int *req_of_token, const int *state_slot,
                      int n, int n_req, int width, int blocks, int taps, hipStream_t stream) {
    if (n <= 0 || n_req <= 0) return LCU_OK;
    if (width <= 0 || blocks <= 0 || width % blocks || width / blocks > RG_MAX_BS || taps < 1 || taps > 16 || n_req > 65535 ||
        !rows || !conv_w || !wa_t || !wi_t || !ba || !bi || !lam || !state || !a || !gx || !y || !out)
        return LCU_BAD_ARGUMENT;
    const int bs = width / blocks;
    if (n > RG_FEW_ROWS) {
        const int bs4 = (bs + 3) / 4 * 4;
        dim3 grid((n + RG_ROWS - 1) / RG_ROWS, blocks), block(bs >= 256 ? 256 : (bs + 63) / 64 * 64);
        const size_t lds = (size_t)RG_ROWS * bs4 * sizeof(float);
        if (in_type == LCU_F32)
            rglru_gates_rows_kernel<float><<<grid, block, lds, stream>>>((const float *)rows, row_stride, x_off, bias, conv_w, conv_b, state, wa_t, wi_t, ba, bi, lam, c_exp, a, gx, y, y_off, q_start, ctx_len, req_of_token, state_slot, n, width, bs, taps);
        else if (in_type == LCU_BF16)
            rglru_gates_rows_kernel<bf16_t><<<grid, block, lds, stream>>>((const bf16_t *)rows, row_stride, x_off, bias, conv_w, conv_b, state, wa_t, wi_t, ba, bi, lam, c_exp, a, gx, y, y_off, q_start, ctx_len, req_of_token, state_slot, n, width, bs, taps);
        else
            return LCU_BAD_ARGUMENT;
        LCU_LAUNCH_CHECK();
    } else {
        dim3 grid((n + RG_TOK - 1) / RG_TOK, blocks, (bs + RG_OUT - 1) / RG_OUT), block(RG_OUT * RG_SLICES);
        if (in_type == LCU_F32)
            rglru_gates_kernel<float><<<grid, block, 0, stream>>>((const float *)rows, row_stride, x_off, bias, conv_w, conv_b, state, wa_t, wi_t, ba, bi, lam, c_exp, a, gx, y, y_off, q_start, ctx_len, req_of_token, state_slot, n, width, bs, taps);
        else if (in_type == LCU_BF16)
            rglru_gates_kernel<bf16_t><<<grid, block, 0, stream>>>((const bf16_t *)rows, row_stride, x_off, bias, conv_w, conv_b, state, wa_t, wi_t, ba, bi, lam, c_exp, a, gx, y, y_off, q_start, ctx_len, req_of_token, state_slot, n, width, bs, taps);
        else
            return LCU_BAD_ARGUMENT;
        LCU_LAUNCH_CHECK();
    }
    {
        // two launches: requests that feed many tokens (if the step's size allows any) are cut into runs, the others not
        dim3 grid((width + 63) / 64, n_req);
#define GO(TI, T) do { rglru_scan_kernel<TI, T, 1><<<grid, dim3(64), 0, stream>>>((const TI *)rows, row_stride, y_off, x_off, bias, a, gx, y, state, (T *)out, q_start, ctx_len, state_slot, n, width, taps, RG_LONG); \
                       if (n >= RG_LONG) rglru_scan_kernel<TI, T, RG_RUNS><<<grid, dim3(64 * RG_RUNS), 0, stream>>>((const TI *)rows, row_stride, y_off, x_off, bias, a, gx, y, state, (T *)out, q_start, ctx_len, state_slot, n, width, taps, RG_LONG); } while (0)
        if (in_type == LCU_F32 && out_type == LCU_F32) GO(float, float);
        else if (in_type == LCU_F32 && out_type == LCU_BF16) GO(float, bf16_t);
        else if (in_type == LCU_BF16 && out_type == LCU_BF16) GO(bf16_t, bf16_t);
        else return LCU_BAD_ARGUMENT;
#undef GO
        LCU_LAUNCH_CHECK();
    }
    return LCU_OK;
}
