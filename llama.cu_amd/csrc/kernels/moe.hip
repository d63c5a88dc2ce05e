// A feed-forward of many small experts of which each token uses a few.
//
//   route:   z = W_router h (32-bit), the `top` experts with the largest z (ties: the lower
//            index), each with the weight sigmoid(z) (not renormalised);
//   group:   the (token, choice) pairs sorted by expert and cut into tiles of 64 rows of one
//            expert, on the device (nothing comes back to the host);
//   up:      act = gelu(W_up[e] (weight * h))    the weight multiplies the expert's INPUT
//   down:    y = W_down[e] act, added to the token's output row (32-bit).
// The products run on the matrix cores: bfloat16 operands with v_mfma_f32_16x16x32_bf16, or
// true 32-bit with v_mfma_f32_16x16x4_f32; sums are 32-bit.  A row's result depends on that
// row and its expert alone (never on which rows share its tile), so it does not depend on
// the batch.
#include "common.h"

constexpr int MOE_MAX_EXPERTS = 1024;
constexpr int MOE_TILE_ROWS = 64;

typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;

// ---------------------------------------------------------------- route
// One block of 256 threads per token.  h: [n, d] of T; router: [experts, d] 32-bit.
// ids, wts: [n, top].
template <class T>
__global__ void __launch_bounds__(256)
moe_route_kernel(const T *__restrict__ h, const float *__restrict__ router, int *__restrict__ ids,
                 float *__restrict__ wts, int d, int experts, int top) {
    __shared__ float z[MOE_MAX_EXPERTS];
    const int t = blockIdx.x, wave = threadIdx.x / WAVE, lane = threadIdx.x % WAVE;
    const T *row = h + (size_t)t * d;
    for (int e = wave; e < experts; e += 256 / WAVE) {
        const float *w = router + (size_t)e * d;
        float acc = 0.f;
        for (int c = lane; c < d; c += WAVE) acc += to_f32(row[c]) * w[c];
        acc = wave_sum(acc);
        if (lane == 0) z[e] = acc;
    }
    __syncthreads();
    for (int k = 0; k < top; ++k) {                  // the first wave chooses; the others only keep the barriers
        if (wave == 0) {
        float best = -INFINITY;
        int arg = 0x7fffffff;
        for (int e = lane; e < experts; e += WAVE) {
            const float v = z[e];
            if (v > best || (v == best && e < arg)) { best = v; arg = e; }
        }
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) {
            const float ob = __shfl_xor(best, off, WAVE);
            const int oa = __shfl_xor(arg, off, WAVE);
            if (ob > best || (ob == best && oa < arg)) { best = ob; arg = oa; }
        }
        if (arg >= experts) arg = 0;                 // every logit NaN: any expert
        if (lane == 0) {
            ids[(size_t)t * top + k] = arg;
            wts[(size_t)t * top + k] = 1.0f / (1.0f + expf(-z[arg]));
            z[arg] = -INFINITY;
        }
        }
        __syncthreads();
    }
}

// ---------------------------------------------------------------- group
// One block.  ids: [total] experts of the (token, choice) pairs in flat order.  Writes
// sorted_to_flat [total] (the pairs sorted by expert), and the tiles: tile_expert, tile_begin
// (first sorted row), tile_rows, each [max_tiles], and n_tiles [1].
__global__ void __launch_bounds__(1024)
moe_group_kernel(const int *__restrict__ ids, int total, int experts, int *__restrict__ sorted_to_flat,
                 int *__restrict__ tile_expert, int *__restrict__ tile_begin, int *__restrict__ tile_rows,
                 int *__restrict__ n_tiles, int max_tiles) {
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
            for (int r = 0; r < count[e] && tiles < max_tiles; r += MOE_TILE_ROWS) {
                tile_expert[tiles] = e;
                tile_begin[tiles] = at + r;
                tile_rows[tiles] = count[e] - r < MOE_TILE_ROWS ? count[e] - r : MOE_TILE_ROWS;
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

enum { MOE_UP = 0, MOE_DOWN = 1 };

// A block of four waves takes one tile (up to 64 sorted rows of one expert) and 64 output
// features, a wave 16 of the features for all rows.  The weight is the instruction's first
// operand (16 features x k), the rows the second (k x 16 rows): a lane then holds four
// neighbouring features of one row.
//   MOE_UP:   x = h [n, K], row = token of the pair, scaled by the pair's weight; out_t = act
//             [total, N] at the sorted row, gelu applied.
//   MOE_DOWN: x = act [total, K] at the sorted row; out_f [total or n, N] 32-bit at the flat pair
//             (add == 0: stored) or at the pair's token (add == 1: added; only with top == 1).
template <class T, int MODE>
__global__ void __launch_bounds__(256)
moe_gemm_kernel(const T *__restrict__ x, int x_stride, const T *__restrict__ w, size_t w_expert_stride, int N, int K,
                const int *__restrict__ sorted_to_flat, const float *__restrict__ wts,
                const int *__restrict__ tile_expert, const int *__restrict__ tile_begin,
                const int *__restrict__ tile_rows, const int *__restrict__ n_tiles, T *__restrict__ out_t,
                float *__restrict__ out_f, int out_stride, int top, int add) {
    typedef Mma<T> M;
    const int tile = blockIdx.x;
    if (tile >= n_tiles[0]) return;
    const int wave = threadIdx.x / WAVE, lane = threadIdx.x % WAVE, g = lane / 16, l16 = lane % 16;
    const int f0 = blockIdx.y * 64 + wave * 16;
    if (f0 >= N) return;
    const int e = tile_expert[tile], row0 = tile_begin[tile], rows = tile_rows[tile];
    const int f = f0 + l16;
    const T *wrow = w + (size_t)e * w_expert_stride + (size_t)(f < N ? f : N - 1) * K;
    const T *xrow[4];
    float sc[4];
    int dst[4];
    bool valid[4];
#pragma unroll
    for (int m = 0; m < 4; ++m) {
        valid[m] = 16 * m + l16 < rows;
        const int srow = row0 + (valid[m] ? 16 * m + l16 : 0);
        const int flat = sorted_to_flat[srow];
        sc[m] = 1.f;
        if (MODE == MOE_UP) {
            xrow[m] = x + (size_t)(flat / top) * x_stride;
            sc[m] = wts[flat];
            dst[m] = srow;
        } else {
            xrow[m] = x + (size_t)srow * x_stride;
            dst[m] = add ? flat / top : flat;
        }
    }
    f32x4 acc[4];
#pragma unroll
    for (int m = 0; m < 4; ++m) acc[m] = f32x4{0.f, 0.f, 0.f, 0.f};

    for (int k0 = 0; k0 < K; k0 += M::KSTEP) {
        const int kk = k0 + g * M::PER_LANE;
        const bool in = kk < K;
        const typename M::frag a = (in && f < N) ? M::load(wrow + kk) : M::zero();
#pragma unroll
        for (int m = 0; m < 4; ++m) {
            if (16 * m < rows) {
                typename M::frag b = (in && valid[m]) ? M::load(xrow[m] + kk) : M::zero();
                if (MODE == MOE_UP) b = M::scaled(b, sc[m]);
                acc[m] = M::mma(a, b, acc[m]);
            }
        }
    }
#pragma unroll
    for (int m = 0; m < 4; ++m) {
        if (!valid[m]) continue;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int col = f0 + 4 * g + i;
            if (col >= N) continue;
            if (MODE == MOE_UP) {
                out_t[(size_t)dst[m] * out_stride + col] = from_f32<T>(gelu_erf(acc[m][i]));
            } else {
                float *o = out_f + (size_t)dst[m] * out_stride + col;
                *o = add ? *o + acc[m][i] : acc[m][i];
            }
        }
    }
}

// out[t, c] += sum_k y[t * top + k, c]  (in the order of k)
__global__ void moe_combine_kernel(float *__restrict__ out, const float *__restrict__ y, int n, int d, int top) {
    const int c = blockIdx.x * blockDim.x + threadIdx.x;
    if (c >= d) return;
    for (size_t t = blockIdx.y; t < (size_t)n; t += gridDim.y) {
        float acc = out[t * d + c];
        for (int k = 0; k < top; ++k) acc += y[(t * top + k) * d + c];
        out[t * d + c] = acc;
    }
}

LCU_API int lcu_moe_tile_rows() { return MOE_TILE_ROWS; }

// h: [n, d] of `type`; router: [experts, d] 32-bit; ids, wts: [n * top].
LCU_API int lcu_moe_route(const void *h, int type, const float *router, int *ids, float *wts, int n, int d, int experts,
                          int top, hipStream_t stream) {
    if (n <= 0) return LCU_OK;
    if (d <= 0 || experts <= 0 || experts > MOE_MAX_EXPERTS || top <= 0 || top > experts) return LCU_BAD_ARGUMENT;
    if (type == LCU_F32) moe_route_kernel<float><<<dim3(n), dim3(256), 0, stream>>>((const float *)h, router, ids, wts, d, experts, top);
    else if (type == LCU_BF16) moe_route_kernel<bf16_t><<<dim3(n), dim3(256), 0, stream>>>((const bf16_t *)h, router, ids, wts, d, experts, top);
    else return LCU_BAD_ARGUMENT;
    LCU_LAUNCH_CHECK();
    return LCU_OK;
}

// ints: scratch of total + 3 * max_tiles + 1 entries, laid out as sorted_to_flat, tile_expert, tile_begin,
// tile_rows, n_tiles.
// w_up: [experts, ff, d], w_down: [experts, d, ff] of `type`.  act: scratch [total, ff] of `type`; y: scratch
// [total, d] 32-bit (only read and written when top > 1).  out: [n, d] 32-bit, added to.
LCU_API int lcu_moe_experts(const void *h, int type, const int *ids, const float *wts, int *ints, int max_tiles,
                            const void *w_up, const void *w_down, void *act, float *y, float *out, int n, int d, int ff,
                            int experts, int top, hipStream_t stream) {
    if (n <= 0) return LCU_OK;
    const int per = type == LCU_BF16 ? 8 : 4;
    if (d <= 0 || ff <= 0 || d % per || ff % per || experts <= 0 || experts > MOE_MAX_EXPERTS || top <= 0 || max_tiles <= 0 ||
        (type != LCU_F32 && type != LCU_BF16))
        return LCU_BAD_ARGUMENT;
    const int total = n * top;
    int *sorted = ints, *t_exp = ints + total, *t_beg = t_exp + max_tiles, *t_rows = t_beg + max_tiles, *n_tiles = t_rows + max_tiles;
    moe_group_kernel<<<dim3(1), dim3(1024), 0, stream>>>(ids, total, experts, sorted, t_exp, t_beg, t_rows, n_tiles, max_tiles);
    LCU_LAUNCH_CHECK();
    const int add = top == 1;
    float *down_to = add ? out : y;
    dim3 block(256), gu(max_tiles, (ff + 63) / 64), gd(max_tiles, (d + 63) / 64);
    if (type == LCU_BF16) {
        moe_gemm_kernel<bf16_t, MOE_UP><<<gu, block, 0, stream>>>((const bf16_t *)h, d, (const bf16_t *)w_up, (size_t)ff * d, ff, d, sorted, wts, t_exp, t_beg, t_rows, n_tiles, (bf16_t *)act, nullptr, ff, top, 0);
        moe_gemm_kernel<bf16_t, MOE_DOWN><<<gd, block, 0, stream>>>((const bf16_t *)act, ff, (const bf16_t *)w_down, (size_t)ff * d, d, ff, sorted, wts, t_exp, t_beg, t_rows, n_tiles, nullptr, down_to, d, top, add);
    } else {
        moe_gemm_kernel<float, MOE_UP><<<gu, block, 0, stream>>>((const float *)h, d, (const float *)w_up, (size_t)ff * d, ff, d, sorted, wts, t_exp, t_beg, t_rows, n_tiles, (float *)act, nullptr, ff, top, 0);
        moe_gemm_kernel<float, MOE_DOWN><<<gd, block, 0, stream>>>((const float *)act, ff, (const float *)w_down, (size_t)ff * d, d, ff, sorted, wts, t_exp, t_beg, t_rows, n_tiles, nullptr, down_to, d, top, add);
    }
    LCU_LAUNCH_CHECK();
    if (!add) {
        moe_combine_kernel<<<dim3((d + 255) / 256, n < 65535 ? n : 65535), dim3(256), 0, stream>>>(out, y, n, d, top);
        LCU_LAUNCH_CHECK();
    }
    return LCU_OK;
}
