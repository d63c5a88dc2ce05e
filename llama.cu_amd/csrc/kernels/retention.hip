// Retention: linear attention with a fixed decay per head, no softmax and no denominator.  Per head, with key
// channels i and value channels j, a state S [d, dv] in 32-bit:
//
//   q, k <- the first rot_dim dims turned by the angle of the token's position (tables; pairing as in the
//           attention's rotation), k then times k_scale
//   S <- decay[h] * S + k v^T          o = S^T q
//
// The scan: a request's tokens are one chain, but column j of S depends on column j alone, so a workgroup takes a
// tile of 16 columns of one head of one request and keeps them in registers from the request's first token of the
// step to its last: sixteen lanes a column, each with a sixteenth of the key channels; the sum over key channels crosses
// the sixteen lanes after a stage's last token.  q and k are rotated by a parallel kernel first (32-bit); they and v go through
// LDS, a stage of tokens at a time, the next stage on its way while the waves work through this one.  The state
// is taken as zero where the request's first token of the step stands at position 0, and is left as the step's
// last token makes it.  The order of every sum depends on d alone: however a prompt is cut into steps, the same
// bits come out.
//
// o is written [head][tile of 16 columns][token][16].  The output: each head's o divided by its root mean square (eps, no weight), times silu(gate) (second kernel).
#include "common.h"

constexpr int RT_THREADS = 256;
constexpr int RT_LANES = 16;                      // lanes that share a column
constexpr int RT_COLS = RT_THREADS / RT_LANES;    // columns a workgroup

// Moves between the lanes of a group of sixteen inside the vector unit (no trip through LDS): the neighbour, the lane two
// away, the mirror image within eight and within sixteen.  After the first two every lane of a quad holds the quad's sum,
// so the mirror image within eight brings the other quad's, and the one within sixteen the other eight's.
__device__ __forceinline__ float lane_xor1(float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, v), 0xB1, 0xF, 0xF, true));     // quad_perm [1, 0, 3, 2]
}
__device__ __forceinline__ float lane_xor2(float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, v), 0x4E, 0xF, 0xF, true));     // quad_perm [2, 3, 0, 1]
}
__device__ __forceinline__ float lane_mirror8(float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, v), 0x141, 0xF, 0xF, true));    // row_half_mirror
}

__device__ __forceinline__ float lane_mirror16(float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, v), 0x140, 0xF, 0xF, true));    // row_mirror
}

// q and k of every (token, head), rotated, k scaled, and v, 32-bit: qkv [nh][n][2 d + dv], a head's tokens one after the
// other, so that the scan's workgroups, which own a head, each stream a run of memory of their own (with rows of all
// heads every workgroup would walk the same few rows at the same time, and those lie in few memory channels).
template <class TI>
__global__ void __launch_bounds__(256)
retention_prep_kernel(const TI *__restrict__ rows, int row_stride, int q_off, int k_off, int v_off, const int *__restrict__ positions,
                      const float *__restrict__ cos_t, const float *__restrict__ sin_t, int max_pos, int rot_dim, int pairing,
                      float k_scale, float *__restrict__ qk, int n, int nh, int d, int dv) {
    const int t = blockIdx.x;
    const TI *row = rows + (size_t)t * row_stride;
    const int half = rot_dim / 2;
    const int pos = cos_t ? positions[t] : 0;
    for (int w = blockIdx.y * blockDim.x + threadIdx.x; w < nh * d; w += gridDim.y * blockDim.x) {
        const int h = w / d, i = w % d;
        float qv = to_f32(row[q_off + w]), kv = to_f32(row[k_off + w]);
        if (cos_t && i < rot_dim) {
            int pi, partner;
            bool first;                                   // whether i is the pair's first dim
            if (pairing == 0) { first = i < half; pi = first ? i : i - half; partner = first ? i + half : i - half; }
            else { first = (i & 1) == 0; pi = i >> 1; partner = i ^ 1; }
            const float qp = to_f32(row[q_off + h * d + partner]), kp = to_f32(row[k_off + h * d + partner]);
            float c = __uint_as_float(0x7fc00000u), sn = c;        // a position outside the table gives NaN
            if (pos >= 0 && pos < max_pos) { c = cos_t[(size_t)pos * half + pi]; sn = sin_t[(size_t)pos * half + pi]; }
            float ra, rb;
            if (first) { rotate_pair(qv, qp, c, sn, ra, rb); qv = ra; rotate_pair(kv, kp, c, sn, ra, rb); kv = ra; }
            else { rotate_pair(qp, qv, c, sn, ra, rb); qv = rb; rotate_pair(kp, kv, c, sn, ra, rb); kv = rb; }
        }
        float *o = qk + ((size_t)h * n + t) * (2 * d + dv);
        o[i] = qv;
        o[d + i] = kv * k_scale;
    }
    for (int w = blockIdx.y * blockDim.x + threadIdx.x; w < nh * dv; w += gridDim.y * blockDim.x)
        qk[((size_t)(w / dv) * n + t) * (2 * d + dv) + 2 * d + w % dv] = to_f32(row[v_off + w]);
}

// The scan.  DPL: key channels per lane (d <= 16 * DPL), a lane's channels neighbours; TOK: tokens staged at a time.  Two
// buffers in LDS: while the waves work through one, every thread holds the next tokens' share in registers (loaded
// before the work began) and writes it into the other afterwards: one barrier a stage.
//
// MODE 0: a request's tokens of the step in one chain (requests that feed fewer than RT_LONG tokens).  A request that
// feeds more is cut into RT_RUNS runs that are walked at once, twice: MODE 1 walks each run from a state of zeros and
// leaves the run's own sum B (S_end = decay^len * S_start + B) in run_b; retention_chain_kernel then gives every run the
// state it really starts from (run_in); MODE 2 walks the runs again from there and writes the outputs, the last run the
// request's state.  (The same recurrence with its sums in another order: the results differ from one chain by rounding.)
constexpr int RT_RUNS = 8;
constexpr int RT_LONG = 512;

// how many of the requests before r feed at least RT_LONG tokens: r's place among those in run_b and run_in
__device__ __forceinline__ int long_index(const int *__restrict__ q_start, int r) {
    int li = 0;
    for (int i = 0; i < r; ++i) li += (q_start[i + 1] - q_start[i] >= RT_LONG);
    return li;
}

template <int DPL, int TOK, int MODE>
__global__ void __launch_bounds__(RT_THREADS)
retention_scan_kernel(const float *__restrict__ qk,
                      const float *__restrict__ decay, float *__restrict__ state, float *__restrict__ o_out,
                      const int *__restrict__ q_start, const int *__restrict__ ctx_len, const int *__restrict__ state_slot,
                      float *__restrict__ run_b, const float *__restrict__ run_in, int n, int nh, int d, int dv) {
    constexpr int D = RT_LANES * DPL;
    constexpr int STAGE = TOK * (2 * D + RT_COLS);                 // floats of a stage: per token q, k, and the tile of v
    constexpr int PER = (STAGE + RT_THREADS - 1) / RT_THREADS;     // of which a thread moves so many
    __shared__ __attribute__((aligned(16))) float lds[2][STAGE];
    const int r = MODE == 0 ? blockIdx.z : blockIdx.z / RT_RUNS, run = MODE == 0 ? 0 : blockIdx.z % RT_RUNS;
    const int h = blockIdx.y, col0 = blockIdx.x * RT_COLS;
    int t0 = q_start[r], t1 = q_start[r + 1];
    if (t1 <= t0 || (MODE != 0) != (t1 - t0 >= RT_LONG)) return;
    const int first_pos = ctx_len[r] - (t1 - t0);
    const int sub = threadIdx.x % RT_LANES, cg = threadIdx.x / RT_LANES, col = col0 + cg;
    const bool live = col < dv;
    float *S = state + ((size_t)state_slot[r] * nh + h) * (size_t)d * dv;
    size_t run_at = 0;
    if (MODE != 0) {
        const int len = (t1 - t0 + RT_RUNS - 1) / RT_RUNS, end = t1;
        t0 = min(end, t0 + run * len);
        t1 = min(end, t0 + len);
        run_at = (((size_t)long_index(q_start, r) * RT_RUNS + run) * nh + h) * (size_t)d * dv;
    }
    const float g = decay[h];
    // the tile of the state goes through LDS (the stages' memory, not yet in use): sixteen lanes read the sixteen
    // neighbouring columns of a row of the state, where the lanes' own elements lie a row apart
    float s[DPL];
    const float *from = MODE == 0 ? (first_pos > 0 ? S : nullptr) : MODE == 2 ? run_in + run_at : nullptr;
    float *tile = &lds[0][0];                                  // [D][RT_COLS + 1]
    if (from) {
        for (int w = threadIdx.x; w < D * RT_COLS; w += RT_THREADS) {
            const int i = w / RT_COLS, c = w % RT_COLS;
            tile[i * (RT_COLS + 1) + c] = (i < d && col0 + c < dv) ? from[(size_t)i * dv + col0 + c] : 0.f;
        }
        __syncthreads();
    }
#pragma unroll
    for (int e = 0; e < DPL; ++e) s[e] = from ? tile[(sub * DPL + e) * (RT_COLS + 1) + cg] : 0.f;
    __syncthreads();
    // element w of a stage: token w / (2D + COLS); within it [0, 2D): q then k (dims beyond d zeros), then the v tile
    auto fetch = [&](int base, int w) -> float {
        const int tt = w / (2 * D + RT_COLS), x = w % (2 * D + RT_COLS), t = base + tt;
        if (w >= STAGE || t >= t1) return 0.f;
        const float *src = qk + ((size_t)h * n + t) * (2 * d + dv);
        if (x < 2 * D) {
            const int which = x / D, i = x % D;
            return i < d ? src[which * d + i] : 0.f;
        }
        const int c = col0 + x - 2 * D;
        return c < dv ? src[2 * d + c] : 0.f;
    };
    float next[PER];
#pragma unroll
    for (int k = 0; k < PER; ++k) next[k] = fetch(t0, threadIdx.x + k * RT_THREADS);
#pragma unroll
    for (int k = 0; k < PER; ++k)
        if (threadIdx.x + k * RT_THREADS < STAGE) lds[0][threadIdx.x + k * RT_THREADS] = next[k];
    __syncthreads();
    int buf = 0;
    for (int base = t0; base < t1; base += TOK, buf ^= 1) {
        const int nt = min(TOK, t1 - base);
        const bool more = base + TOK < t1;
        if (more) {
#pragma unroll
            for (int k = 0; k < PER; ++k) next[k] = fetch(base + TOK, threadIdx.x + k * RT_THREADS);
        }
        const float *cur = lds[buf];
        // the stage's tokens one after the other; each token's sum over the key channels is left in eight lanes' shares
        // and crosses the lanes after the stage's last token, all tokens' at once (nothing in the chain waits for it)
        float acc[TOK];
#pragma unroll
        for (int tt = 0; tt < TOK; ++tt) {
            // (no branch around a token: beyond the request's last one k and v are zeros and the decay is 1, which leaves S)
            const float gt = tt < nt ? g : 1.0f;
            const float *qs = cur + tt * (2 * D + RT_COLS), *ks = qs + D;
            const float v = qs[2 * D + cg];
            acc[tt] = 0.f;
#pragma unroll
            for (int e4 = 0; e4 < DPL / 4; ++e4) {
                const float4 k4 = *(const float4 *)(ks + sub * DPL + 4 * e4), q4 = *(const float4 *)(qs + sub * DPL + 4 * e4);
                s[4 * e4 + 0] = gt * s[4 * e4 + 0] + k4.x * v; acc[tt] += s[4 * e4 + 0] * q4.x;
                s[4 * e4 + 1] = gt * s[4 * e4 + 1] + k4.y * v; acc[tt] += s[4 * e4 + 1] * q4.y;
                s[4 * e4 + 2] = gt * s[4 * e4 + 2] + k4.z * v; acc[tt] += s[4 * e4 + 2] * q4.z;
                s[4 * e4 + 3] = gt * s[4 * e4 + 3] + k4.w * v; acc[tt] += s[4 * e4 + 3] * q4.w;
            }
        }
        // after the moves every lane of a column's sixteen holds the token's sum: lane `tt` of them keeps token tt's, and
        // the stage's outputs leave in one store (o is laid out [head][tile of 16 columns][token][16]: a workgroup's
        // stage is one run of memory)
        float mine = 0.f;
#pragma unroll
        for (int tt = 0; tt < TOK; ++tt) {
            float a = acc[tt];
            a += lane_xor1(a);
            a += lane_xor2(a);
            a += lane_mirror8(a);
            a += lane_mirror16(a);
            if (sub == tt) mine = a;
        }
        if (MODE != 1 && sub < nt && live)
            o_out[(((size_t)h * gridDim.x + blockIdx.x) * n + base + sub) * RT_COLS + cg] = mine;
        if (more) {
#pragma unroll
            for (int k = 0; k < PER; ++k)
                if (threadIdx.x + k * RT_THREADS < STAGE) lds[buf ^ 1][threadIdx.x + k * RT_THREADS] = next[k];
        }
        __syncthreads();
    }
    if (MODE == 2 && run != RT_RUNS - 1) return;              // the last run's end is the request's
    {
        float *dst = MODE == 1 ? run_b + run_at : S;
        float *tile = &lds[0][0];                              // (the last stage's barrier is behind every wave)
#pragma unroll
        for (int e = 0; e < DPL; ++e) tile[(sub * DPL + e) * (RT_COLS + 1) + cg] = s[e];
        __syncthreads();
        for (int w = threadIdx.x; w < D * RT_COLS; w += RT_THREADS) {
            const int i = w / RT_COLS, c = w % RT_COLS;
            if (i < d && col0 + c < dv) dst[(size_t)i * dv + col0 + c] = tile[i * (RT_COLS + 1) + c];
        }
    }
}

// The state that every run of a long request starts from: run 0 from the request's state (zeros at position 0), run k + 1
// from decay^len_k * (run k's start) + (run k's own sum).  A workgroup per (request, head), a thread per element.
__global__ void retention_chain_kernel(const float *__restrict__ decay, const float *__restrict__ state, const float *__restrict__ run_b,
                                       float *__restrict__ run_in, const int *__restrict__ q_start, const int *__restrict__ ctx_len,
                                       const int *__restrict__ state_slot, int nh, int d, int dv) {
    const int r = blockIdx.y, h = blockIdx.x;
    const int t0 = q_start[r], t1 = q_start[r + 1], q = t1 - t0;
    if (q < RT_LONG) return;
    const int first_pos = ctx_len[r] - q;
    const size_t per = (size_t)d * dv;
    const float *S = state + ((size_t)state_slot[r] * nh + h) * per;
    const size_t at = ((size_t)long_index(q_start, r) * RT_RUNS * nh + h) * per;
    const int len = (q + RT_RUNS - 1) / RT_RUNS;
    const float g = decay[h];
    float pw[RT_RUNS];
#pragma unroll
    for (int k = 0; k < RT_RUNS; ++k) {
        const int s0 = min(t1, t0 + k * len), s1 = min(t1, s0 + len);
        pw[k] = powf(g, (float)(s1 - s0));
    }
    for (size_t e = (size_t)blockIdx.z * blockDim.x + threadIdx.x; e < per; e += (size_t)gridDim.z * blockDim.x) {
        float in = first_pos > 0 ? S[e] : 0.f;
#pragma unroll
        for (int k = 0; k < RT_RUNS; ++k) {
            run_in[at + (size_t)k * nh * per + e] = in;
            in = pw[k] * in + run_b[at + (size_t)k * nh * per + e];
        }
    }
}

// out[t, h, :] = o[t, h, :] * rsqrt(mean_j o[t, h, j]^2 + eps) * silu(gate[t, h, :]); one wave per (token, head).
template <class TG, class T>
__global__ void __launch_bounds__(WAVE)
retention_out_kernel(const float *__restrict__ o, const TG *__restrict__ gate, int gate_stride, int g_off, T *__restrict__ out,
                     int n, int nh, int dv, float eps) {
    const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
    const int tiles = (dv + RT_COLS - 1) / RT_COLS;
    auto at = [&](int c) { return o[(((size_t)h * tiles + c / RT_COLS) * n + t) * RT_COLS + c % RT_COLS]; };
    float sq = 0.f;
    for (int c = lane; c < dv; c += WAVE) sq += at(c) * at(c);
    const float f = rsqrtf(wave_sum(sq) / (float)dv + eps);
    for (int c = lane; c < dv; c += WAVE) {
        const float z = to_f32(gate[(size_t)t * gate_stride + g_off + h * dv + c]);
        out[(size_t)t * nh * dv + (size_t)h * dv + c] = from_f32<T>(at(c) * f * (z / (1.0f + expf(-z))));
    }
}

// rows: [n, row_stride] of in_type with q (nh * d) at q_off, k at k_off, v (nh * dv) at v_off and the gate (nh * dv)
// at g_off.  decay: float32 [nh].  state: float32 [slots, nh, d, dv].  qk: float32 scratch [nh, n, 2 d + dv]; o: float32
// scratch of nh * n * (dv rounded up to 16) floats; runs: float32 scratch of 2 * (n / 512) * 8 * nh * d * dv floats (null if n < 512).
// out: [n, nh * dv] of out_type.  cos_t / sin_t may be null (no rotation).
LCU_API int lcu_retention(const void *rows, int in_type, int row_stride, int q_off, int k_off, int v_off, int g_off,
                          const int *positions, const float *cos_t, const float *sin_t, int max_pos, int rot_dim, int pairing,
                          float k_scale, const float *decay, float *state, float *qk, float *o, float *runs, void *out, int out_type,
                          const int *q_start, const int *ctx_len, const int *state_slot, int n, int n_req, int nh, int d,
                          int dv, float eps, hipStream_t stream) {
    if (n <= 0 || n_req <= 0) return LCU_OK;
    if (nh <= 0 || d <= 0 || d > 256 || dv <= 0 || rot_dim < 0 || rot_dim % 2 || rot_dim > d || (pairing != 0 && pairing != 1) ||
        !rows || !decay || !state || !qk || !o || !out || (cos_t && (!sin_t || !positions)) || nh > 65535 || n_req > 65535)
        return LCU_BAD_ARGUMENT;
    {
        dim3 pgrid(n, (nh * (d > dv ? d : dv) + 1023) / 1024), pblock(256);
        if (in_type == LCU_F32)
            retention_prep_kernel<float><<<pgrid, pblock, 0, stream>>>((const float *)rows, row_stride, q_off, k_off, v_off, positions, cos_t, sin_t, max_pos, rot_dim, pairing, k_scale, qk, n, nh, d, dv);
        else if (in_type == LCU_BF16)
            retention_prep_kernel<bf16_t><<<pgrid, pblock, 0, stream>>>((const bf16_t *)rows, row_stride, q_off, k_off, v_off, positions, cos_t, sin_t, max_pos, rot_dim, pairing, k_scale, qk, n, nh, d, dv);
        else
            return LCU_BAD_ARGUMENT;
        LCU_LAUNCH_CHECK();
    }
    dim3 grid((dv + RT_COLS - 1) / RT_COLS, nh, n_req), block(RT_THREADS);
#define SCAN(DPL, TOK, MODE, G) retention_scan_kernel<DPL, TOK, MODE><<<G, block, 0, stream>>>(qk, decay, state, o, q_start, ctx_len, state_slot, runs, runs ? runs + run_floats : nullptr, n, nh, d, dv)
#define BY_DIM(MODE, G) do { if (d <= 64) SCAN(4, 16, MODE, G); else if (d <= 128) SCAN(8, 16, MODE, G); else SCAN(16, 8, MODE, G); } while (0)
    const size_t run_floats = (size_t)(n / RT_LONG) * RT_RUNS * nh * d * dv;
    BY_DIM(0, grid);
    LCU_LAUNCH_CHECK();
    if (n >= RT_LONG) {                 // the step may hold requests that feed many tokens: they are walked in runs
        if (!runs || n_req * RT_RUNS > 65535) return LCU_BAD_ARGUMENT;
        dim3 rgrid(grid.x, nh, n_req * RT_RUNS);
        BY_DIM(1, rgrid);
        LCU_LAUNCH_CHECK();
        retention_chain_kernel<<<dim3(nh, n_req, (unsigned)((d * dv + 1023) / 1024)), dim3(256), 0, stream>>>(decay, state, runs, runs + run_floats, q_start, ctx_len, state_slot, nh, d, dv);
        LCU_LAUNCH_CHECK();
        BY_DIM(2, rgrid);
    }
#undef BY_DIM
#undef SCAN
    LCU_LAUNCH_CHECK();
    dim3 ogrid(n, nh), oblock(WAVE);
#define OUT(TG, T) retention_out_kernel<TG, T><<<ogrid, oblock, 0, stream>>>(o, (const TG *)rows, row_stride, g_off, (T *)out, n, nh, dv, eps)
    if (in_type == LCU_F32 && out_type == LCU_F32) OUT(float, float);
    else if (in_type == LCU_F32 && out_type == LCU_BF16) OUT(float, bf16_t);
    else if (in_type == LCU_BF16 && out_type == LCU_BF16) OUT(bf16_t, bf16_t);
    else return LCU_BAD_ARGUMENT;
#undef OUT
    LCU_LAUNCH_CHECK();
    return LCU_OK;
}
