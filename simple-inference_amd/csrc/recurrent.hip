// Linear attention with a decaying matrix state per head (gated linear attention), token by token.
//
// For every sequence and head, with a state S [D, Dv] of floats that a request keeps in its slot:
//
//   z_t     = A2 a_t + b                       a_t: the token's low-rank decay input [rank]; A2 [H * D, rank]
//   alpha_t = exp(logsigmoid(z_t) / tau)       one decay per key channel, in (0, 1)
//   S_t     = diag(alpha_t) S_(t-1) + k_t v_t^T
//   o_t     = S_t^T (q_t * q_scale)
//   y_t     = o_t * rsqrt(mean(o_t^2) + eps) * w  *  silu(g_t)         w [Dv], shared by the heads
//
// q, k [H * D], v, g [H * Dv] and a [rank] are columns of one projected row (row_stride apart, at the given column
// offsets); y is written as [tokens, H * Dv].  Products' results come in the compute type; decays, their logarithms,
// the state, the sums over channels, the norm and the gate are float, with one rounding of y.
//
// The decays of all tokens and channels are computed first, by a kernel of their own (they do not depend on the
// state, and a step's tokens are thousands of independent little products), into a float workspace.
// A workgroup owns one (sequence, head) and walks the sequence's tokens of this step in order, so a request's
// numbers depend on its own tokens only: not on how its prompt was cut, nor on what else the step holds.
// Thread (j, r) keeps rows r, r + R, r + 2R, ... of column j of S in registers (R a power of two: the lanes of a
// column are neighbours and add their shares of o by lane exchanges).  Blocks of a few tokens are staged through
// LDS (q, k, alpha, v, g as floats), walked, and their outputs normed and gated a token a wave.
//
// A step with few (sequence, head) pairs and runs of many tokens (a prompt) would leave most of the chip idle, and
// the walk along a sequence cannot be shortened.  Such a step gives every pair several workgroups, each with a
// slice of the state's columns (they are independent of one another), more lanes per column and fewer rows per
// lane; the outputs go to a float workspace and a second kernel norms and gates them, since a norm spans a head.
#include "common.h"

__device__ __forceinline__ float log_sigmoid(float z) { return fminf(z, 0.f) - log1pf(expf(-fabsf(z))); }

template <typename T, int ROWS>
__global__ __launch_bounds__(512) void gla_recurrent_kernel(
    const T* __restrict__ proj, int row_stride, int q_col, int k_col, int v_col, int g_col,
    const float* __restrict__ alpha, const float* __restrict__ norm_w, float* __restrict__ state, const int* __restrict__ cu_q, const int* __restrict__ slots, T* __restrict__ out,
    int n_heads, int D, int Dv, int R, int block_tokens, float q_scale, float eps, int slice,
    float* __restrict__ raw_out, const float* __restrict__ k_f32, int q_share, long long state_stride) {
    extern __shared__ float lds[];
    const int seq = blockIdx.x, head = blockIdx.y, tid = threadIdx.x;
    const int j0 = blockIdx.z * slice;     // this workgroup's columns: j0 .. j0 + slice - 1
    const int first = cu_q[seq], last = cu_q[seq + 1];
    if (first >= last) return;
    const int TB = block_tokens;
    float* q_s = lds;                  // [TB][D]
    float* k_s = q_s + TB * D;         // [TB][D]
    float* al_s = k_s + TB * D;        // [TB][D]
    float* v_s = al_s + TB * D;        // [TB][Dv]
    float* g_s = v_s + TB * Dv;        // [TB][Dv]
    float* o_s = g_s + TB * Dv;        // [TB][Dv]

    const int j = j0 + tid / R, r = tid % R;
    const bool owns = tid / R < slice && j < Dv;
    float* S_mem = state + (size_t)slots[seq] * state_stride + (size_t)head * D * Dv;
    float S[ROWS];
#pragma unroll
    for (int i = 0; i < ROWS; ++i) {
        const int d = i * R + r;
        S[i] = (owns && d < D) ? S_mem[(size_t)d * Dv + j] : 0.f;
    }
    const int wave = tid / SIA_WAVE, lane = tid % SIA_WAVE, n_waves = blockDim.x / SIA_WAVE;
    const int q_head = head / q_share;      // q (and a k read from the rows) may be shared by q_share neighbouring heads

    for (int t0 = first; t0 < last; t0 += TB) {
        const int nt = min(TB, last - t0);
        for (int idx = tid; idx < nt * Dv; idx += blockDim.x) {
            const int t = idx / Dv, c = idx % Dv;
            const T* row = proj + (size_t)(t0 + t) * row_stride;
            v_s[t * Dv + c] = to_float(row[v_col + head * Dv + c]);
            g_s[t * Dv + c] = g_col >= 0 ? to_float(row[g_col + head * Dv + c]) : 0.f;
        }
        for (int idx = tid; idx < nt * D; idx += blockDim.x) {
            const int t = idx / D, c = idx % D;
            const T* row = proj + (size_t)(t0 + t) * row_stride;
            q_s[t * D + c] = to_float(row[q_col + q_head * D + c]) * q_scale;
            k_s[t * D + c] = k_f32 ? k_f32[((size_t)(t0 + t) * n_heads + head) * D + c]
                                   : to_float(row[k_col + q_head * D + c]);
            al_s[t * D + c] = alpha[((size_t)(t0 + t) * n_heads + head) * D + c];
        }
        __syncthreads();
        for (int t = 0; t < nt; ++t) {
            float acc = 0.f;
            const float v = owns ? v_s[t * Dv + j] : 0.f;
#pragma unroll
            for (int i = 0; i < ROWS; ++i) {
                const int d = i * R + r;
                if (d < D) {
                    S[i] = al_s[t * D + d] * S[i] + k_s[t * D + d] * v;
                    acc += q_s[t * D + d] * S[i];
                }
            }
            for (int o = R / 2; o > 0; o >>= 1) acc += __shfl_xor(acc, o, SIA_WAVE);
            if (owns && r == 0) {
                if (raw_out) raw_out[((size_t)(t0 + t) * n_heads + head) * Dv + j] = acc;
                else o_s[t * Dv + j] = acc;
            }
        }
        __syncthreads();
        if (raw_out) continue;   // uniform: the norm is another kernel's
        for (int t = wave; t < nt; t += n_waves) {
            float ss = 0.f;
            for (int c = lane; c < Dv; c += SIA_WAVE) ss += o_s[t * Dv + c] * o_s[t * Dv + c];
            const float inv = rsqrtf(wave_sum(ss) / (float)Dv + eps);
            T* dst = out + ((size_t)(t0 + t) * n_heads + head) * Dv;
            for (int c = lane; c < Dv; c += SIA_WAVE) {
                const float g = g_s[t * Dv + c];
                dst[c] = from_float<T>(o_s[t * Dv + c] * inv * norm_w[c] * (g_col >= 0 ? g / (1.f + expf(-g)) : 1.f));
            }
        }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < ROWS; ++i) {
        const int d = i * R + r;
        if (owns && d < D) S_mem[(size_t)d * Dv + j] = S[i];
    }
}

// Sum over the 16 lanes of a row of a wave by lane exchanges inside the vector unit (no trip through LDS's crossbar):
// neighbours, pairs of a quad, the mirrored half, the mirrored row.  Every lane of the row gets the sum.
__device__ __forceinline__ float row16_sum(float v) {
    v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0xB1, 0xF, 0xF, true));    // quad_perm [1,0,3,2]
    v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x4E, 0xF, 0xF, true));    // quad_perm [2,3,0,1]
    v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x141, 0xF, 0xF, true));   // row_half_mirror
    v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x140, 0xF, 0xF, true));   // row_mirror
    return v;
}

// The walk alone, for a prompt's step in bfloat16 whose heads' columns are shared out (D a multiple of 8, rows and
// columns aligned to 16 bytes).  The 16 lanes of one row of a wave share two or four columns of the state, lane r
// keeping rows r * ROWS .. r * ROWS + ROWS - 1 of each (what a lane reads of q, k and the decays serves all its
// columns: LDS bandwidth, which every lane's reads of the same numbers would exhaust, is spent once per
// those columns); a token's outputs are sums over the row.  q, k and the decays lie in LDS so that the 16
// lanes' 16-byte pieces of a read are one contiguous run (no bank meets twice).  Blocks of 32 tokens: their q, k
// (16-byte pieces), decays (float4) and values are requested into registers while the block before is walked, so
// that the walk never waits for memory.  Outputs go to the float workspace; the norm is the finishing kernel's.
#define GLA_WALK_TOKENS 32
#define GLA_WALK_THREADS 256
// KF: what is written (k) comes as floats [tokens, heads, D] from ``k_f32``, as the decays do, not as columns of the
// rows.  ``q_share`` neighbouring heads read the same q columns; a sequence's matrices begin ``state_stride`` floats
// after the sequence before it.
template <int ROWS, int GLA_WALK_COLS, bool KF>
__global__ __launch_bounds__(GLA_WALK_THREADS) void gla_walk_kernel(
    const bf16_t* __restrict__ proj, int row_stride, int q_col, int k_col, int v_col, const float* __restrict__ alpha,
    const float* __restrict__ k_f32, int q_share, float* __restrict__ state, long long state_stride,
    const int* __restrict__ cu_q, const int* __restrict__ slots, int n_heads, int D, int Dv, float q_scale,
    float* __restrict__ raw_out) {
    extern __shared__ float lds[];
    constexpr int TB = GLA_WALK_TOKENS, C = GLA_WALK_COLS, threads = GLA_WALK_THREADS;
    constexpr int slice = threads / 16 * C;      // columns a workgroup
    constexpr int Dp = 16 * ROWS;                // D filled up to the rows the lanes hold: what lies beyond D is zero
    const int seq = blockIdx.x, head = blockIdx.y, tid = threadIdx.x;
    const int j0 = blockIdx.z * slice;
    const int first = cu_q[seq], last = cu_q[seq + 1];
    if (first >= last) return;
    float* q_s = lds;               // [TB][Dp], row d = r * ROWS + i at (i / 4) * 64 + r * 4 + i % 4
    float* k_s = q_s + TB * Dp;
    float* al_s = k_s + TB * Dp;
    float* v_s = al_s + TB * Dp;    // [TB][slice]
    float* o_s = v_s + TB * slice;  // [TB][slice]: a block's outputs, written out together
    auto place = [](int d) { const int r = d / ROWS, i = d % ROWS; return (i / 4) * 64 + r * 4 + i % 4; };
    for (int i = tid; i < 3 * TB * Dp; i += threads) lds[i] = 0.f;
    const int jl = (tid / 16) * C, r = tid % 16;      // this lane's first column inside the slice, and its rows
    float* S_mem = state + (size_t)slots[seq] * state_stride + (size_t)head * D * Dv;
    float S[C][ROWS];
#pragma unroll
    for (int c = 0; c < C; ++c)
#pragma unroll
        for (int i = 0; i < ROWS; ++i) {
            const int d = r * ROWS + i, j = j0 + jl + c;
            S[c][i] = (j < Dv && d < D) ? S_mem[(size_t)d * Dv + j] : 0.f;
        }
    const int d8 = D / 8, d4 = D / 4;
    const int q_at = q_col + (head / q_share) * D, k_at = k_col + (head / q_share) * D;
    // What is on its way from memory is held in named registers, and the two steps below are written out piece by
    // piece: arrays indexed in loops ended up in scratch memory here, and a wave then waited for every piece twice.
    static_assert(TB * slice / threads == 4, "four values a thread and block");
    uint4 rq0, rq1, rq2, rq3, rk0, rk1, rk2, rk3;
    float4 ra0, ra1, ra2, ra3, ra4, ra5, ra6, ra7;
    float4 rf0, rf1, rf2, rf3, rf4, rf5, rf6, rf7;
    float rv0, rv1, rv2, rv3;
    // pieces beyond the block's end repeat its last piece (every load is issued, none is conditional)
#define GLA_REQ_QK(i, Q, K)                                                                          \
    do {                                                                                             \
        const int idx = min(tid + (i) * threads, rnt * d8 - 1);                                       \
        const bf16_t* row = proj + (size_t)(rt0 + idx / d8) * row_stride + (idx % d8) * 8;            \
        Q = *reinterpret_cast<const uint4*>(row + q_at);                                             \
        if constexpr (!KF) K = *reinterpret_cast<const uint4*>(row + k_at);                          \
    } while (0)
#define GLA_REQ_F(i, A, SRC)                                                                         \
    do {                                                                                             \
        const int idx = min(tid + (i) * threads, rnt * d4 - 1);                                       \
        A = *reinterpret_cast<const float4*>(SRC + ((size_t)(rt0 + idx / d4) * n_heads + head) * D + (idx % d4) * 4); \
    } while (0)
#define GLA_REQ_A(i, A) GLA_REQ_F(i, A, alpha)
#define GLA_REQ_V(i, V)                                                                              \
    do {                                                                                             \
        const int idx = min(tid + (i) * threads, rnt * slice - 1);                                    \
        V = bf16_to_float(proj[(size_t)(rt0 + idx / slice) * row_stride + v_col + head * Dv +         \
                               min(j0 + idx % slice, Dv - 1)]);                                      \
    } while (0)
#define GLA_REQUEST(T0)                                                                              \
    do {                                                                                             \
        const int rt0 = (T0), rnt = min(TB, last - rt0);                                                \
        GLA_REQ_QK(0, rq0, rk0); GLA_REQ_QK(1, rq1, rk1); GLA_REQ_QK(2, rq2, rk2); GLA_REQ_QK(3, rq3, rk3); \
        GLA_REQ_A(0, ra0); GLA_REQ_A(1, ra1); GLA_REQ_A(2, ra2); GLA_REQ_A(3, ra3);                  \
        GLA_REQ_A(4, ra4); GLA_REQ_A(5, ra5); GLA_REQ_A(6, ra6); GLA_REQ_A(7, ra7);                  \
        if constexpr (KF) {                                                                          \
            GLA_REQ_F(0, rf0, k_f32); GLA_REQ_F(1, rf1, k_f32); GLA_REQ_F(2, rf2, k_f32); GLA_REQ_F(3, rf3, k_f32); \
            GLA_REQ_F(4, rf4, k_f32); GLA_REQ_F(5, rf5, k_f32); GLA_REQ_F(6, rf6, k_f32); GLA_REQ_F(7, rf7, k_f32); \
        }                                                                                            \
        GLA_REQ_V(0, rv0); GLA_REQ_V(1, rv1); GLA_REQ_V(2, rv2); GLA_REQ_V(3, rv3);                  \
    } while (0)
    // two 16-bit halves of a word are rows d and d + 1
#define GLA_PUT(word_q, word_k, d)                                                                   \
    do {                                                                                             \
        const int p0 = base + place(d), p1 = base + place((d) + 1);                                  \
        q_s[p0] = __uint_as_float((word_q) << 16) * q_scale;                                         \
        q_s[p1] = __uint_as_float((word_q) & 0xffff0000u) * q_scale;                                 \
        if constexpr (!KF) {                                                                         \
            k_s[p0] = __uint_as_float((word_k) << 16);                                               \
            k_s[p1] = __uint_as_float((word_k) & 0xffff0000u);                                       \
        }                                                                                            \
    } while (0)
#define GLA_DEP_QK(i, Q, K)                                                                          \
    do {                                                                                             \
        const int idx = tid + (i) * threads;                                                         \
        if (idx < dnt * d8) {                                                                         \
            const int base = (idx / d8) * Dp, d0 = (idx % d8) * 8;                                   \
            GLA_PUT(Q.x, K.x, d0);                                                                   \
            GLA_PUT(Q.y, K.y, d0 + 2);                                                               \
            GLA_PUT(Q.z, K.z, d0 + 4);                                                               \
            GLA_PUT(Q.w, K.w, d0 + 6);                                                               \
        }                                                                                            \
    } while (0)
#define GLA_DEP_F(i, A, DST)                                                                         \
    do {   /* four rows of one lane (ROWS is a multiple of 4) */                                     \
        const int idx = tid + (i) * threads;                                                         \
        if (idx < dnt * d4) *reinterpret_cast<float4*>(DST + (idx / d4) * Dp + place((idx % d4) * 4)) = A; \
    } while (0)
#define GLA_DEP_A(i, A) GLA_DEP_F(i, A, al_s)
#define GLA_DEP_V(i, V)                                                                              \
    do {                                                                                             \
        const int idx = tid + (i) * threads;                                                         \
        if (idx < dnt * slice) v_s[idx] = (j0 + idx % slice < Dv) ? V : 0.f;                          \
    } while (0)
#define GLA_DEPOSIT(T0)                                                                              \
    do {                                                                                             \
        const int dnt = min(TB, last - (T0));                                                         \
        GLA_DEP_QK(0, rq0, rk0); GLA_DEP_QK(1, rq1, rk1); GLA_DEP_QK(2, rq2, rk2); GLA_DEP_QK(3, rq3, rk3); \
        GLA_DEP_A(0, ra0); GLA_DEP_A(1, ra1); GLA_DEP_A(2, ra2); GLA_DEP_A(3, ra3);                  \
        GLA_DEP_A(4, ra4); GLA_DEP_A(5, ra5); GLA_DEP_A(6, ra6); GLA_DEP_A(7, ra7);                  \
        if constexpr (KF) {                                                                          \
            GLA_DEP_F(0, rf0, k_s); GLA_DEP_F(1, rf1, k_s); GLA_DEP_F(2, rf2, k_s); GLA_DEP_F(3, rf3, k_s); \
            GLA_DEP_F(4, rf4, k_s); GLA_DEP_F(5, rf5, k_s); GLA_DEP_F(6, rf6, k_s); GLA_DEP_F(7, rf7, k_s); \
        }                                                                                            \
        GLA_DEP_V(0, rv0); GLA_DEP_V(1, rv1); GLA_DEP_V(2, rv2); GLA_DEP_V(3, rv3);                  \
    } while (0)
    // One round before the first block only requests it (each of the two steps is written once, so that the pieces
    // on their way stay in registers).
    for (int t0 = first - TB; t0 < last; t0 += TB) {
        const int nt = min(TB, last - t0);
        if (t0 >= first) GLA_DEPOSIT(t0);
        __syncthreads();   // in the first round: the zeros are in place before the first pieces land on them
        if (t0 + TB < last) GLA_REQUEST(t0 + TB);
        if (t0 < first) continue;   // uniform
        // a token's q, k and decays are read from LDS while the token before is worked on
        float4 qn[ROWS / 4], kn[ROWS / 4], an[ROWS / 4];
        auto fetch = [&](int t) {
#pragma unroll
            for (int i = 0; i < ROWS / 4; ++i) {
                const int at = t * Dp + i * 64 + r * 4;
                qn[i] = *reinterpret_cast<const float4*>(q_s + at);
                kn[i] = *reinterpret_cast<const float4*>(k_s + at);
                an[i] = *reinterpret_cast<const float4*>(al_s + at);
            }
        };
        fetch(0);
        for (int t = 0; t < nt; ++t) {
            float4 qv[ROWS / 4], kv[ROWS / 4], av[ROWS / 4];
            float vv[C];
#pragma unroll
            for (int i = 0; i < ROWS / 4; ++i) { qv[i] = qn[i]; kv[i] = kn[i]; av[i] = an[i]; }
#pragma unroll
            for (int c = 0; c < C; ++c) vv[c] = v_s[t * slice + jl + c];
            fetch(min(t + 1, TB - 1));
#pragma unroll
            for (int c = 0; c < C; ++c) {
                const float v = vv[c];
                float acc = 0.f;
#pragma unroll
                for (int i = 0; i < ROWS / 4; ++i) {
                    S[c][4 * i] = av[i].x * S[c][4 * i] + kv[i].x * v;
                    S[c][4 * i + 1] = av[i].y * S[c][4 * i + 1] + kv[i].y * v;
                    S[c][4 * i + 2] = av[i].z * S[c][4 * i + 2] + kv[i].z * v;
                    S[c][4 * i + 3] = av[i].w * S[c][4 * i + 3] + kv[i].w * v;
                    acc += qv[i].x * S[c][4 * i];
                    acc += qv[i].y * S[c][4 * i + 1];
                    acc += qv[i].z * S[c][4 * i + 2];
                    acc += qv[i].w * S[c][4 * i + 3];
                }
                acc = row16_sum(acc);
                if (r == 0) o_s[t * slice + jl + c] = acc;
            }
        }
        __syncthreads();
        for (int idx = tid; idx < nt * slice; idx += threads)
            if (j0 + idx % slice < Dv)
                raw_out[((size_t)(t0 + idx / slice) * n_heads + head) * Dv + j0 + idx % slice] = o_s[idx];
    }
#pragma unroll
    for (int c = 0; c < C; ++c)
#pragma unroll
        for (int i = 0; i < ROWS; ++i) {
            const int d = r * ROWS + i, j = j0 + jl + c;
            if (j < Dv && d < D) S_mem[(size_t)d * Dv + j] = S[c][i];
        }
}

#undef GLA_REQ_QK
#undef GLA_REQ_A
#undef GLA_REQ_F
#undef GLA_DEP_F
#undef GLA_REQ_V
#undef GLA_REQUEST
#undef GLA_PUT
#undef GLA_DEP_QK
#undef GLA_DEP_A
#undef GLA_DEP_V
#undef GLA_DEPOSIT

// alpha[n, c] = exp(logsigmoid(a2_bias[c] + sum_m a[n, m] * A2[c, m]) / tau) for every token n and key channel c of all
// heads: a thread a channel, eight tokens a workgroup (their low-rank inputs staged in LDS, a channel's row of A2
// read once for the eight).
#define GLA_DECAY_TOKENS 8
template <typename T>
__global__ __launch_bounds__(256) void gla_decay_kernel(const T* __restrict__ proj, int row_stride, int a_col,
                                                        const T* __restrict__ a2, const float* __restrict__ a2_bias,
                                                        float* __restrict__ alpha, int n_tokens, int channels, int rank,
                                                        float tau_inv) {
    extern __shared__ float a_s[];   // [GLA_DECAY_TOKENS][rank]
    const int n0 = blockIdx.x * GLA_DECAY_TOKENS, nt = min(GLA_DECAY_TOKENS, n_tokens - n0);
    for (int idx = threadIdx.x; idx < nt * rank; idx += blockDim.x)
        a_s[idx] = to_float(proj[(size_t)(n0 + idx / rank) * row_stride + a_col + idx % rank]);
    __syncthreads();
    const int c = blockIdx.y * blockDim.x + threadIdx.x;
    if (c >= channels) return;
    const T* w = a2 + (size_t)c * rank;
    float z[GLA_DECAY_TOKENS];
    const float b = a2_bias ? a2_bias[c] : 0.f;
#pragma unroll
    for (int t = 0; t < GLA_DECAY_TOKENS; ++t) z[t] = b;
    for (int m = 0; m < rank; ++m) {
        const float wm = to_float(w[m]);
#pragma unroll
        for (int t = 0; t < GLA_DECAY_TOKENS; ++t) z[t] += a_s[min(t, nt - 1) * rank + m] * wm;
    }
#pragma unroll
    for (int t = 0; t < GLA_DECAY_TOKENS; ++t)
        if (t < nt) alpha[(size_t)(n0 + t) * channels + c] = expf(log_sigmoid(z[t]) * tau_inv);
}

// y = o * rsqrt(mean(o^2) + eps) * w * silu(g) for outputs left in a float workspace: a wave a (token, head).
template <typename T>
__global__ __launch_bounds__(SIA_WAVE) void gla_finish_kernel(const float* __restrict__ raw, const T* __restrict__ proj,
                                                              int row_stride, int g_col,
                                                              const float* __restrict__ norm_w, T* __restrict__ out,
                                                              int n_heads, int Dv, float eps) {
    const int n = blockIdx.x, head = blockIdx.y, lane = threadIdx.x;
    const float* o = raw + ((size_t)n * n_heads + head) * Dv;
    float ss = 0.f;
    for (int c = lane; c < Dv; c += SIA_WAVE) ss += o[c] * o[c];
    const float inv = rsqrtf(wave_sum(ss) / (float)Dv + eps);
    const T* g_row = proj + (size_t)n * row_stride + (g_col >= 0 ? g_col : 0) + head * Dv;
    T* dst = out + ((size_t)n * n_heads + head) * Dv;
    for (int c = lane; c < Dv; c += SIA_WAVE) {
        const float g = g_col >= 0 ? to_float(g_row[c]) : 0.f;
        dst[c] = from_float<T>(o[c] * inv * norm_w[c] * (g_col >= 0 ? g / (1.f + expf(-g)) : 1.f));
    }
}

SIA_EXPORT int sia_gla_max_dims() { return 512; }

// Whether a step shares a head's columns out between workgroups (and needs the outputs' part of the workspace).
static bool gla_slices(int n_seqs, int max_q_len, int n_heads) {
    (void)n_seqs; (void)n_heads;
    return max_q_len > 1;
}

// Floats of workspace a step of n_tokens needs: the decays [tokens, heads, D], and room for the raw outputs
// [tokens, heads, Dv] of a step whose heads' columns are shared out.
SIA_EXPORT long long sia_gla_workspace(int n_tokens, int n_seqs, int max_q_len, int n_heads, int D, int Dv) {
    (void)n_seqs; (void)max_q_len;
    return (long long)n_tokens * n_heads * D + (long long)n_tokens * n_heads * Dv;
}

// The recurrence itself for a step's runs of tokens, whoever prepared its inputs: S <- diag(alpha) S + k v^T, o = S^T q.
// q and v (and k, unless k_f32 gives it as floats [tokens, heads, D]) are columns of rows of the compute type; head h
// reads the q (and such a k) of head h / q_share.  A sequence's matrices lie state_stride floats apart from the next
// slot's.  The outputs go to ``raw`` [tokens, heads, Dv] as floats if the caller wants them there (want_raw) or if a
// head's columns are shared out between workgroups; otherwise they are normed over the head (norm_w, eps), gated by
// silu of the columns at g_col (none if negative) and written to ``out``.  Returns through ``raw_used`` whether ``raw``
// holds the outputs.
static int launch_recurrence(const void* proj, int row_stride, int q_col, int k_col, int v_col, int g_col,
                             const float* k_f32, int q_share, const float* alpha, const float* norm_w, float* state,
                             long long state_stride, const int* cu_q, const int* slots, void* out, int n_seqs,
                             int max_q_len, int n_heads, int D, int Dv, float q_scale, float eps, int dtype,
                             float* raw_space, bool want_raw, bool* raw_used, hipStream_t stream) {
    // columns a workgroup: all of a head's, or with a workspace a slice of them, as narrow as it takes to fill the chip
    int slice = Dv;
    const bool prompt = gla_slices(n_seqs, max_q_len, n_heads);
    if (prompt)
        while (slice > 8 && (long long)n_seqs * n_heads * ((Dv + slice - 1) / slice) < 256) slice = (slice + 1) / 2;
    // lanes a column: the largest power of two that keeps the workgroup within 512 threads and a wave's columns whole;
    // a state too tall for the rows a lane can keep is shared out over more workgroups, whatever the step
    int R = 1, rows = D;
    for (;;) {
        R = 1;
        while (R * 2 <= SIA_WAVE && slice * R * 2 <= 512 && R * 2 <= D) R *= 2;
        rows = (D + R - 1) / R;
        if (rows <= 128 || slice <= 1) break;
        slice = (slice + 1) / 2;
    }
    if (rows > 128) return SIA_BAD_ARGUMENT;
    const bool sliced = slice < Dv;
    const int threads = ((slice * R + SIA_WAVE - 1) / SIA_WAVE) * SIA_WAVE;
    int TB = max_q_len >= 16 ? 16 : (max_q_len >= 4 ? 4 : 1);
    auto bytes = [&](int tb) { return (size_t)tb * (3 * D + 3 * Dv) * sizeof(float); };
    while (TB > 1 && bytes(TB) > 60 * 1024) TB /= 2;
    if (bytes(TB) > 60 * 1024) return SIA_BAD_ARGUMENT;
    dim3 grid(n_seqs, n_heads, (Dv + slice - 1) / slice), block(threads);
    // the walk with requests a block ahead, where its pieces are aligned and fit its registers.  (Its workgroups take
    // as many columns as their threads hold whatever the step: the waves of a workgroup share the staged tokens, and
    // what bounds the walk is a wave's own chain of tokens, not the number of workgroups.)
    const int w_cols = 2;
    const int w_slice = GLA_WALK_THREADS / 16 * w_cols;
    const int w_rows = (D + 15) / 16;
    const int w_rows_t = w_rows <= 4 ? 4 : w_rows <= 8 ? 8 : w_rows <= 16 ? 16 : 32;
    const size_t w_lds = (size_t)GLA_WALK_TOKENS * (3 * 16 * w_rows_t + 2 * w_slice) * sizeof(float);
    const bool ahead = prompt && dtype == SIA_BF16 && D % 8 == 0 && row_stride % 8 == 0 && q_col % 8 == 0 &&
                       (k_f32 ? ((uintptr_t)k_f32 % 16) == 0 : k_col % 8 == 0) && ((uintptr_t)alpha % 16) == 0 &&
                       ((uintptr_t)proj % 16) == 0 &&
                       GLA_WALK_TOKENS * (D / 8) <= 4 * GLA_WALK_THREADS && w_lds <= 60 * 1024 && w_rows_t <= 16;
    float* raw = (sliced || ahead || want_raw) ? raw_space : nullptr;
    if (raw_used) *raw_used = raw != nullptr;
    if (ahead) {
        dim3 wgrid(n_seqs, n_heads, (Dv + w_slice - 1) / w_slice), wblock(GLA_WALK_THREADS);
#define WALK_AS(ROWS, COLS, KF)                                                                                      \
    hipLaunchKernelGGL((gla_walk_kernel<ROWS, COLS, KF>), wgrid, wblock, w_lds, stream, (const bf16_t*)proj,         \
                       row_stride, q_col, k_col, v_col, alpha, k_f32, q_share, state, state_stride, cu_q, slots,     \
                       n_heads, D, Dv, q_scale, raw)
#define WALK(ROWS, COLS)                                                                                             \
    do {                                                                                                             \
        if (k_f32) WALK_AS(ROWS, COLS, true);                                                                        \
        else WALK_AS(ROWS, COLS, false);                                                                             \
    } while (0)
        if (w_rows_t == 4) WALK(4, 2);
        else if (w_rows_t == 8) WALK(8, 2);
        else WALK(16, 2);
#undef WALK
#undef WALK_AS
    } else {
#define LAUNCH(T, ROWS)                                                                                              \
    hipLaunchKernelGGL((gla_recurrent_kernel<T, ROWS>), grid, block, bytes(TB), stream, (const T*)proj, row_stride,  \
                       q_col, k_col, v_col, g_col, alpha, norm_w, state, cu_q, slots, (T*)out, n_heads, D, Dv, R, TB,   \
                       q_scale, eps, slice, raw, k_f32, q_share, state_stride)
#define PICK(T)                                                                                                      \
    do {                                                                                                             \
        if (rows <= 4) LAUNCH(T, 4);                                                                                 \
        else if (rows <= 8) LAUNCH(T, 8);                                                                            \
        else if (rows <= 16) LAUNCH(T, 16);                                                                          \
        else if (rows <= 32) LAUNCH(T, 32);                                                                          \
        else if (rows <= 64) LAUNCH(T, 64);                                                                          \
        else LAUNCH(T, 128);                                                                                         \
    } while (0)
    if (dtype == SIA_F32) PICK(float);
    else if (dtype == SIA_BF16) PICK(bf16_t);
    else return SIA_BAD_ARGUMENT;
#undef PICK
#undef LAUNCH
    }
    return 0;
}

SIA_EXPORT int sia_gla_recurrent(const void* proj, int row_stride, int q_col, int k_col, int v_col, int g_col, int a_col,
                                 const void* a2, const float* a2_bias, const float* norm_w, float* state,
                                 const int* cu_q, const int* slots, void* out, int n_seqs, int max_q_len, int n_heads,
                                 int D, int Dv, int rank, float tau, float q_scale, float eps, int dtype,
                                 float* workspace, int n_tokens, hipStream_t stream) {
    if (n_seqs <= 0) return 0;
    if (D <= 0 || Dv <= 0 || D > 512 || Dv > 512 || rank <= 0 || rank > 1024 || n_heads <= 0 || n_heads > 65535 ||
        !(tau > 0.f) || !state || !norm_w || !workspace || n_tokens <= 0)
        return SIA_BAD_ARGUMENT;
    float* alpha = workspace;
    float* raw_space = workspace + (size_t)n_tokens * n_heads * D;
    {
        const int channels = n_heads * D;
        dim3 dgrid((n_tokens + GLA_DECAY_TOKENS - 1) / GLA_DECAY_TOKENS, (channels + 255) / 256), dblock(256);
        const size_t lds = (size_t)GLA_DECAY_TOKENS * rank * sizeof(float);
        if (dtype == SIA_F32)
            hipLaunchKernelGGL(gla_decay_kernel<float>, dgrid, dblock, lds, stream, (const float*)proj, row_stride, a_col,
                               (const float*)a2, a2_bias, alpha, n_tokens, channels, rank, 1.f / tau);
        else if (dtype == SIA_BF16)
            hipLaunchKernelGGL(gla_decay_kernel<bf16_t>, dgrid, dblock, lds, stream, (const bf16_t*)proj, row_stride,
                               a_col, (const bf16_t*)a2, a2_bias, alpha, n_tokens, channels, rank, 1.f / tau);
        else
            return SIA_BAD_ARGUMENT;
    }
    bool raw = false;
    const int code = launch_recurrence(proj, row_stride, q_col, k_col, v_col, g_col, nullptr, 1, alpha, norm_w, state,
                                       (long long)n_heads * D * Dv, cu_q, slots, out, n_seqs, max_q_len, n_heads, D, Dv,
                                       q_scale, eps, dtype, raw_space, false, &raw, stream);
    if (code) return code;
    if (raw) {
        dim3 fgrid(n_tokens, n_heads), fblock(SIA_WAVE);
        if (dtype == SIA_F32)
            hipLaunchKernelGGL(gla_finish_kernel<float>, fgrid, fblock, 0, stream, raw_space, (const float*)proj,
                               row_stride, g_col, norm_w, (float*)out, n_heads, Dv, eps);
        else
            hipLaunchKernelGGL(gla_finish_kernel<bf16_t>, fgrid, fblock, 0, stream, raw_space, (const bf16_t*)proj,
                               row_stride, g_col, norm_w, (bf16_t*)out, n_heads, Dv, eps);
    }
    return SIA_LAUNCH_CHECK();
}

// ---------------------------------------------------------------------------------------------------------------
// The gated linear recurrence whose forget gate also decides what is written:
//   f = l + (1 - l) * sigmoid(z_f + b),  S <- diag(f) S + (1 - f) v^T,  o = S^T silu(z_q),  y = o * rsqrt(mean(o^2) + eps) * w
// Rows are [z_q (H * D) | z_f (H * D) | v (H * Dv)].  A first kernel leaves f and 1 - f in the float workspace and
// silu(z_q) in the rows' own q columns; then the recurrence above, without an output gate.
template <typename T>
__global__ __launch_bounds__(256) void hgrn2_prepare_kernel(T* __restrict__ proj, int row_stride,
                                                            const float* __restrict__ f_bias,
                                                            const float* __restrict__ lower, float* __restrict__ alpha,
                                                            float* __restrict__ k_f32, int channels) {
    const int n = blockIdx.x, c = blockIdx.y * blockDim.x + threadIdx.x;
    if (c >= channels) return;
    T* row = proj + (size_t)n * row_stride;
    const float zq = to_float(row[c]);
    row[c] = from_float<T>(zq / (1.f + expf(-zq)));
    const float z = to_float(row[channels + c]) + (f_bias ? f_bias[c] : 0.f);
    const float l = lower ? lower[c] : 0.f;
    const float f = l + (1.f - l) * (1.f / (1.f + expf(-z)));
    alpha[(size_t)n * channels + c] = f;
    k_f32[(size_t)n * channels + c] = 1.f - f;
}

// floats of workspace: the gates and their complements [tokens, heads, D] each, the raw outputs [tokens, heads, Dv]
SIA_EXPORT long long sia_hgrn2_workspace(int n_tokens, int n_heads, int D, int Dv) {
    return 2LL * n_tokens * n_heads * D + (long long)n_tokens * n_heads * Dv;
}

SIA_EXPORT int sia_hgrn2_scan(void* proj, int row_stride, const float* f_bias, const float* lower, const float* norm_w,
                              float* state, const int* cu_q, const int* slots, void* out, int n_tokens, int n_seqs,
                              int max_q_len, int n_heads, int D, int Dv, float eps, int dtype, float* workspace,
                              hipStream_t stream) {
    if (n_seqs <= 0 || n_tokens <= 0) return 0;
    if (D <= 0 || Dv <= 0 || D > 512 || Dv > 512 || n_heads <= 0 || n_heads > 65535 || !state || !norm_w || !workspace ||
        row_stride < n_heads * (2 * D + Dv))
        return SIA_BAD_ARGUMENT;
    const int channels = n_heads * D;
    float* alpha = workspace;
    float* kf = alpha + (size_t)n_tokens * channels;
    float* raw_space = kf + (size_t)n_tokens * channels;
    dim3 pgrid(n_tokens, (channels + 255) / 256), pblock(256);
    if (dtype == SIA_F32)
        hipLaunchKernelGGL(hgrn2_prepare_kernel<float>, pgrid, pblock, 0, stream, (float*)proj, row_stride, f_bias, lower,
                           alpha, kf, channels);
    else if (dtype == SIA_BF16)
        hipLaunchKernelGGL(hgrn2_prepare_kernel<bf16_t>, pgrid, pblock, 0, stream, (bf16_t*)proj, row_stride, f_bias,
                           lower, alpha, kf, channels);
    else
        return SIA_BAD_ARGUMENT;
    bool raw = false;
    const int code = launch_recurrence(proj, row_stride, 0, 0, 2 * channels, -1, kf, 1, alpha, norm_w, state,
                                       (long long)n_heads * D * Dv, cu_q, slots, out, n_seqs, max_q_len, n_heads, D, Dv,
                                       1.f, eps, dtype, raw_space, false, &raw, stream);
    if (code) return code;
    if (raw) {
        dim3 fgrid(n_tokens, n_heads), fblock(SIA_WAVE);
        if (dtype == SIA_F32)
            hipLaunchKernelGGL(gla_finish_kernel<float>, fgrid, fblock, 0, stream, raw_space, (const float*)proj,
                               row_stride, -1, norm_w, (float*)out, n_heads, Dv, eps);
        else
            hipLaunchKernelGGL(gla_finish_kernel<bf16_t>, fgrid, fblock, 0, stream, raw_space, (const bf16_t*)proj,
                               row_stride, -1, norm_w, (bf16_t*)out, n_heads, Dv, eps);
    }
    return SIA_LAUNCH_CHECK();
}

// ---------------------------------------------------------------------------------------------------------------
// The state-space recurrence with one decay per head:
//   dt = softplus(z_dt + dt_bias),  S <- exp(-exp(A_log) dt) S + (dt B) x^T,  y = S^T C + D x        S [N, P] per head
//   out = y * silu(z), divided by the root mean square of each of norm_groups equal parts of the row, times w
// z and z_dt are columns of the projected rows ([z (H * P) | ... | z_dt (H)], the step sizes last); x, B, C are the
// convolved rows [x (H * P) | B (G * N) | C (G * N)], head h reading the B and C of group h / (H / G).  A first kernel
// leaves the decays and dt * B in the float workspace, the recurrence leaves y there, a last kernel adds D x, gates
// and norms.
template <typename T>
__global__ __launch_bounds__(256) void ssd_prepare_kernel(const T* __restrict__ proj, int row_stride, int dt_col,
                                                          const T* __restrict__ xbc, int xbc_stride, int b_col,
                                                          const float* __restrict__ dt_bias,
                                                          const float* __restrict__ a_log, float* __restrict__ alpha,
                                                          float* __restrict__ k_f32, int n_heads, int N, int share) {
    const int n = blockIdx.x, idx = blockIdx.y * blockDim.x + threadIdx.x;
    if (idx >= n_heads * N) return;
    const int h = idx / N, c = idx % N;
    const float z = to_float(proj[(size_t)n * row_stride + dt_col + h]) + (dt_bias ? dt_bias[h] : 0.f);
    const float dt = fmaxf(z, 0.f) + log1pf(expf(-fabsf(z)));
    alpha[(size_t)n * n_heads * N + idx] = expf(-expf(a_log[h]) * dt);
    k_f32[(size_t)n * n_heads * N + idx] = dt * to_float(xbc[(size_t)n * xbc_stride + b_col + (h / share) * N + c]);
}

template <typename T>
__global__ __launch_bounds__(256) void ssd_finish_kernel(const float* __restrict__ raw, const T* __restrict__ proj,
                                                         int row_stride, const T* __restrict__ xbc, int xbc_stride,
                                                         const float* __restrict__ d_skip,
                                                         const float* __restrict__ norm_w, T* __restrict__ out,
                                                         int inner, int P, int part, float eps) {
    __shared__ float scratch[16];
    const int n = blockIdx.x, c0 = blockIdx.y * part;
    const float* y = raw + (size_t)n * inner;
    const T* z = proj + (size_t)n * row_stride;
    const T* x = xbc + (size_t)n * xbc_stride;
    float ss = 0.f;
    for (int c = c0 + threadIdx.x; c < c0 + part; c += blockDim.x) {
        const float g = to_float(z[c]);
        const float v = (y[c] + (d_skip ? d_skip[c / P] : 0.f) * to_float(x[c])) * (g / (1.f + expf(-g)));
        ss += v * v;
    }
    const float inv = rsqrtf(block_sum(ss, scratch) / (float)part + eps);
    for (int c = c0 + threadIdx.x; c < c0 + part; c += blockDim.x) {
        const float g = to_float(z[c]);
        const float v = (y[c] + (d_skip ? d_skip[c / P] : 0.f) * to_float(x[c])) * (g / (1.f + expf(-g)));
        out[(size_t)n * inner + c] = from_float<T>(v * inv * norm_w[c]);
    }
}

SIA_EXPORT long long sia_ssd_workspace(int n_tokens, int n_heads, int N, int P) {
    return 2LL * n_tokens * n_heads * N + (long long)n_tokens * n_heads * P;
}

SIA_EXPORT int sia_ssd_scan(const void* proj, int row_stride, const void* xbc, int xbc_stride, const float* dt_bias,
                            const float* a_log, const float* d_skip, const float* norm_w, float* state,
                            long long state_stride, const int* cu_q, const int* slots, void* out, int n_tokens,
                            int n_seqs, int max_q_len, int n_heads, int P, int N, int groups, int norm_groups, float eps,
                            int dtype, float* workspace, hipStream_t stream) {
    if (n_seqs <= 0 || n_tokens <= 0) return 0;
    const int inner = n_heads * P;
    if (N <= 0 || P <= 0 || N > 512 || P > 512 || n_heads <= 0 || n_heads > 65535 || groups <= 0 || n_heads % groups ||
        norm_groups <= 0 || inner % norm_groups || norm_groups > 65535 || !state || !norm_w || !a_log || !workspace ||
        row_stride < inner + n_heads || xbc_stride < inner + 2 * groups * N ||
        state_stride < (long long)n_heads * N * P)
        return SIA_BAD_ARGUMENT;
    const int channels = n_heads * N, share = n_heads / groups;
    float* alpha = workspace;
    float* kf = alpha + (size_t)n_tokens * channels;
    float* raw_space = kf + (size_t)n_tokens * channels;
    const int dt_col = row_stride - n_heads, b_col = inner, c_col = inner + groups * N;
    dim3 pgrid(n_tokens, (channels + 255) / 256), pblock(256), fgrid(n_tokens, norm_groups), fblock(256);
    bool raw = false;
#define RUN(T)                                                                                                          \
    do {                                                                                                                \
        hipLaunchKernelGGL(ssd_prepare_kernel<T>, pgrid, pblock, 0, stream, (const T*)proj, row_stride, dt_col,         \
                           (const T*)xbc, xbc_stride, b_col, dt_bias, a_log, alpha, kf, n_heads, N, share);             \
        const int code = launch_recurrence(xbc, xbc_stride, c_col, 0, 0, -1, kf, share, alpha, norm_w, state,           \
                                           state_stride, cu_q, slots, nullptr, n_seqs, max_q_len, n_heads, N, P, 1.f,   \
                                           eps, dtype, raw_space, true, &raw, stream);                                  \
        if (code) return code;                                                                                          \
        hipLaunchKernelGGL(ssd_finish_kernel<T>, fgrid, fblock, 0, stream, raw_space, (const T*)proj, row_stride,       \
                           (const T*)xbc, xbc_stride, d_skip, norm_w, (T*)out, inner, P, inner / norm_groups, eps);     \
    } while (0)
    if (dtype == SIA_F32) RUN(float);
    else if (dtype == SIA_BF16) RUN(bf16_t);
    else return SIA_BAD_ARGUMENT;
#undef RUN
    return SIA_LAUNCH_CHECK();
}

// ---------------------------------------------------------------------------------------------------------------
// Linear attention with a constant decay per head, behind activations:
//   q, k, v = silu(z_q), silu(z_k), silu(z_v);  S <- decay_h S + k v^T;  o = S^T q                  S [D, Dv] per head
//   out = o / sqrt(mean over the whole row of o^2 + eps) * w * sigmoid(z_g)                          w [H * Dv]
// Rows are [z_q (H * D) | z_k (H * D) | z_v (H * Dv) | z_g (H * Dv)].  A first kernel leaves the activations in the
// rows' own columns and the decays, one per head, in the float workspace as the recurrence reads them; then the
// recurrence above with raw outputs, and a kernel that norms a row over all its heads and gates it.
template <typename T>
__global__ __launch_bounds__(256) void decay_prepare_kernel(T* __restrict__ proj, int row_stride,
                                                            const float* __restrict__ decays,
                                                            float* __restrict__ alpha, int n_heads, int D, int active) {
    const int n = blockIdx.x, c = blockIdx.y * blockDim.x + threadIdx.x;
    if (c < active) {
        T* row = proj + (size_t)n * row_stride;
        const float z = to_float(row[c]);
        row[c] = from_float<T>(z / (1.f + expf(-z)));
    }
    if (c < n_heads * D) alpha[(size_t)n * n_heads * D + c] = decays[c / D];
}

template <typename T>
__global__ __launch_bounds__(256) void decay_finish_kernel(const float* __restrict__ raw, const T* __restrict__ proj,
                                                           int row_stride, int g_col,
                                                           const float* __restrict__ norm_w, T* __restrict__ out,
                                                           int inner, float eps) {
    __shared__ float scratch[16];
    const int n = blockIdx.x;
    const float* o = raw + (size_t)n * inner;
    const T* g = proj + (size_t)n * row_stride + g_col;
    float ss = 0.f;
    for (int c = threadIdx.x; c < inner; c += blockDim.x) ss += o[c] * o[c];
    const float inv = rsqrtf(block_sum(ss, scratch) / (float)inner + eps);
    for (int c = threadIdx.x; c < inner; c += blockDim.x) {
        const float z = to_float(g[c]);
        out[(size_t)n * inner + c] = from_float<T>(o[c] * inv * norm_w[c] * (1.f / (1.f + expf(-z))));
    }
}

SIA_EXPORT int sia_decay_attention(void* proj, int row_stride, const float* decays, const float* norm_w, float* state,
                                   const int* cu_q, const int* slots, void* out, int n_tokens, int n_seqs,
                                   int max_q_len, int n_heads, int D, int Dv, float eps, int dtype, float* workspace,
                                   hipStream_t stream) {
    if (n_seqs <= 0 || n_tokens <= 0) return 0;
    if (D <= 0 || Dv <= 0 || D > 512 || Dv > 512 || n_heads <= 0 || n_heads > 65535 || !state || !norm_w || !decays ||
        !workspace || row_stride < n_heads * (2 * D + 2 * Dv))
        return SIA_BAD_ARGUMENT;
    const int qk = n_heads * D, inner = n_heads * Dv, active = 2 * qk + inner;
    float* alpha = workspace;
    float* raw_space = alpha + (size_t)n_tokens * qk;
    dim3 pgrid(n_tokens, (active + 255) / 256), pblock(256), fgrid(n_tokens), fblock(256);
    bool raw = false;
#define RUN(T)                                                                                                          \
    do {                                                                                                                \
        hipLaunchKernelGGL(decay_prepare_kernel<T>, pgrid, pblock, 0, stream, (T*)proj, row_stride, decays, alpha,      \
                           n_heads, D, active);                                                                         \
        const int code = launch_recurrence(proj, row_stride, 0, qk, 2 * qk, -1, nullptr, 1, alpha, norm_w, state,       \
                                           (long long)n_heads * D * Dv, cu_q, slots, nullptr, n_seqs, max_q_len,        \
                                           n_heads, D, Dv, 1.f, eps, dtype, raw_space, true, &raw, stream);             \
        if (code) return code;                                                                                          \
        hipLaunchKernelGGL(decay_finish_kernel<T>, fgrid, fblock, 0, stream, raw_space, (const T*)proj, row_stride,     \
                           active, norm_w, (T*)out, inner, eps);                                                        \
    } while (0)
    if (dtype == SIA_F32) RUN(float);
    else if (dtype == SIA_BF16) RUN(bf16_t);
    else return SIA_BAD_ARGUMENT;
#undef RUN
    return SIA_LAUNCH_CHECK();
}

// ---------------------------------------------------------------------------------------------------------------
// The gated delta rule, token by token:
//   q <- q / sqrt(sum(q^2) + 1e-6) * D^(-1/2),  k <- k / sqrt(sum(k^2) + 1e-6)            per query/key head
//   beta = sigmoid(z_b),  g = exp(-exp(A_log_h) * softplus(z_a + dt_bias_h))              per value head
//   S <- g S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q                          S [D, Dv] per value head
//   out = o * rsqrt(mean(o^2) + eps) * w * silu(z_g)                                      per head, w [Dv]
// q, k [G * D] and v [H * Dv] are columns of the convolved rows (value head h reads query/key head h / (H / G)); z_g
// [H * Dv], z_b and z_a [H] are columns of the projected rows.  A workgroup owns a (sequence, value head) or, in a
// step of few such pairs and many tokens, a slice of the head's columns (a column of S is corrected and read alone:
// S^T k and S^T q are sums down a column).  Thread (j, r) keeps rows r, r + R, ... of column j in registers; a token
// costs two sums over the R lanes of a column, one before the write and one after.  Blocks of tokens are staged
// through LDS as floats, where the unit norms, the write strengths and the decays of the block are taken, by every
// workgroup for itself.  The raw outputs go to the float workspace; the head's norm and gate are a second kernel.
template <typename T, int ROWS>
__global__ __launch_bounds__(512) void delta_rule_kernel(
    const T* __restrict__ qkv, int qkv_stride, const T* __restrict__ proj, int proj_stride, int b_col, int a_col,
    const float* __restrict__ a_log, const float* __restrict__ dt_bias, float* __restrict__ state,
    long long state_stride, const int* __restrict__ cu_q, const int* __restrict__ slots, float* __restrict__ raw_out,
    int n_heads, int n_kv, int D, int Dv, int R, int block_tokens, int slice, int g_col,
    const float* __restrict__ norm_w, T* __restrict__ out, float eps) {
    // raw_out absent: the workgroup owns all of the head's columns (slice == Dv) and norms and gates its outputs itself
    extern __shared__ float lds[];
    const int seq = blockIdx.x, head = blockIdx.y, tid = threadIdx.x;
    const int j0 = blockIdx.z * slice;
    const int first = cu_q[seq], last = cu_q[seq + 1];
    if (first >= last) return;
    const int TB = block_tokens;
    float* q_s = lds;                  // [TB][D]
    float* k_s = q_s + TB * D;         // [TB][D]
    float* v_s = k_s + TB * D;         // [TB][slice]
    float* be_s = v_s + TB * slice;    // [TB]
    float* de_s = be_s + TB;           // [TB]
    float* o_s = de_s + TB;            // [TB][slice], without raw_out only
    const int j = j0 + tid / R, r = tid % R;
    const bool owns = tid / R < slice && j < Dv;
    float* S_mem = state + (size_t)slots[seq] * state_stride + (size_t)head * D * Dv;
    float S[ROWS];
#pragma unroll
    for (int i = 0; i < ROWS; ++i) {
        const int d = i * R + r;
        S[i] = (owns && d < D) ? S_mem[(size_t)d * Dv + j] : 0.f;
    }
    const int wave = tid / SIA_WAVE, lane = tid % SIA_WAVE, n_waves = blockDim.x / SIA_WAVE;
    const int kv_head = head / (n_heads / n_kv);
    const int q_col = kv_head * D, k_col = n_kv * D + kv_head * D, v_col = 2 * n_kv * D + head * Dv;
    const float rate = expf(a_log[head]), bias = dt_bias ? dt_bias[head] : 0.f;
    const float q_scale = rsqrtf((float)D);

    for (int t0 = first; t0 < last; t0 += TB) {
        const int nt = min(TB, last - t0);
        for (int idx = tid; idx < nt * slice; idx += blockDim.x) {
            const int t = idx / slice, c = idx % slice;
            v_s[idx] = j0 + c < Dv ? to_float(qkv[(size_t)(t0 + t) * qkv_stride + v_col + j0 + c]) : 0.f;
        }
        for (int idx = tid; idx < nt * D; idx += blockDim.x) {
            const int t = idx / D, c = idx % D;
            const T* row = qkv + (size_t)(t0 + t) * qkv_stride;
            q_s[idx] = to_float(row[q_col + c]);
            k_s[idx] = to_float(row[k_col + c]);
        }
        if (tid < nt) {
            const T* row = proj + (size_t)(t0 + tid) * proj_stride;
            const float zb = to_float(row[b_col + head]), za = to_float(row[a_col + head]) + bias;
            be_s[tid] = 1.f / (1.f + expf(-zb));
            de_s[tid] = expf(-rate * (fmaxf(za, 0.f) + log1pf(expf(-fabsf(za)))));
        }
        __syncthreads();
        for (int t = wave; t < nt; t += n_waves) {      // unit vectors, a wave a token
            float sq = 0.f, sk = 0.f;
            for (int c = lane; c < D; c += SIA_WAVE) {
                sq += q_s[t * D + c] * q_s[t * D + c];
                sk += k_s[t * D + c] * k_s[t * D + c];
            }
            const float iq = rsqrtf(wave_sum(sq) + 1e-6f) * q_scale, ik = rsqrtf(wave_sum(sk) + 1e-6f);
            for (int c = lane; c < D; c += SIA_WAVE) {
                q_s[t * D + c] *= iq;
                k_s[t * D + c] *= ik;
            }
        }
        __syncthreads();
        for (int t = 0; t < nt; ++t) {
            const float g = de_s[t], b = be_s[t];
            const float v = owns ? v_s[t * slice + (j - j0)] : 0.f;
            float kept = 0.f;
#pragma unroll
            for (int i = 0; i < ROWS; ++i) {
                const int d = i * R + r;
                if (d < D) {
                    S[i] *= g;
                    kept += k_s[t * D + d] * S[i];
                }
            }
            for (int o = R / 2; o > 0; o >>= 1) kept += __shfl_xor(kept, o, SIA_WAVE);
            const float u = b * (v - kept);
            float acc = 0.f;
#pragma unroll
            for (int i = 0; i < ROWS; ++i) {
                const int d = i * R + r;
                if (d < D) {
                    S[i] += k_s[t * D + d] * u;
                    acc += q_s[t * D + d] * S[i];
                }
            }
            for (int o = R / 2; o > 0; o >>= 1) acc += __shfl_xor(acc, o, SIA_WAVE);
            if (owns && r == 0) {
                if (raw_out) raw_out[((size_t)(t0 + t) * n_heads + head) * Dv + j] = acc;
                else o_s[t * slice + (j - j0)] = acc;
            }
        }
        __syncthreads();
        if (raw_out) continue;   // uniform: the norm is another kernel's
        for (int t = wave; t < nt; t += n_waves) {
            float ss = 0.f;
            for (int c = lane; c < Dv; c += SIA_WAVE) ss += o_s[t * slice + c] * o_s[t * slice + c];
            const float inv = rsqrtf(wave_sum(ss) / (float)Dv + eps);
            const T* g_row = proj + (size_t)(t0 + t) * proj_stride + g_col + head * Dv;
            T* dst = out + ((size_t)(t0 + t) * n_heads + head) * Dv;
            for (int c = lane; c < Dv; c += SIA_WAVE) {
                const float z = to_float(g_row[c]);
                dst[c] = from_float<T>(o_s[t * slice + c] * inv * norm_w[c] * (z / (1.f + expf(-z))));
            }
        }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < ROWS; ++i) {
        const int d = i * R + r;
        if (owns && d < D) S_mem[(size_t)d * Dv + j] = S[i];
    }
}

// The same walk for a prompt's step in bfloat16, laid out as the linear attention's walk above: the 16 lanes of one
// row of a wave share C columns of the state, lane r keeping rows r * ROWS .. r * ROWS + ROWS - 1 of each, so that what
// a lane reads of q and k from LDS serves all its columns and the two sums of a token (S^T k before the write, S^T q
// after it) are exchanges inside the vector unit.  q and k lie in LDS as floats so that the 16 lanes' 16-byte pieces
// of a read are one contiguous run; rows beyond D are zero.  Blocks of 32 tokens; a block's unit norms, write
// strengths and decays are taken in LDS before it is walked, and its outputs leave together.
#define DELTA_WALK_TOKENS 32
#define DELTA_WALK_THREADS 256
template <int ROWS, int C>
__global__ __launch_bounds__(DELTA_WALK_THREADS) void delta_walk_kernel(
    const bf16_t* __restrict__ qkv, int qkv_stride, const bf16_t* __restrict__ proj, int proj_stride, int b_col,
    int a_col, const float* __restrict__ a_log, const float* __restrict__ dt_bias, float* __restrict__ state,
    long long state_stride, const int* __restrict__ cu_q, const int* __restrict__ slots, float* __restrict__ raw_out,
    int n_heads, int n_kv, int D, int Dv) {
    extern __shared__ float lds[];
    constexpr int TB = DELTA_WALK_TOKENS, threads = DELTA_WALK_THREADS;
    constexpr int slice = threads / 16 * C;      // columns a workgroup
    constexpr int Dp = 16 * ROWS;
    const int seq = blockIdx.x, head = blockIdx.y, tid = threadIdx.x;
    const int j0 = blockIdx.z * slice;
    const int first = cu_q[seq], last = cu_q[seq + 1];
    if (first >= last) return;
    float* q_s = lds;               // [TB][Dp], row d = r * ROWS + i at (i / 4) * 64 + r * 4 + i % 4
    float* k_s = q_s + TB * Dp;
    float* v_s = k_s + TB * Dp;     // [TB][slice]
    float* o_s = v_s + TB * slice;  // [TB][slice]
    float* be_s = o_s + TB * slice; // [TB]
    float* de_s = be_s + TB;        // [TB]
    auto place = [](int d) { const int r = d / ROWS, i = d % ROWS; return (i / 4) * 64 + r * 4 + i % 4; };
    for (int i = tid; i < 2 * TB * Dp; i += threads) lds[i] = 0.f;
    const int jl = (tid / 16) * C, r = tid % 16;
    float* S_mem = state + (size_t)slots[seq] * state_stride + (size_t)head * D * Dv;
    float S[C][ROWS];
#pragma unroll
    for (int c = 0; c < C; ++c)
#pragma unroll
        for (int i = 0; i < ROWS; ++i) {
            const int d = r * ROWS + i, j = j0 + jl + c;
            S[c][i] = (j < Dv && d < D) ? S_mem[(size_t)d * Dv + j] : 0.f;
        }
    const int wave = tid / SIA_WAVE, lane = tid % SIA_WAVE;
    const int kv_head = head / (n_heads / n_kv);
    const int q_col = kv_head * D, k_col = n_kv * D + kv_head * D, v_col = 2 * n_kv * D + head * Dv;
    const float rate = expf(a_log[head]), bias = dt_bias ? dt_bias[head] : 0.f;
    const float q_scale = rsqrtf((float)D);
    __syncthreads();
    for (int t0 = first; t0 < last; t0 += TB) {
        const int nt = min(TB, last - t0);
        for (int idx = tid; idx < nt * D; idx += threads) {
            const int t = idx / D, d = idx % D;
            const bf16_t* row = qkv + (size_t)(t0 + t) * qkv_stride;
            q_s[t * Dp + place(d)] = bf16_to_float(row[q_col + d]);
            k_s[t * Dp + place(d)] = bf16_to_float(row[k_col + d]);
        }
        for (int idx = tid; idx < nt * slice; idx += threads) {
            const int t = idx / slice, c = idx % slice;
            v_s[idx] = j0 + c < Dv ? bf16_to_float(qkv[(size_t)(t0 + t) * qkv_stride + v_col + j0 + c]) : 0.f;
        }
        if (tid < nt) {
            const bf16_t* row = proj + (size_t)(t0 + tid) * proj_stride;
            const float zb = bf16_to_float(row[b_col + head]), za = bf16_to_float(row[a_col + head]) + bias;
            be_s[tid] = 1.f / (1.f + expf(-zb));
            de_s[tid] = expf(-rate * (fmaxf(za, 0.f) + log1pf(expf(-fabsf(za)))));
        }
        __syncthreads();
        for (int t = wave; t < nt; t += threads / SIA_WAVE) {      // unit vectors, a wave a token (the padding is zero)
            float sq = 0.f, sk = 0.f;
            for (int c = lane; c < Dp; c += SIA_WAVE) {
                sq += q_s[t * Dp + c] * q_s[t * Dp + c];
                sk += k_s[t * Dp + c] * k_s[t * Dp + c];
            }
            const float iq = rsqrtf(wave_sum(sq) + 1e-6f) * q_scale, ik = rsqrtf(wave_sum(sk) + 1e-6f);
            for (int c = lane; c < Dp; c += SIA_WAVE) {
                q_s[t * Dp + c] *= iq;
                k_s[t * Dp + c] *= ik;
            }
        }
        __syncthreads();
        float4 qn[ROWS / 4], kn[ROWS / 4];
        auto fetch = [&](int t) {
#pragma unroll
            for (int i = 0; i < ROWS / 4; ++i) {
                const int at = t * Dp + i * 64 + r * 4;
                qn[i] = *reinterpret_cast<const float4*>(q_s + at);
                kn[i] = *reinterpret_cast<const float4*>(k_s + at);
            }
        };
        fetch(0);
        for (int t = 0; t < nt; ++t) {
            float4 qv[ROWS / 4], kv[ROWS / 4];
            float vv[C];
#pragma unroll
            for (int i = 0; i < ROWS / 4; ++i) { qv[i] = qn[i]; kv[i] = kn[i]; }
#pragma unroll
            for (int c = 0; c < C; ++c) vv[c] = v_s[t * slice + jl + c];
            const float g = de_s[t], b = be_s[t];
            fetch(min(t + 1, TB - 1));
            float kept[C];
#pragma unroll
            for (int c = 0; c < C; ++c) {
                float acc = 0.f;
#pragma unroll
                for (int i = 0; i < ROWS / 4; ++i) {
                    S[c][4 * i] *= g;
                    S[c][4 * i + 1] *= g;
                    S[c][4 * i + 2] *= g;
                    S[c][4 * i + 3] *= g;
                    acc += kv[i].x * S[c][4 * i];
                    acc += kv[i].y * S[c][4 * i + 1];
                    acc += kv[i].z * S[c][4 * i + 2];
                    acc += kv[i].w * S[c][4 * i + 3];
                }
                kept[c] = acc;
            }
#pragma unroll
            for (int c = 0; c < C; ++c) kept[c] = row16_sum(kept[c]);
            float out[C];
#pragma unroll
            for (int c = 0; c < C; ++c) {
                const float u = b * (vv[c] - kept[c]);
                float acc = 0.f;
#pragma unroll
                for (int i = 0; i < ROWS / 4; ++i) {
                    S[c][4 * i] += kv[i].x * u;
                    S[c][4 * i + 1] += kv[i].y * u;
                    S[c][4 * i + 2] += kv[i].z * u;
                    S[c][4 * i + 3] += kv[i].w * u;
                    acc += qv[i].x * S[c][4 * i];
                    acc += qv[i].y * S[c][4 * i + 1];
                    acc += qv[i].z * S[c][4 * i + 2];
                    acc += qv[i].w * S[c][4 * i + 3];
                }
                out[c] = acc;
            }
#pragma unroll
            for (int c = 0; c < C; ++c) {
                out[c] = row16_sum(out[c]);
                if (r == 0) o_s[t * slice + jl + c] = out[c];
            }
        }
        __syncthreads();
        for (int idx = tid; idx < nt * slice; idx += threads)
            if (j0 + idx % slice < Dv)
                raw_out[((size_t)(t0 + idx / slice) * n_heads + head) * Dv + j0 + idx % slice] = o_s[idx];
        // (the next block's staging touches q_s, k_s, v_s and the gates, which nobody reads any more; o_s is written
        // again only behind two more barriers)
    }
#pragma unroll
    for (int c = 0; c < C; ++c)
#pragma unroll
        for (int i = 0; i < ROWS; ++i) {
            const int d = r * ROWS + i, j = j0 + jl + c;
            if (j < Dv && d < D) S_mem[(size_t)d * Dv + j] = S[c][i];
        }
}

// floats of workspace: the raw outputs [tokens, heads, Dv]
SIA_EXPORT long long sia_delta_rule_workspace(int n_tokens, int n_heads, int Dv) {
    return (long long)n_tokens * n_heads * Dv;
}

SIA_EXPORT int sia_delta_rule(const void* qkv, int qkv_stride, const void* proj, int proj_stride, int g_col, int b_col,
                              int a_col, const float* a_log, const float* dt_bias, const float* norm_w, float* state,
                              long long state_stride, const int* cu_q, const int* slots, void* out, int n_tokens,
                              int n_seqs, int max_q_len, int n_heads, int n_kv, int D, int Dv, float eps, int dtype,
                              float* workspace, hipStream_t stream) {
    if (n_seqs <= 0 || n_tokens <= 0) return 0;
    if (D <= 0 || Dv <= 0 || D > 512 || Dv > 512 || n_heads <= 0 || n_heads > 65535 || n_kv <= 0 || n_heads % n_kv ||
        !state || !norm_w || !a_log || !workspace || qkv_stride < 2 * n_kv * D + n_heads * Dv || g_col < 0 ||
        b_col < 0 || a_col < 0 || g_col + n_heads * Dv > proj_stride || b_col + n_heads > proj_stride ||
        a_col + n_heads > proj_stride || state_stride < (long long)n_heads * D * Dv)
        return SIA_BAD_ARGUMENT;
    // columns a workgroup: all of a head's, or in a step of runs of tokens a slice of them, as narrow as it takes to
    // fill the chip; lanes a column: the largest power of two that keeps the workgroup within 512 threads
    int slice = Dv;
    if (max_q_len > 1)
        while (slice > 8 && (long long)n_seqs * n_heads * ((Dv + slice - 1) / slice) < 256) slice = (slice + 1) / 2;
    int R = 1, rows = D;
    for (;;) {
        R = 1;
        while (R * 2 <= SIA_WAVE && slice * R * 2 <= 512 && R * 2 <= D) R *= 2;
        rows = (D + R - 1) / R;
        if (rows <= 128 || slice <= 1) break;
        slice = (slice + 1) / 2;
    }
    if (rows > 128) return SIA_BAD_ARGUMENT;
    const int threads = ((slice * R + SIA_WAVE - 1) / SIA_WAVE) * SIA_WAVE;
    int TB = max_q_len >= 16 ? 16 : (max_q_len >= 4 ? 4 : 1);
    // a workgroup that owns a whole head norms and gates its outputs itself (a decode step: one launch less)
    const bool whole = slice == Dv;
    auto bytes = [&](int tb) { return (size_t)tb * (2 * D + (whole ? 2 : 1) * slice + 2) * sizeof(float); };
    while (TB > 1 && bytes(TB) > 60 * 1024) TB /= 2;
    if (bytes(TB) > 60 * 1024) return SIA_BAD_ARGUMENT;
    float* raw = whole ? nullptr : workspace;
    dim3 grid(n_seqs, n_heads, (Dv + slice - 1) / slice), block(threads), fgrid(n_tokens, n_heads), fblock(SIA_WAVE);
    // a prompt's step in bfloat16: the walk whose lanes share columns, where its rows fit a lane's registers and LDS
    constexpr int w_cols = 2, w_slice = DELTA_WALK_THREADS / 16 * w_cols;
    const int w_rows = (D + 15) / 16;
    const int w_rows_t = w_rows <= 4 ? 4 : w_rows <= 8 ? 8 : w_rows <= 16 ? 16 : 32;
    const size_t w_lds = (size_t)(DELTA_WALK_TOKENS * (2 * 16 * w_rows_t + 2 * w_slice + 2)) * sizeof(float);
    if (max_q_len > 1 && dtype == SIA_BF16 && w_rows_t <= 16 && w_lds <= 60 * 1024) {
        dim3 wgrid(n_seqs, n_heads, (Dv + w_slice - 1) / w_slice), wblock(DELTA_WALK_THREADS);
#define WALK(ROWS)                                                                                                   \
    hipLaunchKernelGGL((delta_walk_kernel<ROWS, w_cols>), wgrid, wblock, w_lds, stream, (const bf16_t*)qkv,          \
                       qkv_stride, (const bf16_t*)proj, proj_stride, b_col, a_col, a_log, dt_bias, state,            \
                       state_stride, cu_q, slots, workspace, n_heads, n_kv, D, Dv)
        if (w_rows_t == 4) WALK(4);
        else if (w_rows_t == 8) WALK(8);
        else WALK(16);
#undef WALK
        hipLaunchKernelGGL(gla_finish_kernel<bf16_t>, fgrid, fblock, 0, stream, workspace, (const bf16_t*)proj,
                           proj_stride, g_col, norm_w, (bf16_t*)out, n_heads, Dv, eps);
        return SIA_LAUNCH_CHECK();
    }
#define LAUNCH(T, ROWS)                                                                                              \
    hipLaunchKernelGGL((delta_rule_kernel<T, ROWS>), grid, block, bytes(TB), stream, (const T*)qkv, qkv_stride,      \
                       (const T*)proj, proj_stride, b_col, a_col, a_log, dt_bias, state, state_stride, cu_q, slots,   \
                       raw, n_heads, n_kv, D, Dv, R, TB, slice, g_col, norm_w, (T*)out, eps)
#define RUN(T)                                                                                                       \
    do {                                                                                                             \
        if (rows <= 4) LAUNCH(T, 4);                                                                                 \
        else if (rows <= 8) LAUNCH(T, 8);                                                                            \
        else if (rows <= 16) LAUNCH(T, 16);                                                                          \
        else if (rows <= 32) LAUNCH(T, 32);                                                                          \
        else if (rows <= 64) LAUNCH(T, 64);                                                                          \
        else LAUNCH(T, 128);                                                                                         \
        if (raw)                                                                                                     \
            hipLaunchKernelGGL(gla_finish_kernel<T>, fgrid, fblock, 0, stream, workspace, (const T*)proj,            \
                               proj_stride, g_col, norm_w, (T*)out, n_heads, Dv, eps);                               \
    } while (0)
    if (dtype == SIA_F32) RUN(float);
    else if (dtype == SIA_BF16) RUN(bf16_t);
    else return SIA_BAD_ARGUMENT;
#undef RUN
#undef LAUNCH
    return SIA_LAUNCH_CHECK();
}
