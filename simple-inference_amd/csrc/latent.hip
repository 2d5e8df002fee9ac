// Latent attention: what is kept of a token, and the products that stand on the query's side of the page attention.
//
// latent_prepare, a workgroup a token, from the projected row [a_q (q_rank) | a (kv_rank) | b (rot_dim)]:
//   c_q = a_q * rsqrt(mean(a_q^2) + eps) * g_q                     -> cq [tokens, q_rank]
//   c   = a * rsqrt(mean(a^2) + eps) * g_kv                        -> the key row's first kv_rank elements, and the
//                                                                     value rows 0 .. kv_rank - 1 of the position
//   k   = b with neighbouring pairs (2i, 2i + 1), i < rotary_dim / 2, turned by the position's cos/sin row
//                                                                  -> the key row's next rot_dim elements
// Key pages [pages, 1, page_size, key_width], value pages [pages, 1, value_rows, page_size]; what lies beyond a row's
// own elements is never written (it is zero since the pool was made).  With kv_rank == 0 only c_q is made.
// Norms and rotation are float on the projection's output, one rounding.
//
// headwise_linear: y[n, h, o] = sum_i x[n, h, i] * w[h, o, i] for every head, x rows in_stride apart per head, y rows
// out_stride apart; a head's ``tail`` elements behind the in_dim inputs are copied behind the out_dim outputs, with
// their first rotary_dim elements turned as above, and the rest of a head's out_stride is set to zero.  Float sums.
// Three forms: a wave an output element for steps of up to 16 rows, matrix cores for more rows in bfloat16 where the
// 16-byte loads are aligned, and an LDS-tiled form on the vector units for everything else (float32, odd sizes).
#include "common.h"

template <typename T>
__global__ __launch_bounds__(256) void latent_prepare_kernel(
    const T* __restrict__ proj, int row_stride, int q_rank, const float* __restrict__ q_gain, int kv_rank,
    const float* __restrict__ kv_gain, int rot_dim, int rotary_dim, const float* __restrict__ cos_t,
    const float* __restrict__ sin_t, float eps, const int* __restrict__ positions, const int* __restrict__ seq_of_token,
    const int* __restrict__ table, int table_width, T* __restrict__ k_pages, T* __restrict__ v_pages, int page_size,
    int key_width, int value_rows, T* __restrict__ cq) {
    __shared__ float scratch[16];
    const int n = blockIdx.x, tid = threadIdx.x;
    const T* row = proj + (size_t)n * row_stride;
    float ss = 0.f;
    for (int i = tid; i < q_rank; i += blockDim.x) {
        const float v = to_float(row[i]);
        ss += v * v;
    }
    float inv = rsqrtf(block_sum(ss, scratch) / (float)q_rank + eps);
    for (int i = tid; i < q_rank; i += blockDim.x)
        cq[(size_t)n * q_rank + i] = from_float<T>(to_float(row[i]) * inv * q_gain[i]);
    if (kv_rank == 0) return;
    const T* a = row + q_rank;
    ss = 0.f;
    for (int i = tid; i < kv_rank; i += blockDim.x) {
        const float v = to_float(a[i]);
        ss += v * v;
    }
    inv = rsqrtf(block_sum(ss, scratch) / (float)kv_rank + eps);
    const int pos = positions[n];
    const int page = table[(size_t)seq_of_token[n] * table_width + pos / page_size];
    if (page < 0) return;
    const int off = pos % page_size;
    T* k_row = k_pages + ((size_t)page * page_size + off) * key_width;
    T* v_col = v_pages + (size_t)page * value_rows * page_size + off;
    for (int i = tid; i < kv_rank; i += blockDim.x) {
        const T c = from_float<T>(to_float(a[i]) * inv * kv_gain[i]);
        k_row[i] = c;
        v_col[(size_t)i * page_size] = c;
    }
    const T* b = a + kv_rank;
    const int half = rotary_dim / 2;
    for (int i = tid; i < rot_dim; i += blockDim.x) {
        float v = to_float(b[i]);
        if (i < rotary_dim) {
            const float other = to_float(b[i ^ 1]);
            const float c = cos_t[(size_t)pos * half + i / 2], s = sin_t[(size_t)pos * half + i / 2];
            v = (i & 1) ? v * c + other * s : v * c - other * s;
        }
        k_row[kv_rank + i] = from_float<T>(v);
    }
}

SIA_EXPORT int sia_latent_prepare(const void* proj, int row_stride, int q_rank, const float* q_gain, int kv_rank,
                                  const float* kv_gain, int rot_dim, int rotary_dim, const float* cos_t,
                                  const float* sin_t, float eps, const int* positions, const int* seq_of_token,
                                  const int* table, int table_width, void* k_pages, void* v_pages, int page_size,
                                  int key_width, int value_rows, void* cq, int n_tokens, int dtype, hipStream_t stream) {
    if (n_tokens <= 0) return 0;
    if (q_rank <= 0 || !q_gain || !cq || kv_rank < 0 || rot_dim < 0 || rotary_dim < 0 || rotary_dim % 2 ||
        rotary_dim > rot_dim || row_stride < q_rank + (kv_rank ? kv_rank + rot_dim : 0))
        return SIA_BAD_ARGUMENT;
    if (kv_rank && (!kv_gain || !table || !k_pages || !v_pages || page_size <= 0 || key_width < kv_rank + rot_dim ||
                    value_rows < kv_rank || !positions || !seq_of_token || (rotary_dim && (!cos_t || !sin_t))))
        return SIA_BAD_ARGUMENT;
    dim3 grid(n_tokens), block(256);
    if (dtype == SIA_F32)
        hipLaunchKernelGGL(latent_prepare_kernel<float>, grid, block, 0, stream, (const float*)proj, row_stride, q_rank,
                           q_gain, kv_rank, kv_gain, rot_dim, rotary_dim, cos_t, sin_t, eps, positions, seq_of_token, table,
                           table_width, (float*)k_pages, (float*)v_pages, page_size, key_width, value_rows, (float*)cq);
    else if (dtype == SIA_BF16)
        hipLaunchKernelGGL(latent_prepare_kernel<bf16_t>, grid, block, 0, stream, (const bf16_t*)proj, row_stride, q_rank,
                           q_gain, kv_rank, kv_gain, rot_dim, rotary_dim, cos_t, sin_t, eps, positions, seq_of_token, table,
                           table_width, (bf16_t*)k_pages, (bf16_t*)v_pages, page_size, key_width, value_rows, (bf16_t*)cq);
    else
        return SIA_BAD_ARGUMENT;
    return SIA_LAUNCH_CHECK();
}

// Behind a head's outputs: the head's tail, its first rotary_dim elements turned in neighbouring pairs, and zeros up to
// the head's stride, for tokens n0 .. n0 + tokens - 1 of head h, by all threads of the workgroup.
template <typename T>
__device__ __forceinline__ void headwise_tail(const T* __restrict__ x, int x_row, int in_stride, T* __restrict__ y,
                                              int y_row, int out_stride, int n_tokens, int in_dim, int out_dim, int tail,
                                              int rotary_dim, const float* __restrict__ cos_t,
                                              const float* __restrict__ sin_t, const int* __restrict__ positions,
                                              int n0, int tokens, int h) {
    const int rest = out_stride - out_dim, half = rotary_dim / 2;
    for (int idx = threadIdx.x; idx < tokens * rest; idx += blockDim.x) {
        const int n = n0 + idx / rest, i = idx % rest;
        if (n >= n_tokens) break;
        float v = 0.f;
        if (i < tail) {
            const T* src = x + (size_t)n * x_row + (size_t)h * in_stride + in_dim;
            v = to_float(src[i]);
            if (i < rotary_dim) {
                const int pos = positions[n];
                const float other = to_float(src[i ^ 1]);
                const float c = cos_t[(size_t)pos * half + i / 2], s = sin_t[(size_t)pos * half + i / 2];
                v = (i & 1) ? v * c + other * s : v * c - other * s;
            }
        }
        y[(size_t)n * y_row + (size_t)h * out_stride + out_dim + i] = from_float<T>(v);
    }
}

#define HW_TOKENS 16
#define HW_OUTS 64
#define HW_K 32

template <typename T>
__global__ __launch_bounds__(256) void headwise_linear_kernel(const T* __restrict__ x, int x_row, int in_stride,
                                                              const T* __restrict__ w, T* __restrict__ y, int y_row,
                                                              int out_stride, int n_tokens, int in_dim, int out_dim,
                                                              int tail, int rotary_dim, const float* __restrict__ cos_t,
                                                              const float* __restrict__ sin_t,
                                                              const int* __restrict__ positions) {
    __shared__ float xs[HW_TOKENS][HW_K];
    __shared__ float ws[HW_OUTS][HW_K + 1];
    const int n0 = blockIdx.x * HW_TOKENS, h = blockIdx.y, o0 = blockIdx.z * HW_OUTS, tid = threadIdx.x;
    const int o = tid % HW_OUTS, tg = tid / HW_OUTS;     // this thread: one output column, four tokens
    const T* wh = w + (size_t)h * out_dim * in_dim;
    float acc[4] = {0.f, 0.f, 0.f, 0.f};
    for (int k0 = 0; k0 < in_dim; k0 += HW_K) {
        for (int idx = tid; idx < HW_TOKENS * HW_K; idx += blockDim.x) {
            const int t = idx / HW_K, kk = idx % HW_K;
            xs[t][kk] = (n0 + t < n_tokens && k0 + kk < in_dim)
                            ? to_float(x[(size_t)(n0 + t) * x_row + (size_t)h * in_stride + k0 + kk]) : 0.f;
        }
        for (int idx = tid; idx < HW_OUTS * HW_K; idx += blockDim.x) {
            const int oo = idx / HW_K, kk = idx % HW_K;
            ws[oo][kk] = (o0 + oo < out_dim && k0 + kk < in_dim) ? to_float(wh[(size_t)(o0 + oo) * in_dim + k0 + kk]) : 0.f;
        }
        __syncthreads();
#pragma unroll
        for (int kk = 0; kk < HW_K; ++kk) {
            const float a = ws[o][kk];
#pragma unroll
            for (int t = 0; t < 4; ++t) acc[t] += xs[tg * 4 + t][kk] * a;
        }
        __syncthreads();
    }
#pragma unroll
    for (int t = 0; t < 4; ++t) {
        const int n = n0 + tg * 4 + t;
        if (n < n_tokens && o0 + o < out_dim) y[(size_t)n * y_row + (size_t)h * out_stride + o0 + o] = from_float<T>(acc[t]);
    }
    if (blockIdx.z != 0) return;
    headwise_tail<T>(x, x_row, in_stride, y, y_row, out_stride, n_tokens, in_dim, out_dim, tail, rotary_dim, cos_t, sin_t,
                     positions, n0, HW_TOKENS, h);
}

// A step of few rows (decode): a wave an output element of a head, for all the rows; the head's weight row is read once
// from memory (again from the cache for every further row), sums in float.
template <typename T>
__global__ __launch_bounds__(256) void headwise_rows_kernel(const T* __restrict__ x, int x_row, int in_stride,
                                                            const T* __restrict__ w, T* __restrict__ y, int y_row,
                                                            int out_stride, int n_tokens, int in_dim, int out_dim,
                                                            int tail, int rotary_dim, const float* __restrict__ cos_t,
                                                            const float* __restrict__ sin_t,
                                                            const int* __restrict__ positions) {
    const int h = blockIdx.y, wave = threadIdx.x / SIA_WAVE, lane = threadIdx.x % SIA_WAVE;
    const int o = blockIdx.x * (blockDim.x / SIA_WAVE) + wave;
    if (o < out_dim) {
        const T* wr = w + ((size_t)h * out_dim + o) * in_dim;
        for (int n = 0; n < n_tokens; ++n) {
            const T* xr = x + (size_t)n * x_row + (size_t)h * in_stride;
            float acc = 0.f;
            for (int k = lane; k < in_dim; k += SIA_WAVE) acc += to_float(wr[k]) * to_float(xr[k]);
            acc = wave_sum(acc);
            if (lane == 0) y[(size_t)n * y_row + (size_t)h * out_stride + o] = from_float<T>(acc);
        }
    }
    if (blockIdx.x != 0) return;
    headwise_tail<T>(x, x_row, in_stride, y, y_row, out_stride, n_tokens, in_dim, out_dim, tail, rotary_dim, cos_t, sin_t,
                     positions, 0, n_tokens, h);
}

// Many rows in bfloat16 (prompts): matrix cores.  A workgroup 128 tokens and 32 output columns of a head, a wave 32 of
// the tokens: v_mfma_f32_16x16x32_bf16 with the weights' rows as first operand and the tokens' rows as second, both read
// k-contiguous from memory in 16-byte pieces (in_dim, the strides and the rows' starts multiples of 8 elements); what
// lies beyond in_dim in the last step of 32 is zero.
typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 hw_bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float hw_floatx4;

__global__ __launch_bounds__(256) void headwise_mfma_kernel(const bf16_t* __restrict__ x, int x_row, int in_stride,
                                                            const bf16_t* __restrict__ w, bf16_t* __restrict__ y,
                                                            int y_row, int out_stride, int n_tokens, int in_dim,
                                                            int out_dim, int tail, int rotary_dim,
                                                            const float* __restrict__ cos_t,
                                                            const float* __restrict__ sin_t,
                                                            const int* __restrict__ positions) {
    const int h = blockIdx.y, o0 = blockIdx.z * 32, n0 = blockIdx.x * 128;
    const int wave = threadIdx.x / SIA_WAVE, lane = threadIdx.x % SIA_WAVE, r = lane & 15, g = lane >> 4;
    const int t0 = n0 + wave * 32;
    if (t0 < n_tokens) {
        const bf16_t* xp[2];
        const bf16_t* wp[2];
#pragma unroll
        for (int mb = 0; mb < 2; ++mb)
            xp[mb] = x + (size_t)min(t0 + mb * 16 + r, n_tokens - 1) * x_row + (size_t)h * in_stride + g * 8;
#pragma unroll
        for (int nb = 0; nb < 2; ++nb)
            wp[nb] = w + ((size_t)h * out_dim + min(o0 + nb * 16 + r, out_dim - 1)) * in_dim + g * 8;
        hw_floatx4 acc[2][2];
#pragma unroll
        for (int nb = 0; nb < 2; ++nb)
#pragma unroll
            for (int mb = 0; mb < 2; ++mb) acc[nb][mb] = hw_floatx4{0.f, 0.f, 0.f, 0.f};
        const hw_bf16x8 zero = {0, 0, 0, 0, 0, 0, 0, 0};
        for (int k = 0; k < in_dim; k += 32) {
            const bool live = k + g * 8 < in_dim;
            hw_bf16x8 a[2], b[2];
#pragma unroll
            for (int mb = 0; mb < 2; ++mb) b[mb] = live ? *reinterpret_cast<const hw_bf16x8*>(xp[mb] + k) : zero;
#pragma unroll
            for (int nb = 0; nb < 2; ++nb) a[nb] = live ? *reinterpret_cast<const hw_bf16x8*>(wp[nb] + k) : zero;
#pragma unroll
            for (int nb = 0; nb < 2; ++nb)
#pragma unroll
                for (int mb = 0; mb < 2; ++mb)
                    acc[nb][mb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[nb], b[mb], acc[nb][mb], 0, 0, 0);
        }
        // acc[nb][mb][i]: output column o0 + nb * 16 + 4g + i of token t0 + mb * 16 + r
#pragma unroll
        for (int mb = 0; mb < 2; ++mb) {
            const int n = t0 + mb * 16 + r;
            if (n >= n_tokens) continue;
#pragma unroll
            for (int nb = 0; nb < 2; ++nb)
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const int c = o0 + nb * 16 + 4 * g + i;
                    if (c < out_dim) y[(size_t)n * y_row + (size_t)h * out_stride + c] = float_to_bf16(acc[nb][mb][i]);
                }
        }
    }
    if (blockIdx.z != 0) return;
    headwise_tail<bf16_t>(x, x_row, in_stride, y, y_row, out_stride, n_tokens, in_dim, out_dim, tail, rotary_dim, cos_t,
                          sin_t, positions, n0, 128, h);
}

SIA_EXPORT int sia_headwise_linear(const void* x, int x_row, int in_stride, const void* w, void* y, int y_row,
                                   int out_stride, int n_tokens, int n_heads, int in_dim, int out_dim, int tail,
                                   int rotary_dim, const float* cos_t, const float* sin_t, const int* positions, int dtype,
                                   hipStream_t stream) {
    if (n_tokens <= 0) return 0;
    if (n_heads <= 0 || n_heads > 65535 || in_dim <= 0 || out_dim <= 0 || tail < 0 || in_dim + tail > in_stride ||
        out_dim + tail > out_stride || x_row < n_heads * in_stride || y_row < n_heads * out_stride || rotary_dim < 0 ||
        rotary_dim % 2 || rotary_dim > tail || (rotary_dim && (!cos_t || !sin_t || !positions)) ||
        (out_dim + HW_OUTS - 1) / HW_OUTS > 65535)
        return SIA_BAD_ARGUMENT;
    dim3 grid((n_tokens + HW_TOKENS - 1) / HW_TOKENS, n_heads, (out_dim + HW_OUTS - 1) / HW_OUTS), block(256);
    if (n_tokens <= 16 && (out_dim + 3) / 4 <= 65535) {
        dim3 rgrid((out_dim + 3) / 4, n_heads);
        if (dtype == SIA_F32)
            hipLaunchKernelGGL(headwise_rows_kernel<float>, rgrid, block, 0, stream, (const float*)x, x_row, in_stride,
                               (const float*)w, (float*)y, y_row, out_stride, n_tokens, in_dim, out_dim, tail,
                               rotary_dim, cos_t, sin_t, positions);
        else if (dtype == SIA_BF16)
            hipLaunchKernelGGL(headwise_rows_kernel<bf16_t>, rgrid, block, 0, stream, (const bf16_t*)x, x_row, in_stride,
                               (const bf16_t*)w, (bf16_t*)y, y_row, out_stride, n_tokens, in_dim, out_dim, tail,
                               rotary_dim, cos_t, sin_t, positions);
        else
            return SIA_BAD_ARGUMENT;
        return SIA_LAUNCH_CHECK();
    }
    if (dtype == SIA_BF16 && in_dim % 8 == 0 && x_row % 8 == 0 && in_stride % 8 == 0 && ((uintptr_t)x % 16) == 0 &&
        ((uintptr_t)w % 16) == 0 && (out_dim + 31) / 32 <= 65535) {
        dim3 mgrid((n_tokens + 127) / 128, n_heads, (out_dim + 31) / 32);
        hipLaunchKernelGGL(headwise_mfma_kernel, mgrid, block, 0, stream, (const bf16_t*)x, x_row, in_stride,
                           (const bf16_t*)w, (bf16_t*)y, y_row, out_stride, n_tokens, in_dim, out_dim, tail, rotary_dim,
                           cos_t, sin_t, positions);
        return SIA_LAUNCH_CHECK();
    }
    if (dtype == SIA_F32)
        hipLaunchKernelGGL(headwise_linear_kernel<float>, grid, block, 0, stream, (const float*)x, x_row, in_stride,
                           (const float*)w, (float*)y, y_row, out_stride, n_tokens, in_dim, out_dim, tail, rotary_dim,
                           cos_t, sin_t, positions);
    else if (dtype == SIA_BF16)
        hipLaunchKernelGGL(headwise_linear_kernel<bf16_t>, grid, block, 0, stream, (const bf16_t*)x, x_row, in_stride,
                           (const bf16_t*)w, (bf16_t*)y, y_row, out_stride, n_tokens, in_dim, out_dim, tail, rotary_dim,
                           cos_t, sin_t, positions);
    else
        return SIA_BAD_ARGUMENT;
    return SIA_LAUNCH_CHECK();
}
