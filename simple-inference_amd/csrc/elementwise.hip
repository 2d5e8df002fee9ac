// Embedding gather, residual add + RMS norm, RMS norm of a sublayer's output + residual add, SwiGLU and plain
// activations.
//
// These are bound by memory traffic or by launch latency.  The residual stream is float
// in both modes; rows are handled by one workgroup each, with vector accesses where the
// row length allows.
#include "common.h"

// ---------------------------------------------------------------------------------------
// Embedding: out[n, :] = float(table[ids[n], :]) * scale   (reference: ops/embedding.py:57-60; scale 1 there)
// ---------------------------------------------------------------------------------------
template <typename T>
__global__ void embed_kernel(const int* __restrict__ ids, const T* __restrict__ table,
                             float* __restrict__ out, int hidden, float scale) {
    const int n = blockIdx.x;
    const T* src = table + (size_t)ids[n] * hidden;
    float* dst = out + (size_t)n * hidden;
    for (int i = threadIdx.x; i < hidden; i += blockDim.x) dst[i] = to_float(src[i]) * scale;
}

SIA_EXPORT int sia_embed(const int* ids, const void* table, float* out, int n_tokens, int hidden,
                         int table_dtype, float scale, hipStream_t stream) {
    if (n_tokens <= 0) return 0;
    dim3 grid(n_tokens), block(256);
    if (table_dtype == SIA_F32)
        hipLaunchKernelGGL(embed_kernel<float>, grid, block, 0, stream, ids, (const float*)table, out, hidden, scale);
    else if (table_dtype == SIA_BF16)
        hipLaunchKernelGGL(embed_kernel<bf16_t>, grid, block, 0, stream, ids, (const bf16_t*)table, out, hidden, scale);
    else
        return SIA_BAD_ARGUMENT;
    return SIA_LAUNCH_CHECK();
}

// ---------------------------------------------------------------------------------------
// Residual add + RMS norm  (reference: ops/rmsnorm.py:41-46, kernels/rmsnorm_kernel.py:105-113)
//
//   x = residual[row] + delta[row]            (float; delta may be absent)
//   y = x * rsqrt(mean(x^2) + eps) * w        (float, one rounding to the output type)
//
// rows == nullptr: every row r of the batch; x is written back into residual[r].
// rows != nullptr: out[i] comes from row rows[i]; residual is not written.
// The sum of squares is reduced in a fixed order that depends on the row length only.
// ---------------------------------------------------------------------------------------
// SCALED: the delta is multiplied by a constant, and a second delta with a constant of its own may join it
// (x = residual + f1 * delta + f2 * delta2); without a weight only the sum is made.
template <typename T, bool SCALED>
__global__ void add_rmsnorm_kernel(float* __restrict__ residual, const T* __restrict__ delta,
                                   const float* __restrict__ weight, T* __restrict__ out,
                                   const int* __restrict__ rows, int hidden, float eps, float f1,
                                   const T* __restrict__ delta2, float f2) {
    __shared__ float scratch[16];
    const int i_out = blockIdx.x;
    const int row = rows ? rows[i_out] : i_out;
    float* res = residual + (size_t)row * hidden;
    const T* del = delta ? delta + (size_t)row * hidden : nullptr;
    const T* del2 = (SCALED && delta2) ? delta2 + (size_t)row * hidden : nullptr;
    T* dst = out + (size_t)i_out * hidden;

    float ss = 0.f;
    for (int i = threadIdx.x; i < hidden; i += blockDim.x) {
        float x = res[i];
        if (del) x += SCALED ? f1 * to_float(del[i]) : to_float(del[i]);
        if (del2) x += f2 * to_float(del2[i]);
        if (!rows && del) res[i] = x;
        ss += x * x;
    }
    if (SCALED && !weight) return;   // uniform
    ss = block_sum(ss, scratch);
    const float inv = rsqrtf(ss / (float)hidden + eps);
    for (int i = threadIdx.x; i < hidden; i += blockDim.x) {
        float x = res[i];
        if (rows && del) x += SCALED ? f1 * to_float(del[i]) : to_float(del[i]);
        if (rows && del2) x += f2 * to_float(del2[i]);
        dst[i] = from_float<T>(x * inv * weight[i]);
    }
}

// The same for rows that one workgroup holds in registers (hidden % 8 == 0, hidden <= 8 * 1024): each
// thread takes 8 consecutive elements with 16- and 32-byte accesses, every input is read once and all
// loads (the gain's included) are issued before the first is used.
template <typename T, bool SCALED>
__global__ void add_rmsnorm_row_kernel(float* __restrict__ residual, const T* __restrict__ delta,
                                       const float* __restrict__ weight, T* __restrict__ out,
                                       const int* __restrict__ rows, int hidden, float eps, float f1,
                                       const T* __restrict__ delta2, float f2) {
    __shared__ float scratch[16];
    const int i_out = blockIdx.x;
    const int row = rows ? rows[i_out] : i_out;
    const int i0 = threadIdx.x * 8;
    const bool live = i0 < hidden;
    float x[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f}, w[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f}, d[8];
    if (live) {
        Vec8<float> vr, vw;
        Vec8<T> vd, vd2;
        vr.load(residual + (size_t)row * hidden + i0);
        if (!SCALED || weight) vw.load(weight + i0);
        if (delta) vd.load(delta + (size_t)row * hidden + i0);
        if (SCALED && delta2) vd2.load(delta2 + (size_t)row * hidden + i0);
        vr.get(x);
        if (!SCALED || weight) vw.get(w);
        if (delta) {
            vd.get(d);
#pragma unroll
            for (int i = 0; i < 8; ++i) x[i] += SCALED ? f1 * d[i] : d[i];
            if (SCALED && delta2) {
                vd2.get(d);
#pragma unroll
                for (int i = 0; i < 8; ++i) x[i] += f2 * d[i];
            }
            if (!rows) {
                vr.set(x);
                vr.store(residual + (size_t)row * hidden + i0);
            }
        }
    }
    if (SCALED && !weight) return;   // uniform: only the sum was asked for
    float ss = 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i) ss += x[i] * x[i];
    ss = block_sum(ss, scratch);
    if (live) {
        const float inv = rsqrtf(ss / (float)hidden + eps);
#pragma unroll
        for (int i = 0; i < 8; ++i) x[i] = x[i] * inv * w[i];
        Vec8<T> vo;
        vo.set(x);
        vo.store(out + (size_t)i_out * hidden + i0);
    }
}

template <bool SCALED>
static int launch_add_rmsnorm(float* residual, const void* delta, float f1, const void* delta2, float f2,
                              const float* weight, void* out, const int* rows, int n_out, int hidden, float eps,
                              int dtype, hipStream_t stream) {
    if (n_out <= 0) return 0;
    if (dtype != SIA_F32 && dtype != SIA_BF16) return SIA_BAD_ARGUMENT;
    dim3 grid(n_out);
    if (hidden % 8 == 0 && hidden <= 8 * 1024) {
        dim3 block(((hidden / 8 + SIA_WAVE - 1) / SIA_WAVE) * SIA_WAVE);
        if (dtype == SIA_F32)
            hipLaunchKernelGGL((add_rmsnorm_row_kernel<float, SCALED>), grid, block, 0, stream, residual,
                               (const float*)delta, weight, (float*)out, rows, hidden, eps, f1, (const float*)delta2, f2);
        else
            hipLaunchKernelGGL((add_rmsnorm_row_kernel<bf16_t, SCALED>), grid, block, 0, stream, residual,
                               (const bf16_t*)delta, weight, (bf16_t*)out, rows, hidden, eps, f1, (const bf16_t*)delta2,
                               f2);
        return SIA_LAUNCH_CHECK();
    }
    dim3 block(hidden >= 2048 ? 512 : 256);
    if (dtype == SIA_F32)
        hipLaunchKernelGGL((add_rmsnorm_kernel<float, SCALED>), grid, block, 0, stream, residual, (const float*)delta,
                           weight, (float*)out, rows, hidden, eps, f1, (const float*)delta2, f2);
    else
        hipLaunchKernelGGL((add_rmsnorm_kernel<bf16_t, SCALED>), grid, block, 0, stream, residual, (const bf16_t*)delta,
                           weight, (bf16_t*)out, rows, hidden, eps, f1, (const bf16_t*)delta2, f2);
    return SIA_LAUNCH_CHECK();
}

SIA_EXPORT int sia_add_rmsnorm(float* residual, const void* delta, const float* weight, void* out,
                               const int* rows, int n_out, int hidden, float eps, int dtype,
                               hipStream_t stream) {
    return launch_add_rmsnorm<false>(residual, delta, 1.f, nullptr, 0.f, weight, out, rows, n_out, hidden, eps, dtype,
                                     stream);
}

// x = residual + f1 * delta + f2 * delta2 (delta2 may be absent) and, with a weight, the RMS norm of x; without one
// only the sum is made (rows must then be absent, so that the residual keeps it).
SIA_EXPORT int sia_add_rmsnorm_scaled(float* residual, const void* delta, float f1, const void* delta2, float f2,
                                      const float* weight, void* out, const int* rows, int n_out, int hidden,
                                      float eps, int dtype, hipStream_t stream) {
    if (!delta || (!weight && rows) || (weight && !out)) return SIA_BAD_ARGUMENT;
    return launch_add_rmsnorm<true>(residual, delta, f1, delta2, f2, weight, out, rows, n_out, hidden, eps, dtype,
                                    stream);
}

// ---------------------------------------------------------------------------------------
// RMS norm of a sublayer's output, added into the residual:
//
//   residual[row] += y[row] * rsqrt(mean(y[row]^2) + eps) * w         (all float)
//   lowered[row]   = the new residual[row], rounded to T               (if lowered is given)
//
// for layers whose norm sits behind the sublayer and whose sublayers read the residual itself.  One workgroup a
// row; the sum of squares is reduced in a fixed order that depends on the row length only.
// ---------------------------------------------------------------------------------------
template <typename T>
__global__ void norm_add_kernel(float* __restrict__ residual, const T* __restrict__ y,
                                const float* __restrict__ weight, T* __restrict__ lowered, int hidden, float eps) {
    __shared__ float scratch[16];
    const size_t base = (size_t)blockIdx.x * hidden;
    float ss = 0.f;
    for (int i = threadIdx.x; i < hidden; i += blockDim.x) {
        const float v = to_float(y[base + i]);
        ss += v * v;
    }
    ss = block_sum(ss, scratch);
    const float inv = rsqrtf(ss / (float)hidden + eps);
    for (int i = threadIdx.x; i < hidden; i += blockDim.x) {
        const float x = residual[base + i] + to_float(y[base + i]) * inv * weight[i];
        residual[base + i] = x;
        if (lowered) lowered[base + i] = from_float<T>(x);
    }
}

// The same for rows that one workgroup holds in registers (hidden % 8 == 0, hidden <= 8 * 1024): 8 consecutive
// elements a thread, every input read once, all loads issued before the first is used.
template <typename T>
__global__ void norm_add_row_kernel(float* __restrict__ residual, const T* __restrict__ y,
                                    const float* __restrict__ weight, T* __restrict__ lowered, int hidden, float eps) {
    __shared__ float scratch[16];
    const size_t base = (size_t)blockIdx.x * hidden;
    const int i0 = threadIdx.x * 8;
    const bool live = i0 < hidden;
    float x[8], w[8], v[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    if (live) {
        Vec8<float> vr, vw;
        Vec8<T> vy;
        vr.load(residual + base + i0);
        vw.load(weight + i0);
        vy.load(y + base + i0);
        vr.get(x);
        vw.get(w);
        vy.get(v);
    }
    float ss = 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i) ss += v[i] * v[i];
    ss = block_sum(ss, scratch);
    if (live) {
        const float inv = rsqrtf(ss / (float)hidden + eps);
#pragma unroll
        for (int i = 0; i < 8; ++i) x[i] += v[i] * inv * w[i];
        Vec8<float> vr;
        vr.set(x);
        vr.store(residual + base + i0);
        if (lowered) {
            Vec8<T> vo;
            vo.set(x);
            vo.store(lowered + base + i0);
        }
    }
}

SIA_EXPORT int sia_norm_add(float* residual, const void* y, const float* weight, void* lowered, int n_rows,
                            int hidden, float eps, int dtype, hipStream_t stream) {
    if (n_rows <= 0) return 0;
    if ((dtype != SIA_F32 && dtype != SIA_BF16) || hidden <= 0 || !residual || !y || !weight) return SIA_BAD_ARGUMENT;
    dim3 grid(n_rows);
    const bool row = hidden % 8 == 0 && hidden <= 8 * 1024;
    dim3 block(row ? ((hidden / 8 + SIA_WAVE - 1) / SIA_WAVE) * SIA_WAVE : (hidden >= 2048 ? 512 : 256));
#define LAUNCH(KERNEL, T)                                                                                         \
    hipLaunchKernelGGL(KERNEL<T>, grid, block, 0, stream, residual, (const T*)y, weight, (T*)lowered, hidden, eps)
    if (row) {
        if (dtype == SIA_F32) LAUNCH(norm_add_row_kernel, float);
        else LAUNCH(norm_add_row_kernel, bf16_t);
    } else {
        if (dtype == SIA_F32) LAUNCH(norm_add_kernel, float);
        else LAUNCH(norm_add_kernel, bf16_t);
    }
#undef LAUNCH
    return SIA_LAUNCH_CHECK();
}

// ---------------------------------------------------------------------------------------
// Plain activations, in float on the stored value, rounded once:
//   SIA_RELU2:      max(z, 0)^2
//   SIA_GELU_TANH:  0.5 z (1 + tanh(sqrt(2/pi) (z + 0.044715 z^3)))
// ---------------------------------------------------------------------------------------
template <typename T>
__global__ void activation_kernel(const T* __restrict__ in, T* __restrict__ out, size_t n, int kind) {
    const size_t i = ((size_t)blockIdx.x * blockDim.x + threadIdx.x) * 8;
    if (i >= n) return;
    if (i + 8 <= n) {
        Vec8<T> v;
        float z[8];
        v.load(in + i);
        v.get(z);
#pragma unroll
        for (int j = 0; j < 8; ++j) z[j] = activate(z[j], kind);
        v.set(z);
        v.store(out + i);
    } else {
        for (size_t j = i; j < n; ++j) out[j] = from_float<T>(activate(to_float(in[j]), kind));
    }
}

// Eight elements a thread; the last thread takes what is left one by one.
SIA_EXPORT int sia_activation(const void* in, void* out, long long n, int kind, int dtype, hipStream_t stream) {
    if (n <= 0) return 0;
    if ((dtype != SIA_F32 && dtype != SIA_BF16) || (kind != SIA_RELU2 && kind != SIA_GELU_TANH && kind != SIA_GELU)) return SIA_BAD_ARGUMENT;
    dim3 block(256), grid((unsigned)(((n + 7) / 8 + 255) / 256));
    if (dtype == SIA_F32)
        hipLaunchKernelGGL(activation_kernel<float>, grid, block, 0, stream, (const float*)in, (float*)out, (size_t)n, kind);
    else
        hipLaunchKernelGGL(activation_kernel<bf16_t>, grid, block, 0, stream, (const bf16_t*)in, (bf16_t*)out, (size_t)n, kind);
    return SIA_LAUNCH_CHECK();
}

// ---------------------------------------------------------------------------------------
// A gated activation of another kind than SwiGLU over rows [gate (I) | up (I)] (``gated_activation`` of common.h),
// and the sum of up to two matrices with a constant factor each.
// ---------------------------------------------------------------------------------------
template <typename T>
__global__ void glu_kernel(const T* __restrict__ gu, T* __restrict__ out, int inter, int kind, float limit) {
    const int n = blockIdx.y;
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= inter) return;
    const T* row = gu + (size_t)n * 2 * inter;
    out[(size_t)n * inter + i] = from_float<T>(gated_activation(to_float(row[i]), to_float(row[inter + i]), kind, limit));
}

// Eight elements a thread, 16- or 32-byte accesses (inter % 8 == 0).
template <typename T>
__global__ void glu_vec_kernel(const T* __restrict__ gu, T* __restrict__ out, int inter, int kind, float limit) {
    const int n = blockIdx.y;
    const int i = (blockIdx.x * blockDim.x + threadIdx.x) * 8;
    if (i >= inter) return;
    const T* row = gu + (size_t)n * 2 * inter;
    Vec8<T> vg, vu;
    vg.load(row + i);
    vu.load(row + inter + i);
    float g[8], u[8];
    vg.get(g);
    vu.get(u);
#pragma unroll
    for (int j = 0; j < 8; ++j) g[j] = gated_activation(g[j], u[j], kind, limit);
    vg.set(g);
    vg.store(out + (size_t)n * inter + i);
}

SIA_EXPORT int sia_glu(const void* gu, void* out, int n_tokens, int inter, int kind, float limit, int dtype,
                       hipStream_t stream) {
    if (n_tokens <= 0) return 0;
    if (n_tokens > 65535 || inter <= 0 || (dtype != SIA_F32 && dtype != SIA_BF16) ||
        (kind != SIA_GLU_SILU && kind != SIA_GLU_CLAMPED))
        return SIA_BAD_ARGUMENT;
    if (inter % 8 == 0) {
        dim3 block(256), grid((inter / 8 + 255) / 256, n_tokens);
        if (dtype == SIA_F32)
            hipLaunchKernelGGL(glu_vec_kernel<float>, grid, block, 0, stream, (const float*)gu, (float*)out, inter, kind,
                               limit);
        else
            hipLaunchKernelGGL(glu_vec_kernel<bf16_t>, grid, block, 0, stream, (const bf16_t*)gu, (bf16_t*)out, inter,
                               kind, limit);
        return SIA_LAUNCH_CHECK();
    }
    dim3 block(256), grid((inter + 255) / 256, n_tokens);
    if (dtype == SIA_F32)
        hipLaunchKernelGGL(glu_kernel<float>, grid, block, 0, stream, (const float*)gu, (float*)out, inter, kind, limit);
    else
        hipLaunchKernelGGL(glu_kernel<bf16_t>, grid, block, 0, stream, (const bf16_t*)gu, (bf16_t*)out, inter, kind, limit);
    return SIA_LAUNCH_CHECK();
}

template <typename T>
__global__ void scaled_sum_kernel(const T* __restrict__ a, float fa, const T* __restrict__ b, float fb,
                                  T* __restrict__ out, size_t n) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    float x = fa * to_float(a[i]);
    if (b) x += fb * to_float(b[i]);
    out[i] = from_float<T>(x);
}

SIA_EXPORT int sia_scaled_sum(const void* a, float fa, const void* b, float fb, void* out, long long n, int dtype,
                              hipStream_t stream) {
    if (n <= 0) return 0;
    if (!a || !out || (dtype != SIA_F32 && dtype != SIA_BF16)) return SIA_BAD_ARGUMENT;
    dim3 block(256), grid((unsigned)((n + 255) / 256));
    if (dtype == SIA_F32)
        hipLaunchKernelGGL(scaled_sum_kernel<float>, grid, block, 0, stream, (const float*)a, fa, (const float*)b, fb,
                           (float*)out, (size_t)n);
    else
        hipLaunchKernelGGL(scaled_sum_kernel<bf16_t>, grid, block, 0, stream, (const bf16_t*)a, fa, (const bf16_t*)b, fb,
                           (bf16_t*)out, (size_t)n);
    return SIA_LAUNCH_CHECK();
}

// ---------------------------------------------------------------------------------------
// SwiGLU: out[n, i] = silu(gu[n, i]) * gu[n, I + i], silu(g) = g / (1 + exp(-g)), in float
// (reference: ops/mlp.py:117-128, kernels/swiglu_kernel.py:142-150)
// ---------------------------------------------------------------------------------------
template <typename T>
__global__ void swiglu_kernel(const T* __restrict__ gu, T* __restrict__ out, int inter) {
    const int n = blockIdx.y;
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= inter) return;
    const T* row = gu + (size_t)n * 2 * inter;
    const float g = to_float(row[i]);
    const float u = to_float(row[inter + i]);
    out[(size_t)n * inter + i] = from_float<T>(g / (1.f + expf(-g)) * u);
}

// Eight elements a thread, 16- or 32-byte accesses (inter % 8 == 0).
template <typename T>
__global__ void swiglu_vec_kernel(const T* __restrict__ gu, T* __restrict__ out, int inter) {
    const int n = blockIdx.y;
    const int i = (blockIdx.x * blockDim.x + threadIdx.x) * 8;
    if (i >= inter) return;
    const T* row = gu + (size_t)n * 2 * inter;
    Vec8<T> vg, vu;
    vg.load(row + i);
    vu.load(row + inter + i);
    float g[8], u[8];
    vg.get(g);
    vu.get(u);
#pragma unroll
    for (int j = 0; j < 8; ++j) g[j] = g[j] / (1.f + expf(-g[j])) * u[j];
    vg.set(g);
    vg.store(out + (size_t)n * inter + i);
}

SIA_EXPORT int sia_swiglu(const void* gu, void* out, int n_tokens, int inter, int dtype, hipStream_t stream) {
    if (n_tokens <= 0) return 0;
    if (n_tokens > 65535) return SIA_BAD_ARGUMENT;
    if (dtype != SIA_F32 && dtype != SIA_BF16) return SIA_BAD_ARGUMENT;
    if (inter % 8 == 0) {
        dim3 block(256), grid((inter / 8 + 255) / 256, n_tokens);
        if (dtype == SIA_F32)
            hipLaunchKernelGGL(swiglu_vec_kernel<float>, grid, block, 0, stream, (const float*)gu, (float*)out, inter);
        else
            hipLaunchKernelGGL(swiglu_vec_kernel<bf16_t>, grid, block, 0, stream, (const bf16_t*)gu, (bf16_t*)out, inter);
        return SIA_LAUNCH_CHECK();
    }
    dim3 block(256), grid((inter + 255) / 256, n_tokens);
    if (dtype == SIA_F32)
        hipLaunchKernelGGL(swiglu_kernel<float>, grid, block, 0, stream, (const float*)gu, (float*)out, inter);
    else
        hipLaunchKernelGGL(swiglu_kernel<bf16_t>, grid, block, 0, stream, (const bf16_t*)gu, (bf16_t*)out, inter);
    return SIA_LAUNCH_CHECK();
}

// ---------------------------------------------------------------------------------------
// Casts between the two element types (used where a float32-stored matrix meets bfloat16
// activations).
// ---------------------------------------------------------------------------------------
__global__ void cast_bf16_to_f32_kernel(const bf16_t* __restrict__ in, float* __restrict__ out, size_t n) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) out[i] = bf16_to_float(in[i]);
}
__global__ void cast_f32_to_bf16_kernel(const float* __restrict__ in, bf16_t* __restrict__ out, size_t n) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) out[i] = float_to_bf16(in[i]);
}

SIA_EXPORT int sia_cast(const void* in, void* out, long long n, int in_dtype, hipStream_t stream) {
    if (n <= 0) return 0;
    dim3 block(256), grid((unsigned)((n + 255) / 256));
    if (in_dtype == SIA_BF16)
        hipLaunchKernelGGL(cast_bf16_to_f32_kernel, grid, block, 0, stream, (const bf16_t*)in, (float*)out, (size_t)n);
    else if (in_dtype == SIA_F32)
        hipLaunchKernelGGL(cast_f32_to_bf16_kernel, grid, block, 0, stream, (const float*)in, (bf16_t*)out, (size_t)n);
    else
        return SIA_BAD_ARGUMENT;
    return SIA_LAUNCH_CHECK();
}

// out[m][k] = scaled[m][k] * rsqrt(sum_p partials[p][m] / width + eps): finishes the norm that a product with a
// residual epilogue left unfinished, for a consumer that cannot scale its own rows.
__global__ __launch_bounds__(256) void scale_rows_kernel(const bf16_t* __restrict__ scaled,
                                                         const float* __restrict__ partials, bf16_t* __restrict__ out,
                                                         int width, int n_partials, float eps) {
    __shared__ float sums[256];
    const int m = blockIdx.x;
    float ss = 0.f;
    for (int p = threadIdx.x; p < n_partials; p += 256) ss += partials[p * 16 + m];
    sums[threadIdx.x] = ss;
    __syncthreads();
    for (int half = 128; half > 0; half >>= 1) {
        if ((int)threadIdx.x < half) sums[threadIdx.x] += sums[threadIdx.x + half];
        __syncthreads();
    }
    const float rs = rsqrtf(sums[0] / (float)width + eps);
    for (int k = threadIdx.x; k < width; k += 256)
        out[(size_t)m * width + k] = float_to_bf16(bf16_to_float(scaled[(size_t)m * width + k]) * rs);
}

SIA_EXPORT int sia_scale_rows(const void* scaled, const float* partials, void* out, int rows, int width,
                              int n_partials, float eps, hipStream_t stream) {
    if (rows <= 0) return 0;
    if (rows > 16 || width <= 0 || n_partials <= 0) return SIA_BAD_ARGUMENT;
    hipLaunchKernelGGL(scale_rows_kernel, dim3(rows), dim3(256), 0, stream, (const bf16_t*)scaled, partials,
                       (bf16_t*)out, width, n_partials, eps);
    return SIA_LAUNCH_CHECK();
}

// dst[dst_rows[i]] = src[src_rows[i]]: token ids that a sampler has left on the device become the input of the
// next step without a trip through the host.
__global__ __launch_bounds__(256) void place_tokens_kernel(int* __restrict__ dst, const int* __restrict__ dst_rows,
                                                           const int* __restrict__ src,
                                                           const int* __restrict__ src_rows, int n) {
    const int i = blockIdx.x * 256 + threadIdx.x;
    if (i < n) dst[dst_rows[i]] = src[src_rows[i]];
}

SIA_EXPORT int sia_place_tokens(int* dst, const int* dst_rows, const int* src, const int* src_rows, int n,
                                hipStream_t stream) {
    if (n <= 0) return 0;
    if (!dst || !dst_rows || !src || !src_rows) return SIA_BAD_ARGUMENT;
    hipLaunchKernelGGL(place_tokens_kernel, dim3((n + 255) / 256), dim3(256), 0, stream, dst, dst_rows, src, src_rows,
                       n);
    return SIA_LAUNCH_CHECK();
}
