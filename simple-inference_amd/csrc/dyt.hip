// A norm without a statistic (dynamic tanh), with the residual add in front of it.
//
//   x   = residual (+ d)            d = delta, or if the delta passes a norm of this kind on its way:
//                                   d = (tanh(a1 * delta) * w1 + b1) * s1        (s1 optional: a layer scale)
//   out = (tanh(a2 * x) * w2 + b2) * s2                                          (s2 optional; the whole norm optional)
//
// All rows (the residual is left updated) or selected rows (the residual is left as it was: the model's last norm).
// Everything is float; delta and out are of the compute type, rounded once.  The scalars a1, a2 are read from
// device memory.  Elementwise: a workgroup a row, eight elements a thread and step where rows are aligned.
#include "common.h"

struct DytTerms {
    const float* w;
    const float* b;
    const float* alpha;
    const float* scale;
};

__device__ __forceinline__ float dyt_apply(float x, float a, float w, float b, float s) { return (tanhf(a * x) * w + b) * s; }

template <typename T, bool VEC>
__global__ __launch_bounds__(256) void dyt_norm_kernel(float* __restrict__ residual, const T* __restrict__ delta,
                                                       DytTerms post, DytTerms pre, T* __restrict__ out,
                                                       const int* __restrict__ rows, int width) {
    const int r_out = blockIdx.x;
    const int r = rows ? rows[r_out] : r_out;
    float* x = residual + (size_t)r * width;
    const T* d = delta ? delta + (size_t)r * width : nullptr;
    T* o = out ? out + (size_t)r_out * width : nullptr;
    const float a1 = (d && post.w) ? post.alpha[0] : 0.f;
    const float a2 = pre.w ? pre.alpha[0] : 0.f;
    const bool keep = rows == nullptr && d != nullptr;
    if (VEC) {
        for (int i = threadIdx.x * 8; i < width; i += blockDim.x * 8) {
            Vec8<float> xv;
            xv.load(x + i);
            float v[8];
            xv.get(v);
            if (d) {
                Vec8<T> dv;
                dv.load(d + i);
                float e[8];
                dv.get(e);
                if (post.w) {
                    Vec8<float> wv, bv;
                    wv.load(post.w + i);
                    bv.load(post.b + i);
                    float w[8], b[8], s[8];
                    wv.get(w);
                    bv.get(b);
                    if (post.scale) {
                        Vec8<float> sv;
                        sv.load(post.scale + i);
                        sv.get(s);
                    } else {
#pragma unroll
                        for (int j = 0; j < 8; ++j) s[j] = 1.f;
                    }
#pragma unroll
                    for (int j = 0; j < 8; ++j) e[j] = dyt_apply(e[j], a1, w[j], b[j], s[j]);
                }
#pragma unroll
                for (int j = 0; j < 8; ++j) v[j] += e[j];
                if (keep) {
                    xv.set(v);
                    xv.store(x + i);
                }
            }
            if (o) {
                Vec8<float> wv, bv;
                wv.load(pre.w + i);
                bv.load(pre.b + i);
                float w[8], b[8], s[8];
                wv.get(w);
                bv.get(b);
                if (pre.scale) {
                    Vec8<float> sv;
                    sv.load(pre.scale + i);
                    sv.get(s);
                } else {
#pragma unroll
                    for (int j = 0; j < 8; ++j) s[j] = 1.f;
                }
#pragma unroll
                for (int j = 0; j < 8; ++j) v[j] = dyt_apply(v[j], a2, w[j], b[j], s[j]);
                Vec8<T> ov;
                ov.set(v);
                ov.store(o + i);
            }
        }
    } else {
        for (int i = threadIdx.x; i < width; i += blockDim.x) {
            float v = x[i];
            if (d) {
                float e = to_float(d[i]);
                if (post.w) e = dyt_apply(e, a1, post.w[i], post.b[i], post.scale ? post.scale[i] : 1.f);
                v += e;
                if (keep) x[i] = v;
            }
            if (o) o[i] = from_float<T>(dyt_apply(v, a2, pre.w[i], pre.b[i], pre.scale ? pre.scale[i] : 1.f));
        }
    }
}

SIA_EXPORT int sia_dyt_norm(float* residual, const void* delta, const float* post_w, const float* post_b,
                            const float* post_alpha, const float* post_scale, const float* pre_w, const float* pre_b,
                            const float* pre_alpha, const float* pre_scale, void* out, const int* rows, int n_rows,
                            int width, int dtype, hipStream_t stream) {
    if (n_rows <= 0) return 0;
    if (!residual || width <= 0 || (post_w && (!post_b || !post_alpha)) || (pre_w && (!pre_b || !pre_alpha || !out)) ||
        (!pre_w && out) || (!delta && !pre_w))
        return SIA_BAD_ARGUMENT;
    DytTerms post{post_w, post_b, post_alpha, post_scale}, pre{pre_w, pre_b, pre_alpha, pre_scale};
    auto aligned = [](const void* p, size_t a) { return p == nullptr || ((uintptr_t)p % a) == 0; };
    const bool vec = width % 8 == 0 && aligned(residual, 16) && aligned(delta, 16) && aligned(out, 16) &&
                     aligned(post_w, 16) && aligned(post_b, 16) && aligned(post_scale, 16) && aligned(pre_w, 16) &&
                     aligned(pre_b, 16) && aligned(pre_scale, 16);
    const int per = vec ? 8 : 1;
    int threads = ((width / per + SIA_WAVE - 1) / SIA_WAVE) * SIA_WAVE;
    threads = threads < SIA_WAVE ? SIA_WAVE : (threads > 256 ? 256 : threads);
    dim3 grid(n_rows), block(threads);
#define LAUNCH(T, V)                                                                                              \
    hipLaunchKernelGGL((dyt_norm_kernel<T, V>), grid, block, 0, stream, residual, (const T*)delta, post, pre, (T*)out, \
                       rows, width)
    if (dtype == SIA_F32) {
        if (vec) LAUNCH(float, true); else LAUNCH(float, false);
    } else if (dtype == SIA_BF16) {
        if (vec) LAUNCH(bf16_t, true); else LAUNCH(bf16_t, false);
    } else {
        return SIA_BAD_ARGUMENT;
    }
#undef LAUNCH
    return SIA_LAUNCH_CHECK();
}
