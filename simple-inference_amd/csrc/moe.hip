// Mixture of experts: the router, and the experts' products for a token's chosen experts.
//
//   route:    z = R h (float, R float [E, width]); the ``top`` largest logits (ties: the lower index) and the softmax
//             over those alone:  ids [N, top] int32,  weights [N, top] float; or sigmoid scores, the choice among the
//             best groups of experts, weights normalised over the chosen and scaled
//   gate/up:  a[s, f] = silu(h[n] . Wg[e][f]) * (h[n] . Wu[e][f])      s = n * top + k, e = ids[s]
//             the experts' matrices are stacked: W1 [E, 2 * ff, width], gate rows first
//   down:     y[n, c] = sum_k weights[n, k] * (a[n * top + k] . W2[e_k][c])  (+ sigmoid(sg[n]) * shared[n, c])
//             W2 [E, width, ff]
//
// These forms walk the slots one by one: every (token, choice) streams the rows of its expert, a wave an output
// element at a time, sums in float.  That is the shape of a decode step (few slots, the weights read once each).
#include "common.h"

#define MOE_MAX_EXPERTS 1024
#define MOE_MAX_TOP 64

// score_mode 0: the softmax over the chosen logits alone.  score_mode 1: scores s = sigmoid(z); with n_groups > 0 the
// experts form n_groups equal groups of neighbours, a group's score is the sum of its two largest s, and only
// experts of the keep_groups best groups (ties: the lower group) can be chosen; the weights are the chosen s divided
// by their sum (+ 1e-20), times weight_scale.  score_mode 2: scores s = softmax(z) over all experts; the choice goes by
// s + correction (a float per expert, if given), the weights are the chosen s divided by their sum (+ 1e-20).
template <typename T>
__global__ __launch_bounds__(256) void moe_route_kernel(const T* __restrict__ h, const float* __restrict__ router,
                                                         int* __restrict__ ids, float* __restrict__ weights, int width,
                                                         int n_experts, int top, int score_mode, int n_groups,
                                                         int keep_groups, float weight_scale,
                                                         const float* __restrict__ correction) {
    __shared__ float logit_s[MOE_MAX_EXPERTS];
    __shared__ float group_s[MOE_MAX_EXPERTS];
    const int n = blockIdx.x, wave = threadIdx.x / SIA_WAVE, lane = threadIdx.x % SIA_WAVE;
    const T* x = h + (size_t)n * width;
    // a wave an expert at a time; four independent runs of loads a lane, so that a row's latency is paid once
    for (int e = wave; e < n_experts; e += blockDim.x / SIA_WAVE) {
        const float* w = router + (size_t)e * width;
        float acc[4] = {0.f, 0.f, 0.f, 0.f};
        int i = lane;
        for (; i + 3 * SIA_WAVE < width; i += 4 * SIA_WAVE) {
#pragma unroll
            for (int u = 0; u < 4; ++u) acc[u] += to_float(x[i + u * SIA_WAVE]) * w[i + u * SIA_WAVE];
        }
        for (; i < width; i += SIA_WAVE) acc[0] += to_float(x[i]) * w[i];
        const float total = wave_sum((acc[0] + acc[1]) + (acc[2] + acc[3]));
        if (lane == 0) logit_s[e] = score_mode == 1 ? 1.f / (1.f + expf(-total)) : total;
    }
    __syncthreads();
    if (wave != 0) return;
    if (score_mode == 2) {
        // the scores stay in group_s, what the choice goes by takes the logits' place
        float top_z = -INFINITY, sum = 0.f;
        for (int e = lane; e < n_experts; e += SIA_WAVE) top_z = fmaxf(top_z, logit_s[e]);
        top_z = wave_max(top_z);
        for (int e = lane; e < n_experts; e += SIA_WAVE) sum += expf(logit_s[e] - top_z);
        sum = wave_sum(sum);
        for (int e = lane; e < n_experts; e += SIA_WAVE) {
            const float sc = expf(logit_s[e] - top_z) / sum;
            group_s[e] = sc;
            logit_s[e] = correction ? sc + correction[e] : sc;
        }
        __builtin_amdgcn_wave_barrier();
        __threadfence_block();
    }
    if (score_mode == 1 && n_groups > 0) {
        // a lane a group at a time: the sum of its two largest scores; then keep_groups rounds of a wave-wide best
        // group, and the experts of every other group leave the choice
        const int per = n_experts / n_groups;
        for (int g = lane; g < n_groups; g += SIA_WAVE) {
            float a = -INFINITY, b = -INFINITY;
            for (int e = g * per; e < (g + 1) * per; ++e) {
                const float z = logit_s[e];
                if (z > a) { b = a; a = z; } else if (z > b) { b = z; }
            }
            group_s[g] = per > 1 ? a + b : a;
        }
        __builtin_amdgcn_wave_barrier();
        __threadfence_block();
        for (int k = 0; k < keep_groups; ++k) {
            float best = -INFINITY;
            int which = 0x7fffffff;
            for (int g = lane; g < n_groups; g += SIA_WAVE) {
                const float z = group_s[g];
                if (z != INFINITY && z > best) { best = z; which = g; }      // a kept group is out of the next rounds
            }
#pragma unroll
            for (int off = SIA_WAVE / 2; off > 0; off >>= 1) {
                const float ob = __shfl_xor(best, off, SIA_WAVE);
                const int ow = __shfl_xor(which, off, SIA_WAVE);
                if (ob > best || (ob == best && ow < which)) { best = ob; which = ow; }
            }
            if (which >= n_groups) break;
            if (lane == 0) group_s[which] = INFINITY;      // kept
            __builtin_amdgcn_wave_barrier();
            __threadfence_block();
        }
        for (int e = lane; e < n_experts; e += SIA_WAVE)
            if (group_s[e / per] != INFINITY) logit_s[e] = -INFINITY;
        __builtin_amdgcn_wave_barrier();
        __threadfence_block();
    }
    float chosen = 0.f, first = 0.f, total = 0.f;   // lane k keeps the k-th choice
    int chosen_id = 0;
    for (int k = 0; k < top; ++k) {
        float best = -INFINITY;
        int which = 0x7fffffff;
        for (int e = lane; e < n_experts; e += SIA_WAVE) {
            const float z = logit_s[e];
            if (z > best) { best = z; which = e; }     // ascending e: the lower index wins a tie
        }
#pragma unroll
        for (int off = SIA_WAVE / 2; off > 0; off >>= 1) {
            const float ob = __shfl_xor(best, off, SIA_WAVE);
            const int ow = __shfl_xor(which, off, SIA_WAVE);
            if (ob > best || (ob == best && ow < which)) { best = ob; which = ow; }
        }
        if (which >= n_experts) { which = k; best = 0.f; }   // logits that are not numbers order nothing: still an expert that exists
        if (k == 0) first = best;
        const float p = score_mode == 1 ? best : score_mode == 2 ? group_s[which] : expf(best - first);
        total += p;
        if (lane == k) { chosen = p; chosen_id = which; }
        if (lane == 0 && which < n_experts) logit_s[which] = -INFINITY;
        __builtin_amdgcn_wave_barrier();
        __threadfence_block();
    }
    if (lane < top) {
        ids[(size_t)n * top + lane] = chosen_id;
        weights[(size_t)n * top + lane] = score_mode == 1 ? chosen / (total + 1e-20f) * weight_scale
                                          : score_mode == 2 ? chosen / (total + 1e-20f) : chosen / total;
    }
}

static int route(const void* h, const float* router, int* ids, float* weights, int n_tokens, int width, int n_experts,
                 int top, int dtype, int score_mode, int n_groups, int keep_groups, float weight_scale,
                 const float* correction, hipStream_t stream) {
    if (n_tokens <= 0) return 0;
    if (n_experts <= 0 || n_experts > MOE_MAX_EXPERTS || top <= 0 || top > n_experts || top > MOE_MAX_TOP ||
        (score_mode != 0 && score_mode != 1 && score_mode != 2) || n_groups < 0 || (correction && score_mode != 2) ||
        (n_groups > 0 && (score_mode != 1 || n_experts % n_groups || keep_groups <= 0 || keep_groups > n_groups ||
                          top > n_experts / n_groups * keep_groups)))
        return SIA_BAD_ARGUMENT;
    dim3 grid(n_tokens), block(256);
    if (dtype == SIA_F32)
        hipLaunchKernelGGL(moe_route_kernel<float>, grid, block, 0, stream, (const float*)h, router, ids, weights, width,
                           n_experts, top, score_mode, n_groups, keep_groups, weight_scale, correction);
    else if (dtype == SIA_BF16)
        hipLaunchKernelGGL(moe_route_kernel<bf16_t>, grid, block, 0, stream, (const bf16_t*)h, router, ids, weights,
                           width, n_experts, top, score_mode, n_groups, keep_groups, weight_scale, correction);
    else
        return SIA_BAD_ARGUMENT;
    return SIA_LAUNCH_CHECK();
}

SIA_EXPORT int sia_moe_route_ex(const void* h, const float* router, int* ids, float* weights, int n_tokens, int width,
                                int n_experts, int top, int dtype, int score_mode, int n_groups, int keep_groups,
                                float weight_scale, hipStream_t stream) {
    return route(h, router, ids, weights, n_tokens, width, n_experts, top, dtype, score_mode, n_groups, keep_groups,
                 weight_scale, nullptr, stream);
}

// scores over all experts (score_mode 2) with the vector that corrects the choice
SIA_EXPORT int sia_moe_route_corrected(const void* h, const float* router, const float* correction, int* ids,
                                       float* weights, int n_tokens, int width, int n_experts, int top, int dtype,
                                       hipStream_t stream) {
    return route(h, router, ids, weights, n_tokens, width, n_experts, top, dtype, 2, 0, 0, 1.f, correction, stream);
}

SIA_EXPORT int sia_moe_route(const void* h, const float* router, int* ids, float* weights, int n_tokens, int width,
                             int n_experts, int top, int dtype, hipStream_t stream) {
    return sia_moe_route_ex(h, router, ids, weights, n_tokens, width, n_experts, top, dtype, 0, 0, 0, 1.f, stream);
}

// dot product of two rows of K elements by one wave (every lane gets the sum)
template <typename T>
__device__ __forceinline__ float wave_dot(const T* __restrict__ a, const T* __restrict__ b, int K, int lane, bool vec) {
    float acc = 0.f;
    if (vec) {
        for (int i = lane * 8; i < K; i += SIA_WAVE * 8) {
            Vec8<T> va, vb;
            va.load(a + i);
            vb.load(b + i);
            float x[8], y[8];
            va.get(x);
            vb.get(y);
#pragma unroll
            for (int e = 0; e < 8; ++e) acc += x[e] * y[e];
        }
    } else {
        for (int i = lane; i < K; i += SIA_WAVE) acc += to_float(a[i]) * to_float(b[i]);
    }
    return wave_sum(acc);
}

#define MOE_WAVES 4
#define MOE_PER_WAVE 4    // output elements a wave takes in turn

template <typename T>
__global__ __launch_bounds__(MOE_WAVES* SIA_WAVE) void moe_gate_up_kernel(
    const T* __restrict__ h, const T* __restrict__ w1, const int* __restrict__ ids, T* __restrict__ act, int width,
    int ff, int top, bool vec, int n_real, int glu, float limit) {
    const int slot = blockIdx.x, wave = threadIdx.x / SIA_WAVE, lane = threadIdx.x % SIA_WAVE;
    const int e = ids[slot];
    if (e >= n_real) return;     // an expert without tensors: the down kernel hands the token's input on
    const T* x = h + (size_t)(slot / top) * width;
    const T* w = w1 + (size_t)e * 2 * ff * width;
    const int f0 = (blockIdx.y * MOE_WAVES + wave) * MOE_PER_WAVE;
    for (int f = f0; f < min(ff, f0 + MOE_PER_WAVE); ++f) {
        const float g = wave_dot<T>(x, w + (size_t)f * width, width, lane, vec);
        const float u = wave_dot<T>(x, w + (size_t)(ff + f) * width, width, lane, vec);
        if (lane == 0) act[(size_t)slot * ff + f] = from_float<T>(gated_activation(g, u, glu, limit));
    }
}

template <typename T>
__global__ __launch_bounds__(MOE_WAVES* SIA_WAVE) void moe_down_kernel(
    const T* __restrict__ act, const T* __restrict__ w2, const int* __restrict__ ids, const float* __restrict__ weights,
    const T* __restrict__ shared, const T* __restrict__ shared_gate, int shared_gate_stride, T* __restrict__ out,
    int width, int ff, int top, bool vec, const T* __restrict__ h, int n_real) {
    const int n = blockIdx.x, wave = threadIdx.x / SIA_WAVE, lane = threadIdx.x % SIA_WAVE;
    const int c0 = (blockIdx.y * MOE_WAVES + wave) * MOE_PER_WAVE;
    for (int c = c0; c < min(width, c0 + MOE_PER_WAVE); ++c) {
        float y = 0.f;
        for (int k = 0; k < top; ++k) {
            const int slot = n * top + k;
            if (ids[slot] >= n_real) {      // wave-uniform
                y += weights[slot] * to_float(h[(size_t)n * width + c]);
                continue;
            }
            const T* w = w2 + ((size_t)ids[slot] * width + c) * ff;
            y += weights[slot] * wave_dot<T>(act + (size_t)slot * ff, w, ff, lane, vec);
        }
        if (shared) {
            float s = to_float(shared[(size_t)n * width + c]);
            if (shared_gate) s *= 1.f / (1.f + expf(-to_float(shared_gate[(size_t)n * shared_gate_stride])));
            y += s;
        }
        if (lane == 0) out[(size_t)n * width + c] = from_float<T>(y);
    }
}

// n_real: ids from there on name experts without tensors, which return their input; glu, limit: the experts' gated
// activation (``gated_activation`` of common.h).
SIA_EXPORT int sia_moe_gate_up_ex(const void* h, const void* w1, const int* ids, void* act, int n_tokens, int width,
                                  int ff, int top, int n_real, int glu, float limit, int dtype, hipStream_t stream) {
    if (n_tokens <= 0) return 0;
    if (width <= 0 || ff <= 0 || top <= 0 || (long long)n_tokens * top > 0x7fffffffLL || n_real <= 0 ||
        (glu != SIA_GLU_SILU && glu != SIA_GLU_CLAMPED))
        return SIA_BAD_ARGUMENT;
    const int per_block = MOE_WAVES * MOE_PER_WAVE;
    dim3 grid(n_tokens * top, (ff + per_block - 1) / per_block), block(MOE_WAVES * SIA_WAVE);
    if (grid.y > 65535) return SIA_BAD_ARGUMENT;
    const bool vec = width % 8 == 0;
    if (dtype == SIA_F32)
        hipLaunchKernelGGL(moe_gate_up_kernel<float>, grid, block, 0, stream, (const float*)h, (const float*)w1, ids,
                           (float*)act, width, ff, top, vec, n_real, glu, limit);
    else if (dtype == SIA_BF16)
        hipLaunchKernelGGL(moe_gate_up_kernel<bf16_t>, grid, block, 0, stream, (const bf16_t*)h, (const bf16_t*)w1, ids,
                           (bf16_t*)act, width, ff, top, vec, n_real, glu, limit);
    else
        return SIA_BAD_ARGUMENT;
    return SIA_LAUNCH_CHECK();
}

SIA_EXPORT int sia_moe_gate_up(const void* h, const void* w1, const int* ids, void* act, int n_tokens, int width, int ff,
                               int top, int dtype, hipStream_t stream) {
    return sia_moe_gate_up_ex(h, w1, ids, act, n_tokens, width, ff, top, 0x7fffffff, SIA_GLU_SILU, 0.f, dtype, stream);
}

// h, n_real: a slot whose id is n_real or more adds its weight times the token's own input h.
SIA_EXPORT int sia_moe_down_ex(const void* act, const void* w2, const int* ids, const float* weights, const void* shared,
                               const void* shared_gate, int shared_gate_stride, void* out, int n_tokens, int width,
                               int ff, int top, const void* h, int n_real, int dtype, hipStream_t stream) {
    if (n_tokens <= 0) return 0;
    if (width <= 0 || ff <= 0 || top <= 0 || (shared_gate && !shared) || n_real <= 0 || (n_real != 0x7fffffff && !h))
        return SIA_BAD_ARGUMENT;
    const int per_block = MOE_WAVES * MOE_PER_WAVE;
    dim3 grid(n_tokens, (width + per_block - 1) / per_block), block(MOE_WAVES * SIA_WAVE);
    if (grid.y > 65535) return SIA_BAD_ARGUMENT;
    const bool vec = ff % 8 == 0;
    if (dtype == SIA_F32)
        hipLaunchKernelGGL(moe_down_kernel<float>, grid, block, 0, stream, (const float*)act, (const float*)w2, ids,
                           weights, (const float*)shared, (const float*)shared_gate, shared_gate_stride, (float*)out,
                           width, ff, top, vec, (const float*)h, n_real);
    else if (dtype == SIA_BF16)
        hipLaunchKernelGGL(moe_down_kernel<bf16_t>, grid, block, 0, stream, (const bf16_t*)act, (const bf16_t*)w2, ids,
                           weights, (const bf16_t*)shared, (const bf16_t*)shared_gate, shared_gate_stride, (bf16_t*)out,
                           width, ff, top, vec, (const bf16_t*)h, n_real);
    else
        return SIA_BAD_ARGUMENT;
    return SIA_LAUNCH_CHECK();
}

SIA_EXPORT int sia_moe_down(const void* act, const void* w2, const int* ids, const float* weights, const void* shared,
                            const void* shared_gate, int shared_gate_stride, void* out, int n_tokens, int width, int ff,
                            int top, int dtype, hipStream_t stream) {
    return sia_moe_down_ex(act, w2, ids, weights, shared, shared_gate, shared_gate_stride, out, n_tokens, width, ff, top,
                           nullptr, 0x7fffffff, dtype, stream);
}

// ---------------------------------------------------------------------------------------------------------------
// Steps of many tokens (bfloat16): the slots are sorted by expert on the device and the experts' products run on the
// matrix cores, a tile of 32 slots of one expert at a time.
//
//   sort:     counts the slots of every expert, gives every expert whole tiles of 32 places (the places a tile does
//             not fill hold -1) and writes, for every place, its slot, and for every tile, its expert.  One workgroup;
//             nothing comes back to the host: the products are launched for the most tiles there can be
//             (ceil(slots / 32) + experts) and the tiles beyond the count leave at once.  Which place of its expert's
//             tiles a slot gets depends on the order of atomic adds; a slot's numbers do not (a row of a product
//             does not depend on the other rows).
//   gate/up:  a[s, f] for a tile's slots and 128 columns f a workgroup: v_mfma_f32_16x16x32_bf16 with the weights'
//             rows as the first operand and the tokens' rows as the second, both read from memory k-contiguous
//             (lane (r, g): row r, elements 8g .. 8g + 7 of a step of 32); a wave holds 32 columns x 32 slots of
//             gate and of up and writes 4 consecutive columns of a slot at a time.
//   down:     y[s, c] the same way, bfloat16, one row per slot;
//   combine:  out[n, c] = sum_k weights[n, k] * y[n * top + k, c] (+ sigmoid(sg[n]) * shared[n, c]), float sums.
// ---------------------------------------------------------------------------------------------------------------
typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 moe_bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float moe_floatx4;

#define MOE_TILE 32

__global__ __launch_bounds__(1024) void moe_sort_kernel(const int* __restrict__ ids, int n_slots, int n_experts,
                                                        int* __restrict__ place_slot, int* __restrict__ tile_expert,
                                                        int* __restrict__ n_tiles_out, int max_tiles) {
    __shared__ int count_s[MOE_MAX_EXPERTS];
    __shared__ int first_s[MOE_MAX_EXPERTS];   // first place of the expert's tiles
    for (int e = threadIdx.x; e < n_experts; e += blockDim.x) count_s[e] = 0;
    for (int i = threadIdx.x; i < max_tiles * MOE_TILE; i += blockDim.x) place_slot[i] = -1;
    __syncthreads();
    // a slot whose id lies beyond the experts (an expert without tensors) gets no place: the combine kernel serves it
    auto expert_of = [&](int s) { return max(ids[s], 0); };
    for (int s = threadIdx.x; s < n_slots; s += blockDim.x)
        if (expert_of(s) < n_experts) atomicAdd(&count_s[expert_of(s)], 1);
    __syncthreads();
    if (threadIdx.x == 0) {
        int tile = 0;
        for (int e = 0; e < n_experts; ++e) {
            first_s[e] = tile * MOE_TILE;
            const int tiles = (count_s[e] + MOE_TILE - 1) / MOE_TILE;
            for (int t = 0; t < tiles; ++t) tile_expert[tile + t] = e;
            tile += tiles;
            count_s[e] = 0;   // from here on: the next free place of the expert
        }
        *n_tiles_out = tile;
    }
    __syncthreads();
    for (int s = threadIdx.x; s < n_slots; s += blockDim.x) {
        const int e = expert_of(s);
        if (e < n_experts) place_slot[first_s[e] + atomicAdd(&count_s[e], 1)] = s;
    }
}

__device__ __forceinline__ moe_bf16x8 moe_ld8(const bf16_t* p) { return *reinterpret_cast<const moe_bf16x8*>(p); }

// GATED: rows f and ff + f of W make silu(gate) * up; else a plain product.  Output row stride n_out.
template <bool GATED>
__global__ __launch_bounds__(256) void moe_tile_kernel(const bf16_t* __restrict__ x, int rows_per_slot,
                                                       const bf16_t* __restrict__ w, const int* __restrict__ place_slot,
                                                       const int* __restrict__ tile_expert,
                                                       const int* __restrict__ n_tiles, bf16_t* __restrict__ out,
                                                       int K, int n_out, int glu, float limit) {
    const int tile = blockIdx.x;
    if (tile >= *n_tiles) return;
    const int wave = threadIdx.x / SIA_WAVE, lane = threadIdx.x % SIA_WAVE, r = lane & 15, g = lane >> 4;
    const int e = tile_expert[tile];
    const int c0 = blockIdx.y * 128 + wave * 32;          // this wave's 32 output columns
    if (c0 >= n_out) return;
    const size_t expert_rows = GATED ? 2 * (size_t)n_out : (size_t)n_out;
    const bf16_t* we = w + (size_t)e * expert_rows * K;
    int slot[2];
    const bf16_t* xp[2];
    const bf16_t* wp[2][2];
#pragma unroll
    for (int mb = 0; mb < 2; ++mb) {
        slot[mb] = place_slot[tile * MOE_TILE + mb * 16 + r];
        xp[mb] = x + (size_t)(max(slot[mb], 0) / rows_per_slot) * K + g * 8;
    }
#pragma unroll
    for (int nb = 0; nb < 2; ++nb) {
        const int c = min(c0 + nb * 16 + r, n_out - 1);
        wp[nb][0] = we + (size_t)c * K + g * 8;
        wp[nb][1] = we + (size_t)(n_out + c) * K + g * 8;     // the up rows (GATED only)
    }
    moe_floatx4 acc[2][2][2];
#pragma unroll
    for (int nb = 0; nb < 2; ++nb)
#pragma unroll
        for (int mb = 0; mb < 2; ++mb)
#pragma unroll
            for (int h = 0; h < 2; ++h) acc[nb][mb][h] = moe_floatx4{0.f, 0.f, 0.f, 0.f};
    for (int k = 0; k < K; k += 32) {
        moe_bf16x8 a[2][2], b[2];
#pragma unroll
        for (int mb = 0; mb < 2; ++mb) b[mb] = moe_ld8(xp[mb] + k);
#pragma unroll
        for (int nb = 0; nb < 2; ++nb) {
            a[nb][0] = moe_ld8(wp[nb][0] + k);
            if (GATED) a[nb][1] = moe_ld8(wp[nb][1] + k);
        }
#pragma unroll
        for (int nb = 0; nb < 2; ++nb)
#pragma unroll
            for (int mb = 0; mb < 2; ++mb) {
                acc[nb][mb][0] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[nb][0], b[mb], acc[nb][mb][0], 0, 0, 0);
                if (GATED)
                    acc[nb][mb][1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[nb][1], b[mb], acc[nb][mb][1], 0, 0, 0);
            }
    }
    // acc[nb][mb][.][i]: column c0 + nb * 16 + 4g + i of the slot at place mb * 16 + r
#pragma unroll
    for (int mb = 0; mb < 2; ++mb) {
        if (slot[mb] < 0) continue;
        const size_t row = GATED ? (size_t)slot[mb] : (size_t)slot[mb];
#pragma unroll
        for (int nb = 0; nb < 2; ++nb) {
            const int c = c0 + nb * 16 + 4 * g;
            bf16_t v[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                float y = acc[nb][mb][0][i];
                if (GATED) y = gated_activation(y, acc[nb][mb][1][i], glu, limit);
                v[i] = float_to_bf16(y);
            }
            bf16_t* dst = out + row * n_out + c;
            if (c + 3 < n_out && n_out % 4 == 0) {
                *reinterpret_cast<uint2*>(dst) = make_uint2((uint32_t)v[0] | ((uint32_t)v[1] << 16),
                                                            (uint32_t)v[2] | ((uint32_t)v[3] << 16));
            } else {
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    if (c + i < n_out) dst[i] = v[i];
            }
        }
    }
}

__global__ __launch_bounds__(256) void moe_combine_kernel(const bf16_t* __restrict__ y, const float* __restrict__ weights,
                                                          const bf16_t* __restrict__ shared,
                                                          const bf16_t* __restrict__ shared_gate, int shared_gate_stride,
                                                          bf16_t* __restrict__ out, int width, int top,
                                                          const int* __restrict__ ids, const bf16_t* __restrict__ h,
                                                          int n_real) {
    const int n = blockIdx.x;
    float scale = 1.f;
    if (shared && shared_gate) scale = 1.f / (1.f + expf(-bf16_to_float(shared_gate[(size_t)n * shared_gate_stride])));
    for (int c = threadIdx.x; c < width; c += blockDim.x) {
        float acc = 0.f;
        for (int k = 0; k < top; ++k) {
            const size_t slot = (size_t)n * top + k;
            // an expert without tensors returns the token's input; its row of y was never written
            acc += weights[slot] * bf16_to_float(ids[slot] >= n_real ? h[(size_t)n * width + c] : y[slot * width + c]);
        }
        if (shared) acc += scale * bf16_to_float(shared[(size_t)n * width + c]);
        out[(size_t)n * width + c] = float_to_bf16(acc);
    }
}

// ints of workspace the tiled form needs for a step of n_tokens (0: the step is too small for it, or the sizes
// do not fit: the slot-by-slot form runs)
SIA_EXPORT long long sia_moe_tiled_workspace(int n_tokens, int top, int n_experts, int width, int ff) {
    const long long slots = (long long)n_tokens * top;
    if (slots < 64 || width % 32 || ff % 32 || slots > 0x3fffffffLL) return 0;
    const long long max_tiles = (slots + MOE_TILE - 1) / MOE_TILE + n_experts;
    return max_tiles * MOE_TILE + max_tiles + 4;
}

// act [slots, ff] and y [slots, width] are the caller's scratch (bfloat16).
// glu, limit: the experts' gated activation; ids of n_experts and more name experts without tensors.
SIA_EXPORT int sia_moe_tiled_ex(const void* h, const void* w1, const void* w2, const int* ids, const float* weights,
                                const void* shared, const void* shared_gate, int shared_gate_stride, void* act, void* y,
                                void* out, int* workspace, int n_tokens, int width, int ff, int top, int n_experts,
                                int glu, float limit, hipStream_t stream) {
    if (n_tokens <= 0) return 0;
    if (sia_moe_tiled_workspace(n_tokens, top, n_experts, width, ff) == 0 || n_experts > MOE_MAX_EXPERTS ||
        (shared_gate && !shared) || (glu != SIA_GLU_SILU && glu != SIA_GLU_CLAMPED))
        return SIA_BAD_ARGUMENT;
    const int slots = n_tokens * top;
    const int max_tiles = (slots + MOE_TILE - 1) / MOE_TILE + n_experts;
    int* place_slot = workspace;
    int* tile_expert = workspace + (size_t)max_tiles * MOE_TILE;
    int* n_tiles = tile_expert + max_tiles;
    hipLaunchKernelGGL(moe_sort_kernel, dim3(1), dim3(1024), 0, stream, ids, slots, n_experts, place_slot, tile_expert,
                       n_tiles, max_tiles);
    hipLaunchKernelGGL(moe_tile_kernel<true>, dim3(max_tiles, (ff + 127) / 128), dim3(256), 0, stream,
                       (const bf16_t*)h, top, (const bf16_t*)w1, place_slot, tile_expert, n_tiles, (bf16_t*)act, width, ff,
                       glu, limit);
    hipLaunchKernelGGL(moe_tile_kernel<false>, dim3(max_tiles, (width + 127) / 128), dim3(256), 0, stream,
                       (const bf16_t*)act, 1, (const bf16_t*)w2, place_slot, tile_expert, n_tiles, (bf16_t*)y, ff, width,
                       SIA_GLU_SILU, 0.f);
    hipLaunchKernelGGL(moe_combine_kernel, dim3(n_tokens), dim3(256), 0, stream, (const bf16_t*)y, weights,
                       (const bf16_t*)shared, (const bf16_t*)shared_gate, shared_gate_stride, (bf16_t*)out, width, top,
                       ids, (const bf16_t*)h, n_experts);
    return SIA_LAUNCH_CHECK();
}

SIA_EXPORT int sia_moe_tiled(const void* h, const void* w1, const void* w2, const int* ids, const float* weights,
                             const void* shared, const void* shared_gate, int shared_gate_stride, void* act, void* y,
                             void* out, int* workspace, int n_tokens, int width, int ff, int top, int n_experts,
                             hipStream_t stream) {
    return sia_moe_tiled_ex(h, w1, w2, ids, weights, shared, shared_gate, shared_gate_stride, act, y, out, workspace,
                            n_tokens, width, ff, top, n_experts, SIA_GLU_SILU, 0.f, stream);
}
