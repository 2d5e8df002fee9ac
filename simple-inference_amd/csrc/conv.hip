// A short causal convolution per channel over each sequence's tokens, with the inputs before a step's first token
// kept in the sequence's state.
//
//   out[t, c] = act(b[c] + sum_j w[c, j] * u[t - (taps - 1) + j, c])        j = 0 .. taps - 1; the last tap meets t
//
// u are columns first_col .. first_col + channels - 1 of the projected rows (row_stride apart).  Inputs at places
// before the step's first token of the sequence come from the sequence's state row: state[slot * state_stride +
// state_offset + i * channels + c] holds the input i places after the oldest kept one (taps - 1 of them, zeros before a
// sequence's first token).  After the step the row holds the last taps - 1 inputs again.  Sums in float, one rounding.
//
// Two launches: every (token, channel) is independent once the old state may still be read, so the state is
// rewritten by a second, small kernel (a thread reads what it overwrites first).  A step in which every sequence
// brings one token does both in one kernel: the thread of a (sequence, channel) is the only one that touches its
// part of the state.
#include "common.h"

#define CONV_MAX_TAPS 16

template <typename T>
__global__ __launch_bounds__(256) void conv_tokens_kernel(const T* __restrict__ proj, int row_stride, int first_col,
                                                          const float* __restrict__ w, const float* __restrict__ b,
                                                          float* __restrict__ state, long long state_stride,
                                                          int state_offset, const int* __restrict__ cu_q,
                                                          const int* __restrict__ seq_of_token,
                                                          const int* __restrict__ slots, T* __restrict__ out,
                                                          int channels, int taps, int silu, int single) {
    const int t = blockIdx.x, c = blockIdx.y * blockDim.x + threadIdx.x;
    if (c >= channels) return;
    const int seq = seq_of_token[t];
    const int first = cu_q[seq];
    float* st = state + (size_t)slots[seq] * state_stride + state_offset;
    float acc = b ? b[c] : 0.f;
    float window[CONV_MAX_TAPS];
    for (int j = 0; j < taps; ++j) {
        const int src = t - (taps - 1) + j;     // a token of this step, or a place in the state
        float u;
        if (src >= first) u = to_float(proj[(size_t)src * row_stride + first_col + c]);
        else u = st[(size_t)(taps - 1 - (first - src)) * channels + c];
        window[j] = u;
        acc += w[(size_t)c * taps + j] * u;
    }
    if (silu) acc = acc / (1.f + expf(-acc));
    out[(size_t)t * channels + c] = from_float<T>(acc);
    if (single)     // the sequence's only token of the step: the window without its oldest input is the new state
        for (int j = 1; j < taps; ++j) st[(size_t)(j - 1) * channels + c] = window[j];
}

template <typename T>
__global__ __launch_bounds__(256) void conv_state_kernel(const T* __restrict__ proj, int row_stride, int first_col,
                                                         float* __restrict__ state, long long state_stride,
                                                         int state_offset, const int* __restrict__ cu_q,
                                                         const int* __restrict__ slots, int channels, int taps) {
    const int seq = blockIdx.x, c = blockIdx.y * blockDim.x + threadIdx.x;
    if (c >= channels) return;
    const int first = cu_q[seq], last = cu_q[seq + 1];
    const int n = last - first, keep = taps - 1;
    if (n <= 0) return;
    float* st = state + (size_t)slots[seq] * state_stride + state_offset;
    float fresh[CONV_MAX_TAPS];
    for (int i = 0; i < keep; ++i) {
        const int src = last - keep + i;        // the i-th of the last taps - 1 inputs
        fresh[i] = src >= first ? to_float(proj[(size_t)src * row_stride + first_col + c])
                                : st[(size_t)(keep - (first - src)) * channels + c];
    }
    for (int i = 0; i < keep; ++i) st[(size_t)i * channels + c] = fresh[i];
}

SIA_EXPORT int sia_causal_conv(const void* proj, int row_stride, int first_col, const float* w, const float* b,
                               float* state, long long state_stride, int state_offset, const int* cu_q,
                               const int* seq_of_token, const int* slots, void* out, int n_tokens, int n_seqs,
                               int max_q_len, int channels, int taps, int silu, int dtype, hipStream_t stream) {
    if (n_tokens <= 0 || n_seqs <= 0) return 0;
    if (channels <= 0 || taps <= 0 || taps > CONV_MAX_TAPS || !proj || !w || !state || !out || first_col < 0 ||
        first_col + channels > row_stride || state_offset < 0 ||
        (long long)state_offset + (long long)channels * (taps - 1) > state_stride)
        return SIA_BAD_ARGUMENT;
    const int single = max_q_len <= 1;
    dim3 block(256), grid(n_tokens, (channels + 255) / 256), sgrid(n_seqs, (channels + 255) / 256);
    if (dtype == SIA_F32) {
        hipLaunchKernelGGL(conv_tokens_kernel<float>, grid, block, 0, stream, (const float*)proj, row_stride, first_col, w,
                           b, state, state_stride, state_offset, cu_q, seq_of_token, slots, (float*)out, channels, taps,
                           silu, single);
        if (!single && taps > 1)
            hipLaunchKernelGGL(conv_state_kernel<float>, sgrid, block, 0, stream, (const float*)proj, row_stride,
                               first_col, state, state_stride, state_offset, cu_q, slots, channels, taps);
    } else if (dtype == SIA_BF16) {
        hipLaunchKernelGGL(conv_tokens_kernel<bf16_t>, grid, block, 0, stream, (const bf16_t*)proj, row_stride, first_col,
                           w, b, state, state_stride, state_offset, cu_q, seq_of_token, slots, (bf16_t*)out, channels,
                           taps, silu, single);
        if (!single && taps > 1)
            hipLaunchKernelGGL(conv_state_kernel<bf16_t>, sgrid, block, 0, stream, (const bf16_t*)proj, row_stride,
                               first_col, state, state_stride, state_offset, cu_q, slots, channels, taps);
    } else {
        return SIA_BAD_ARGUMENT;
    }
    return SIA_LAUNCH_CHECK();
}
