// What lies between the q/k/v product and attention for mixers that do more there than rotate: bias, a per-head
// RMS norm of q and k, rotation of the first rotary_dim elements of a head, and the write of k and v into the
// cache pages, in one kernel.
//
// The projected row is [q heads | k heads | v heads]; q and k heads are head_dim wide, v heads value_dim.
// For every q and k head x (all of it float, one rounding at the end):
//
//   x += bias                                                     (if bias is given)
//   x  = x * rsqrt(mean(x^2) + eps) * gain                         (if gains are given; one gain of head_dim for
//                                                                   all q heads, one for all k heads)
//   x *= 1 + coef * ln(floor((pos + 1) / every) + 1)               (q heads only, if a query temperature is given)
//   (x_i, x_{i+r/2}) <- (x_i c_i - x_{i+r/2} s_i, x_{i+r/2} c_i + x_i s_i),  i < r/2, r = rotary_dim,
//                       c, s from the float tables at the token's absolute position; elements from r on pass
//
// q is written back in place, k goes to the token's place in its page, v (with its bias) too.
//
// Page layout:  keys   [page][kv_head][offset][k_row]
//               values [page][kv_head][v_rows][offset]      (positions innermost)
// k_row and v_rows are head_dim and value_dim, or larger: pages may be wider than the heads (a mixer whose keys and
// values differ in width can keep both at one width, for kernels that want them alike); what lies beyond a head's
// own elements is never written and stays as the pages were made (zero).  q goes back in place, or to a matrix of
// its own with heads q_head_stride apart (the elements between heads are the caller's: zero).
//
// A wave takes one q or k head of one token: a lane holds the elements lane, lane + 64, ... of the head, the sum
// of squares is a butterfly over the wave, and the rotation's partner of an element comes from the lane that holds
// it by a lane exchange; waves never wait for one another.  A workgroup is four such waves (grid: tokens x groups
// of four heads), and one more workgroup per token writes the values.  Values lie in a page with positions
// innermost: where 8 or 16 consecutive tokens of a sequence fill an aligned run of a page, their workgroups share
// the (head, dim) rows and each writes all the run's positions of its rows at once (16 or 32 contiguous bytes in
// bfloat16) instead of one element per token and row.
#include "common.h"

#define QKP_MAX_HEAD_DIM 256
#define QKP_WAVES 4
#define QKP_PER_LANE (QKP_MAX_HEAD_DIM / SIA_WAVE)

// A query's temperature: 1 + coef * ln(floor((pos + 1) / every) + 1), a step function of the position that sharpens
// the scores of late queries (every <= 0: none).
__device__ __forceinline__ float query_temperature(int pos, float coef, int every) {
    return 1.f + coef * logf((float)((pos + 1) / every + 1));
}

template <typename T>
__device__ __forceinline__ void write_values(const T* __restrict__ qkv, int row_stride, const float* __restrict__ bias,
                                             const int* __restrict__ positions, const int* __restrict__ seq_of_token,
                                             T* __restrict__ v_pages, int n, int n_tokens, int page, int off, int pos,
                                             int v_first, int rows, int value_dim, int v_rows, int page_size,
                                             int v_group) {
    const size_t page_rows = (size_t)(rows / value_dim) * v_rows;   // value rows of a page, over its kv heads
    auto page_row = [&](int i) { return (size_t)(i / value_dim) * v_rows + i % value_dim; };
    const T* x = qkv + (size_t)n * row_stride + v_first;
    const float* b = bias ? bias + v_first : nullptr;
    bool whole = false;
    int place = 0, first = n;
    if (v_group > 0) {
        const int seq = seq_of_token[n];
        place = off % v_group;
        first = n - place;
        whole = first >= 0 && first + v_group <= n_tokens && seq_of_token[first] == seq &&
                seq_of_token[first + v_group - 1] == seq && positions[first] == pos - place &&
                positions[first + v_group - 1] == pos - place + v_group - 1;
    }
    if (!whole) {  // an incomplete run: every token writes its own values
        for (int i = threadIdx.x; i < rows; i += blockDim.x) {
            float v = to_float(x[i]);
            if (b) v += b[i];
            v_pages[((size_t)page * page_rows + page_row(i)) * page_size + off] = from_float<T>(v);
        }
        return;
    }
    constexpr int V_MAX = 16;
    constexpr int PER = 16 / sizeof(T);  // elements of a 16-byte store
    const int slice = (rows + v_group - 1) / v_group;
    const T* x0 = qkv + (size_t)first * row_stride + v_first;
    for (int i = place * slice + threadIdx.x; i < min(rows, (place + 1) * slice); i += blockDim.x) {
        __attribute__((aligned(16))) T vals[V_MAX];
        const float add = b ? b[i] : 0.f;
#pragma unroll
        for (int j = 0; j < V_MAX; ++j)
            vals[j] = j < v_group ? from_float<T>(to_float(x0[(size_t)j * row_stride + i]) + add) : T(0);
        T* dst = v_pages + ((size_t)page * page_rows + page_row(i)) * page_size + (off - place);
#pragma unroll
        for (int j = 0; j < V_MAX; j += PER)
            if (j < v_group) *reinterpret_cast<uint4*>(dst + j) = *reinterpret_cast<const uint4*>(vals + j);
    }
}

template <typename T>
__global__ __launch_bounds__(QKP_WAVES* SIA_WAVE) void qk_prepare_kernel(
    T* qkv, int row_stride, const float* __restrict__ bias, const float* __restrict__ q_gain,
    const float* __restrict__ k_gain, float eps, const float* __restrict__ cos_table,
    const float* __restrict__ sin_table, const int* __restrict__ positions, const int* __restrict__ seq_of_token,
    const int* __restrict__ block_table, int table_width, T* __restrict__ k_pages, T* __restrict__ v_pages,
    int n_tokens, int n_heads, int n_kv, int head_dim, int value_dim, int rotary_dim, int page_size, int v_group,
    int k_row, int v_rows, T* q_out, int q_row_stride, int q_head_stride, float temp_coef,
    int temp_every, int values_are_keys) {   // q_out may be qkv
    const int n = blockIdx.x, wave = threadIdx.x / SIA_WAVE, lane = threadIdx.x % SIA_WAVE;
    const int pos = positions[n];
    const int half = rotary_dim / 2;
    int page = -1, off = 0;
    if (n_kv > 0) {
        page = block_table[(size_t)seq_of_token[n] * table_width + pos / page_size];
        off = pos % page_size;
    }
    // values that are the keys as projected: the value rows are read from the k columns, and the row has no v columns
    const int k_first = n_heads * head_dim, v_first = values_are_keys ? k_first : k_first + n_kv * head_dim;
    const int qk_groups = (n_heads + n_kv + QKP_WAVES - 1) / QKP_WAVES;
    if ((int)blockIdx.y >= qk_groups) {  // the token's values
        if (page >= 0)
            write_values<T>(qkv, row_stride, bias, positions, seq_of_token, v_pages, n, n_tokens, page, off, pos, v_first,
                            n_kv * value_dim, value_dim, v_rows, page_size, v_group);
        return;
    }
    const int item = blockIdx.y * QKP_WAVES + wave;
    if (item >= n_heads + n_kv) return;  // wave-uniform
    T* row = qkv + (size_t)n * row_stride;
    const bool is_q = item < n_heads;
    const int h = is_q ? item : item - n_heads;
    const int col0 = is_q ? h * head_dim : k_first + h * head_dim;
    const float* gain = is_q ? q_gain : k_gain;
    float x[QKP_PER_LANE];
    float ss = 0.f;
#pragma unroll
    for (int j = 0; j < QKP_PER_LANE; ++j) {
        const int d = lane + j * SIA_WAVE;
        x[j] = 0.f;
        if (d < head_dim) {
            x[j] = to_float(row[col0 + d]);
            if (bias) x[j] += bias[col0 + d];
        }
        ss += x[j] * x[j];
    }
    if (gain) {
        const float inv = rsqrtf(wave_sum(ss) / (float)head_dim + eps);
#pragma unroll
        for (int j = 0; j < QKP_PER_LANE; ++j) {
            const int d = lane + j * SIA_WAVE;
            if (d < head_dim) x[j] = x[j] * inv * gain[d];
        }
    }
    if (is_q && temp_every > 0) {
        const float temp = query_temperature(pos, temp_coef, temp_every);
#pragma unroll
        for (int j = 0; j < QKP_PER_LANE; ++j) x[j] *= temp;
    }
    T* dst = is_q ? q_out + (size_t)n * q_row_stride + h * q_head_stride
                  : (page >= 0 ? k_pages + (((size_t)page * n_kv + h) * page_size + off) * k_row : nullptr);
#pragma unroll
    for (int j = 0; j < QKP_PER_LANE; ++j) {
        if (j * SIA_WAVE >= head_dim) break;  // wave-uniform: the exchanges below are taken by all lanes or by none
        const int d = lane + j * SIA_WAVE;
        // element d turns with element d + half (d < half) or d - half (half <= d < rotary_dim)
        const int mate = d < half ? d + half : (d < rotary_dim ? d - half : d);
        float other = 0.f;
#pragma unroll
        for (int jj = 0; jj < QKP_PER_LANE; ++jj) {
            if (jj * SIA_WAVE >= head_dim) break;
            const float got = __shfl(x[jj], mate % SIA_WAVE, SIA_WAVE);
            if (mate / SIA_WAVE == jj) other = got;
        }
        if (d >= head_dim) continue;
        float v = x[j];
        if (d < half) v = x[j] * cos_table[(size_t)pos * half + d] - other * sin_table[(size_t)pos * half + d];
        else if (d < rotary_dim) v = x[j] * cos_table[(size_t)pos * half + d - half] + other * sin_table[(size_t)pos * half + d - half];
        if (dst) dst[d] = from_float<T>(v);
    }
}

// The same for head sizes of 16, 32, 64, 128 or 256 with rotary_dim a multiple of 16: a lane takes 8 consecutive
// elements with 16- and 32-byte accesses, a head is head_dim / 8 neighbouring lanes, a wave 64 / (head_dim / 8)
// heads; sums and the rotation's partners cross lanes inside a head's group only.  All of a lane's loads are
// independent of one another and issued before the first is used.
template <typename T>
__global__ __launch_bounds__(QKP_WAVES* SIA_WAVE) void qk_prepare_vec_kernel(
    T* qkv, int row_stride, const float* __restrict__ bias, const float* __restrict__ q_gain,
    const float* __restrict__ k_gain, float eps, const float* __restrict__ cos_table,
    const float* __restrict__ sin_table, const int* __restrict__ positions, const int* __restrict__ seq_of_token,
    const int* __restrict__ block_table, int table_width, T* __restrict__ k_pages, T* __restrict__ v_pages,
    int n_tokens, int n_heads, int n_kv, int head_dim, int value_dim, int rotary_dim, int page_size, int v_group,
    int k_row, int v_rows, T* q_out, int q_row_stride, int q_head_stride, float temp_coef,
    int temp_every, int values_are_keys) {   // q_out may be qkv
    const int n = blockIdx.x, wave = threadIdx.x / SIA_WAVE, lane = threadIdx.x % SIA_WAVE;
    const int pos = positions[n];
    const int half = rotary_dim / 2;
    const int group = head_dim / 8, heads_a_wave = SIA_WAVE / group;   // lanes of a head; a power of two up to 32
    // values that are the keys as projected: the value rows are read from the k columns, and the row has no v columns
    const int k_first = n_heads * head_dim, v_first = values_are_keys ? k_first : k_first + n_kv * head_dim;
    const int qk_groups = (n_heads + n_kv + QKP_WAVES * heads_a_wave - 1) / (QKP_WAVES * heads_a_wave);
    if ((int)blockIdx.y >= qk_groups) {  // the token's values
        const int page = block_table[(size_t)seq_of_token[n] * table_width + pos / page_size];
        if (page >= 0)
            write_values<T>(qkv, row_stride, bias, positions, seq_of_token, v_pages, n, n_tokens, page, pos % page_size,
                            pos, v_first, n_kv * value_dim, value_dim, v_rows, page_size, v_group);
        return;
    }
    const int item = (blockIdx.y * QKP_WAVES + wave) * heads_a_wave + lane / group;
    const bool live = item < n_heads + n_kv;
    const int it = live ? item : 0;      // lanes without a head go along (the exchanges are taken by all) and store nothing
    const bool is_q = it < n_heads;
    const int h = is_q ? it : it - n_heads;
    const int d0 = (lane % group) * 8;
    const int col = (is_q ? h * head_dim : k_first + h * head_dim) + d0;
    T* row = qkv + (size_t)n * row_stride;
    const bool turns = d0 < rotary_dim, low = d0 < half;
    const int t0 = low ? d0 : d0 - half;   // where this piece's angles lie in the tables' row
    Vec8<T> vx;
    Vec8<float> vb, vg, vc, vs;
    vx.load(row + col);
    if (bias) vb.load(bias + col);
    const float* gain = is_q ? q_gain : k_gain;
    if (gain) vg.load(gain + d0);
    if (turns) {
        vc.load(cos_table + (size_t)pos * half + t0);
        vs.load(sin_table + (size_t)pos * half + t0);
    }
    int page = -1;
    if (!is_q) page = block_table[(size_t)seq_of_token[n] * table_width + pos / page_size];
    float x[8], b[8], g[8], c[8], sn[8];
    vx.get(x);
    if (bias) {
        vb.get(b);
#pragma unroll
        for (int i = 0; i < 8; ++i) x[i] += b[i];
    }
    if (gain) {
        float ss = 0.f;
#pragma unroll
        for (int i = 0; i < 8; ++i) ss += x[i] * x[i];
        for (int o = group / 2; o > 0; o >>= 1) ss += __shfl_xor(ss, o, SIA_WAVE);   // fixed order inside the head's lanes
        const float inv = rsqrtf(ss / (float)head_dim + eps);
        vg.get(g);
#pragma unroll
        for (int i = 0; i < 8; ++i) x[i] = x[i] * inv * g[i];
    }
    if (is_q && temp_every > 0) {
        const float temp = query_temperature(pos, temp_coef, temp_every);
#pragma unroll
        for (int i = 0; i < 8; ++i) x[i] *= temp;
    }
    if (rotary_dim > 0) {   // wave-uniform: every lane takes the exchange
        const int mate = turns ? (low ? lane + half / 8 : lane - half / 8) : lane;
        float other[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) other[i] = __shfl(x[i], mate, SIA_WAVE);
        if (turns) {
            vc.get(c);
            vs.get(sn);
#pragma unroll
            for (int i = 0; i < 8; ++i) x[i] = low ? x[i] * c[i] - other[i] * sn[i] : x[i] * c[i] + other[i] * sn[i];
        }
    }
    if (!live) return;
    vx.set(x);
    if (is_q) vx.store(q_out + (size_t)n * q_row_stride + h * q_head_stride + d0);
    else if (page >= 0) vx.store(k_pages + (((size_t)page * n_kv + h) * page_size + pos % page_size) * k_row + d0);
}

SIA_EXPORT int sia_qk_prepare_max_head_dim() { return QKP_MAX_HEAD_DIM; }

// values_are_keys: the row is [q heads | k heads] and a position's value rows are its k heads as projected (with
// their bias, before norm and rotation); value_dim is then head_dim.
SIA_EXPORT int sia_qk_prepare_ex(void* qkv, int row_stride, const float* bias, const float* q_gain, const float* k_gain,
                                 float eps, const float* cos_table, const float* sin_table, const int* positions,
                                 const int* seq_of_token, const int* block_table, int table_width, void* k_pages,
                                 void* v_pages, int n_tokens, int n_heads, int n_kv, int head_dim, int value_dim,
                                 int rotary_dim, int page_size, int k_row, int v_rows, void* q_out, int q_row_stride,
                                 int q_head_stride, float temp_coef, int temp_every, int values_are_keys, int dtype,
                                 hipStream_t stream) {
    if (n_tokens <= 0) return 0;
    if (values_are_keys && value_dim != head_dim) return SIA_BAD_ARGUMENT;
    if (head_dim <= 0 || head_dim > QKP_MAX_HEAD_DIM || value_dim <= 0 || n_heads < 0 || n_kv < 0) return SIA_BAD_ARGUMENT;
    if (rotary_dim < 0 || rotary_dim > head_dim || (rotary_dim & 1)) return SIA_BAD_ARGUMENT;
    if (rotary_dim > 0 && (!cos_table || !sin_table)) return SIA_BAD_ARGUMENT;
    if ((q_gain == nullptr) != (k_gain == nullptr)) return SIA_BAD_ARGUMENT;
    if (n_kv > 0 && (!k_pages || !v_pages || !block_table || page_size <= 0)) return SIA_BAD_ARGUMENT;
    if (row_stride < n_heads * head_dim + n_kv * (head_dim + (values_are_keys ? 0 : value_dim))) return SIA_BAD_ARGUMENT;
    if (n_kv > 0 && (k_row < head_dim || v_rows < value_dim)) return SIA_BAD_ARGUMENT;
    if (!q_out) {  // q goes back where it came from
        q_out = qkv;
        q_row_stride = row_stride;
        q_head_stride = head_dim;
    }
    if (q_head_stride < head_dim || q_row_stride < n_heads * q_head_stride) return SIA_BAD_ARGUMENT;
    if (n_heads + n_kv > 65535 * QKP_WAVES) return SIA_BAD_ARGUMENT;
    // tokens whose values one workgroup writes together (0: every token its own); needs runs aligned to 16 bytes
    const int v_group = (n_kv > 0 && n_tokens > 1 && page_size % 16 == 0) ? 16 : (n_kv > 0 && n_tokens > 1 && page_size % 8 == 0) ? 8 : 0;
    const bool vec = (head_dim == 16 || head_dim == 32 || head_dim == 64 || head_dim == 128 || head_dim == 256) &&
                     rotary_dim % 16 == 0 && row_stride % 8 == 0 && q_row_stride % 8 == 0 && q_head_stride % 8 == 0 &&
                     k_row % 8 == 0;
    const int heads_a_group = QKP_WAVES * (vec ? SIA_WAVE / (head_dim / 8) : 1);
    dim3 grid(n_tokens, (n_heads + n_kv + heads_a_group - 1) / heads_a_group + (n_kv > 0 ? 1 : 0)), block(QKP_WAVES * SIA_WAVE);
#define LAUNCH(T)                                                                                                    \
    do {                                                                                                             \
        if (vec)                                                                                                     \
            hipLaunchKernelGGL(qk_prepare_vec_kernel<T>, grid, block, 0, stream, (T*)qkv, row_stride, bias, q_gain,  \
                               k_gain, eps, cos_table, sin_table, positions, seq_of_token, block_table, table_width, \
                               (T*)k_pages, (T*)v_pages, n_tokens, n_heads, n_kv, head_dim, value_dim, rotary_dim,   \
                               page_size, v_group, k_row, v_rows, (T*)q_out, q_row_stride, q_head_stride, temp_coef,  \
                               temp_every, values_are_keys);                                                                       \
        else                                                                                                         \
            hipLaunchKernelGGL(qk_prepare_kernel<T>, grid, block, 0, stream, (T*)qkv, row_stride, bias, q_gain,      \
                               k_gain, eps, cos_table, sin_table, positions, seq_of_token, block_table, table_width, \
                               (T*)k_pages, (T*)v_pages, n_tokens, n_heads, n_kv, head_dim, value_dim, rotary_dim,   \
                               page_size, v_group, k_row, v_rows, (T*)q_out, q_row_stride, q_head_stride, temp_coef,  \
                               temp_every, values_are_keys);                                                                       \
    } while (0)
    if (dtype == SIA_F32) LAUNCH(float);
    else if (dtype == SIA_BF16) LAUNCH(bf16_t);
    else return SIA_BAD_ARGUMENT;
#undef LAUNCH
    return SIA_LAUNCH_CHECK();
}

SIA_EXPORT int sia_qk_prepare(void* qkv, int row_stride, const float* bias, const float* q_gain, const float* k_gain,
                              float eps, const float* cos_table, const float* sin_table, const int* positions,
                              const int* seq_of_token, const int* block_table, int table_width, void* k_pages,
                              void* v_pages, int n_tokens, int n_heads, int n_kv, int head_dim, int value_dim,
                              int rotary_dim, int page_size, int k_row, int v_rows, void* q_out, int q_row_stride,
                              int q_head_stride, float temp_coef, int temp_every, int dtype, hipStream_t stream) {
    return sia_qk_prepare_ex(qkv, row_stride, bias, q_gain, k_gain, eps, cos_table, sin_table, positions, seq_of_token,
                             block_table, table_width, k_pages, v_pages, n_tokens, n_heads, n_kv, head_dim, value_dim,
                             rotary_dim, page_size, k_row, v_rows, q_out, q_row_stride, q_head_stride, temp_coef,
                             temp_every, 0, dtype, stream);
}
