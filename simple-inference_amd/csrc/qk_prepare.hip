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
//   (x_i, x_{i+r/2}) <- (x_i c_i - x_{i+r/2} s_i, x_{i+r/2} c_i + x_i s_i),  i < r/2, r = rotary_dim,
//                       c, s from the float tables at the token's absolute position; elements from r on pass
//
// q is written back in place, k goes to the token's place in its page, v (with its bias) too.
//
// Page layout:  keys   [page][kv_head][offset][head_dim]
//               values [page][kv_head][value_dim][offset]      (positions innermost)
//
// One workgroup a token, one wave a head at a time (the workgroup's waves take the heads in turns), a lane the
// elements lane, lane + 64, ...
#include "common.h"

#define QKP_MAX_HEAD_DIM 256
#define QKP_WAVES 4

template <typename T>
__global__ __launch_bounds__(QKP_WAVES* SIA_WAVE) void qk_prepare_kernel(
    T* __restrict__ qkv, int row_stride, const float* __restrict__ bias, const float* __restrict__ q_gain,
    const float* __restrict__ k_gain, float eps, const float* __restrict__ cos_table,
    const float* __restrict__ sin_table, const int* __restrict__ positions, const int* __restrict__ seq_of_token,
    const int* __restrict__ block_table, int table_width, T* __restrict__ k_pages, T* __restrict__ v_pages,
    int n_heads, int n_kv, int head_dim, int value_dim, int rotary_dim, int page_size) {
    __shared__ float normed[QKP_WAVES][QKP_MAX_HEAD_DIM];
    const int n = blockIdx.x, wave = threadIdx.x / SIA_WAVE, lane = threadIdx.x % SIA_WAVE;
    const int pos = positions[n];
    const int half = rotary_dim / 2;
    T* row = qkv + (size_t)n * row_stride;
    const float* cs = cos_table ? cos_table + (size_t)pos * half : nullptr;
    const float* sn = sin_table ? sin_table + (size_t)pos * half : nullptr;
    int page = -1, off = 0;
    if (n_kv > 0) {
        page = block_table[(size_t)seq_of_token[n] * table_width + pos / page_size];
        off = pos % page_size;
    }
    const int k_first = n_heads * head_dim, v_first = k_first + n_kv * head_dim;

    const int total = n_heads + 2 * n_kv;
    for (int first = 0; first < total; first += QKP_WAVES) {   // every wave takes every turn: the barriers are shared
        const int item = first + wave;
        const bool qk = item < n_heads + n_kv;
        if (item < total && !qk && page >= 0) {   // a value head: bias, then into the page
            const int h = item - n_heads - n_kv;
            for (int d = lane; d < value_dim; d += SIA_WAVE) {
                const int col = v_first + h * value_dim + d;
                float v = to_float(row[col]);
                if (bias) v += bias[col];
                v_pages[(((size_t)page * n_kv + h) * value_dim + d) * page_size + off] = from_float<T>(v);
            }
        }
        const bool is_q = item < n_heads;
        const int h = is_q ? item : item - n_heads;
        const int col0 = is_q ? h * head_dim : k_first + h * head_dim;
        const float* gain = is_q ? q_gain : k_gain;
        float x[QKP_MAX_HEAD_DIM / SIA_WAVE];
        if (qk) {
            float ss = 0.f;
#pragma unroll
            for (int j = 0; j < QKP_MAX_HEAD_DIM / SIA_WAVE; ++j) {
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
                for (int j = 0; j < QKP_MAX_HEAD_DIM / SIA_WAVE; ++j) {
                    const int d = lane + j * SIA_WAVE;
                    if (d < head_dim) x[j] = x[j] * inv * gain[d];
                }
            }
            // the rotation's partner of an element lies in another lane: through the wave's row of LDS
#pragma unroll
            for (int j = 0; j < QKP_MAX_HEAD_DIM / SIA_WAVE; ++j) {
                const int d = lane + j * SIA_WAVE;
                if (d < head_dim) normed[wave][d] = x[j];
            }
        }
        __syncthreads();
        if (qk) {
            T* dst = is_q ? row + col0
                          : (page >= 0 ? k_pages + (((size_t)page * n_kv + h) * page_size + off) * head_dim : nullptr);
#pragma unroll
            for (int j = 0; j < QKP_MAX_HEAD_DIM / SIA_WAVE; ++j) {
                const int d = lane + j * SIA_WAVE;
                if (d >= head_dim) continue;
                float v = x[j];
                if (d < half) v = x[j] * cs[d] - normed[wave][d + half] * sn[d];
                else if (d < rotary_dim) v = x[j] * cs[d - half] + normed[wave][d - half] * sn[d - half];
                if (dst) dst[d] = from_float<T>(v);
            }
        }
        __syncthreads();   // the rows of LDS are free for the next turn
    }
}

SIA_EXPORT int sia_qk_prepare_max_head_dim() { return QKP_MAX_HEAD_DIM; }

SIA_EXPORT int sia_qk_prepare(void* qkv, int row_stride, const float* bias, const float* q_gain, const float* k_gain,
                              float eps, const float* cos_table, const float* sin_table, const int* positions,
                              const int* seq_of_token, const int* block_table, int table_width, void* k_pages,
                              void* v_pages, int n_tokens, int n_heads, int n_kv, int head_dim, int value_dim,
                              int rotary_dim, int page_size, int dtype, hipStream_t stream) {
    if (n_tokens <= 0) return 0;
    if (head_dim <= 0 || head_dim > QKP_MAX_HEAD_DIM || value_dim <= 0 || n_heads < 0 || n_kv < 0) return SIA_BAD_ARGUMENT;
    if (rotary_dim < 0 || rotary_dim > head_dim || (rotary_dim & 1)) return SIA_BAD_ARGUMENT;
    if (rotary_dim > 0 && (!cos_table || !sin_table)) return SIA_BAD_ARGUMENT;
    if ((q_gain == nullptr) != (k_gain == nullptr)) return SIA_BAD_ARGUMENT;
    if (n_kv > 0 && (!k_pages || !v_pages || !block_table || page_size <= 0)) return SIA_BAD_ARGUMENT;
    if (row_stride < n_heads * head_dim + n_kv * (head_dim + value_dim)) return SIA_BAD_ARGUMENT;
    dim3 grid(n_tokens), block(QKP_WAVES * SIA_WAVE);
#define LAUNCH(T)                                                                                                  \
    hipLaunchKernelGGL(qk_prepare_kernel<T>, grid, block, 0, stream, (T*)qkv, row_stride, bias, q_gain, k_gain, eps, \
                       cos_table, sin_table, positions, seq_of_token, block_table, table_width, (T*)k_pages,       \
                       (T*)v_pages, n_heads, n_kv, head_dim, value_dim, rotary_dim, page_size)
    if (dtype == SIA_F32) LAUNCH(float);
    else if (dtype == SIA_BF16) LAUNCH(bf16_t);
    else return SIA_BAD_ARGUMENT;
#undef LAUNCH
    return SIA_LAUNCH_CHECK();
}
