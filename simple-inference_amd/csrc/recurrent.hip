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
// A workgroup owns one (sequence, head) and walks the sequence's tokens of this step in order, so a request's
// numbers depend on its own tokens only: not on how its prompt was cut, nor on what else the step holds.
// Thread (j, r) keeps rows r, r + R, r + 2R, ... of column j of S in registers (R a power of two: the lanes of a
// column are neighbours and add their shares of o by lane exchanges).  Blocks of a few tokens are staged through
// LDS (q, k, alpha, v, g as floats), walked, and their outputs normed and gated a token a wave.
#include "common.h"

__device__ __forceinline__ float log_sigmoid(float z) { return fminf(z, 0.f) - log1pf(expf(-fabsf(z))); }

template <typename T, int ROWS>
__global__ __launch_bounds__(512) void gla_recurrent_kernel(
    const T* __restrict__ proj, int row_stride, int q_col, int k_col, int v_col, int g_col, int a_col,
    const T* __restrict__ a2, const float* __restrict__ a2_bias, const float* __restrict__ norm_w,
    float* __restrict__ state, const int* __restrict__ cu_q, const int* __restrict__ slots, T* __restrict__ out,
    int n_heads, int D, int Dv, int rank, int R, int block_tokens, float tau_inv, float q_scale, float eps) {
    extern __shared__ float lds[];
    const int seq = blockIdx.x, head = blockIdx.y, tid = threadIdx.x;
    const int first = cu_q[seq], last = cu_q[seq + 1];
    if (first >= last) return;
    const int TB = block_tokens;
    float* q_s = lds;                  // [TB][D]
    float* k_s = q_s + TB * D;         // [TB][D]
    float* al_s = k_s + TB * D;        // [TB][D]
    float* v_s = al_s + TB * D;        // [TB][Dv]
    float* g_s = v_s + TB * Dv;        // [TB][Dv]
    float* o_s = g_s + TB * Dv;        // [TB][Dv]
    float* a_s = o_s + TB * Dv;        // [TB][rank]

    const int j = tid / R, r = tid % R;
    const bool owns = j < Dv;
    float* S_mem = state + ((size_t)slots[seq] * n_heads + head) * D * Dv;
    float S[ROWS];
#pragma unroll
    for (int i = 0; i < ROWS; ++i) {
        const int d = i * R + r;
        S[i] = (owns && d < D) ? S_mem[(size_t)d * Dv + j] : 0.f;
    }
    const int wave = tid / SIA_WAVE, lane = tid % SIA_WAVE, n_waves = blockDim.x / SIA_WAVE;

    for (int t0 = first; t0 < last; t0 += TB) {
        const int nt = min(TB, last - t0);
        for (int idx = tid; idx < nt * rank; idx += blockDim.x) {
            const int t = idx / rank, c = idx % rank;
            a_s[idx] = to_float(proj[(size_t)(t0 + t) * row_stride + a_col + c]);
        }
        for (int idx = tid; idx < nt * Dv; idx += blockDim.x) {
            const int t = idx / Dv, c = idx % Dv;
            const T* row = proj + (size_t)(t0 + t) * row_stride;
            v_s[t * Dv + c] = to_float(row[v_col + head * Dv + c]);
            g_s[t * Dv + c] = to_float(row[g_col + head * Dv + c]);
        }
        __syncthreads();
        for (int idx = tid; idx < nt * D; idx += blockDim.x) {
            const int t = idx / D, c = idx % D;
            const T* row = proj + (size_t)(t0 + t) * row_stride;
            q_s[t * D + c] = to_float(row[q_col + head * D + c]) * q_scale;
            k_s[t * D + c] = to_float(row[k_col + head * D + c]);
            const T* w = a2 + (size_t)(head * D + c) * rank;
            float z = a2_bias ? a2_bias[head * D + c] : 0.f;
            for (int m = 0; m < rank; ++m) z += a_s[t * rank + m] * to_float(w[m]);
            al_s[t * D + c] = expf(log_sigmoid(z) * tau_inv);
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
            if (owns && r == 0) o_s[t * Dv + j] = acc;
        }
        __syncthreads();
        for (int t = wave; t < nt; t += n_waves) {
            float ss = 0.f;
            for (int c = lane; c < Dv; c += SIA_WAVE) ss += o_s[t * Dv + c] * o_s[t * Dv + c];
            const float inv = rsqrtf(wave_sum(ss) / (float)Dv + eps);
            T* dst = out + ((size_t)(t0 + t) * n_heads + head) * Dv;
            for (int c = lane; c < Dv; c += SIA_WAVE) {
                const float g = g_s[t * Dv + c];
                dst[c] = from_float<T>(o_s[t * Dv + c] * inv * norm_w[c] * (g / (1.f + expf(-g))));
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

SIA_EXPORT int sia_gla_max_dims() { return 512; }

SIA_EXPORT int sia_gla_recurrent(const void* proj, int row_stride, int q_col, int k_col, int v_col, int g_col, int a_col,
                                 const void* a2, const float* a2_bias, const float* norm_w, float* state,
                                 const int* cu_q, const int* slots, void* out, int n_seqs, int max_q_len, int n_heads,
                                 int D, int Dv, int rank, float tau, float q_scale, float eps, int dtype,
                                 hipStream_t stream) {
    if (n_seqs <= 0) return 0;
    if (D <= 0 || Dv <= 0 || D > 512 || Dv > 512 || rank <= 0 || rank > 1024 || n_heads <= 0 || n_heads > 65535 ||
        !(tau > 0.f) || !state || !norm_w)
        return SIA_BAD_ARGUMENT;
    // lanes a column: the largest power of two that keeps the workgroup within 512 threads and a wave's columns whole
    int R = 1;
    while (R * 2 <= SIA_WAVE && Dv * R * 2 <= 512 && R * 2 <= D) R *= 2;
    const int rows = (D + R - 1) / R;
    if (rows > 128) return SIA_BAD_ARGUMENT;
    const int threads = ((Dv * R + SIA_WAVE - 1) / SIA_WAVE) * SIA_WAVE;
    int TB = max_q_len >= 16 ? 16 : (max_q_len >= 4 ? 4 : 1);
    auto bytes = [&](int tb) { return (size_t)tb * (3 * D + 3 * Dv + rank) * sizeof(float); };
    while (TB > 1 && bytes(TB) > 60 * 1024) TB /= 2;
    if (bytes(TB) > 60 * 1024) return SIA_BAD_ARGUMENT;
    dim3 grid(n_seqs, n_heads), block(threads);
#define LAUNCH(T, ROWS)                                                                                              \
    hipLaunchKernelGGL((gla_recurrent_kernel<T, ROWS>), grid, block, bytes(TB), stream, (const T*)proj, row_stride,  \
                       q_col, k_col, v_col, g_col, a_col, (const T*)a2, a2_bias, norm_w, state, cu_q, slots, (T*)out, \
                       n_heads, D, Dv, rank, R, TB, 1.f / tau, q_scale, eps)
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
    return SIA_LAUNCH_CHECK();
}
