// Mixture of experts: the router, and the experts' products for a token's chosen experts.
//
//   route:    z = R h (float, R float [E, width]); the ``top`` largest logits (ties: the lower index) and the softmax
//             over those alone:  ids [N, top] int32,  weights [N, top] float
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

template <typename T>
__global__ __launch_bounds__(256) void moe_route_kernel(const T* __restrict__ h, const float* __restrict__ router,
                                                         int* __restrict__ ids, float* __restrict__ weights, int width,
                                                         int n_experts, int top) {
    __shared__ float logit_s[MOE_MAX_EXPERTS];
    const int n = blockIdx.x, wave = threadIdx.x / SIA_WAVE, lane = threadIdx.x % SIA_WAVE;
    const T* x = h + (size_t)n * width;
    for (int e = wave; e < n_experts; e += blockDim.x / SIA_WAVE) {
        const float* w = router + (size_t)e * width;
        float acc = 0.f;
        for (int i = lane; i < width; i += SIA_WAVE) acc += to_float(x[i]) * w[i];
        acc = wave_sum(acc);
        if (lane == 0) logit_s[e] = acc;
    }
    __syncthreads();
    if (wave != 0) return;
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
        if (k == 0) first = best;
        const float p = expf(best - first);
        total += p;
        if (lane == k) { chosen = p; chosen_id = which; }
        if (lane == 0 && which < n_experts) logit_s[which] = -INFINITY;
        __builtin_amdgcn_wave_barrier();
        __threadfence_block();
    }
    if (lane < top) {
        ids[(size_t)n * top + lane] = chosen_id;
        weights[(size_t)n * top + lane] = chosen / total;
    }
}

SIA_EXPORT int sia_moe_route(const void* h, const float* router, int* ids, float* weights, int n_tokens, int width,
                             int n_experts, int top, int dtype, hipStream_t stream) {
    if (n_tokens <= 0) return 0;
    if (n_experts <= 0 || n_experts > MOE_MAX_EXPERTS || top <= 0 || top > n_experts || top > MOE_MAX_TOP)
        return SIA_BAD_ARGUMENT;
    dim3 grid(n_tokens), block(256);
    if (dtype == SIA_F32)
        hipLaunchKernelGGL(moe_route_kernel<float>, grid, block, 0, stream, (const float*)h, router, ids, weights, width,
                           n_experts, top);
    else if (dtype == SIA_BF16)
        hipLaunchKernelGGL(moe_route_kernel<bf16_t>, grid, block, 0, stream, (const bf16_t*)h, router, ids, weights,
                           width, n_experts, top);
    else
        return SIA_BAD_ARGUMENT;
    return SIA_LAUNCH_CHECK();
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
    int ff, int top, bool vec) {
    const int slot = blockIdx.x, wave = threadIdx.x / SIA_WAVE, lane = threadIdx.x % SIA_WAVE;
    const int e = ids[slot];
    const T* x = h + (size_t)(slot / top) * width;
    const T* w = w1 + (size_t)e * 2 * ff * width;
    const int f0 = (blockIdx.y * MOE_WAVES + wave) * MOE_PER_WAVE;
    for (int f = f0; f < min(ff, f0 + MOE_PER_WAVE); ++f) {
        const float g = wave_dot<T>(x, w + (size_t)f * width, width, lane, vec);
        const float u = wave_dot<T>(x, w + (size_t)(ff + f) * width, width, lane, vec);
        if (lane == 0) act[(size_t)slot * ff + f] = from_float<T>(g / (1.f + expf(-g)) * u);
    }
}

template <typename T>
__global__ __launch_bounds__(MOE_WAVES* SIA_WAVE) void moe_down_kernel(
    const T* __restrict__ act, const T* __restrict__ w2, const int* __restrict__ ids, const float* __restrict__ weights,
    const T* __restrict__ shared, const T* __restrict__ shared_gate, int shared_gate_stride, T* __restrict__ out,
    int width, int ff, int top, bool vec) {
    const int n = blockIdx.x, wave = threadIdx.x / SIA_WAVE, lane = threadIdx.x % SIA_WAVE;
    const int c0 = (blockIdx.y * MOE_WAVES + wave) * MOE_PER_WAVE;
    for (int c = c0; c < min(width, c0 + MOE_PER_WAVE); ++c) {
        float y = 0.f;
        for (int k = 0; k < top; ++k) {
            const int slot = n * top + k;
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

SIA_EXPORT int sia_moe_gate_up(const void* h, const void* w1, const int* ids, void* act, int n_tokens, int width, int ff,
                               int top, int dtype, hipStream_t stream) {
    if (n_tokens <= 0) return 0;
    if (width <= 0 || ff <= 0 || top <= 0 || (long long)n_tokens * top > 0x7fffffffLL) return SIA_BAD_ARGUMENT;
    const int per_block = MOE_WAVES * MOE_PER_WAVE;
    dim3 grid(n_tokens * top, (ff + per_block - 1) / per_block), block(MOE_WAVES * SIA_WAVE);
    if (grid.y > 65535) return SIA_BAD_ARGUMENT;
    const bool vec = width % 8 == 0;
    if (dtype == SIA_F32)
        hipLaunchKernelGGL(moe_gate_up_kernel<float>, grid, block, 0, stream, (const float*)h, (const float*)w1, ids,
                           (float*)act, width, ff, top, vec);
    else if (dtype == SIA_BF16)
        hipLaunchKernelGGL(moe_gate_up_kernel<bf16_t>, grid, block, 0, stream, (const bf16_t*)h, (const bf16_t*)w1, ids,
                           (bf16_t*)act, width, ff, top, vec);
    else
        return SIA_BAD_ARGUMENT;
    return SIA_LAUNCH_CHECK();
}

SIA_EXPORT int sia_moe_down(const void* act, const void* w2, const int* ids, const float* weights, const void* shared,
                            const void* shared_gate, int shared_gate_stride, void* out, int n_tokens, int width, int ff,
                            int top, int dtype, hipStream_t stream) {
    if (n_tokens <= 0) return 0;
    if (width <= 0 || ff <= 0 || top <= 0 || (shared_gate && !shared)) return SIA_BAD_ARGUMENT;
    const int per_block = MOE_WAVES * MOE_PER_WAVE;
    dim3 grid(n_tokens, (width + per_block - 1) / per_block), block(MOE_WAVES * SIA_WAVE);
    if (grid.y > 65535) return SIA_BAD_ARGUMENT;
    const bool vec = ff % 8 == 0;
    if (dtype == SIA_F32)
        hipLaunchKernelGGL(moe_down_kernel<float>, grid, block, 0, stream, (const float*)act, (const float*)w2, ids,
                           weights, (const float*)shared, (const float*)shared_gate, shared_gate_stride, (float*)out,
                           width, ff, top, vec);
    else if (dtype == SIA_BF16)
        hipLaunchKernelGGL(moe_down_kernel<bf16_t>, grid, block, 0, stream, (const bf16_t*)act, (const bf16_t*)w2, ids,
                           weights, (const bf16_t*)shared, (const bf16_t*)shared_gate, shared_gate_stride, (bf16_t*)out,
                           width, ff, top, vec);
    else
        return SIA_BAD_ARGUMENT;
    return SIA_LAUNCH_CHECK();
}
