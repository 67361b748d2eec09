// Gates on the way into the residual stream and small steps around them.
//
//   gated add + RMS norm:   x = residual[row] + (delta[row] + delta_bias) * sigmoid(gate[row] + gate_bias)
//                           y = x * rsqrt(mean(x^2) + eps) * w
//     the counterpart of the plain residual add + RMS norm for blocks whose sublayers' results pass an elementwise
//     sigmoid gate.  ``gate`` holds the gate's logits (a product's columns: rows gate_stride apart; without it the
//     factor is 1); the sigmoid,
//     the product with the delta, the sum and the norm are float with one rounding of y.  Without w nothing is
//     normed and only the residual is updated (the sum is wanted by itself: where a stream is re-mixed).  With
//     ``rows`` only those rows are normed and the residual is left as it was.
//   bias:                   y[n, :] += b                                in place
//   head gate:              out[n, h, :] *= sigmoid(logit[n, h])        a scalar for every token and head
//   side by side:           out[n, :] = [T(a[n, :]), T(b[n, :])]        two float streams lowered into one row
//   scale + soft cap:       z <- cap * tanh(z * scale / cap)            (cap <= 0: z <- z * scale), in place, float
#include "common.h"

__device__ __forceinline__ float sigmoidf_(float z) { return 1.f / (1.f + expf(-z)); }

template <typename T>
__global__ void gated_add_rmsnorm_kernel(float* __restrict__ residual, const T* __restrict__ delta,
                                         const float* __restrict__ delta_bias, const T* __restrict__ gate,
                                         int gate_stride, const float* __restrict__ gate_bias,
                                         const float* __restrict__ weight, T* __restrict__ out,
                                         const int* __restrict__ rows, int hidden, float eps) {
    __shared__ float scratch[16];
    const int i_out = blockIdx.x;
    const int row = rows ? rows[i_out] : i_out;
    float* res = residual + (size_t)row * hidden;
    const T* del = delta + (size_t)row * hidden;
    const T* g = gate ? gate + (size_t)row * gate_stride : nullptr;
    float ss = 0.f;
    for (int i = threadIdx.x; i < hidden; i += blockDim.x) {
        float d = to_float(del[i]);
        if (delta_bias) d += delta_bias[i];
        if (g) {
            float z = to_float(g[i]);
            if (gate_bias) z += gate_bias[i];
            d *= sigmoidf_(z);
        }
        const float x = res[i] + d;
        if (!rows) res[i] = x;
        ss += x * x;
    }
    if (!weight) return;   // uniform over the grid
    ss = block_sum(ss, scratch);
    const float inv = rsqrtf(ss / (float)hidden + eps);
    T* dst = out + (size_t)i_out * hidden;
    for (int i = threadIdx.x; i < hidden; i += blockDim.x) {
        float x = res[i];
        if (rows) {   // the residual was not written: the same sum once more
            float d = to_float(del[i]);
            if (delta_bias) d += delta_bias[i];
            if (g) {
                float z = to_float(g[i]);
                if (gate_bias) z += gate_bias[i];
                d *= sigmoidf_(z);
            }
            x += d;
        }
        dst[i] = from_float<T>(x * inv * weight[i]);
    }
}

// The same for rows that one workgroup holds in registers (hidden % 8 == 0, hidden <= 8 * 1024, gate rows aligned
// to 8 elements): every input is read once, with 16- and 32-byte accesses issued before the first is used.
template <typename T>
__global__ void gated_add_rmsnorm_row_kernel(float* __restrict__ residual, const T* __restrict__ delta,
                                             const float* __restrict__ delta_bias, const T* __restrict__ gate,
                                             int gate_stride, const float* __restrict__ gate_bias,
                                             const float* __restrict__ weight, T* __restrict__ out,
                                             const int* __restrict__ rows, int hidden, float eps) {
    __shared__ float scratch[16];
    const int i_out = blockIdx.x;
    const int row = rows ? rows[i_out] : i_out;
    const int i0 = threadIdx.x * 8;
    const bool live = i0 < hidden;
    float x[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f}, w[8];
    if (live) {
        Vec8<float> vr, vw, vdb, vgb;
        Vec8<T> vd, vg;
        vr.load(residual + (size_t)row * hidden + i0);
        vd.load(delta + (size_t)row * hidden + i0);
        if (gate) vg.load(gate + (size_t)row * gate_stride + i0);
        if (weight) vw.load(weight + i0);
        if (delta_bias) vdb.load(delta_bias + i0);
        if (gate_bias) vgb.load(gate_bias + i0);
        float d[8], z[8], b[8];
        vr.get(x);
        vd.get(d);
        if (gate) vg.get(z);
        if (weight) vw.get(w);
        if (delta_bias) {
            vdb.get(b);
#pragma unroll
            for (int i = 0; i < 8; ++i) d[i] += b[i];
        }
        if (gate && gate_bias) {
            vgb.get(b);
#pragma unroll
            for (int i = 0; i < 8; ++i) z[i] += b[i];
        }
#pragma unroll
        for (int i = 0; i < 8; ++i) x[i] += gate ? d[i] * sigmoidf_(z[i]) : d[i];
        if (!rows) {
            vr.set(x);
            vr.store(residual + (size_t)row * hidden + i0);
        }
    }
    if (!weight) return;
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

SIA_EXPORT int sia_gated_add_rmsnorm(float* residual, const void* delta, const float* delta_bias, const void* gate,
                                     int gate_stride, const float* gate_bias, const float* weight, void* out,
                                     const int* rows, int n_out, int hidden, float eps, int dtype,
                                     hipStream_t stream) {
    if (n_out <= 0) return 0;
    if ((dtype != SIA_F32 && dtype != SIA_BF16) || !delta || (gate && gate_stride < hidden) || (weight && !out) ||
        (!weight && rows) || (!gate && gate_bias))
        return SIA_BAD_ARGUMENT;
    dim3 grid(n_out);
    const int el = dtype == SIA_F32 ? 4 : 2;
    const bool aligned = !gate || (gate_stride % 8 == 0 && ((uintptr_t)gate % (8 * el)) == 0);
    if (hidden % 8 == 0 && hidden <= 8 * 1024 && aligned) {
        dim3 block(((hidden / 8 + SIA_WAVE - 1) / SIA_WAVE) * SIA_WAVE);
        if (dtype == SIA_F32)
            hipLaunchKernelGGL(gated_add_rmsnorm_row_kernel<float>, grid, block, 0, stream, residual,
                               (const float*)delta, delta_bias, (const float*)gate, gate_stride, gate_bias, weight,
                               (float*)out, rows, hidden, eps);
        else
            hipLaunchKernelGGL(gated_add_rmsnorm_row_kernel<bf16_t>, grid, block, 0, stream, residual,
                               (const bf16_t*)delta, delta_bias, (const bf16_t*)gate, gate_stride, gate_bias, weight,
                               (bf16_t*)out, rows, hidden, eps);
        return SIA_LAUNCH_CHECK();
    }
    dim3 block(hidden >= 2048 ? 512 : 256);
    if (dtype == SIA_F32)
        hipLaunchKernelGGL(gated_add_rmsnorm_kernel<float>, grid, block, 0, stream, residual, (const float*)delta,
                           delta_bias, (const float*)gate, gate_stride, gate_bias, weight, (float*)out, rows, hidden, eps);
    else
        hipLaunchKernelGGL(gated_add_rmsnorm_kernel<bf16_t>, grid, block, 0, stream, residual, (const bf16_t*)delta,
                           delta_bias, (const bf16_t*)gate, gate_stride, gate_bias, weight, (bf16_t*)out, rows, hidden,
                           eps);
    return SIA_LAUNCH_CHECK();
}

// ---------------------------------------------------------------------------------------
// out[n, h, d] *= sigmoid(logits[n * logit_stride + h])
// ---------------------------------------------------------------------------------------
template <typename T>
__global__ void head_gate_kernel(T* __restrict__ out, const T* __restrict__ logits, int logit_stride, int n_heads,
                                 int head_dim) {
    const int n = blockIdx.x;
    T* row = out + (size_t)n * n_heads * head_dim;
    const T* g = logits + (size_t)n * logit_stride;
    for (int i = threadIdx.x; i < n_heads * head_dim; i += blockDim.x)
        row[i] = from_float<T>(to_float(row[i]) * sigmoidf_(to_float(g[i / head_dim])));
}

SIA_EXPORT int sia_head_gate(void* out, const void* logits, int logit_stride, int n_tokens, int n_heads, int head_dim,
                             int dtype, hipStream_t stream) {
    if (n_tokens <= 0) return 0;
    if (n_heads <= 0 || head_dim <= 0 || logit_stride < n_heads) return SIA_BAD_ARGUMENT;
    dim3 grid(n_tokens), block(256);
    if (dtype == SIA_F32)
        hipLaunchKernelGGL(head_gate_kernel<float>, grid, block, 0, stream, (float*)out, (const float*)logits,
                           logit_stride, n_heads, head_dim);
    else if (dtype == SIA_BF16)
        hipLaunchKernelGGL(head_gate_kernel<bf16_t>, grid, block, 0, stream, (bf16_t*)out, (const bf16_t*)logits,
                           logit_stride, n_heads, head_dim);
    else
        return SIA_BAD_ARGUMENT;
    return SIA_LAUNCH_CHECK();
}

// ---------------------------------------------------------------------------------------
// out[n, 0:w] = T(a[n, :]), out[n, w:2w] = T(b[n, :])
// ---------------------------------------------------------------------------------------
template <typename T>
__global__ void side_by_side_kernel(const float* __restrict__ a, const float* __restrict__ b, T* __restrict__ out,
                                    int width) {
    const int n = blockIdx.x;
    for (int i = threadIdx.x; i < width; i += blockDim.x) {
        out[(size_t)n * 2 * width + i] = from_float<T>(a[(size_t)n * width + i]);
        out[(size_t)n * 2 * width + width + i] = from_float<T>(b[(size_t)n * width + i]);
    }
}

SIA_EXPORT int sia_side_by_side(const float* a, const float* b, void* out, int n_rows, int width, int dtype,
                                hipStream_t stream) {
    if (n_rows <= 0) return 0;
    dim3 grid(n_rows), block(256);
    if (dtype == SIA_F32)
        hipLaunchKernelGGL(side_by_side_kernel<float>, grid, block, 0, stream, a, b, (float*)out, width);
    else if (dtype == SIA_BF16)
        hipLaunchKernelGGL(side_by_side_kernel<bf16_t>, grid, block, 0, stream, a, b, (bf16_t*)out, width);
    else
        return SIA_BAD_ARGUMENT;
    return SIA_LAUNCH_CHECK();
}

// ---------------------------------------------------------------------------------------
// z <- cap * tanh(z * scale / cap)   (cap <= 0: z <- z * scale)
// ---------------------------------------------------------------------------------------
__global__ void scale_softcap_kernel(float* __restrict__ z, long long n, float scale, float cap) {
    const long long i0 = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    for (long long i = i0; i < n; i += (long long)gridDim.x * blockDim.x) {
        const float v = z[i] * scale;
        z[i] = cap > 0.f ? cap * tanhf(v / cap) : v;
    }
}

SIA_EXPORT int sia_scale_softcap(float* z, long long n, float scale, float cap, hipStream_t stream) {
    if (n <= 0) return 0;
    const long long blocks = (n + 255) / 256;
    dim3 grid((unsigned)(blocks < 65535 ? blocks : 65535)), block(256);
    hipLaunchKernelGGL(scale_softcap_kernel, grid, block, 0, stream, z, n, scale, cap);
    return SIA_LAUNCH_CHECK();
}

// ---------------------------------------------------------------------------------------
// y[n, :] += bias
// ---------------------------------------------------------------------------------------
template <typename T>
__global__ void add_bias_kernel(T* __restrict__ y, const float* __restrict__ bias, int width) {
    T* row = y + (size_t)blockIdx.x * width;
    for (int i = threadIdx.x; i < width; i += blockDim.x) row[i] = from_float<T>(to_float(row[i]) + bias[i]);
}

SIA_EXPORT int sia_add_bias(void* y, const float* bias, int n_rows, int width, int dtype, hipStream_t stream) {
    if (n_rows <= 0) return 0;
    dim3 grid(n_rows), block(256);
    if (dtype == SIA_F32) hipLaunchKernelGGL(add_bias_kernel<float>, grid, block, 0, stream, (float*)y, bias, width);
    else if (dtype == SIA_BF16) hipLaunchKernelGGL(add_bias_kernel<bf16_t>, grid, block, 0, stream, (bf16_t*)y, bias, width);
    else return SIA_BAD_ARGUMENT;
    return SIA_LAUNCH_CHECK();
}
