// The small per-layer operators of the reference's batched decode step
// (compiler/runtime/batched_walker.cpp:246-405) for gfx950: RMSNorm over a batch of rows,
// residual add, SiLU(gate)*up and its form fused with the gate/up split.  All are
// launch-latency bound at decode batch sizes (a few hundred KB); the point of having them is
// that the whole layer stays on the device between the attention calls.
//
// Arithmetic follows the reference kernels so that results agree with its CPU path to the last
// few bits: no fused multiply-adds where the reference has separate roundings, a correctly
// rounded 1/sqrtf and division, expf instead of a fast approximation.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace mlc_hip {

// MSL rms_norm_kernel_v2_batched (compiler/runtime/metal_runtime.mm:166-208), CPU rmsNorm
// (compiler/runtime/operator_backend.cpp:186-203): out[r][i] = in[r][i] * scale_r * weight[i],
// scale_r = 1 / sqrt(mean_i(in[r][i]^2) + eps).  One workgroup of 256 threads per row.
__global__ __launch_bounds__(256) void rms_norm_batched_kernel(const float* __restrict__ in,
                                                               const float* __restrict__ weight,
                                                               uint32_t n_weight, float epsilon,
                                                               uint32_t length,
                                                               float* __restrict__ out) {
    __shared__ float partial[4];
    const float* x = in + (size_t)blockIdx.x * length;
    float* y = out + (size_t)blockIdx.x * length;
    float sum = 0.f;
    for (uint32_t i = threadIdx.x; i < length; i += 256) {
        const float v = x[i];
        sum = fmaf(v, v, sum);
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) sum += __shfl_xor(sum, off);
    if (threadIdx.x % 64 == 0) partial[threadIdx.x / 64] = sum;
    __syncthreads();
    const float total = (partial[0] + partial[1]) + (partial[2] + partial[3]);
    const float scale = 1.0f / sqrtf(total / (float)length + epsilon);
    for (uint32_t i = threadIdx.x; i < length; i += 256) {
        const float gamma = i < n_weight ? weight[i] : 1.0f;
        y[i] = x[i] * scale * gamma;
    }
}

// MSL add_vectors (metal_runtime.mm:44-52) over a flat range.
__global__ __launch_bounds__(256) void add_kernel(const float* __restrict__ a,
                                                  const float* __restrict__ b,
                                                  float* __restrict__ out, uint32_t n) {
    const uint32_t i = blockIdx.x * 256 + threadIdx.x;
    if (i < n) out[i] = a[i] + b[i];
}

__device__ __forceinline__ float silu_times(float g, float u) {
    const float silu = g / (1.0f + expf(-g));
    return silu * u;
}

// MSL feedforward_silu_mul (metal_runtime.mm:32-42).
__global__ __launch_bounds__(256) void silu_mul_kernel(const float* __restrict__ gate,
                                                       const float* __restrict__ up,
                                                       float* __restrict__ out, uint32_t n) {
    const uint32_t i = blockIdx.x * 256 + threadIdx.x;
    if (i < n) out[i] = silu_times(gate[i], up[i]);
}

// MetalExecutor::encodeGateUpSplitSiluMul (metal_runtime.mm:8029-8091): two strided copies and
// the SiLU product, here one pass that writes all three outputs.
__global__ __launch_bounds__(256) void gate_up_split_silu_mul_kernel(
    const float* __restrict__ gate_up, float* __restrict__ gate, float* __restrict__ up,
    float* __restrict__ out, uint32_t batch, uint32_t ffn_inner, uint32_t gate_up_rows) {
    const uint32_t i = blockIdx.x * 256 + threadIdx.x;
    if (i >= batch * ffn_inner) return;
    const uint32_t r = i / ffn_inner, c = i - r * ffn_inner;
    const float g = gate_up[(size_t)r * gate_up_rows + c];
    const float u = gate_up[(size_t)r * gate_up_rows + ffn_inner + c];
    gate[i] = g;
    up[i] = u;
    out[i] = silu_times(g, u);
}

}  // namespace mlc_hip
