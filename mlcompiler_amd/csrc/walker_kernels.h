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

// ---- several row-local operators of one pass in one launch.  At decode batch sizes every one
// of the operators above is a few microseconds of launch and drain around a few hundred KB of
// data, so a chain like  sum of matmul K slices -> + residual -> RMSNorm -> fp16 split for the
// next matmul  costs four launches for work that one workgroup per row does in one.  The host
// collects such a chain while the operators are encoded and hands it over as a RowProgram; the
// results every operator is specified to write are all still written.
//
// Stages, in this order, each optional except the source:
//   source   row = src[row]                                   (plain buffer, row length len_src)
//            or   slice 0 + slice 1 + ...  in that order      (K slices of a matmul), stored to
//            src_store when that is set (the matmul's output buffer)
//   silu     gate = row[0:len], up = row[len:2 len] -> gate_out, up_out;
//            row = gate / (1 + exp(-gate)) * up -> silu_out   (len = len_src / 2)
//   add      row = row + addend[row] -> add_out
//   rms      row = row * 1/sqrt(mean(row^2) + eps) * weight -> rms_out
//   split    row * 2^e = hi + lo (fp16 each) in the matmul's B-operand layout -> frag, 2^-e ->
//            inv_scale  (q4_split_activations_kernel's arithmetic; rows >= batch are zero padding)
// One workgroup of 1024 threads per row (there are only as many rows as requests, so the row
// is spread as wide as a workgroup goes).  A thread keeps its part of the row in registers from
// the first stage to the last: groups of 8 consecutive elements, group number j * 1024 + thread.
// Row lengths are multiples of 8, at most 16384 (twice that for the source of silu).
struct RowProgram {
    const float* src;
    uint32_t n_slices;       // 1 = plain buffer
    uint32_t slice_stride;   // elements between slices
    uint32_t len_src;
    float* src_store;
    uint32_t silu;
    float* gate_out;
    float* up_out;
    float* silu_out;
    const float* addend;     // nullptr = no add
    float* add_out;
    const float* rms_weight; // used when rms != 0
    uint32_t rms, n_weight;
    float epsilon;
    float* rms_out;
    _Float16* frag;          // nullptr = no split
    float* inv_scale;
    uint32_t batch;          // rows that exist; the grid may be padded to a multiple of 32 for split
};

typedef _Float16 row_half8 __attribute__((ext_vector_type(8)));

static constexpr int kRowThreads = 1024;

template <int NG>  // groups of 8 elements per thread
__global__ __launch_bounds__(kRowThreads) void row_program_kernel(const RowProgram p) {
    constexpr int NWAVE = kRowThreads / 64;
    constexpr int SB = 8;  // K slices whose loads are in flight together
    __shared__ float red[NWAVE];      // sum of squares per wave (rms)
    __shared__ float red_max[NWAVE];  // largest magnitude per wave (split)
    const uint32_t row = blockIdx.x;
    const uint32_t tid = threadIdx.x;
    const bool live = row < p.batch;
    const uint32_t len = p.silu ? p.len_src / 2 : p.len_src;
    float v[NG][8];
    if (live) {
        // ---- source (and silu, which reads the two halves of the source row)
        auto load_src = [&](uint32_t col, float (&out)[8]) __attribute__((always_inline)) {
            const float* q = p.src + (size_t)row * p.len_src + col;
            float4 a = reinterpret_cast<const float4*>(q)[0], b = reinterpret_cast<const float4*>(q)[1];
            for (uint32_t s0 = 1; s0 < p.n_slices; s0 += SB) {
                float4 c[SB], d[SB];
#pragma unroll
                for (int ss = 0; ss < SB; ++ss) {
                    const uint32_t sl = min(s0 + ss, p.n_slices - 1);  // past the end: a repeat, not added
                    const float4* qs = reinterpret_cast<const float4*>(q + (size_t)sl * p.slice_stride);
                    c[ss] = qs[0];
                    d[ss] = qs[1];
                }
#pragma unroll
                for (int ss = 0; ss < SB; ++ss)
                    if (s0 + ss < p.n_slices) {  // slice order, like q4_sum_slices_kernel
                        a.x += c[ss].x; a.y += c[ss].y; a.z += c[ss].z; a.w += c[ss].w;
                        b.x += d[ss].x; b.y += d[ss].y; b.z += d[ss].z; b.w += d[ss].w;
                    }
            }
            if (p.src_store) {
                float4* w = reinterpret_cast<float4*>(p.src_store + (size_t)row * p.len_src + col);
                w[0] = a;
                w[1] = b;
            }
            out[0] = a.x; out[1] = a.y; out[2] = a.z; out[3] = a.w;
            out[4] = b.x; out[5] = b.y; out[6] = b.z; out[7] = b.w;
        };
        auto store8 = [&](float* base, uint32_t col, const float (&x)[8]) __attribute__((always_inline)) {
            float4* w = reinterpret_cast<float4*>(base + (size_t)row * len + col);
            w[0] = make_float4(x[0], x[1], x[2], x[3]);
            w[1] = make_float4(x[4], x[5], x[6], x[7]);
        };
#pragma unroll
        for (int j = 0; j < NG; ++j) {
            const uint32_t col = (j * kRowThreads + tid) * 8;
            if (col >= len) continue;
            if (p.silu) {
                float gt[8], u[8];
                load_src(col, gt);
                load_src(len + col, u);
#pragma unroll
                for (int e = 0; e < 8; ++e) v[j][e] = silu_times(gt[e], u[e]);
                store8(p.gate_out, col, gt);
                store8(p.up_out, col, u);
                store8(p.silu_out, col, v[j]);
            } else {
                load_src(col, v[j]);
            }
            if (p.addend) {
                const float4* q = reinterpret_cast<const float4*>(p.addend + (size_t)row * len + col);
                const float4 a = q[0], b = q[1];
                v[j][0] += a.x; v[j][1] += a.y; v[j][2] += a.z; v[j][3] += a.w;
                v[j][4] += b.x; v[j][5] += b.y; v[j][6] += b.z; v[j][7] += b.w;
                store8(p.add_out, col, v[j]);
            }
        }
        // ---- rms (the weights are fetched before the reduction, not behind its barrier)
        if (p.rms) {
            float gamma[NG][8];
#pragma unroll
            for (int j = 0; j < NG; ++j) {
                const uint32_t col = (j * kRowThreads + tid) * 8;
#pragma unroll
                for (int e = 0; e < 8; ++e)
                    gamma[j][e] = (col < len && col + e < p.n_weight) ? p.rms_weight[col + e] : 1.0f;
            }
            float sum = 0.f;
#pragma unroll
            for (int j = 0; j < NG; ++j) {
                if ((j * kRowThreads + tid) * 8 >= len) continue;
#pragma unroll
                for (int e = 0; e < 8; ++e) sum = fmaf(v[j][e], v[j][e], sum);
            }
#pragma unroll
            for (int off = 32; off > 0; off >>= 1) sum += __shfl_xor(sum, off);
            if (tid % 64 == 0) red[tid / 64] = sum;
            __syncthreads();
            float total = 0.f;
#pragma unroll
            for (int w = 0; w < NWAVE; ++w) total += red[w];
            const float scale = 1.0f / sqrtf(total / (float)len + p.epsilon);
#pragma unroll
            for (int j = 0; j < NG; ++j) {
                const uint32_t col = (j * kRowThreads + tid) * 8;
                if (col >= len) continue;
#pragma unroll
                for (int e = 0; e < 8; ++e) v[j][e] = v[j][e] * scale * gamma[j][e];
                store8(p.rms_out, col, v[j]);
            }
        }
    }
    if (!p.frag) return;

    // ---- split (the whole workgroup takes part, padding rows write zeros)
    float amax = 0.f;
    if (live) {
#pragma unroll
        for (int j = 0; j < NG; ++j) {
            if ((j * kRowThreads + tid) * 8 >= len) continue;
#pragma unroll
            for (int e = 0; e < 8; ++e) amax = fmaxf(amax, fabsf(v[j][e]));
        }
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) amax = fmaxf(amax, __shfl_xor(amax, off));
    if (tid % 64 == 0) red_max[tid / 64] = amax;
    __syncthreads();
#pragma unroll
    for (int w = 0; w < NWAVE; ++w) amax = fmaxf(amax, red_max[w]);
    int ex = 0;
    if (amax > 0.f && amax < INFINITY) (void)frexpf(amax, &ex);
    int se = 14 - ex;
    se = se > 100 ? 100 : (se < -100 ? -100 : se);
    const float s = ldexpf(1.0f, se);
    if (tid == 0 && live) p.inv_scale[row] = ldexpf(1.0f, -se);
    const uint32_t ksteps = len / 16;
#pragma unroll
    for (int j = 0; j < NG; ++j) {
        const uint32_t k = (j * kRowThreads + tid) * 8;
        if (k >= len) continue;
        row_half8 hi, lo;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const float t = live ? v[j][e] * s : 0.f;
            hi[e] = (_Float16)t;
            lo[e] = (_Float16)(t - (float)hi[e]);
        }
        const size_t base = ((size_t)(row / 32) * ksteps + k / 16) * 2;
        const uint32_t lane = ((k % 16) / 8) * 32 + row % 32;
        *reinterpret_cast<row_half8*>(p.frag + ((base + 0) * 64 + lane) * 8) = hi;
        *reinterpret_cast<row_half8*>(p.frag + ((base + 1) * 64 + lane) * 8) = lo;
    }
}

}  // namespace mlc_hip
