// The step before the paged KV write, for gfx950: split the fused qkv row of every
// request into q / k / v, rotate q and k (RoPE), cast k and v to fp16 -- and, in the
// fused form, write those fp16 rows straight into their KV pages.
//
// Reference: MetalExecutor::encodeQkvSplitRopeCast (compiler/runtime/metal_runtime.mm:7915-8025)
// runs seven dispatches for this (3x strided_copy_f32 :447-455, 2x batched_rope :287-314,
// 2x cast_f32_to_f16 :457-464) and the walker then two scatter_kv_paged_batched_f16 (:405-424).
// Here it is one launch: every thread owns one (even, odd) pair of one request's qkv row,
// so the rotation is thread-local and every buffer is touched once.
//
// Arithmetic follows the reference exactly: x0' = x0*c - x1*s, x1' = x0*s + x1*c with every
// product and sum rounded to fp32 on its own (no FMA contraction, so the result is bit-equal
// to the CPU applyRotaryEmbedding, compiler/runtime/quantization.cpp:772-793), and `half(x)`
// is round-to-nearest-even (v_cvt_f16_f32).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace mlc_hip {

struct RopeArgs {
    const float* qkv;        // [batch][qkv_rows]
    float* q;                // [batch][q_rows]            (never null)
    float* k;                // [batch][k_rows] fp32       (may be null in the fused form)
    float* v;                // [batch][v_rows] fp32       (may be null in the fused form)
    _Float16* k_f16;         // [batch][k_rows]            (may be null: no fp16 staging copy)
    _Float16* v_f16;         // [batch][v_rows]
    _Float16* k_pages;       // KV pools [page][slot][kv_head][dim] (may be null: no paged write)
    _Float16* v_pages;
    const float* cos_table;  // [batch][rotary_dim / 2]
    const float* sin_table;
    const uint32_t* page_ids;  // [batch], needed when k_pages or v_pages is set
    const uint32_t* slots;     // [batch]
    uint32_t batch, head_dim, qkv_rows, q_rows, k_rows, v_rows, rotary_dim, page_size;
};

// (x0, x1) -> (x0*c - x1*s, x0*s + x1*c): four products, one difference, one sum, each
// rounded on its own -- contraction into v_fma is switched off for this function.
__device__ __forceinline__ float2 rope_rotate(float2 x, float c, float s) {
#pragma clang fp contract(off)
    const float a0 = x.x * c, a1 = x.y * s, b0 = x.x * s, b1 = x.y * c;
    return make_float2(a0 - a1, b0 + b1);
}

// One thread per pair.  Pair index pi of a request counts pairs of the q, then k, then v
// segment (every segment length is even on this path).  Which of the k / v outputs exist
// (fp32 copy, fp16 staging copy, paged write) is decided per launch by the pointers.
__global__ __launch_bounds__(256) void qkv_split_rope_cast_kernel(const RopeArgs a) {
    const uint32_t pairs_row = (a.q_rows + a.k_rows + a.v_rows) / 2;
    const uint32_t gid = blockIdx.x * blockDim.x + threadIdx.x;
    if (gid >= a.batch * pairs_row) return;
    const uint32_t req = gid / pairs_row;
    const uint32_t e = (gid - req * pairs_row) * 2;  // element offset within q|k|v
    const float2 x = *reinterpret_cast<const float2*>(a.qkv + (size_t)req * a.qkv_rows + e);
    float2 y = x;
    const bool is_q = e < a.q_rows;
    const bool is_k = !is_q && e < a.q_rows + a.k_rows;
    const uint32_t local = is_q ? e : (is_k ? e - a.q_rows : e - a.q_rows - a.k_rows);
    if (is_q || is_k) {
        const uint32_t d = local % a.head_dim;  // even
        if (d < a.rotary_dim) {
            const uint32_t ci = req * (a.rotary_dim / 2) + d / 2;
            y = rope_rotate(x, a.cos_table[ci], a.sin_table[ci]);
        }
    }
    if (is_q) {
        *reinterpret_cast<float2*>(a.q + (size_t)req * a.q_rows + local) = y;
        return;
    }
    float* f32 = is_k ? a.k : a.v;
    const uint32_t rows = is_k ? a.k_rows : a.v_rows;
    if (f32) *reinterpret_cast<float2*>(f32 + (size_t)req * rows + local) = y;
    typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
    const half2_t h = {(_Float16)y.x, (_Float16)y.y};
    _Float16* f16 = is_k ? a.k_f16 : a.v_f16;
    if (f16) *reinterpret_cast<half2_t*>(f16 + (size_t)req * rows + local) = h;
    _Float16* pool = is_k ? a.k_pages : a.v_pages;
    if (pool) {
        // scatter_kv_paged_batched_f16 (metal_runtime.mm:418-422): a row of all KV heads is
        // contiguous at page_ids[r]*P*rows + slots[r]*rows
        const size_t dst = ((size_t)a.page_ids[req] * a.page_size + a.slots[req]) * rows + local;
        *reinterpret_cast<half2_t*>(pool + dst) = h;
    }
}

inline void launch_qkv_split_rope_cast(const RopeArgs& a, hipStream_t stream) {
    const uint32_t total = a.batch * ((a.q_rows + a.k_rows + a.v_rows) / 2);
    hipLaunchKernelGGL(qkv_split_rope_cast_kernel, dim3((total + 255) / 256), dim3(256), 0, stream, a);
}

}  // namespace mlc_hip
