// Shape-agnostic paged decode attention for gfx950: the fallback for shapes the
// tiled kernel does not cover.  Same semantics (compiler/runtime/metal_runtime.mm:2216-2335).
#pragma once

#include "paged_decode_kernels.h"

namespace mlc_hip {

// Shape-agnostic kernel: any head_dim <= 256, any page size, any GQA ratio.  One
// wave per (request, query head); lanes own tokens for QK and dims for PV.  Used
// for the shapes the fast kernel does not cover (small pages, odd head sizes).
struct GenericArgs {
    const float* q;
    const _Float16* k_pages;
    const _Float16* v_pages;
    float* o;
    const uint32_t* pt_flat;
    const uint32_t* pt_off;    // [B]
    const uint32_t* limits;    // [B] visible kv positions (causal rule applied)
    uint32_t num_heads;
    uint32_t kv_heads;
    uint32_t head_dim;
    uint32_t page_size;
    float scale_log2e;
};

__global__ __launch_bounds__(64) void paged_decode_generic_kernel(const GenericArgs a) {
    const uint32_t req = blockIdx.x / a.num_heads;
    const uint32_t head = blockIdx.x % a.num_heads;
    const uint32_t kvh = (uint32_t)(((uint64_t)head * a.kv_heads) / a.num_heads);
    const uint32_t D = a.head_dim;
    const uint32_t limit = a.limits[req];
    const uint32_t pt_base = a.pt_off[req];
    const int lane = threadIdx.x;
    __shared__ float s_q[256];
    const float* qrow = a.q + ((size_t)req * a.num_heads + head) * D;
    for (uint32_t d = lane; d < D; d += 64) s_q[d] = qrow[d] * a.scale_log2e;
    __syncthreads();

    constexpr int DPL = 4;  // dims per lane: covers head_dim <= 256
    float oacc[DPL] = {0.f, 0.f, 0.f, 0.f};
    float m = kNegBig, l = 0.f;
    const size_t row_elems = (size_t)a.kv_heads * D;

    for (uint32_t t0 = 0; t0 < limit; t0 += 64) {
        const uint32_t pos = t0 + lane;
        const bool visible = pos < limit;
        size_t row = 0;
        float s = -INFINITY;
        if (visible) {
            const uint32_t page_idx = pos / a.page_size;
            const uint32_t slot = pos - page_idx * a.page_size;
            const uint32_t page_id = a.pt_flat[pt_base + page_idx];
            row = ((size_t)page_id * a.page_size + slot) * row_elems + (size_t)kvh * D;
            const _Float16* kr = a.k_pages + row;
            float dot = 0.f;
            for (uint32_t d = 0; d < D; ++d) dot = fmaf(s_q[d], (float)kr[d], dot);
            s = dot;
        }
        float tmax = s;
#pragma unroll
        for (int off = 1; off < 64; off <<= 1) tmax = fmaxf(tmax, __shfl_xor(tmax, off));
        const float m_new = fmaxf(m, tmax);
        const float alpha = fast_exp2(m - m_new);
        const float p = fast_exp2(s - m_new);  // s = -inf -> 0
        float psum = p;
#pragma unroll
        for (int off = 1; off < 64; off <<= 1) psum += __shfl_xor(psum, off);
        l = l * alpha + psum;
        m = m_new;
#pragma unroll
        for (int k = 0; k < DPL; ++k) oacc[k] *= alpha;
        const uint32_t n_here = (limit - t0) < 64u ? (limit - t0) : 64u;
        const uint32_t row_lo = (uint32_t)(row & 0xFFFFFFFFu);
        const uint32_t row_hi = (uint32_t)(row >> 32);
        for (uint32_t t = 0; t < n_here; ++t) {
            const float pt = __shfl(p, (int)t);
            const size_t rt = ((size_t)__shfl((int)row_hi, (int)t) << 32) |
                              (uint32_t)__shfl((int)row_lo, (int)t);
            const _Float16* vr = a.v_pages + rt;
#pragma unroll
            for (int k = 0; k < DPL; ++k) {
                const uint32_t d = lane + 64u * k;
                if (d < D) oacc[k] = fmaf(pt, (float)vr[d], oacc[k]);
            }
        }
    }
    const float inv = l > 0.f ? 1.0f / l : 0.f;
    float* orow = a.o + ((size_t)req * a.num_heads + head) * D;
#pragma unroll
    for (int k = 0; k < DPL; ++k) {
        const uint32_t d = lane + 64u * k;
        if (d < D) orow[d] = oacc[k] * inv;
    }
}

}  // namespace mlc_hip
