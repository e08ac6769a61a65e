// Paged flash-attention decode kernels for gfx950 (MI355X), wave64.
//
// Semantics: MSL kernel paged_flash_attention of the reference
// (compiler/runtime/metal_runtime.mm:2216-2335): for each (request, query head)
//   O = softmax(q . K^T / sqrt(D), causal: kv_pos <= q_pos) . V
// with K/V rows read through the request's page table from fp16 pages laid out
// [page][slot][kv_head][dim], fp32 arithmetic and fp32 output.
//
// Layout of the work: the host flattens the batch into WORK ITEMS
// (request, kv head, head group, token range) of roughly equal length -- split-K
// over pages -- and launches one 64-lane wavefront per item.  All query heads
// that share the KV head (GQA) are processed by the same wave, so every K/V byte
// is fetched from HBM once.  Items that cover a whole request write O directly;
// split requests write un-normalised (o, m, l) partials that a small second
// kernel merges.
//
// Lane layout of the fast kernel (D = 64 or 128):
//   a K (or V) row of one KV head is D halves = D/8 16-byte chunks; lane
//   (r, c) = (lane / CPR, lane % CPR), CPR = D/8, loads chunk c of row r of a
//   "row group" of RPI = 64/CPR consecutive tokens, so one global_load_dwordx4
//   per wave reads RPI whole rows, fully coalesced.  A tile is 8 row groups
//   (64 tokens for D=64, 32 for D=128).
//   QK: every lane forms the partial dot over its 8 dims for HPW heads x 8 row
//   groups, then a 3-step reduce-scatter over the 8 c-lanes (DPP half-mirror,
//   quad xor 2, quad xor 1 fused into v_add_f32) leaves lane (r, c) holding the
//   complete scores of ONE token for all HPW heads.  To keep that exchange free
//   of selects, register j' of lane c holds row group j' ^ g(c), g(c) = c ^
//   ((c & 4) ? 3 : 0): the swizzle is applied to the load address, which costs
//   nothing.
//   Softmax: exp2 with log2(e)/sqrt(D) folded into q; the running reference
//   maximum is kept per r-set (the 8 tokens x 8 tiles a row of lanes owns) and
//   only raised when a tile exceeds it by more than 2^8 (exact math, any
//   reference works; this removes almost all accumulator rescales).
//   PV: p is gathered back over the same 8 lanes (7 DPP moves per head) and
//   applied to the V rows held in the same (r, c) layout; accumulators are
//   [HPW][8 dims] per lane, reduced over r once, at the end of the item.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace mlc_hip {

struct DecodeWorkItem {
    uint32_t req;        // request index
    uint32_t head0;      // first query head handled by this wave
    uint32_t kv_head;    // KV head those query heads read
    uint32_t pt_base;    // offset of the request's page ids in page_tables_flat
    uint32_t tok_begin;  // first kv position (multiple of the tile size)
    uint32_t tok_end;    // one past the last visible kv position of this item
    uint32_t part_idx;   // partial slot, or kNoPartial to write O directly
    uint32_t pad;
};
static constexpr uint32_t kNoPartial = 0xFFFFFFFFu;

struct DecodeArgs {
    const float* q;             // [B][H][D]
    const uint4* k_pages;       // fp16 pages, viewed as 16-byte chunks
    const uint4* v_pages;
    float* o;                   // [B][H][D]
    const uint32_t* pt_flat;    // device copy of page_tables_flat
    const DecodeWorkItem* items;
    float* part_o;              // [n_part][HPW][D] un-normalised partial outputs
    float2* part_ml;            // [n_part][HPW]    (m in log2 units, l)
    uint32_t num_heads;
    uint32_t kv_heads;
    uint32_t page_size;         // tokens per page
    uint32_t n_items;
    float scale_log2e;          // log2(e) / sqrt(D)
};

typedef _Float16 half8_t __attribute__((ext_vector_type(8)));

// DPP controls (GFX9 encoding)
static constexpr int kDppQuadXor1 = 0xB1;     // quad_perm:[1,0,3,2]
static constexpr int kDppQuadXor2 = 0x4E;     // quad_perm:[2,3,0,1]
static constexpr int kDppQuadXor3 = 0x1B;     // quad_perm:[3,2,1,0]
static constexpr int kDppHalfMirror = 0x141;  // row_half_mirror: i -> 7-i within 8 lanes
static constexpr int kDppRowRor8 = 0x128;     // row_ror:8: i -> i^8 within 16 lanes

template <int CTRL>
__device__ __forceinline__ float dpp_f(float v) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xF, 0xF, true));
}

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// -inf substitute for running maxima: finite, so (m - m) and exp2(-inf - m) stay NaN-free.
static constexpr float kNegBig = -1.0e30f;
// A tile may exceed the running reference by 2^kLazyTau before accumulators are rescaled.
static constexpr float kLazyTau = 8.0f;

template <int D, int HPW>
__global__ __launch_bounds__(64) void paged_decode_fast_kernel(const DecodeArgs a) {
    static_assert(D == 64 || D == 128, "fast path covers head_dim 64 and 128");
    constexpr int CPR = D / 8;       // 16-byte chunks per row
    constexpr int RPI = 64 / CPR;    // rows fetched by one wave-wide load
    constexpr int TT = 8 * RPI;      // tokens per tile
    constexpr int OPL = HPW * D / 64;  // outputs per lane in the epilogue

    __shared__ float s_acc[RPI * HPW * D];

    const uint32_t item_idx = blockIdx.x;
    if (item_idx >= a.n_items) return;
    const DecodeWorkItem it = a.items[item_idx];
    const int lane = threadIdx.x;
    const int c = lane % CPR;
    const int r = lane / CPR;
    const int c7 = c & 7;
    const int gsw = c7 ^ ((c7 & 4) ? 3 : 0);  // row-group swizzle g(c)

    // q for this wave's heads, dims c*8 .. c*8+7, pre-scaled.
    float qv[HPW][8];
    {
        const float* qbase = a.q + ((size_t)it.req * a.num_heads + it.head0) * D + c * 8;
#pragma unroll
        for (int h = 0; h < HPW; ++h) {
            const float4 lo = *reinterpret_cast<const float4*>(qbase + h * D);
            const float4 hi = *reinterpret_cast<const float4*>(qbase + h * D + 4);
            qv[h][0] = lo.x * a.scale_log2e; qv[h][1] = lo.y * a.scale_log2e;
            qv[h][2] = lo.z * a.scale_log2e; qv[h][3] = lo.w * a.scale_log2e;
            qv[h][4] = hi.x * a.scale_log2e; qv[h][5] = hi.y * a.scale_log2e;
            qv[h][6] = hi.z * a.scale_log2e; qv[h][7] = hi.w * a.scale_log2e;
        }
    }

    float acc[HPW][8];
    float m_ref[HPW], l_sum[HPW];
#pragma unroll
    for (int h = 0; h < HPW; ++h) {
        m_ref[h] = kNegBig;
        l_sum[h] = 0.f;
#pragma unroll
        for (int i = 0; i < 8; ++i) acc[h][i] = 0.f;
    }

    const uint32_t row_u4 = a.kv_heads * CPR;  // 16-byte chunks per token row (all KV heads)
    const uint32_t lane_u4 = it.kv_head * CPR + c;

    // Addresses of the 8 rows this lane reads in a tile; rows past the visible end are
    // clamped onto the last visible row (in bounds, masked out of the softmax below).
    auto load_tile = [&](const uint4* pages, uint32_t tile_start, uint4 (&reg)[8]) {
        const uint32_t page_idx = tile_start / a.page_size;
        const uint32_t slot0 = tile_start - page_idx * a.page_size;
        const uint32_t page_id = a.pt_flat[it.pt_base + page_idx];
        const uint32_t last = it.tok_end - 1u - tile_start;  // last visible row of the tile
        const uint4* base = pages + ((size_t)page_id * a.page_size + slot0) * row_u4 + lane_u4;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            uint32_t t = (uint32_t)((j ^ gsw) * RPI + r);
            t = t < last ? t : last;
            reg[j] = base[(size_t)t * row_u4];
        }
    };

    uint4 kreg[8], vreg[8];
    if (it.tok_begin < it.tok_end) {
        load_tile(a.k_pages, it.tok_begin, kreg);
        load_tile(a.v_pages, it.tok_begin, vreg);
    }

    for (uint32_t tile_start = it.tok_begin; tile_start < it.tok_end; tile_start += TT) {
        const uint32_t next = tile_start + TT;
        const bool has_next = next < it.tok_end;

        // ---- QK: per head, partial dots over this lane's 8 dims for the 8 row groups,
        // then a reduce-scatter over the 8 c-lanes (lane keeps row group g(c)).
        float sc[HPW];
#pragma unroll
        for (int h = 0; h < HPW; ++h) {
            float part[8];
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const half8_t kh = __builtin_bit_cast(half8_t, kreg[j]);
                float s = qv[h][0] * (float)kh[0];
#pragma unroll
                for (int i = 1; i < 8; ++i) s = fmaf(qv[h][i], (float)kh[i], s);
                part[j] = s;
            }
#pragma unroll
            for (int j = 0; j < 4; ++j) part[j] += dpp_f<kDppHalfMirror>(part[j + 4]);
#pragma unroll
            for (int j = 0; j < 2; ++j) part[j] += dpp_f<kDppQuadXor2>(part[j + 2]);
            float s = part[0] + dpp_f<kDppQuadXor1>(part[1]);
            if (CPR == 16) s += dpp_f<kDppRowRor8>(s);
            sc[h] = s;
        }
        if (has_next) load_tile(a.k_pages, next, kreg);

        // ---- mask, tile maximum over the r-set, lazy reference update
        const uint32_t my_tok = tile_start + (uint32_t)(gsw * RPI + r);
        const bool visible = my_tok < it.tok_end;
        bool raise = false;
        float tmax[HPW];
#pragma unroll
        for (int h = 0; h < HPW; ++h) {
            sc[h] = visible ? sc[h] : -INFINITY;
            float m = sc[h];
            m = fmaxf(m, dpp_f<kDppQuadXor1>(m));
            m = fmaxf(m, dpp_f<kDppQuadXor2>(m));
            m = fmaxf(m, dpp_f<kDppHalfMirror>(m));
            if (CPR == 16) m = fmaxf(m, dpp_f<kDppRowRor8>(m));
            tmax[h] = m;
            raise |= (m > m_ref[h] + kLazyTau);
        }
        if (__any(raise)) {
#pragma unroll
            for (int h = 0; h < HPW; ++h) {
                const float m_new = fmaxf(m_ref[h], tmax[h]);
                const float alpha = fast_exp2(m_ref[h] - m_new);
                m_ref[h] = m_new;
                l_sum[h] *= alpha;
#pragma unroll
                for (int i = 0; i < 8; ++i) acc[h][i] *= alpha;
            }
        }
        float p[HPW];
#pragma unroll
        for (int h = 0; h < HPW; ++h) {
            p[h] = fast_exp2(sc[h] - m_ref[h]);
            l_sum[h] += p[h];
        }

        // ---- PV: register j of this lane holds the V row whose weight lives in the
        // lane at swizzle distance j; fetch it with DPP moves.
#pragma unroll
        for (int h = 0; h < HPW; ++h) {
            float pj[8];
            pj[0] = p[h];
            pj[1] = dpp_f<kDppQuadXor1>(p[h]);
            pj[2] = dpp_f<kDppQuadXor2>(p[h]);
            pj[3] = dpp_f<kDppQuadXor3>(p[h]);
            pj[4] = dpp_f<kDppHalfMirror>(p[h]);
            pj[5] = dpp_f<kDppQuadXor1>(pj[4]);
            pj[6] = dpp_f<kDppQuadXor2>(pj[4]);
            pj[7] = dpp_f<kDppQuadXor3>(pj[4]);
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const half8_t vh = __builtin_bit_cast(half8_t, vreg[j]);
#pragma unroll
                for (int i = 0; i < 8; ++i) acc[h][i] = fmaf(pj[j], (float)vh[i], acc[h][i]);
            }
        }
        if (has_next) load_tile(a.v_pages, next, vreg);
    }

    // ---- epilogue: bring the RPI r-sets onto one reference, sum over r through LDS
    float m_all[HPW], l_all[HPW];
#pragma unroll
    for (int h = 0; h < HPW; ++h) {
        float m = m_ref[h];
#pragma unroll
        for (int off = CPR; off < 64; off <<= 1) m = fmaxf(m, __shfl_xor(m, off));
        m_all[h] = m;
        const float w = fast_exp2(m_ref[h] - m);
        // with CPR == 16 every token's weight sits in two lanes (c and c^8): count it once
        float l = (CPR == 16 && (c & 8)) ? 0.f : l_sum[h] * w;
#pragma unroll
        for (int off = 1; off < 64; off <<= 1) l += __shfl_xor(l, off);
        l_all[h] = l;
        float4* dst = reinterpret_cast<float4*>(&s_acc[((r * HPW + h) * CPR + c) * 8]);
        dst[0] = make_float4(acc[h][0] * w, acc[h][1] * w, acc[h][2] * w, acc[h][3] * w);
        dst[1] = make_float4(acc[h][4] * w, acc[h][5] * w, acc[h][6] * w, acc[h][7] * w);
    }
    __syncthreads();

#pragma unroll
    for (int k = 0; k < OPL; ++k) {
        const int idx = k * 64 + lane;  // index into [HPW][D]
        const int h = idx / D;
        const int d = idx % D;
        float sum = 0.f;
#pragma unroll
        for (int rr = 0; rr < RPI; ++rr) sum += s_acc[(rr * HPW + h) * D + d];
        // m_all[h], l_all[h] for a run-time h: select without indexing registers dynamically
        float mh = m_all[0], l = l_all[0];
#pragma unroll
        for (int hh = 1; hh < HPW; ++hh) {
            mh = (h == hh) ? m_all[hh] : mh;
            l = (h == hh) ? l_all[hh] : l;
        }
        if (it.part_idx == kNoPartial) {
            const float inv = l > 0.f ? 1.0f / l : 0.f;
            a.o[((size_t)it.req * a.num_heads + it.head0 + h) * D + d] = sum * inv;
        } else {
            a.part_o[((size_t)it.part_idx * HPW + h) * D + d] = sum;
            if (d == 0) a.part_ml[(size_t)it.part_idx * HPW + h] = make_float2(mh, l);
        }
    }
}

// Merges the split-K partials of one (request, head group): grid = number of
// merge entries, block = D threads... one thread per output dim, loop over heads.
struct MergeEntry {
    uint32_t req;
    uint32_t head0;
    uint32_t first_part;
    uint32_t n_parts;
};

template <int HPW>
__global__ void paged_decode_merge_kernel(const MergeEntry* entries, const float* part_o,
                                          const float2* part_ml, float* o, uint32_t num_heads,
                                          uint32_t head_dim) {
    const MergeEntry e = entries[blockIdx.x];
    const uint32_t h = blockIdx.y;
    const float2* ml = part_ml + (size_t)e.first_part * HPW + h;
    float m = kNegBig;
    for (uint32_t s = 0; s < e.n_parts; ++s) m = fmaxf(m, ml[(size_t)s * HPW].x);
    float l = 0.f;
    for (uint32_t s = 0; s < e.n_parts; ++s) {
        const float2 v = ml[(size_t)s * HPW];
        l += v.y * fast_exp2(v.x - m);
    }
    const float inv = l > 0.f ? 1.0f / l : 0.f;
    for (uint32_t d = threadIdx.x; d < head_dim; d += blockDim.x) {
        float acc = 0.f;
        for (uint32_t s = 0; s < e.n_parts; ++s) {
            const float w = fast_exp2(ml[(size_t)s * HPW].x - m);
            acc += w * part_o[(((size_t)e.first_part + s) * HPW + h) * head_dim + d];
        }
        o[((size_t)e.req * num_heads + e.head0 + h) * head_dim + d] = acc * inv;
    }
}

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
