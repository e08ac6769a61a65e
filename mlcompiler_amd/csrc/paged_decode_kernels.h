// Paged flash-attention decode kernels for gfx950 (MI355X), wave64.
//
// Semantics: MSL kernel paged_flash_attention of the reference
// (compiler/runtime/metal_runtime.mm:2216-2335): for each (request, query head)
//   O = softmax(q . K^T / sqrt(D), causal: kv_pos <= q_pos) . V
// with K/V rows read through the request's page table from fp16 pages laid out
// [page][slot][kv_head][dim], fp32 accumulation and fp32 output.
//
// Layout of the work: the host flattens the batch into WORK ITEMS
// (request, kv head, token range) of roughly equal length -- split-K over pages --
// and launches one workgroup per item.  A workgroup has NW x NS wavefronts: the
// GQA group of the KV head is spread over NW waves (HPW query heads each, so
// every K/V byte is fetched from HBM once and re-read from the CU's vector cache
// by the other head waves), and the item's tiles are dealt round-robin to NS
// wave rows.  Partial softmax states of the NS rows are merged through LDS; an
// item that covers its whole request writes O directly, split requests publish
// (o, m, l) partials and the last workgroup to arrive merges them.
//
// Lane layout (D = 64 or 128):
//   a K (or V) row of one KV head is D halves = D/8 16-byte chunks; lane
//   (r, c) = (lane / CPR, lane % CPR), CPR = D/8, loads chunk c of row r of a
//   "row group" of RPI = 64/CPR consecutive tokens, so one global_load_dwordx4
//   per wave reads RPI whole rows, fully coalesced.  A tile is 8 row groups
//   (64 tokens for D=64, 32 for D=128).
//   QK: every lane forms the partial dot over its 8 dims for 8 row groups, then a
//   3-step reduce-scatter over the 8 c-lanes (DPP half-mirror, quad xor 2, quad
//   xor 1 fused into v_add_f32) leaves lane (r, c) holding the complete scores of
//   ONE token for all HPW heads.  To keep that exchange free of selects, register
//   j' of lane c holds row group j' ^ g(c), g(c) = c ^ ((c & 4) ? 3 : 0): the
//   swizzle is applied to the load address, which costs nothing.
//   Softmax: exp2 with log2(e)/sqrt(D) folded into q; the running reference
//   maximum is kept per r-set (the tokens a row of lanes owns) and only raised
//   when a tile exceeds it by more than 2^8 (exact math, any reference works;
//   this removes almost all accumulator rescales).
//   PV: weights are rounded to fp16 (and the normaliser is summed from the
//   rounded values), gathered back over the same 8 lanes with DPP moves and
//   applied with v_dot2_f32_f16 to V rows held in the same (r, c) layout;
//   accumulators are fp32 [HPW][8 dims] per lane, reduced over r once per item.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace mlc_hip {

struct DecodeWorkItem {
    uint32_t req;         // request index
    uint32_t kv_head;     // KV head; the workgroup's waves cover its query-head group
    uint32_t pt_base;     // offset of the request's page ids in page_tables_flat
    uint32_t tok_begin;   // first kv position (multiple of the tile size)
    uint32_t tok_end;     // one past the last visible kv position of this item
    uint32_t part_first;  // first partial slot of this (request, kv head), or kNoPartial
    uint32_t split;       // this item's split index | number of splits << 16
    uint32_t first_pages[4];  // page ids of the item's first four tiles: the first tile loads
                              // then depend on the item alone, not on a page-table fetch
    uint32_t group_size;  // 0: the last arriver merges all splits; otherwise the splits are
                          // merged in groups of this many, and the groups' results after them
};
static_assert(sizeof(DecodeWorkItem) == 48, "work items are uploaded as raw bytes");
static constexpr uint32_t kNoPartial = 0xFFFFFFFFu;
static constexpr uint32_t kMaxSplits = 512;      // per (request, KV head)
static constexpr uint32_t kFlatMergeSplits = 16;  // up to here one wave merges all partials;
                                                  // beyond, in two levels (each merge <= 64)

struct DecodeArgs {
    const float* q;             // [B][H][D]
    const uint4* k_pages;       // fp16 pages, viewed as 16-byte chunks
    const uint4* v_pages;
    float* o;                   // [B][H][D]
    const uint32_t* pt_flat;    // device copy of page_tables_flat
    const DecodeWorkItem* items;
    float* part_o;              // [n_part][G][D] un-normalised partial outputs
    float* part_ml;             // [n_part][G][2] (m in log2 units, l)
    uint32_t* counters;         // [n_part][NW] arrival counters, zero between launches
    uint32_t num_heads;
    uint32_t kv_heads;
    uint32_t page_size;         // tokens per page
    uint32_t n_items;
    float scale_log2e;          // log2(e) / sqrt(D)
    // The step's KV write done by this launch (null: none): the new fp16 K / V row of every
    // request, [B][Hkv][D], goes to its newest position (new_rows[r] = page id * page size +
    // slot, which the caller has checked to be position seq_len - 1 of request r) before the
    // item that reads that position loads anything.
    const uint4* new_k;
    const uint4* new_v;
    const uint32_t* new_ids;    // [B] page ids
    const uint32_t* new_slots;  // [B] slots in page
};

typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef _Float16 half2_t __attribute__((ext_vector_type(2)));

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
template <int CTRL>
__device__ __forceinline__ uint32_t dpp_u(uint32_t v) {
    return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, CTRL, 0xF, 0xF, true);
}

// Device-scope accesses: the store is written through to memory, the load bypasses the
// (per-XCD, mutually non-coherent) L2 caches.
__device__ __forceinline__ void st_dev(float* p, float v) {
    __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ float ld_dev(const float* p) {
    return __hip_atomic_load(const_cast<float*>(p), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// plain maximum; the file is compiled with -fno-honor-nans so no NaN-quieting moves are added
__device__ __forceinline__ float max_nn(float a, float b) { return __builtin_fmaxf(a, b); }

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) v = max_nn(v, __shfl_xor(v, off));
    return v;
}
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) v += __shfl_xor(v, off);
    return v;
}

// -inf substitute for running maxima: finite, so (m - m) and exp2(-inf - m) stay NaN-free.
static constexpr float kNegBig = -1.0e30f;
// A tile may exceed the running reference by 2^kLazyTau before accumulators are rescaled.
static constexpr float kLazyTau = 8.0f;

// Static LDS of one workgroup of the tiled kernel (staging buffers, reused by the epilogue).
static constexpr int kMaxStaticLds = 65536;
constexpr int decode_lds_bytes(int D, int HPW, int NW, int NS, int NBUF) {
    const int rpi = 64 / (D / 8);
    const int stage = NS * 2 * (8 * rpi * D * 2);  // one staging buffer: [NS][K, V] tiles
    const int epi = NW * NS * rpi * HPW * D * 4;   // the epilogue's sums must fit one buffer
    return NBUF * (epi > stage ? epi : stage) + (NBUF == 1 ? 512 : 0);
}

// 16-byte global -> LDS copy that bypasses the register file: lane i's 16 bytes land at
// lds_base + 16*i (lds_base is wave-uniform), whatever global address lane i reads.
__device__ __forceinline__ void g2lds16(const uint4* g, void* lds_base) {
    __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)g,
                                     (__attribute__((address_space(3))) void*)lds_base, 16, 0, 0);
}

// s_waitcnt vmcnt(N) with the other counters left alone (gfx9 encoding).
template <int N>
__device__ __forceinline__ void wait_vmcnt() {
    __builtin_amdgcn_s_waitcnt((N & 0xF) | ((N >> 4) << 14) | (0x7 << 4) | (0xF << 8));
}

template <int D, int HPW, int NW, int NS, int NBUF, bool PV16>
__global__ __launch_bounds__(64 * NW * NS) void paged_decode_fast_kernel(const DecodeArgs a) {
    static_assert(D == 64 || D == 128, "fast path covers head_dim 64 and 128");
    static_assert(NW == 1 || NW == 2 || NW == 4, "waves per GQA group");
    constexpr int CPR = D / 8;         // 16-byte chunks per row
    constexpr int RPI = 64 / CPR;      // rows fetched by one wave-wide load
    constexpr int TT = 8 * RPI;        // tokens per tile
    constexpr int OPL = HPW * D / 64;  // outputs per lane in the epilogue
    constexpr int HPK = D / 64;        // epilogue registers per head: idx = k*64+lane -> h = k/HPK
    constexpr int G = HPW * NW;        // query heads per KV head
    constexpr int NWAVES = NW * NS;
    constexpr int TILE_BYTES = TT * D * 2;  // one tensor, one KV head: 8 KiB for both head sizes
    constexpr int LPW = 16 / NW;            // tile-load instructions per wave and step (8 K + 8 V per tile)
    // LDS: [2 buffers][NS tile rows][K, V][TILE_BYTES] staging, reused by the epilogue as
    // [NWAVES][RPI*HPW*D] floats + [NWAVES][HPW][2] floats.
    // one buffer: [NS tile rows][K, V], at least as large as the epilogue's [NWAVES][RPI*HPW*D] floats
    constexpr int STAGE_BYTES = (decode_lds_bytes(D, HPW, NW, NS, NBUF) - (NBUF == 1 ? 512 : 0)) / NBUF;
    static_assert(NBUF * STAGE_BYTES <= kMaxStaticLds, "workgroup LDS budget");
    // Two separate arrays (not one indexed by the step parity): the compiler then knows that
    // reads of the buffer being consumed do not alias the global -> LDS loads in flight into
    // the other one, and does not wait for those loads before every LDS read.
    __shared__ __attribute__((aligned(16))) unsigned char stage0[STAGE_BYTES];
    // With one buffer (NBUF == 1) the second array only holds the epilogue's (m, l) pairs;
    // latency is then hidden by the other workgroups of the CU instead of by prefetching.
    __shared__ __attribute__((aligned(16))) unsigned char stage1[NBUF == 2 ? STAGE_BYTES : 512];

    const uint32_t item_idx = blockIdx.x;
    if (item_idx >= a.n_items) return;
    // The item is read once, into scalar registers: any vector load issued after the tile
    // loads would have to wait for them (loads return in order).
    struct {
        uint32_t req, kv_head, pt_base, tok_begin, tok_end, part_first, split, pg[4], group_size;
    } it;
    {
        const DecodeWorkItem* gi = a.items + item_idx;
        it.req = __builtin_amdgcn_readfirstlane(gi->req);
        it.kv_head = __builtin_amdgcn_readfirstlane(gi->kv_head);
        it.pt_base = __builtin_amdgcn_readfirstlane(gi->pt_base);
        it.tok_begin = __builtin_amdgcn_readfirstlane(gi->tok_begin);
        it.tok_end = __builtin_amdgcn_readfirstlane(gi->tok_end);
        it.part_first = __builtin_amdgcn_readfirstlane(gi->part_first);
        it.split = __builtin_amdgcn_readfirstlane(gi->split);
        it.group_size = __builtin_amdgcn_readfirstlane(gi->group_size);
#pragma unroll
        for (int i = 0; i < 4; ++i) it.pg[i] = __builtin_amdgcn_readfirstlane(gi->first_pages[i]);
    }
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / 64);  // wave-uniform, in an SGPR
    const int lane = threadIdx.x % 64;
    const int hg = wave % NW;   // head group of this wave
    const int sub = wave / NW;  // tile row of this wave
    const int c = lane % CPR;
    const int r = lane / CPR;
    const int c7 = c & 7;
    const int gsw = c7 ^ ((c7 & 4) ? 3 : 0);  // row-group swizzle g(c)
    const uint32_t head0 = it.kv_head * G + hg * HPW;

    // An item without visible tokens (only a request of length 0 makes one; it is never
    // split) writes its zeros and leaves before anything is loaded.
    if (it.tok_end == it.tok_begin) {
        float* orow = a.o + ((size_t)it.req * a.num_heads + head0) * D;
        if (wave < NW)
            for (int i = lane; i < HPW * D; i += 64) orow[i] = 0.f;
        return;
    }

    // The step's KV write, when this launch carries it: the item that ends at the request's
    // newest position (the last split, or the only item) copies its KV head's slice of the new K
    // and V rows into the pages and waits for the stores, so that its own tile loads below see
    // them; no other item reads that position.  Nothing is in flight after this block, so the
    // waits further down count the same loads as without it.
    if (a.new_k != nullptr) {
        const bool newest = it.part_first == kNoPartial || (it.split & 0xFFFFu) + 1u == (it.split >> 16);
        if (newest) {
            if (wave == 0 && lane < 2 * CPR) {
                const bool is_v = lane >= CPR;
                const uint32_t cc = lane % CPR;
                const size_t row = (size_t)a.new_ids[it.req] * a.page_size + a.new_slots[it.req];
                const uint4 val = (is_v ? a.new_v : a.new_k)[((size_t)it.req * a.kv_heads + it.kv_head) * CPR + cc];
                uint4* dst = const_cast<uint4*>(is_v ? a.v_pages : a.k_pages);
                dst[(row * a.kv_heads + it.kv_head) * CPR + cc] = val;
            }
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
            wait_vmcnt<0>();  // the row has left this wave before any wave of the workgroup loads it
            __syncthreads();
        }
    }

    // q for this wave's heads, dims c*8 .. c*8+7 (issued before the tile loads, so that waiting
    // for it does not wait for them).
    float qv[HPW][8];
    {
        const float* qbase = a.q + ((size_t)it.req * a.num_heads + head0) * D + c * 8;
#pragma unroll
        for (int h = 0; h < HPW; ++h) {
            const float4 lo = *reinterpret_cast<const float4*>(qbase + h * D);
            const float4 hi = *reinterpret_cast<const float4*>(qbase + h * D + 4);
            qv[h][0] = lo.x; qv[h][1] = lo.y; qv[h][2] = lo.z; qv[h][3] = lo.w;
            qv[h][4] = hi.x; qv[h][5] = hi.y; qv[h][6] = hi.z; qv[h][7] = hi.w;
        }
    }

    const uint32_t row_u4 = a.kv_heads * CPR;  // 16-byte chunks per token row (all KV heads)
    const uint32_t lane_u4 = it.kv_head * CPR + c;
    const uint32_t n_tiles = (it.tok_end - it.tok_begin + TT - 1) / TT;
    const uint32_t n_steps = (n_tiles + NS - 1) / NS;

    // This wave's share of the global -> LDS loads of tile `t` of the item (row `sub` of
    // buffer `buf`).  Load instruction j of a tensor brings row group j ^ g(c) to lane (r, c),
    // at LDS offset j*1024 + lane*16; rows past the visible end are clamped onto the last
    // visible row (in bounds, masked out of the softmax).
    auto issue_tile = [&](uint32_t t, unsigned char* stage, uint32_t page_id) {
        const uint32_t tile_start = it.tok_begin + t * TT;
        const uint32_t slot0 = tile_start % a.page_size;
        const uint32_t last = it.tok_end - 1u - tile_start;
        const size_t row0 = ((size_t)page_id * a.page_size + slot0) * row_u4 + lane_u4;
        unsigned char* slot = stage + (size_t)(sub * 2) * TILE_BYTES;
        constexpr int PARTS = (NW == 1) ? 2 : 1;
        constexpr int JN = (NW == 4) ? 4 : 8;
#pragma unroll
        for (int p = 0; p < PARTS; ++p) {
            const int tensor = (NW == 1) ? p : (NW == 2 ? hg : hg / 2);
            const int j0 = (NW == 4) ? (hg % 2) * 4 : 0;
            const uint4* base = (tensor ? a.v_pages : a.k_pages) + row0;
            unsigned char* dst = slot + tensor * TILE_BYTES;
#pragma unroll
            for (int jj = 0; jj < JN; ++jj) {
                const int j = j0 + jj;
                uint32_t tr = (uint32_t)((j ^ gsw) * RPI + r);
                tr = tr < last ? tr : last;
                g2lds16(base + (size_t)tr * row_u4, dst + j * 1024);
            }
        }
    };
    // Page ids: the first four tiles' come with the item, later ones are fetched 64 steps at a
    // time (tile sub + i*NS in lane i) -- the first batch after this wave's first tile loads
    // were issued, later batches when nothing else is in flight.
    uint32_t page_vec = 0;
    auto fetch_pages = [&](uint32_t step0) {
        const uint32_t t = (step0 + lane) * NS + sub;
        page_vec = 0;
        if (t < n_tiles) page_vec = a.pt_flat[it.pt_base + (it.tok_begin + t * TT) / a.page_size];
    };
    // (selected without indexing: a runtime index would move the item to scratch memory)
    const uint32_t pg0 = (NS == 2 && sub) ? it.pg[1] : it.pg[0];
    const uint32_t pg1 = (NS == 2) ? (sub ? it.pg[3] : it.pg[2]) : it.pg[1];
    auto page_of_step = [&](uint32_t step) {
        if (step == 0) return pg0;
        if (step == 1) return pg1;
        return (uint32_t)__builtin_amdgcn_readlane((int)page_vec, (int)(step & 63u));
    };
    static_assert(2 * NS <= 4, "the item carries the page ids of the first two steps");

    // Order of the first loads: q, page ids (long items only), tile 0, tile 1.  The wait that
    // precedes the first use of q or of tile 0 then leaves exactly tile 1 in flight; tile 0 is
    // issued unconditionally (NS == 1) because a conditional load here would turn that wait
    // into a wait for everything.
    const bool have1 = NBUF == 2 && (uint32_t)(NS + sub) < n_tiles;
    if (n_tiles > 2u * NS) fetch_pages(0);
    if (NS == 1 || (uint32_t)sub < n_tiles) issue_tile(sub, stage0, pg0);
    if (have1) issue_tile(NS + sub, stage1, pg1);

#pragma unroll
    for (int h = 0; h < HPW; ++h)
#pragma unroll
        for (int i = 0; i < 8; ++i) qv[h][i] *= a.scale_log2e;

    float acc[HPW][8];
    float m_ref[HPW], l_sum[HPW];
#pragma unroll
    for (int h = 0; h < HPW; ++h) {
        m_ref[h] = kNegBig;
        l_sum[h] = 0.f;
#pragma unroll
        for (int i = 0; i < 8; ++i) acc[h][i] = 0.f;
    }

    // One step of the pipeline: consume `cur`, refill `nxt` (which the previous step consumed).
    auto do_step = [&](uint32_t step, unsigned char* cur, unsigned char* nxt) {
        const uint32_t t = step * NS + sub;
        if (NBUF == 1 && step >= 1) {
            __syncthreads();  // everyone left the previous step: the buffer can be refilled
            if ((step & 63u) == 0) fetch_pages(step);
            if (t < n_tiles) issue_tile(t, cur, page_of_step(step));
        }
        // own loads of this step have landed (at step 0 the loads of step 1 may stay in flight)
        if (step == 0 && have1) wait_vmcnt<LPW>(); else wait_vmcnt<0>();
        __syncthreads();  // everyone's loads of this step landed; everyone left the previous step
        if (NBUF == 2 && step >= 1 && step + 1 < n_steps) {
            if (((step + 1) & 63u) == 0) fetch_pages(step + 1);  // nothing else is in flight here
            const uint32_t t2 = (step + 1) * NS + sub;
            if (t2 < n_tiles) issue_tile(t2, nxt, page_of_step(step + 1));
        }
        if (t >= n_tiles) return;
        const uint32_t tile_start = it.tok_begin + t * TT;
        const uint4* kl = reinterpret_cast<const uint4*>(cur + (size_t)(sub * 2) * TILE_BYTES) + lane;
        const uint4* vl = kl + TILE_BYTES / 16;

        // ---- QK: partial dots over this lane's 8 dims for the 8 row groups, then per head a
        // reduce-scatter over the 8 c-lanes (lane keeps row group g(c)).
        float part[HPW][8];
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const uint4 kq = kl[j * 64];
            const half8_t kh = __builtin_bit_cast(half8_t, kq);
#pragma unroll
            for (int h = 0; h < HPW; ++h) {
                float s = qv[h][0] * (float)kh[0];
#pragma unroll
                for (int i = 1; i < 8; ++i) s = fmaf(qv[h][i], (float)kh[i], s);
                part[h][j] = s;
            }
        }
        float sc[HPW];
#pragma unroll
        for (int h = 0; h < HPW; ++h) {
#pragma unroll
            for (int j = 0; j < 4; ++j) part[h][j] += dpp_f<kDppHalfMirror>(part[h][j + 4]);
#pragma unroll
            for (int j = 0; j < 2; ++j) part[h][j] += dpp_f<kDppQuadXor2>(part[h][j + 2]);
            float s = part[h][0] + dpp_f<kDppQuadXor1>(part[h][1]);
            if (CPR == 16) s += dpp_f<kDppRowRor8>(s);
            sc[h] = s;
        }

        // ---- mask, tile maximum over the r-set, lazy reference update
        const uint32_t my_tok = tile_start + (uint32_t)(gsw * RPI + r);
        const bool visible = my_tok < it.tok_end;
        bool raise = false;
        float tmax[HPW];
#pragma unroll
        for (int h = 0; h < HPW; ++h) {
            sc[h] = visible ? sc[h] : -INFINITY;
            float m = sc[h];
            m = max_nn(m, dpp_f<kDppQuadXor1>(m));
            m = max_nn(m, dpp_f<kDppQuadXor2>(m));
            m = max_nn(m, dpp_f<kDppHalfMirror>(m));
            if (CPR == 16) m = max_nn(m, dpp_f<kDppRowRor8>(m));
            tmax[h] = m;
            raise |= (m > m_ref[h] + kLazyTau);
        }
        if (__any(raise)) {
#pragma unroll
            for (int h = 0; h < HPW; ++h) {
                const float m_new = max_nn(m_ref[h], tmax[h]);
                const float alpha = fast_exp2(m_ref[h] - m_new);
                m_ref[h] = m_new;
                l_sum[h] *= alpha;
#pragma unroll
                for (int i = 0; i < 8; ++i) acc[h][i] *= alpha;
            }
        }

        if constexpr (PV16) {
            // ---- weights rounded to fp16 (the sum l uses the rounded values, so the result
            // is an exactly normalised average with weights perturbed by <= 2^-11), packed
            // two heads to a register and gathered over the 8 c-lanes: register j of the
            // gather holds the weights of the token whose V row sits in V register j.
            constexpr int H2 = (HPW + 1) / 2;
            uint32_t g8[H2][8];
#pragma unroll
            for (int h2 = 0; h2 < H2; ++h2) {
                const _Float16 p0 = (_Float16)fast_exp2(sc[2 * h2] - m_ref[2 * h2]);
                l_sum[2 * h2] += (float)p0;
                _Float16 p1 = (_Float16)0.f;
                if (2 * h2 + 1 < HPW) {
                    p1 = (_Float16)fast_exp2(sc[2 * h2 + 1] - m_ref[2 * h2 + 1]);
                    l_sum[2 * h2 + 1] += (float)p1;
                }
                half2_t pk = {p0, p1};
                const uint32_t pp = __builtin_bit_cast(uint32_t, pk);
                g8[h2][0] = pp;
                g8[h2][1] = dpp_u<kDppQuadXor1>(pp);
                g8[h2][2] = dpp_u<kDppQuadXor2>(pp);
                g8[h2][3] = dpp_u<kDppQuadXor3>(pp);
                g8[h2][4] = dpp_u<kDppHalfMirror>(pp);
                g8[h2][5] = dpp_u<kDppQuadXor1>(g8[h2][4]);
                g8[h2][6] = dpp_u<kDppQuadXor2>(g8[h2][4]);
                g8[h2][7] = dpp_u<kDppQuadXor3>(g8[h2][4]);
            }
            // ---- PV with v_dot2_f32_f16 on row pairs (2k, 2k+1)
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                const uint4 va4 = vl[(2 * k) * 64];
                const uint4 vb4 = vl[(2 * k + 1) * 64];
                const uint32_t* va = reinterpret_cast<const uint32_t*>(&va4);
                const uint32_t* vb = reinterpret_cast<const uint32_t*>(&vb4);
                uint32_t vp[8];  // (v[2k][i], v[2k+1][i])
#pragma unroll
                for (int w = 0; w < 4; ++w) {
                    vp[2 * w] = __builtin_amdgcn_perm(vb[w], va[w], 0x05040100u);
                    vp[2 * w + 1] = __builtin_amdgcn_perm(vb[w], va[w], 0x07060302u);
                }
#pragma unroll
                for (int h2 = 0; h2 < H2; ++h2) {
                    const uint32_t w0 =
                        __builtin_amdgcn_perm(g8[h2][2 * k + 1], g8[h2][2 * k], 0x05040100u);
                    const half2_t pw0 = __builtin_bit_cast(half2_t, w0);
#pragma unroll
                    for (int i = 0; i < 8; ++i)
                        acc[2 * h2][i] = __builtin_amdgcn_fdot2(
                            __builtin_bit_cast(half2_t, vp[i]), pw0, acc[2 * h2][i], false);
                    if (2 * h2 + 1 < HPW) {
                        const uint32_t w1 =
                            __builtin_amdgcn_perm(g8[h2][2 * k + 1], g8[h2][2 * k], 0x07060302u);
                        const half2_t pw1 = __builtin_bit_cast(half2_t, w1);
#pragma unroll
                        for (int i = 0; i < 8; ++i)
                            acc[2 * h2 + 1][i] = __builtin_amdgcn_fdot2(
                                __builtin_bit_cast(half2_t, vp[i]), pw1, acc[2 * h2 + 1][i], false);
                    }
                }
            }
        } else {
            // ---- exact fp32 weights: gather them over the 8 lanes, fp16 V widened in the FMA
            float pj[HPW][8];
#pragma unroll
            for (int h = 0; h < HPW; ++h) {
                const float p = fast_exp2(sc[h] - m_ref[h]);
                l_sum[h] += p;
                pj[h][0] = p;
                pj[h][1] = dpp_f<kDppQuadXor1>(p);
                pj[h][2] = dpp_f<kDppQuadXor2>(p);
                pj[h][3] = dpp_f<kDppQuadXor3>(p);
                pj[h][4] = dpp_f<kDppHalfMirror>(p);
                pj[h][5] = dpp_f<kDppQuadXor1>(pj[h][4]);
                pj[h][6] = dpp_f<kDppQuadXor2>(pj[h][4]);
                pj[h][7] = dpp_f<kDppQuadXor3>(pj[h][4]);
            }
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const uint4 vq = vl[j * 64];
                const half8_t vh = __builtin_bit_cast(half8_t, vq);
#pragma unroll
                for (int h = 0; h < HPW; ++h)
#pragma unroll
                    for (int i = 0; i < 8; ++i) acc[h][i] = fmaf(pj[h][j], (float)vh[i], acc[h][i]);
            }
        }
    };
    if constexpr (NBUF == 2) {
        for (uint32_t step = 0; step < n_steps; step += 2) {
            do_step(step, stage0, stage1);
            if (step + 1 < n_steps) do_step(step + 1, stage1, stage0);
        }
    } else {
        for (uint32_t step = 0; step < n_steps; ++step) do_step(step, stage0, stage0);
    }
    __syncthreads();  // staging memory is reused below

    static_assert(NWAVES * RPI * HPW * D * 4 <= STAGE_BYTES, "epilogue sums fit the first buffer");
    float* s_acc = reinterpret_cast<float*>(stage0) + (size_t)wave * (RPI * HPW * D);
    float* s_ml = reinterpret_cast<float*>(stage1);  // [NWAVES][HPW][2]

    // ---- epilogue 1: bring the RPI r-sets of this wave onto one reference, sum over r
    // through this wave's LDS region.
    float m_all[HPW], l_all[HPW];
#pragma unroll
    for (int h = 0; h < HPW; ++h) {
        float m = m_ref[h];
#pragma unroll
        for (int off = CPR; off < 64; off <<= 1) m = max_nn(m, __shfl_xor(m, off));
        m_all[h] = m;
        const float w = fast_exp2(m_ref[h] - m);
        // with CPR == 16 every token's weight sits in two lanes (c and c^8): count it once
        l_all[h] = wave_sum((CPR == 16 && (c & 8)) ? 0.f : l_sum[h] * w);
        float4* dst = reinterpret_cast<float4*>(&s_acc[((r * HPW + h) * CPR + c) * 8]);
        dst[0] = make_float4(acc[h][0] * w, acc[h][1] * w, acc[h][2] * w, acc[h][3] * w);
        dst[1] = make_float4(acc[h][4] * w, acc[h][5] * w, acc[h][6] * w, acc[h][7] * w);
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");

    // Output k of this lane is element idx = k*64 + lane of [HPW][D]: head k / HPK.
    float o_un[OPL];
#pragma unroll
    for (int k = 0; k < OPL; ++k) {
        const int idx = k * 64 + lane;
        float sum = 0.f;
#pragma unroll
        for (int rr = 0; rr < RPI; ++rr) sum += s_acc[rr * HPW * D + idx];
        o_un[k] = sum;
    }

    // ---- epilogue 2: merge the NS tile rows of the workgroup through LDS
    if constexpr (NS > 1) {
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
#pragma unroll
        for (int k = 0; k < OPL; ++k) s_acc[k * 64 + lane] = o_un[k];
        if (lane < HPW) {
            // m_all / l_all are wave-uniform: pick this lane's head without dynamic indexing
            float mh = m_all[0], lh = l_all[0];
#pragma unroll
            for (int hh = 1; hh < HPW; ++hh) {
                mh = (lane == hh) ? m_all[hh] : mh;
                lh = (lane == hh) ? l_all[hh] : lh;
            }
            s_ml[(wave * HPW + lane) * 2] = mh;
            s_ml[(wave * HPW + lane) * 2 + 1] = lh;
        }
        __syncthreads();
        if (sub != 0) return;
#pragma unroll
        for (int h = 0; h < HPW; ++h) {
            float m = kNegBig;
#pragma unroll
            for (int s = 0; s < NS; ++s) m = max_nn(m, s_ml[((s * NW + hg) * HPW + h) * 2]);
            float l = 0.f;
            float w[NS];
#pragma unroll
            for (int s = 0; s < NS; ++s) {
                w[s] = fast_exp2(s_ml[((s * NW + hg) * HPW + h) * 2] - m);
                l += w[s] * s_ml[((s * NW + hg) * HPW + h) * 2 + 1];
            }
            m_all[h] = m;
            l_all[h] = l;
#pragma unroll
            for (int kk = 0; kk < HPK; ++kk) {
                const int k = h * HPK + kk;
                float sum = 0.f;
#pragma unroll
                for (int s = 0; s < NS; ++s)
                    sum += w[s] * reinterpret_cast<const float*>(stage0)[(size_t)(s * NW + hg) * (RPI * HPW * D) + k * 64 + lane];
                o_un[k] = sum;
            }
        }
    }

    if (it.part_first == kNoPartial) {
#pragma unroll
        for (int k = 0; k < OPL; ++k) {
            const float l = l_all[k / HPK];
            const float inv = l > 0.f ? 1.0f / l : 0.f;
            a.o[((size_t)it.req * a.num_heads + head0) * D + k * 64 + lane] = o_un[k] * inv;
        }
        return;
    }

    if (it.group_size != 0) {
        // Many splits: groups of group_size partials are merged by their own last arrivers
        // into the n_groups slots behind the request's partials, and the last of those merges
        // the groups' results.  (Kept apart from the common case below, whose code is laid out
        // for the shortest path through publish, ticket and merge.)
        const uint32_t n_splits = it.split >> 16;
        const uint32_t my_split = it.split & 0xFFFFu;
        // Partial state of this wave's heads -> slot `slot`: unnormalised o, running max m, sum l.
        auto publish = [&](size_t slot, const float (&o)[OPL], const float (&m)[HPW],
                           const float (&l)[HPW]) __attribute__((always_inline)) {
            float* po = a.part_o + (slot * G + hg * HPW) * D;
            float* ml = a.part_ml + (slot * G + hg * HPW) * 2;
#pragma unroll
            for (int k = 0; k < OPL; ++k) st_dev(po + k * 64 + lane, o[k]);
            if (lane < HPW) {
                float mh = m[0], lh = l[0];
#pragma unroll
                for (int hh = 1; hh < HPW; ++hh) {
                    mh = (lane == hh) ? m[hh] : mh;
                    lh = (lane == hh) ? l[hh] : lh;
                }
                st_dev(ml + lane * 2, mh);
                st_dev(ml + lane * 2 + 1, lh);
            }
            // The partial must have reached memory before the arrival counter is bumped: the
            // write-through stores above are complete once this wave's store counter is zero.
            // (A workgroup-scope release alone emits no such wait on this target.)
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
            wait_vmcnt<0>();
        };
        // Bumps the arrival counter of slot `slot`; true for the last of `expected` arrivers, which
        // also puts the counter back to zero for the next launch.
        auto last_arriver = [&](size_t slot, uint32_t expected) __attribute__((always_inline)) {
            uint32_t ticket = 0;
            uint32_t* counter = &a.counters[slot * NW + hg];
            if (lane == 0)
                ticket = __hip_atomic_fetch_add(counter, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            ticket = __shfl(ticket, 0);
            if (ticket != expected - 1) return false;
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
            if (lane == 0) __hip_atomic_store(counter, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            return true;
        };
        // Merges the `count` (<= 64) partials from slot `first` on.  Lane s holds the (m, l) of
        // partial s for every head; all loads of a round are issued before any is consumed, so
        // eight partials cost about one memory round trip.
        auto merge = [&](size_t first, uint32_t count, float (&acc_o)[OPL], float (&m_fin)[HPW],
                         float (&l_fin)[HPW]) __attribute__((always_inline)) {
            const float* ml_base = a.part_ml + (first * G + hg * HPW) * 2;
            const float* po_base = a.part_o + (first * G + hg * HPW) * D;
            float ms[HPW], ls[HPW];
#pragma unroll
            for (int h = 0; h < HPW; ++h) {
                ms[h] = kNegBig;
                ls[h] = 0.f;
                if ((uint32_t)lane < count) {
                    ms[h] = ld_dev(ml_base + ((size_t)lane * G + h) * 2);
                    ls[h] = ld_dev(ml_base + ((size_t)lane * G + h) * 2 + 1);
                }
            }
            constexpr int UNR = 8;
#pragma unroll
            for (int k = 0; k < OPL; ++k) acc_o[k] = 0.f;
            float wgt[HPW];
            bool have_w = false;
            for (uint32_t s0 = 0; s0 < count; s0 += UNR) {
                float pv[UNR][OPL];
#pragma unroll
                for (int u = 0; u < UNR; ++u) {
#pragma unroll
                    for (int k = 0; k < OPL; ++k) {
                        pv[u][k] = 0.f;
                        if (s0 + u < count) pv[u][k] = ld_dev(po_base + (size_t)(s0 + u) * G * D + k * 64 + lane);
                    }
                }
                if (!have_w) {
#pragma unroll
                    for (int h = 0; h < HPW; ++h) {
                        m_fin[h] = wave_max(ms[h]);
                        wgt[h] = fast_exp2(ms[h] - m_fin[h]);  // lanes >= count: exp2(-1e30 - m) = 0
                        l_fin[h] = wave_sum(wgt[h] * ls[h]);
                    }
                    have_w = true;
                }
#pragma unroll
                for (int u = 0; u < UNR; ++u) {
                    if (s0 + u < count) {
#pragma unroll
                        for (int k = 0; k < OPL; ++k)
                            acc_o[k] += __shfl(wgt[k / HPK], (int)(s0 + u)) * pv[u][k];
                    }
                }
            }
        };

        const uint32_t gs = it.group_size;
        const uint32_t group = my_split / gs;
        float acc_o[OPL], m_fin[HPW], l_fin[HPW];
        publish((size_t)it.part_first + my_split, o_un, m_all, l_all);
        size_t first = (size_t)it.part_first + (size_t)group * gs;
        uint32_t count = min(gs, n_splits - group * gs);
        uint32_t groups_left = (n_splits + gs - 1) / gs;
        for (;;) {
            if (!last_arriver(first, count)) return;
            merge(first, count, acc_o, m_fin, l_fin);
            if (groups_left == 0) break;
            first = (size_t)it.part_first + n_splits;
            count = groups_left;
            groups_left = 0;
            publish(first + group, acc_o, m_fin, l_fin);
        }
#pragma unroll
        for (int k = 0; k < OPL; ++k) {
            const float l = l_fin[k / HPK];
            const float inv = l > 0.f ? 1.0f / l : 0.f;
            a.o[((size_t)it.req * a.num_heads + head0) * D + k * 64 + lane] = acc_o[k] * inv;
        }
        return;
    }

    // ---- split request: publish this item's partial, the last arriver merges all of them.
    // Partials are written and read with device-scope (write-through / cache-bypassing)
    // accesses, so no L2 write-back or invalidate is needed around the arrival counter:
    // waiting for the stores to complete before the counter is bumped is enough.
    const uint32_t n_splits = it.split >> 16;
    const uint32_t my_split = it.split & 0xFFFFu;
    {
        const size_t slot = (size_t)it.part_first + my_split;
        float* po = a.part_o + (slot * G + hg * HPW) * D;
        float* ml = a.part_ml + (slot * G + hg * HPW) * 2;
#pragma unroll
        for (int k = 0; k < OPL; ++k) st_dev(po + k * 64 + lane, o_un[k]);
        if (lane < HPW) {
            float mh = m_all[0], lh = l_all[0];
#pragma unroll
            for (int hh = 1; hh < HPW; ++hh) {
                mh = (lane == hh) ? m_all[hh] : mh;
                lh = (lane == hh) ? l_all[hh] : lh;
            }
            st_dev(ml + lane * 2, mh);
            st_dev(ml + lane * 2 + 1, lh);
        }
    }
    // (a workgroup-scope release alone emits no wait on this target: wait for this wave's
    // write-through stores explicitly, so that whoever wins the ticket finds them in memory)
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    wait_vmcnt<0>();
    uint32_t ticket = 0;
    uint32_t* counter = &a.counters[(size_t)it.part_first * NW + hg];
    if (lane == 0)
        ticket = __hip_atomic_fetch_add(counter, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    ticket = __shfl(ticket, 0);
    if (ticket != n_splits - 1) return;
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
    if (lane == 0)  // ready for the next launch
        __hip_atomic_store(counter, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);

    // Lane s holds the (m, l) of split s for every head; all loads are issued before any
    // is consumed, so the merge costs about one memory round trip.
    const float* ml_base = a.part_ml + ((size_t)it.part_first * G + hg * HPW) * 2;
    const float* po_base = a.part_o + ((size_t)it.part_first * G + hg * HPW) * D;
    float ms[HPW], ls[HPW];
#pragma unroll
    for (int h = 0; h < HPW; ++h) {
        ms[h] = kNegBig;
        ls[h] = 0.f;
        if ((uint32_t)lane < n_splits) {
            ms[h] = ld_dev(ml_base + ((size_t)lane * G + h) * 2);
            ls[h] = ld_dev(ml_base + ((size_t)lane * G + h) * 2 + 1);
        }
    }
    constexpr int UNR = 8;
    float acc_o[OPL];
#pragma unroll
    for (int k = 0; k < OPL; ++k) acc_o[k] = 0.f;
    float wgt[HPW], l_fin[HPW];
    bool have_w = false;
    for (uint32_t s0 = 0; s0 < n_splits; s0 += UNR) {
        float pv[UNR][OPL];
#pragma unroll
        for (int u = 0; u < UNR; ++u) {
#pragma unroll
            for (int k = 0; k < OPL; ++k) {
                pv[u][k] = 0.f;
                if (s0 + u < n_splits) pv[u][k] = ld_dev(po_base + (size_t)(s0 + u) * G * D + k * 64 + lane);
            }
        }
        if (!have_w) {
#pragma unroll
            for (int h = 0; h < HPW; ++h) {
                const float m = wave_max(ms[h]);
                wgt[h] = fast_exp2(ms[h] - m);  // lanes >= n_splits: exp2(-1e30 - m) = 0
                l_fin[h] = wave_sum(wgt[h] * ls[h]);
            }
            have_w = true;
        }
#pragma unroll
        for (int u = 0; u < UNR; ++u) {
            if (s0 + u < n_splits) {
#pragma unroll
                for (int k = 0; k < OPL; ++k)
                    acc_o[k] += __shfl(wgt[k / HPK], (int)(s0 + u)) * pv[u][k];
            }
        }
    }
#pragma unroll
    for (int k = 0; k < OPL; ++k) {
        const float l = l_fin[k / HPK];
        const float inv = l > 0.f ? 1.0f / l : 0.f;
        a.o[((size_t)it.req * a.num_heads + head0) * D + k * 64 + lane] = acc_o[k] * inv;
    }
}

}  // namespace mlc_hip
