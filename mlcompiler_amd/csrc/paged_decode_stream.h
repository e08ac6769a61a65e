// Tile-balanced paged flash-attention decode for gfx950 (MI355X), wave64.
//
// Same semantics as paged_decode_fast_kernel (MSL paged_flash_attention of the reference,
// compiler/runtime/metal_runtime.mm:2216-2335) and the same per-tile arithmetic; what differs
// is who decides the work.  Here the kernel does, from the caller's tables alone:
//
//   * The KV tiles of the whole batch are numbered in the order
//     [request][kv head][tile of the request]; with T tiles and W workgroups, workgroup w
//     takes tiles [w*T/W, (w+1)*T/W): every workgroup gets the same number of tiles (+-1)
//     whatever the context lengths are, and the grid size does not depend on the tables.
//   * A workgroup walks its range as one stream: tile k+1 is in flight while tile k is
//     consumed, also across the boundary between two (request, kv head) pairs; the running
//     softmax state is kept across the tiles of a pair and finalised when the pair (or the
//     range) ends.
//   * A pair that lies inside one range is written to O directly.  A pair cut by range
//     boundaries is published as partials by the workgroups that share it (at most two
//     partials per workgroup: the first and the last pair of its range); the last of them
//     to arrive merges.  Which workgroups share a pair follows from the numbering, so
//     nobody needs a list.
//   * The per-request arrays (lengths, query positions, page-table offsets) either travel
//     inside the kernel arguments or are read from device memory; the flat page table is
//     always in device memory.  Nothing is planned on the host.
#pragma once

#include "paged_decode_kernels.h"

namespace mlc_hip {

static constexpr uint32_t kStreamEmbBatch = 256;    // requests whose arrays fit the kernel arguments
static constexpr uint32_t kStreamMaxBatch = 4096;   // 64-ary search over the tile prefix in two levels
static constexpr uint32_t kStreamMaxWgs = 2048;     // workgroups per launch, at most

struct StreamArgs {
    const float* q;             // [B][H][D]
    const uint4* k_pages;       // fp16 pages, viewed as 16-byte chunks
    const uint4* v_pages;
    float* o;                   // [B][H][D]
    const uint32_t* pt_flat;    // device copy of page_tables_flat
    const uint32_t* meta;       // device [3][meta_stride]: seq_lens, q_positions, page_table_offsets;
                                // null: the arrays are in emb (stride kStreamEmbBatch)
    float* part_o;              // [2 * n_wg][G][D] un-normalised partial outputs
    float* part_ml;             // [2 * n_wg][G][2] (m in log2 units, l)
    uint32_t* counters;         // [n_wg][NW] arrival counters, zero between launches
    uint32_t batch;
    uint32_t num_heads;
    uint32_t kv_heads;
    uint32_t page_size;         // tokens per page
    uint32_t causal;
    uint32_t capacity_pages;    // page ids are clamped below this (0: not clamped)
    uint32_t meta_stride;
    float scale_log2e;          // log2(e) / sqrt(D)
    // The step's KV write done by this launch (null: none), as in DecodeArgs: the workgroup
    // that owns a pair's last tile writes that pair's slice of the new rows before it loads
    // anything.
    const uint4* new_k;
    const uint4* new_v;
    const uint32_t* new_ids;
    const uint32_t* new_slots;
    uint32_t emb[3 * kStreamEmbBatch];
};

constexpr int stream_static_lds_bytes(int D, int G) {
    const int rpi = 64 / (D / 8);
    return 2 * 2 * (8 * rpi * D * 2) + G * D * rpi * 4;  // two staging buffers (K, V tiles) + epilogue sums
}
// dynamic LDS: tile prefix [B + 1], visible lengths [B], page-table offsets [B]
inline size_t stream_dynamic_lds_bytes(size_t batch) { return (3 * batch + 1) * 4; }

template <int D, int HPW, int NW, bool PV16>
__global__ __launch_bounds__(64 * NW) void paged_decode_stream_kernel(const StreamArgs a) {
    static_assert(D == 64 || D == 128, "head_dim 64 and 128");
    static_assert(NW == 1 || NW == 2 || NW == 4, "waves per GQA group");
    constexpr int CPR = D / 8;         // 16-byte chunks per row
    constexpr int RPI = 64 / CPR;      // rows fetched by one wave-wide load
    constexpr int TT = 8 * RPI;        // tokens per tile
    constexpr int OPL = HPW * D / 64;  // outputs per lane in the epilogue
    constexpr int HPK = D / 64;        // epilogue registers per head
    constexpr int G = HPW * NW;        // query heads per KV head
    constexpr int TILE_BYTES = TT * D * 2;  // one tensor, one KV head: 8 KiB
    // Separate arrays: reads of the buffer being consumed do not alias the global -> LDS loads
    // in flight into the other one, and the epilogue has memory of its own because tile loads
    // stay in flight across it.
    __shared__ __attribute__((aligned(16))) unsigned char stage0[2 * TILE_BYTES];
    __shared__ __attribute__((aligned(16))) unsigned char stage1[2 * TILE_BYTES];
    __shared__ __attribute__((aligned(16))) float s_epi[NW * RPI * HPW * D];
    extern __shared__ uint32_t s_meta[];
    const uint32_t B = a.batch;
    uint32_t* s_start = s_meta;            // [B + 1] tiles of the requests before r (one KV head)
    uint32_t* s_lim = s_meta + B + 1;      // [B] visible tokens
    uint32_t* s_off = s_lim + B;           // [B] offset of the request's page ids

    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / 64);
    const int lane = threadIdx.x % 64;
    const int hg = wave;  // head group of this wave
    const int c = lane % CPR;
    const int r_l = lane / CPR;
    const int c7 = c & 7;
    const int gsw = c7 ^ ((c7 & 4) ? 3 : 0);  // row-group swizzle g(c)
    const uint32_t Hkv = a.kv_heads;
    const uint32_t row_u4 = Hkv * CPR;  // 16-byte chunks per token row (all KV heads)

    // ---- the per-request arrays -> LDS: visible length, page-table offset, tile prefix
    if (wave == 0) {
        const uint32_t* meta = a.meta ? a.meta : a.emb;
        const uint32_t stride = a.meta ? a.meta_stride : kStreamEmbBatch;
        uint32_t carry = 0;
        for (uint32_t b0 = 0; b0 < B; b0 += 64) {
            const uint32_t i = b0 + lane;
            uint32_t seq = 0, qp = 0, off = 0;
            if (i < B) {
                seq = meta[i];
                qp = meta[stride + i];
                off = meta[2 * stride + i];
            }
            const uint32_t lim = (a.causal && qp < seq) ? qp + 1u : seq;  // metal_runtime.mm:2286
            const uint32_t tiles = (lim + TT - 1) / TT;
            uint32_t x = tiles;
#pragma unroll
            for (int d = 1; d < 64; d <<= 1) {
                const uint32_t y = __shfl_up(x, d);
                if (lane >= d) x += y;
            }
            if (i < B) {
                s_start[i] = carry + x - tiles;
                s_lim[i] = lim;
                s_off[i] = off;
            }
            carry += __shfl(x, 63);
        }
        if (lane == 0) s_start[B] = carry;
    }
    __syncthreads();

    // ---- requests without visible tokens are in nobody's range: their rows are zero
    // (metal_runtime.mm:2254-2257)
    for (uint32_t rr = blockIdx.x; rr < B; rr += gridDim.x) {
        if (s_lim[rr] == 0) {
            float* orow = a.o + (size_t)rr * a.num_heads * D;
            for (uint32_t i = threadIdx.x; i < a.num_heads * D; i += 64 * NW) orow[i] = 0.f;
        }
    }

    const uint32_t tiles_head = s_start[B];
    const uint32_t T = tiles_head * Hkv;                       // the host keeps this below 2^31
    const uint32_t W = gridDim.x < T ? gridDim.x : T;          // every workgroup below W has work
    const uint32_t w = blockIdx.x;
    if (w >= W) return;
    const uint32_t g0 = (uint32_t)(((uint64_t)w * T) / W);
    const uint32_t g1 = (uint32_t)(((uint64_t)(w + 1) * T) / W);
    const uint32_t n = g1 - g0;  // >= 1

    // Position in the tile stream: request, KV head, tile of the request, and the request's
    // figures.  All wave-uniform (kept in scalar registers).
    struct Cursor {
        uint32_t r, kvh, t, tiles, lim, off;
    };
    auto load_request = [&](Cursor& cu) {
        cu.tiles = __builtin_amdgcn_readfirstlane(s_start[cu.r + 1] - s_start[cu.r]);
        cu.lim = __builtin_amdgcn_readfirstlane(s_lim[cu.r]);
        cu.off = __builtin_amdgcn_readfirstlane(s_off[cu.r]);
    };
    // largest r with s_start[r] <= key (key < tiles_head): 64-ary search, two levels
    auto find_request = [&](uint32_t key) {
        uint32_t base = 0;
        if (B > 64) {
            const uint32_t idx = (uint32_t)lane * 64u;
            const uint32_t v = idx < B ? s_start[idx] : 0xFFFFFFFFu;
            base = (uint32_t)(__builtin_popcountll(__ballot(v <= key)) - 1) * 64u;
        }
        const uint32_t idx = base + (uint32_t)lane;
        const uint32_t v = idx < B ? s_start[idx] : 0xFFFFFFFFu;
        return (uint32_t)__builtin_amdgcn_readfirstlane(base + (uint32_t)__builtin_popcountll(__ballot(v <= key)) - 1u);
    };
    auto seek = [&](Cursor& cu, uint32_t g) {
        cu.r = find_request(g / Hkv);
        load_request(cu);
        const uint32_t rem = g - __builtin_amdgcn_readfirstlane(s_start[cu.r]) * Hkv;
        cu.kvh = __builtin_amdgcn_readfirstlane(rem / cu.tiles);
        cu.t = rem - cu.kvh * cu.tiles;
    };
    // one tile on; only called while tiles of the range remain, so a next pair exists
    auto advance = [&](Cursor& cu) {
        if (++cu.t < cu.tiles) return;
        cu.t = 0;
        if (++cu.kvh < Hkv) return;
        cu.kvh = 0;
        do {
            ++cu.r;
        } while (__builtin_amdgcn_readfirstlane(s_start[cu.r + 1] - s_start[cu.r]) == 0);
        load_request(cu);
    };
    const uint32_t tpp = a.page_size / TT;  // tiles per page (page size is a multiple of the tile)

    Cursor ci, cc;  // issue side (one tile ahead) and consume side
    seek(cc, g0);
    ci = cc;

    // Page ids of the issue side's request, 64 tiles at a time: lane i holds the page of tile
    // pv_win + i.  Refetched when the issue side enters another request or another window.
    uint32_t pv = 0, pv_win = 0, pv_req = 0xFFFFFFFFu;
    auto fetch_pages = [&](const Cursor& cu) {
        pv_req = cu.r;
        pv_win = cu.t & ~63u;
        const uint32_t t = pv_win + (uint32_t)lane;
        pv = 0;
        if (t < cu.tiles) pv = a.pt_flat[cu.off + t / tpp];
    };
    auto pages_ready = [&](const Cursor& cu) { return pv_req == cu.r && (cu.t & ~63u) == pv_win; };
    fetch_pages(ci);

    // ---- the step's KV write: this workgroup owns the last tile of every pair that ends in
    // its range, so it writes those pairs' slices of the new rows, waits for the stores, and
    // only then loads anything.  2 * CPR lanes move one pair's K and V slice.
    if (a.new_k != nullptr) {
        constexpr int LPP = 2 * CPR;           // lanes per pair
        constexpr int PPW = 64 / LPP;          // pairs per wave and round
        // pairs that end in [g0, g1): the one under the cursor, then every following one that
        // ends before g1.  Pair index p counts pairs with tiles only, from the cursor's.
        const uint32_t first_end = g0 + (cc.tiles - cc.t);  // one past the last tile of the first pair
        if (first_end <= g1) {
            // walk the pairs with a cursor of their own; each wave takes PPW pairs per round
            Cursor cw = cc;
            uint32_t end = first_end, idx = 0;
            for (;;) {
                const uint32_t slot = idx % (uint32_t)(PPW * NW);
                if (slot / PPW == (uint32_t)wave && (uint32_t)lane / LPP == slot % PPW) {
                    const uint32_t l2 = (uint32_t)lane % LPP;
                    const bool is_v = l2 >= (uint32_t)CPR;
                    const uint32_t cch = l2 % CPR;
                    const size_t row = (size_t)a.new_ids[cw.r] * a.page_size + a.new_slots[cw.r];
                    const uint4 val = (is_v ? a.new_v : a.new_k)[((size_t)cw.r * Hkv + cw.kvh) * CPR + cch];
                    uint4* dst = const_cast<uint4*>(is_v ? a.v_pages : a.k_pages);
                    dst[(row * Hkv + cw.kvh) * CPR + cch] = val;
                }
                ++idx;
                if (end >= g1) break;  // no tile of the range is left behind this pair
                cw.t = cw.tiles - 1;
                advance(cw);           // first tile of the next pair
                if (end + cw.tiles > g1) break;  // the next pair ends in a later range
                end += cw.tiles;
            }
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
        wait_vmcnt<0>();  // the rows have left this wave before any wave of the workgroup loads them
        __syncthreads();
    }

    // q of this wave's heads, dims c*8 .. c*8+7, scaled
    float qv[HPW][8];
    auto load_q = [&](const Cursor& cu) {
        const float* qbase = a.q + ((size_t)cu.r * a.num_heads + cu.kvh * G + hg * HPW) * D + c * 8;
#pragma unroll
        for (int h = 0; h < HPW; ++h) {
            const float4 lo = *reinterpret_cast<const float4*>(qbase + h * D);
            const float4 hi = *reinterpret_cast<const float4*>(qbase + h * D + 4);
            qv[h][0] = lo.x * a.scale_log2e; qv[h][1] = lo.y * a.scale_log2e;
            qv[h][2] = lo.z * a.scale_log2e; qv[h][3] = lo.w * a.scale_log2e;
            qv[h][4] = hi.x * a.scale_log2e; qv[h][5] = hi.y * a.scale_log2e;
            qv[h][6] = hi.z * a.scale_log2e; qv[h][7] = hi.w * a.scale_log2e;
        }
    };

    // This wave's share of the global -> LDS loads of the tile under `cu`.  Load instruction j
    // of a tensor brings row group j ^ g(c) to lane (r, c), at LDS offset j*1024 + lane*16; rows
    // past the visible end are clamped onto the last visible row (in bounds, masked out later).
    auto issue_tile = [&](const Cursor& cu, unsigned char* stage) {
        uint32_t page_id = (uint32_t)__builtin_amdgcn_readlane((int)pv, (int)(cu.t & 63u));
        if (a.capacity_pages && page_id >= a.capacity_pages) page_id = a.capacity_pages - 1u;
        const uint32_t tile_start = cu.t * TT;
        const uint32_t slot0 = tile_start % a.page_size;
        const uint32_t last = cu.lim - 1u - tile_start;
        const size_t row0 = ((size_t)page_id * a.page_size + slot0) * row_u4 + cu.kvh * CPR + c;
        constexpr int PARTS = (NW == 1) ? 2 : 1;
        constexpr int JN = (NW == 4) ? 4 : 8;
#pragma unroll
        for (int p = 0; p < PARTS; ++p) {
            const int tensor = (NW == 1) ? p : (NW == 2 ? hg : hg / 2);
            const int j0 = (NW == 4) ? (hg % 2) * 4 : 0;
            const uint4* base = (tensor ? a.v_pages : a.k_pages) + row0;
            unsigned char* dst = stage + tensor * TILE_BYTES;
#pragma unroll
            for (int jj = 0; jj < JN; ++jj) {
                const int j = j0 + jj;
                uint32_t tr = (uint32_t)((j ^ gsw) * RPI + r_l);
                tr = tr < last ? tr : last;
                g2lds16(base + (size_t)tr * row_u4, dst + j * 1024);
            }
        }
    };

    float acc[HPW][8];
    float m_ref[HPW], l_sum[HPW];
    auto reset_state = [&]() {
#pragma unroll
        for (int h = 0; h < HPW; ++h) {
            m_ref[h] = kNegBig;
            l_sum[h] = 0.f;
#pragma unroll
            for (int i = 0; i < 8; ++i) acc[h][i] = 0.f;
        }
    };
    reset_state();

    // ---- one tile: QK, softmax update, PV (the arithmetic of paged_decode_fast_kernel)
    auto consume_tile = [&](const unsigned char* cur, uint32_t t, uint32_t lim) {
        const uint32_t tile_start = t * TT;
        const uint4* kl = reinterpret_cast<const uint4*>(cur) + lane;
        const uint4* vl = kl + TILE_BYTES / 16;
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
        const uint32_t my_tok = tile_start + (uint32_t)(gsw * RPI + r_l);
        const bool visible = my_tok < lim;
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
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                const uint4 va4 = vl[(2 * k) * 64];
                const uint4 vb4 = vl[(2 * k + 1) * 64];
                const uint32_t* va = reinterpret_cast<const uint32_t*>(&va4);
                const uint32_t* vb = reinterpret_cast<const uint32_t*>(&vb4);
                uint32_t vp[8];
#pragma unroll
                for (int q4 = 0; q4 < 4; ++q4) {
                    vp[2 * q4] = __builtin_amdgcn_perm(vb[q4], va[q4], 0x05040100u);
                    vp[2 * q4 + 1] = __builtin_amdgcn_perm(vb[q4], va[q4], 0x07060302u);
                }
#pragma unroll
                for (int h2 = 0; h2 < H2; ++h2) {
                    const uint32_t w0 = __builtin_amdgcn_perm(g8[h2][2 * k + 1], g8[h2][2 * k], 0x05040100u);
                    const half2_t pw0 = __builtin_bit_cast(half2_t, w0);
#pragma unroll
                    for (int i = 0; i < 8; ++i)
                        acc[2 * h2][i] = __builtin_amdgcn_fdot2(__builtin_bit_cast(half2_t, vp[i]), pw0,
                                                                acc[2 * h2][i], false);
                    if (2 * h2 + 1 < HPW) {
                        const uint32_t w1 = __builtin_amdgcn_perm(g8[h2][2 * k + 1], g8[h2][2 * k], 0x07060302u);
                        const half2_t pw1 = __builtin_bit_cast(half2_t, w1);
#pragma unroll
                        for (int i = 0; i < 8; ++i)
                            acc[2 * h2 + 1][i] = __builtin_amdgcn_fdot2(__builtin_bit_cast(half2_t, vp[i]), pw1,
                                                                        acc[2 * h2 + 1][i], false);
                    }
                }
            }
        } else {
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

    // ---- end of a pair's tiles inside this range: sum over the rows of lanes, then either
    // the output (the whole pair was ours) or a partial, whose last arriver merges.
    // seg_first: global index of the first tile this workgroup consumed for the pair.
    auto finalize = [&](const Cursor& cu, uint32_t seg_first, uint32_t seg_end) {
        float* s_acc = s_epi + (size_t)wave * (RPI * HPW * D);
        float m_all[HPW], l_all[HPW];
#pragma unroll
        for (int h = 0; h < HPW; ++h) {
            float m = m_ref[h];
#pragma unroll
            for (int off = CPR; off < 64; off <<= 1) m = max_nn(m, __shfl_xor(m, off));
            m_all[h] = m;
            const float wgt = fast_exp2(m_ref[h] - m);
            // with CPR == 16 every token's weight sits in two lanes (c and c^8): count it once
            l_all[h] = wave_sum((CPR == 16 && (c & 8)) ? 0.f : l_sum[h] * wgt);
            float4* dst = reinterpret_cast<float4*>(&s_acc[((r_l * HPW + h) * CPR + c) * 8]);
            dst[0] = make_float4(acc[h][0] * wgt, acc[h][1] * wgt, acc[h][2] * wgt, acc[h][3] * wgt);
            dst[1] = make_float4(acc[h][4] * wgt, acc[h][5] * wgt, acc[h][6] * wgt, acc[h][7] * wgt);
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        float o_un[OPL];
#pragma unroll
        for (int k = 0; k < OPL; ++k) {
            const int idx = k * 64 + lane;
            float sum = 0.f;
#pragma unroll
            for (int rr = 0; rr < RPI; ++rr) sum += s_acc[rr * HPW * D + idx];
            o_un[k] = sum;
        }
        // (the next pair's sums are written to the same memory: reads above come first)
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();

        const uint32_t head0 = cu.kvh * G + hg * HPW;
        float* orow = a.o + ((size_t)cu.r * a.num_heads + head0) * D;
        const uint32_t ps = __builtin_amdgcn_readfirstlane(s_start[cu.r]) * Hkv + cu.kvh * cu.tiles;  // pair's first tile
        const uint32_t pe = ps + cu.tiles;
        if (seg_first == ps && seg_end == pe) {
#pragma unroll
            for (int k = 0; k < OPL; ++k) {
                const float l = l_all[k / HPK];
                const float inv = l > 0.f ? 1.0f / l : 0.f;
                orow[k * 64 + lane] = o_un[k] * inv;
            }
            return;
        }
        // workgroup of tile g: the largest w with w*T/W <= g
        auto wg_of = [&](uint32_t g) { return (uint32_t)((((uint64_t)g + 1u) * W - 1u) / T); };
        const uint32_t w_lo = wg_of(ps), w_hi = wg_of(pe - 1u);
        const uint32_t n_splits = w_hi - w_lo + 1u;
        // A workgroup's first pair uses slot 2w, a later (so: its last) pair slot 2w + 1.
        const uint32_t g0_lo = (uint32_t)(((uint64_t)w_lo * T) / W);
        const uint32_t slot_first = 2u * w_lo + (g0_lo == ps ? 0u : 1u);
        const uint32_t my_slot = (ps <= g0) ? 2u * w : 2u * w + 1u;
        {
            float* po = a.part_o + ((size_t)my_slot * G + hg * HPW) * D;
            float* ml = a.part_ml + ((size_t)my_slot * G + hg * HPW) * 2;
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
        // The partial must have reached memory before the arrival counter is bumped: the
        // write-through stores are complete once this wave's memory counter is zero.
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
        wait_vmcnt<0>();
        uint32_t ticket = 0;
        uint32_t* counter = &a.counters[(size_t)w_lo * NW + hg];
        if (lane == 0) ticket = __hip_atomic_fetch_add(counter, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        ticket = __shfl(ticket, 0);
        if (ticket != n_splits - 1u) return;
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
        if (lane == 0)  // ready for the next launch
            __hip_atomic_store(counter, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);

        // Merge, 64 partials at a time: lane s holds the (m, l) of partial s for every head; the
        // partial outputs are loaded eight at a time, all issued before any is consumed.
        auto slot_of = [&](uint32_t i) { return i == 0 ? slot_first : 2u * (w_lo + i); };
        float acc_o[OPL], m_run[HPW], l_run[HPW];
#pragma unroll
        for (int k = 0; k < OPL; ++k) acc_o[k] = 0.f;
#pragma unroll
        for (int h = 0; h < HPW; ++h) {
            m_run[h] = kNegBig;
            l_run[h] = 0.f;
        }
        for (uint32_t s0 = 0; s0 < n_splits; s0 += 64) {
            const uint32_t cnt = min(64u, n_splits - s0);
            float wgt[HPW];
            {
                const size_t my = slot_of(s0 + (uint32_t)lane);
                const float* ml = a.part_ml + (my * G + hg * HPW) * 2;
#pragma unroll
                for (int h = 0; h < HPW; ++h) {
                    float ms = kNegBig, ls = 0.f;
                    if ((uint32_t)lane < cnt) {
                        ms = ld_dev(ml + h * 2);
                        ls = ld_dev(ml + h * 2 + 1);
                    }
                    const float m_new = max_nn(m_run[h], wave_max(ms));
                    const float keep = fast_exp2(m_run[h] - m_new);
                    wgt[h] = fast_exp2(ms - m_new);  // lanes >= cnt: exp2(-1e30 - m) = 0
                    l_run[h] = l_run[h] * keep + wave_sum(wgt[h] * ls);
                    m_run[h] = m_new;
#pragma unroll
                    for (int kk = 0; kk < HPK; ++kk) acc_o[h * HPK + kk] *= keep;
                }
            }
            constexpr int UNR = 8;
            for (uint32_t u0 = 0; u0 < cnt; u0 += UNR) {
                float pvv[UNR][OPL];
#pragma unroll
                for (int u = 0; u < UNR; ++u) {
                    const float* po = a.part_o + ((size_t)slot_of(s0 + u0 + u) * G + hg * HPW) * D;
#pragma unroll
                    for (int k = 0; k < OPL; ++k) {
                        pvv[u][k] = 0.f;
                        if (u0 + u < cnt) pvv[u][k] = ld_dev(po + k * 64 + lane);
                    }
                }
#pragma unroll
                for (int u = 0; u < UNR; ++u) {
                    if (u0 + u < cnt) {
#pragma unroll
                        for (int k = 0; k < OPL; ++k) acc_o[k] += __shfl(wgt[k / HPK], (int)(u0 + u)) * pvv[u][k];
                    }
                }
            }
        }
#pragma unroll
        for (int k = 0; k < OPL; ++k) {
            const float l = l_run[k / HPK];
            const float inv = l > 0.f ? 1.0f / l : 0.f;
            orow[k * 64 + lane] = acc_o[k] * inv;
        }
    };

    // ---- the stream: tiles 0 and 1 of the range go out together, then one tile per step
    load_q(cc);
    issue_tile(ci, stage0);
    if (n > 1) {
        advance(ci);
        if (!pages_ready(ci)) fetch_pages(ci);
        issue_tile(ci, stage1);
    }
    uint32_t seg_first = g0;  // first tile consumed for the pair under cc
    auto do_step = [&](uint32_t k, unsigned char* cur, unsigned char* nxt) {
        wait_vmcnt<0>();   // own loads of tile k (and the page ids fetched with them) have landed
        __syncthreads();   // everyone's have; everyone left tile k-1, whose buffer is free
        if (k >= 1 && k + 1 < n) {
            advance(ci);
            if (!pages_ready(ci)) {  // rare (a new request, or 64 tiles on): fetched on demand
                fetch_pages(ci);
            }
            issue_tile(ci, nxt);
        }
        consume_tile(cur, cc.t, cc.lim);
        const bool pair_done = cc.t + 1u == cc.tiles;
        if (pair_done || k + 1 == n) {
            finalize(cc, seg_first, g0 + k + 1u);
            reset_state();
            seg_first = g0 + k + 1u;
        }
        if (k + 1 < n) {
            advance(cc);
            if (pair_done) load_q(cc);
        }
    };
    for (uint32_t k = 0; k < n; k += 2) {
        do_step(k, stage0, stage1);
        if (k + 1 < n) do_step(k + 1, stage1, stage0);
    }
}

}  // namespace mlc_hip
