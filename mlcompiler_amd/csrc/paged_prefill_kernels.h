// Chunked-prefill attention over paged KV for gfx950 (MI355X): the MFMA path.
//
// Semantics (no kernel of this kind exists in the reference, which prefills by
// looping its decode kernel once per prompt token,
// compiler/runtime/batched_executor.cpp:454-466): for request r, chunk row i at
// absolute position p = q_start[r] + i and query head h,
//   O[r][i][h][:] = softmax_{key <= p, key < seq_len[r]} (q . K[key] / sqrt(D)) . V[key]
// i.e. the decode kernel's causal rule (metal_runtime.mm:2286) applied per row.
// q is fp16 [B][C][H][D], K/V are the same fp16 pages the decode path reads, O is
// fp32 [B][C][H][D]; products run on v_mfma_f32_32x32x16_f16 with fp32 accumulate.
//
// One workgroup = 8 waves = the G query heads of one KV head x 8/G blocks of 32
// consecutive chunk rows, so a K/V tile is fetched once for 256 query rows.
// Per 32-key tile and wave:
//   S^T = K . Q^T    A = K rows (32 keys x 16 dims per step) read from LDS,
//                    B = Q^T, resident in registers.  In the 32x32 accumulator layout
//                    lane l owns query row l%32, so every softmax statistic is
//                    lane-local (plus one exchange with lane l^32).
//   O^T += V^T . P^T A = V^T rows (32 dims x 16 keys per step) read from LDS,
//                    B = P^T, which is exactly what lane l already holds of S^T (keys
//                    of the 16-key group in the order 0-3, 8-11 | 4-7, 12-15); V^T is
//                    stored in LDS with that key order so no cross-lane traffic is needed.
// Pipeline: NST stages in LDS, each one K tile plus one raw V tile, filled by direct
// global -> LDS loads issued NST-1 tiles ahead (K chunks XOR-swizzled by row to spread
// banks).  One tile ahead of its use every thread reads back the 16 bytes of V its own
// load delivered and writes them transposed into one of two V^T buffers, so the only
// wait is on the thread's own oldest loads and there is one barrier per tile.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <type_traits>

namespace mlc_hip {

struct PrefillArgs {
    const _Float16* q;
    const _Float16* k_pages;
    const _Float16* v_pages;
    float* o;
    const uint32_t* pt_flat;
    const uint32_t* pt_off;
    const uint32_t* seq_lens;
    const uint32_t* q_start;
    uint32_t batch, chunk, num_heads, kv_heads, page_size;
    uint32_t row_blocks;  // workgroups along the chunk
    float scale_log2e;
};

typedef _Float16 pf_half8 __attribute__((ext_vector_type(8)));
typedef float pf_float16 __attribute__((ext_vector_type(16)));

static constexpr int kPfKeys = 32;   // keys per tile
static constexpr int kPfRows = 32;   // chunk rows per wave
static constexpr int kPfWaves = 8;   // waves per workgroup

// 16-byte global -> LDS load that bypasses the register file: lane i's 16 bytes land at LDS
// byte address lds_base + 16*i (lds_base wave-uniform).  Issued as inline assembly on
// purpose: the compiler tracks the builtin form of this load and, at the head of the tile
// loop, waits for ALL outstanding loads before the first LDS read (it cannot prove which of
// them target the stage being read), which would stall the pipeline once per round.  Here the
// ordering is explicit instead: pf_wait_vmcnt + pf_barrier below.
__device__ __forceinline__ void pf_g2lds16(const void* g, uint32_t lds_base) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off"
                 :
                 : "s"(lds_base), "v"(g)
                 : "memory", "m0");
}

// Byte address of an LDS object, as the M0 base of pf_g2lds16 wants it.
__device__ __forceinline__ uint32_t pf_lds_addr(const void* p) {
    return (uint32_t)(uintptr_t)(const __attribute__((address_space(3))) void*)p;
}

// s_waitcnt vmcnt(N), other counters untouched.  Also a compiler barrier for memory accesses:
// the LDS reads that follow it depend on loads the compiler does not know about.
template <int N>
__device__ __forceinline__ void pf_wait_vmcnt() {
    asm volatile("s_waitcnt vmcnt(%0)" : : "n"(N) : "memory");
}

// Workgroup barrier that orders LDS traffic only: __syncthreads() would also wait for every
// global -> LDS load still in flight, which is exactly what the pipeline must not do.
__device__ __forceinline__ void pf_barrier() {
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

// D: head_dim (64 or 128); G: query heads per KV head (1, 2, 4, 8); NST: pipeline stages (even).
template <int D, int G, int NST>
__global__ __launch_bounds__(64 * kPfWaves) void paged_prefill_mfma_kernel(const PrefillArgs a) {
    static_assert(D == 64 || D == 128, "head_dim 64 or 128");
    static_assert(kPfWaves % G == 0, "waves cover whole GQA groups");
    static_assert(NST >= 2 && NST <= 8 && NST % 2 == 0, "2, 4, 6 or 8 stages");
    constexpr int NT = 64 * kPfWaves;
    constexpr int CPR = D / 8;            // 16-byte chunks per K/V row of one head
    constexpr int KSTEPS = D / 16;        // MFMA steps over head_dim for S^T
    constexpr int MB = D / 32;            // 32-row blocks of O^T
    constexpr int RB = kPfWaves / G;      // row blocks per workgroup
    constexpr int K_TILE = kPfKeys * D * 2;          // bytes of one tensor's tile
    constexpr int VS = kPfKeys * 2 + 16;             // V^T row stride in bytes (padded)
    constexpr int V_TILE = D * VS;
    constexpr int CHUNKS = kPfKeys * CPR;            // 16-byte chunks per tile and tensor
    static_assert(CHUNKS <= NT, "one chunk of K and one of V per thread and tile");
    constexpr int AHEAD = NST - 1;                   // tiles in flight
    constexpr int KEEP = (AHEAD - 1) * 2;            // own loads that may stay in flight

    // One array per stage: loads into one stage are then known not to touch another.
    __shared__ __attribute__((aligned(16))) unsigned char st0[2 * K_TILE];
    __shared__ __attribute__((aligned(16))) unsigned char st1[2 * K_TILE];
    __shared__ __attribute__((aligned(16))) unsigned char st2[NST > 2 ? 2 * K_TILE : 16];
    __shared__ __attribute__((aligned(16))) unsigned char st3[NST > 2 ? 2 * K_TILE : 16];
    __shared__ __attribute__((aligned(16))) unsigned char st4[NST > 4 ? 2 * K_TILE : 16];
    __shared__ __attribute__((aligned(16))) unsigned char st5[NST > 4 ? 2 * K_TILE : 16];
    __shared__ __attribute__((aligned(16))) unsigned char st6[NST > 6 ? 2 * K_TILE : 16];
    __shared__ __attribute__((aligned(16))) unsigned char st7[NST > 6 ? 2 * K_TILE : 16];
    __shared__ __attribute__((aligned(16))) unsigned char vt0[V_TILE];
    __shared__ __attribute__((aligned(16))) unsigned char vt1[V_TILE];
#define PF_STAGE(S) ((S) == 0 ? st0 : (S) == 1 ? st1 : (S) == 2 ? st2 : (S) == 3 ? st3 : \
                     (S) == 4 ? st4 : (S) == 5 ? st5 : (S) == 6 ? st6 : st7)

    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid / 64);
    const int lane = tid % 64;
    const int l32 = lane % 32;
    const int half = lane / 32;

    // Workgroup -> (row block, KV head, request).  Consecutive workgroup ids go to different
    // XCDs (8 of them, each with its own L2), so ids that share an XCD are made neighbours in
    // the logical order: the row blocks that read the same K/V then share one L2.
    uint32_t wg = blockIdx.x;
    if (gridDim.x % 8u == 0) wg = (wg % 8u) * (gridDim.x / 8u) + wg / 8u;
    const uint32_t rbk = wg % a.row_blocks;
    const uint32_t kvh = (wg / a.row_blocks) % a.kv_heads;
    const uint32_t req = wg / (a.row_blocks * a.kv_heads);
    const uint32_t row0_wg = rbk * (kPfRows * RB);
    const uint32_t head = kvh * G + (wave % G);
    const uint32_t row0 = row0_wg + (wave / G) * kPfRows;  // first chunk row of this wave

    const uint32_t seq_len = a.seq_lens[req];
    const uint32_t qs = a.q_start[req];
    const uint32_t pt_base = a.pt_off[req];
    // keys any row of this workgroup may see
    const uint32_t last_row = min(row0_wg + kPfRows * RB, a.chunk) - 1u;
    const uint64_t lim64 = (uint64_t)qs + last_row + 1u;
    const uint32_t wg_limit = (uint32_t)(lim64 < seq_len ? lim64 : seq_len);
    const uint32_t n_tiles = (wg_limit + kPfKeys - 1) / kPfKeys;

    // this lane's query row and its absolute position
    const uint32_t my_row = row0 + l32;
    const bool row_ok = my_row < a.chunk;
    const uint32_t my_pos = qs + my_row;
    const size_t out_row = (((size_t)req * a.chunk + (row_ok ? my_row : 0)) * a.num_heads + head) * D;

    // Q^T fragments: B operand, lane (n = row l32, k group = half) holds dims ks*16 + half*8 .. +8
    pf_half8 qf[KSTEPS];
    {
        const _Float16* qrow = a.q + out_row;
#pragma unroll
        for (int ks = 0; ks < KSTEPS; ++ks) {
            qf[ks] = *reinterpret_cast<const pf_half8*>(qrow + ks * 16 + half * 8);
            if (!row_ok) qf[ks] = pf_half8{0, 0, 0, 0, 0, 0, 0, 0};
        }
    }

    const uint32_t row_elems = a.kv_heads * D;  // halves per token row (all KV heads)
    // Every thread issues its two loads on every tile, unconditionally: a load under a branch
    // would make the compiler's count of "loads issued since" uncertain and turn the partial
    // waits below into waits for everything.  With head_dim 64 a tile has only 256 chunks per
    // tensor, so the upper four waves repeat the lower four's loads (same bytes to the same LDS
    // addresses).
    const int ltid = tid % CHUNKS;          // chunk position served by this thread
    const int lwave = wave % (CHUNKS / 64);

    // ---- tile loader: thread tid fetches K chunk position tid and V chunk position tid.
    // K position p (row = p / CPR, slot = p % CPR) is filled with global chunk
    // slot ^ (row % CPR) of key `row`: rows are 2*D bytes apart in LDS, the XOR spreads the 32
    // rows an MFMA operand read touches over the banks.  V position p is chunk p / 32 of key
    // p % 32.  Rows past the last key of the workgroup are clamped (in bounds, masked later).
    const uint32_t k_row = (uint32_t)ltid / CPR;
    const uint32_t k_col = ((((uint32_t)ltid % CPR) ^ (k_row % CPR)) * 8u) + kvh * D;
    const uint32_t v_row = (uint32_t)ltid % kPfKeys;
    const uint32_t v_col = ((uint32_t)ltid / kPfKeys) * 8u + kvh * D;
    // Page ids are kept 64 at a time in one register (lane j: page 64*group + j) and picked
    // with readlane: a vector load issued between the tile loads would have to wait for all
    // of them, since loads return in order.  The register is refilled when the loader enters
    // the next group of 64 pages.
    const uint32_t n_pages = a.pt_off[req + 1] - pt_base;
    uint32_t page_vec = 0;
    auto fetch_pages = [&](uint32_t group) {
        const uint32_t idx = group * 64u + (uint32_t)lane;
        page_vec = n_pages ? a.pt_flat[pt_base + (idx < n_pages ? idx : n_pages - 1u)] : 0u;
        pf_wait_vmcnt<0>();  // here, so that the paths that skip the refill carry no pending load
    };
    auto issue = [&](uint32_t tile, unsigned char* st) {
        tile = tile < n_tiles ? tile : n_tiles - 1u;  // past the end: refetch, never used
        const uint32_t key0 = tile * kPfKeys;
        const uint32_t page = key0 / a.page_size;
        if (page % 64u == 0 && key0 % a.page_size == 0) fetch_pages(page / 64u);
        const uint32_t page_id = __builtin_amdgcn_readlane(page_vec, page % 64u);
        const size_t tok0 = (size_t)page_id * a.page_size + key0 % a.page_size;
        const uint32_t last = wg_limit - 1u - key0;  // last valid row of the tile
        const uint32_t kr = k_row < last ? k_row : last;
        const uint32_t vr = v_row < last ? v_row : last;
        const _Float16* kbase = a.k_pages + tok0 * row_elems;
        const _Float16* vbase = a.v_pages + tok0 * row_elems;
        const uint32_t dst = __builtin_amdgcn_readfirstlane(pf_lds_addr(st) + lwave * 1024);
        pf_g2lds16(kbase + (kr * row_elems + k_col), dst);
        pf_g2lds16(vbase + (vr * row_elems + v_col), dst + K_TILE);
    };
    // ---- V transposer: the thread's own 16 bytes (key v_row, dims 8*(tid/32)..+8) go to
    // V^T[dim][pos(key)], keys of each 16-key group ordered 0-3, 8-11, 4-7, 12-15 (the order in
    // which the S^T accumulators hold them).
    const uint32_t vt_off = [&] {
        const uint32_t x = v_row & 15u;
        const uint32_t pos = (v_row & 16u) | (x & 3u) | ((x & 8u) >> 1) | ((x & 4u) << 1);
        return ((uint32_t)ltid / kPfKeys) * 8u * VS + pos * 2u;
    }();
    auto transpose_v = [&](const unsigned char* st, unsigned char* vt) {
        if (tid < CHUNKS) {
            const pf_half8 h8 = *reinterpret_cast<const pf_half8*>(st + K_TILE + tid * 16);
#pragma unroll
            for (int e = 0; e < 8; ++e)
                *reinterpret_cast<_Float16*>(vt + vt_off + e * VS) = h8[e];
        }
    };

    pf_float16 oacc[MB];
#pragma unroll
    for (int mb = 0; mb < MB; ++mb)
#pragma unroll
        for (int i = 0; i < 16; ++i) oacc[mb][i] = 0.f;
    float m_run = -1.0e30f, l_run = 0.f;  // m_run is identical in lanes l and l^32

    auto compute_tile = [&](uint32_t tile, const unsigned char* kbuf, const unsigned char* vbuf) {
        const uint32_t key0 = tile * kPfKeys;
        // ---- S^T = K . Q^T.  All operand reads of a phase are issued before its first MFMA,
        // and the V^T reads before the softmax, so LDS latency is paid once per phase and
        // mostly behind other work instead of once per MFMA.
        pf_half8 kf[KSTEPS];
#pragma unroll
        for (int ks = 0; ks < KSTEPS; ++ks) {
            const int chunk = ks * 2 + half;
            kf[ks] = *reinterpret_cast<const pf_half8*>(
                kbuf + (size_t)l32 * (D * 2) + ((chunk ^ (l32 % CPR)) * 16));
        }
        pf_float16 s;
#pragma unroll
        for (int i = 0; i < 16; ++i) s[i] = 0.f;
#pragma unroll
        for (int ks = 0; ks < KSTEPS; ++ks)
            s = __builtin_amdgcn_mfma_f32_32x32x16_f16(kf[ks], qf[ks], s, 0, 0, 0);
        pf_half8 vf[MB][2];
#pragma unroll
        for (int mb = 0; mb < MB; ++mb)
#pragma unroll
            for (int t = 0; t < 2; ++t)
                vf[mb][t] = *reinterpret_cast<const pf_half8*>(
                    vbuf + (size_t)(mb * 32 + l32) * VS + (t * 16 + half * 8) * 2);
        __builtin_amdgcn_sched_barrier(0);  // keep the V^T reads ahead of the softmax
        // ---- mask + online softmax on the raw scores (the scale is folded into the exp2
        // argument); register i holds key (i/4)*8 + half*4 + i%4 of the tile.  The running
        // reference is only raised when a tile exceeds it by more than 2^8, so the O^T
        // accumulators are rescaled on very few tiles.
        const bool need_mask = (key0 + kPfKeys > wg_limit) || (key0 + kPfKeys - 1u > qs + row0);
        if (need_mask) {
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                const uint32_t key = key0 + (uint32_t)((i / 4) * 8 + half * 4 + (i % 4));
                if (key > my_pos || key >= seq_len) s[i] = -INFINITY;
            }
        }
        float mx = s[0];
#pragma unroll
        for (int i = 1; i < 16; ++i) mx = fmaxf(mx, s[i]);
        mx = fmaxf(mx, __shfl_xor(mx, 32)) * a.scale_log2e;  // scale > 0: max commutes
        if (__any(mx > m_run + 8.0f)) {
            const float m_new = fmaxf(m_run, mx);
            const float alpha = __builtin_amdgcn_exp2f(m_run - m_new);
            m_run = m_new;
            l_run *= alpha;
#pragma unroll
            for (int mb = 0; mb < MB; ++mb)
#pragma unroll
                for (int i = 0; i < 16; ++i) oacc[mb][i] *= alpha;
        }
        float rs = 0.f;
        pf_half8 pfrag[2];
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            const float p = __builtin_amdgcn_exp2f(fmaf(s[i], a.scale_log2e, -m_run));
            rs += p;
            pfrag[i / 8][i % 8] = (_Float16)p;
        }
        l_run += rs;  // this lane's keys only; the two halves are added at the end
        // ---- O^T += V^T . P^T
#pragma unroll
        for (int mb = 0; mb < MB; ++mb)
#pragma unroll
            for (int t = 0; t < 2; ++t)
                oacc[mb] = __builtin_amdgcn_mfma_f32_32x32x16_f16(vf[mb][t], pfrag[t], oacc[mb], 0, 0, 0);
    };

    // Tile t lives in stage t % NST and V^T buffer t % 2.  Step S (t % NST == S): start the
    // loads of tile t + NST - 1 into the stage tile t - 1 just left, multiply tile t, then
    // transpose tile t + 1's V, whose loads are this thread's oldest and have landed once at
    // most KEEP newer ones remain in flight.
    auto step = [&](auto sc, uint32_t tile) {
        constexpr int S = decltype(sc)::value;
        issue(tile + AHEAD, PF_STAGE((S + AHEAD) % NST));
        compute_tile(tile, PF_STAGE(S), (S % 2) ? vt1 : vt0);
        pf_wait_vmcnt<KEEP>();
        if (tile + 1 < n_tiles) transpose_v(PF_STAGE((S + 1) % NST), (S % 2) ? vt0 : vt1);
        pf_barrier();
    };

    if (n_tiles > 0) {
        issue(0, st0);
        if (AHEAD > 1) issue(1, st1);
        if (AHEAD > 2) issue(2, st2);
        if (AHEAD > 3) issue(3, st3);
        if (AHEAD > 4) issue(4, st4);
        if (AHEAD > 5) issue(5, st5);
        if (AHEAD > 6) issue(6, st6);
        pf_wait_vmcnt<KEEP>();
        transpose_v(st0, vt0);
        pf_barrier();
        for (uint32_t base = 0; base < n_tiles; base += NST) {
            step(std::integral_constant<int, 0>{}, base);
            if (base + 1 >= n_tiles) break;
            step(std::integral_constant<int, 1>{}, base + 1);
            if constexpr (NST > 2) {
                if (base + 2 >= n_tiles) break;
                step(std::integral_constant<int, 2>{}, base + 2);
                if (base + 3 >= n_tiles) break;
                step(std::integral_constant<int, 3>{}, base + 3);
            }
            if constexpr (NST > 4) {
                if (base + 4 >= n_tiles) break;
                step(std::integral_constant<int, 4>{}, base + 4);
                if (base + 5 >= n_tiles) break;
                step(std::integral_constant<int, 5>{}, base + 5);
            }
            if constexpr (NST > 6) {
                if (base + 6 >= n_tiles) break;
                step(std::integral_constant<int, 6>{}, base + 6);
                if (base + 7 >= n_tiles) break;
                step(std::integral_constant<int, 7>{}, base + 7);
            }
        }
        pf_wait_vmcnt<0>();  // refetches past the last tile still target this workgroup's LDS
    }
#undef PF_STAGE

    // ---- write O: lane owns row my_row; register i of block mb is dim mb*32 + (i/4)*8 + half*4 + i%4
    if (row_ok) {
        l_run += __shfl_xor(l_run, 32);
        const float inv = l_run > 0.f ? 1.0f / l_run : 0.f;
        float* orow = a.o + out_row;
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) {
#pragma unroll
            for (int g4 = 0; g4 < 4; ++g4) {
                const float4 v = make_float4(oacc[mb][g4 * 4 + 0] * inv, oacc[mb][g4 * 4 + 1] * inv,
                                             oacc[mb][g4 * 4 + 2] * inv, oacc[mb][g4 * 4 + 3] * inv);
                *reinterpret_cast<float4*>(orow + mb * 32 + g4 * 8 + half * 4) = v;
            }
        }
    }
}

inline bool prefill_shape_supported(size_t head_dim, size_t page_size, size_t num_heads,
                                    size_t kv_heads) {
    const size_t g = kv_heads ? num_heads / kv_heads : 0;
    return (head_dim == 64 || head_dim == 128) && page_size % kPfKeys == 0 &&
           (g == 1 || g == 2 || g == 4 || g == 8);
}

template <int D, int G>
inline void launch_prefill_dg(PrefillArgs a, int stages, hipStream_t stream) {
    const uint32_t rows_per_wg = kPfRows * (kPfWaves / G);
    a.row_blocks = (a.chunk + rows_per_wg - 1) / rows_per_wg;
    const dim3 grid(a.row_blocks * a.kv_heads * a.batch), block(64 * kPfWaves);
    switch (stages) {
        case 2: hipLaunchKernelGGL((paged_prefill_mfma_kernel<D, G, 2>), grid, block, 0, stream, a); break;
        case 4: hipLaunchKernelGGL((paged_prefill_mfma_kernel<D, G, 4>), grid, block, 0, stream, a); break;
        case 8: hipLaunchKernelGGL((paged_prefill_mfma_kernel<D, G, 8>), grid, block, 0, stream, a); break;
        default: hipLaunchKernelGGL((paged_prefill_mfma_kernel<D, G, 6>), grid, block, 0, stream, a); break;
    }
}

template <int D>
inline void launch_prefill_d(const PrefillArgs& a, int stages, hipStream_t stream) {
    switch (a.num_heads / a.kv_heads) {
        case 8: launch_prefill_dg<D, 8>(a, stages, stream); break;
        case 4: launch_prefill_dg<D, 4>(a, stages, stream); break;
        case 2: launch_prefill_dg<D, 2>(a, stages, stream); break;
        default: launch_prefill_dg<D, 1>(a, stages, stream); break;
    }
}

// stages: LDS pipeline depth (2, 4, 6 or 8; anything else selects 6).
inline void launch_prefill(const PrefillArgs& a, size_t head_dim, int stages, hipStream_t stream) {
    if (head_dim == 64) launch_prefill_d<64>(a, stages, stream); else launch_prefill_d<128>(a, stages, stream);
}

}  // namespace mlc_hip
