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
// (GQA ratios up to 4 run the second kernel of this file, 64 chunk rows per wave; see there.)
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
    const uint32_t n_pages = (seq_len + a.page_size - 1u) / a.page_size;  // the table covers the sequence
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

// ---- the same computation with 64 chunk rows per wave (GQA ratios 1, 2 and 4).  One workgroup
// = 4 waves = the G query heads of one KV head x 4/G blocks of 64 consecutive chunk rows (the
// same 256 (row, head) pairs per K/V tile as above), one wave per SIMD with the whole register
// file to itself.  Every A operand read from LDS (a K row block, a V^T row block) feeds two
// MFMAs, one per 32-row half of the wave's rows, which halves the LDS operand traffic per MFMA.
//   * V stays row-major in LDS, as the global -> LDS loads deliver it: the V^T operand is read
//     with the transposing LDS read of gfx950 (ds_read_b64_tr_b16), so there is no transposition
//     pass and no V^T buffer.
//   * With one wave per SIMD nothing but the wave's own instruction order overlaps the matrix
//     pipe with the vector pipe, so the tile loop is software-pipelined across tiles and its
//     instruction order is fixed by hand.  A step is a sequence of slots, each one MFMA plus a
//     few instructions for the other pipes (head_dim 128: 32 slots),
//       slots  0-15  S(t+1) = K(t+1).Q^T                     + V^T(t) operand reads
//       slots 16-23  O^T += V^T(t).P(t)^T, rows 0-31         + K(t+2) operand reads
//       slots 24-31  the same for rows 32-63                 + global -> LDS loads of a later tile
//     and the weights P = exp2(S.scale - m), one per slot: those of tile t in slots 0-21 (the
//     first 8 were done in the step before), lane maxima of S(t+1) in slots 18-21, the growth
//     test of the running maxima in slot 22, the first 8 weights of tile t+1 in slots 23-31.
//     K(t+2) therefore has to be in LDS two steps ahead (NST >= 4).
//   * The scores are produced by MFMAs written as inline assembly so that they land in ordinary
//     vector registers (with 512 registers per lane the compiler would place every MFMA result
//     in the accumulation registers, which the softmax arithmetic cannot read without one move
//     per value); O stays in accumulation registers.
// Timing experiments (results are wrong, only the time is of interest): compile with
//   -DMLC_PF_NO_MFMA_S / -DMLC_PF_NO_MFMA_PV  without the MFMAs of S / of P.V
//   -DMLC_PF_NO_WEIGHTS    without fma + exp2 + rounding + row sums
//   -DMLC_PF_NO_MAXIMA     without lane maxima and growth test
//   -DMLC_PF_NO_LDS_READS  without the K and V^T operand reads
//   -DMLC_PF_NO_LOADS      without the global -> LDS loads behind the first tiles
typedef _Float16 pf_half2 __attribute__((ext_vector_type(2)));
typedef uint32_t pf_u32x4 __attribute__((ext_vector_type(4)));

// 16-byte global -> LDS load, address = 64-bit uniform base + 32-bit per-lane byte offset.
__device__ __forceinline__ void pf_g2lds16_base(const void* base, uint32_t off, uint32_t lds_base) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                 :
                 : "s"(lds_base), "v"(off), "s"(base)
                 : "memory", "m0");
}

// MFMAs written as inline assembly.  All of them are volatile, so they and the empty "tie"
// statements below keep their order in the instruction stream; the compiler does not see an
// MFMA in them and inserts no wait states, which the step layout provides instead: the result
// of pf_mfma_v is read by vector instructions two whole slots (two MFMAs and about twenty other
// instructions) after the last one of its chain, pf_mfma_a results only by the next MFMA of
// their chain (other MFMAs in between), by the rare rescale and by the epilogue, both behind
// explicit wait states.
__device__ __forceinline__ void pf_mfma_v_first(pf_float16& acc, const pf_half8& x, const pf_half8& y) {
    asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, 0" : "=&v"(acc) : "v"(x), "v"(y));
}
__device__ __forceinline__ void pf_mfma_v(pf_float16& acc, const pf_half8& x, const pf_half8& y) {
#ifdef MLC_PF_NO_MFMA_S
    asm volatile("" : "+v"(acc) : "v"(x), "v"(y)); return;
#endif
    asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+v"(acc) : "v"(x), "v"(y));
}
// accumulate into accumulation registers; also a fence for LDS traffic
__device__ __forceinline__ void pf_mfma_a(pf_float16& acc, const pf_half8& x, const pf_u32x4& y) {
#ifdef MLC_PF_NO_MFMA_PV
    asm volatile("" : "+a"(acc) : "v"(x), "v"(y) : "memory"); return;
#endif
    asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+a"(acc) : "v"(x), "v"(y) : "memory");
}
// Compile-time loop: f(integral_constant<int, I>) for I in [I0, N).
template <int I, int N, class F>
__device__ __forceinline__ void pf_static_for(F&& f) {
    if constexpr (I < N) {
        f(std::integral_constant<int, I>{});
        pf_static_for<I + 1, N>(f);
    }
}
// Empty volatile statements that pin the instructions computing their operands between the
// neighbouring MFMAs: what produces an operand comes before, what consumes it comes after.
__device__ __forceinline__ void pf_tie(float& x, float& y) { asm volatile("" : "+v"(x), "+v"(y)); }
__device__ __forceinline__ void pf_tie(uint32_t& x, float& y) { asm volatile("" : "+v"(x), "+v"(y)); }
__device__ __forceinline__ void pf_tie(float& x) { asm volatile("" : "+v"(x)); }
__device__ __forceinline__ void pf_tie(pf_float16& x) { asm volatile("" : "+v"(x)); }

template <int D, int G, int NST>
__global__ __launch_bounds__(256) void paged_prefill_mfma64_kernel(const PrefillArgs a) {
    static_assert(D == 64 || D == 128, "head_dim 64 or 128");
    static_assert(G == 1 || G == 2 || G == 4, "waves cover whole GQA groups");
    static_assert(NST >= 4 && NST <= 8 && NST % 2 == 0, "4, 6 or 8 stages");
    constexpr int WAVES = 4;
    constexpr int NT = 64 * WAVES;
    constexpr int HALVES = 2;             // 32-row blocks per wave
    constexpr int CPR = D / 8;            // 16-byte chunks per K/V row of one head
    constexpr int KSTEPS = D / 16;        // MFMA steps over head_dim for S^T
    constexpr int MB = D / 32;            // 32-row blocks of O^T
    constexpr int RB = WAVES / G;         // 64-row blocks per workgroup
    constexpr int K_TILE = kPfKeys * D * 2;          // bytes of one tensor's tile
    constexpr int CHUNKS = kPfKeys * CPR;            // 16-byte chunks per tile and tensor
    constexpr int LPT = CHUNKS / NT;                 // chunks of each tensor per thread and tile
    static_assert(CHUNKS % NT == 0 && LPT >= 1, "whole chunks per thread");
    // Eight stages: the waves meet only after every second step.  A step reads V(tile) and
    // K(tile + 2), so what the two steps behind a barrier read (up to tile + 4 of the barrier's
    // step) must have landed there, and what they load (tiles + 6, + 7) replaces the tiles of
    // the two steps before the barrier.
    constexpr bool B2 = NST == 8;
    constexpr int AHEAD = B2 ? NST - 2 : NST - 1;    // tiles issued ahead of the one in work
    constexpr int KEEP = (AHEAD - (B2 ? 4 : 3)) * 2 * LPT;  // own loads that may stay in flight
    constexpr int SLOTS_S = 2 * KSTEPS;              // MFMAs of S per step
    constexpr int SLOTS_PV = 2 * MB;                 // MFMAs of P.V per step and half
    static_assert(SLOTS_PV == KSTEPS, "one K operand read per slot of the first P.V half");

    // stage s: K tile at s * 2 * K_TILE, V tile behind it, both as rows of D halves per key with
    // the 16-byte chunks of a row permuted (see the loader)
    __shared__ __attribute__((aligned(1024))) unsigned char smem[NST * 2 * K_TILE];
#define PF_INLINE __attribute__((always_inline))

    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid / 64);
    const int lane = tid % 64;
    const int l32 = lane % 32;
    const int half = lane / 32;

    // workgroup -> (row block, KV head, request), XCD-aware as above
    uint32_t wg = blockIdx.x;
    if (gridDim.x % 8u == 0) wg = (wg % 8u) * (gridDim.x / 8u) + wg / 8u;
    const uint32_t rbk = wg % a.row_blocks;
    const uint32_t kvh = (wg / a.row_blocks) % a.kv_heads;
    const uint32_t req = wg / (a.row_blocks * a.kv_heads);
    constexpr uint32_t ROWS_WG = kPfRows * HALVES * RB;
    const uint32_t row0_wg = rbk * ROWS_WG;
    const uint32_t head = kvh * G + (wave % G);
    const uint32_t row0 = row0_wg + (wave / G) * (kPfRows * HALVES);  // first chunk row of this wave

    const uint32_t seq_len = a.seq_lens[req];
    const uint32_t qs = a.q_start[req];
    const uint32_t pt_base = a.pt_off[req];
    const uint32_t last_row = min(row0_wg + ROWS_WG, a.chunk) - 1u;
    const uint64_t lim64 = (uint64_t)qs + last_row + 1u;
    const uint32_t wg_limit = (uint32_t)(lim64 < seq_len ? lim64 : seq_len);
    const uint32_t n_tiles = (wg_limit + kPfKeys - 1) / kPfKeys;

    // this lane's two query rows (one per half) and their absolute positions
    uint32_t my_pos[HALVES];
    bool row_ok[HALVES];
    size_t out_row[HALVES];
    pf_half8 qf[HALVES][KSTEPS];
#pragma unroll
    for (int hb = 0; hb < HALVES; ++hb) {
        const uint32_t my_row = row0 + hb * kPfRows + l32;
        row_ok[hb] = my_row < a.chunk;
        my_pos[hb] = qs + my_row;
        out_row[hb] = (((size_t)req * a.chunk + (row_ok[hb] ? my_row : 0)) * a.num_heads + head) * D;
        const _Float16* qrow = a.q + out_row[hb];
#pragma unroll
        for (int ks = 0; ks < KSTEPS; ++ks) {
            qf[hb][ks] = *reinterpret_cast<const pf_half8*>(qrow + ks * 16 + half * 8);
            if (!row_ok[hb]) qf[hb][ks] = pf_half8{0, 0, 0, 0, 0, 0, 0, 0};
        }
    }

    const uint32_t row_bytes = a.kv_heads * D * 2;  // bytes per token row (all KV heads)
    // ---- tile loader: thread tid fetches K and V chunk positions tid + j*NT (j < LPT).
    // Position p (row = p / CPR, slot = p % CPR) is filled with the global chunk
    // slot ^ (row % CPR) of key `row` for K and slot ^ 2 * (row % 4) for V: the first spreads
    // the 16-byte operand reads of 16 keys over the banks, the second the transposing 8-byte
    // reads of 4 keys x 2 chunks.  Tiles are issued in ascending
    // order, so the position in the page table advances by one tile per call; past the last
    // tile the last one is fetched again (never used).  In the last tile V rows beyond the
    // sequence are replaced by its last valid row: their weights are zero, but whatever an
    // unwritten slot of the page holds must not reach the 0 x V products.  (K rows beyond the
    // sequence only produce scores that the mask replaces.)
    uint32_t k_off[LPT], v_row[LPT], v_colb[LPT];
#pragma unroll
    for (int j = 0; j < LPT; ++j) {
        const uint32_t p = (uint32_t)tid + j * NT;
        const uint32_t row = p / CPR;
        k_off[j] = row * row_bytes + ((((p % CPR) ^ (row % CPR)) * 8u) + kvh * D) * 2u;
        v_row[j] = row;
        v_colb[j] = ((((p % CPR) ^ (2u * (row % 4u))) * 8u) + kvh * D) * 2u;
    }
    const uint32_t n_pages = (seq_len + a.page_size - 1u) / a.page_size;  // the table covers the sequence
    uint32_t page_vec = 0;
    // (the load and its wait are one assembly statement: a load the compiler tracks would make
    // it wait for every load in flight, the tile loads included, wherever page_vec is read)
    auto fetch_pages = [&](uint32_t group) PF_INLINE {
        const uint32_t idx = group * 64u + (uint32_t)lane;
        const uint32_t* src = a.pt_flat + pt_base + (idx < n_pages ? idx : (n_pages ? n_pages - 1u : 0u));
        if (n_pages)
            asm volatile("global_load_dword %0, %1, off\n\ts_waitcnt vmcnt(0)" : "=v"(page_vec) : "v"(src) : "memory");
    };
    uint32_t nx_tile = 0, nx_page = 0, nx_off = 0;  // next tile to issue: index, page, token in page
    struct TileSrc { const char* kbase; const char* vbase; uint32_t last; };
    auto tile_src = [&]() PF_INLINE {
        const uint32_t page_id = __builtin_amdgcn_readlane(page_vec, nx_page % 64u);
        const size_t tok0 = (size_t)page_id * a.page_size + nx_off;
        TileSrc ts;
        ts.kbase = reinterpret_cast<const char*>(a.k_pages) + tok0 * row_bytes;
        ts.vbase = reinterpret_cast<const char*>(a.v_pages) + tok0 * row_bytes;
        ts.last = wg_limit - 1u - nx_tile * kPfKeys;  // last valid row of the tile
        return ts;
    };
    // load l (0 .. 2*LPT-1) of the tile described by ts into stage st
    auto tile_load = [&](const TileSrc& ts, int st, int l) PF_INLINE {
        const int j = l / 2;
        const uint32_t dst = __builtin_amdgcn_readfirstlane(
            pf_lds_addr(smem) + st * 2 * K_TILE + (j * WAVES + wave) * 1024);
        if (l % 2 == 0) pf_g2lds16_base(ts.kbase, k_off[j], dst);
        else pf_g2lds16_base(ts.vbase, min(v_row[j], ts.last) * row_bytes + v_colb[j], dst + K_TILE);
    };
    auto tile_advance = [&]() PF_INLINE {
        // (selects instead of branches: this runs once per step)
        const bool adv = nx_tile + 1u < n_tiles;
        const uint32_t off2 = nx_off + kPfKeys;
        const bool wrap = adv && off2 == a.page_size;
        nx_tile += adv ? 1u : 0u;
        nx_off = wrap ? 0u : (adv ? off2 : nx_off);
        nx_page += wrap ? 1u : 0u;
        if (__builtin_expect(wrap && nx_page % 64u == 0, 0)) fetch_pages(nx_page / 64u);
    };

    // ---- LDS operand addresses (per lane, stage base added at the use)
    uint32_t kf_off[KSTEPS];
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ++ks)
        kf_off[ks] = (uint32_t)l32 * (D * 2) + (((ks * 2 + half) ^ (l32 % CPR)) * 16);
    auto read_k = [&](int st, int ks) PF_INLINE {
        return *reinterpret_cast<const pf_half8*>(smem + st * 2 * K_TILE + kf_off[ks]);
    };
    // V^T operand (32 head dims x 16 keys per MFMA) straight from the row-major V tile with the
    // transposing LDS read: within 16 lanes, the lanes 4e .. 4e+3 point at 16 consecutive halves
    // of row e (4 each) and lane j receives column j of those 4 rows.  A lane's 8 keys are, in
    // the order of its P fragment, 4*half + {0..3} and 8 + 4*half + {0..3} of the 16-key group.
    uint32_t vf_off[MB];
    {
        const uint32_t e = (lane % 16) / 4, q = lane % 4, gbit = (lane / 16) % 2;
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) {
            const uint32_t c = mb * 4 + gbit * 2 + q / 2;
            vf_off[mb] = (half * 4 + e) * (D * 2) + ((c ^ (2u * e)) * 16) + (q % 2) * 8;
        }
    }
    auto read_vt = [&](int st, int mb, int t) PF_INLINE {
        typedef __fp16 pf_fp16x4 __attribute__((vector_size(8)));
        typedef uint32_t pf_u32x2 __attribute__((ext_vector_type(2)));
        const unsigned char* base = smem + st * 2 * K_TILE + K_TILE + t * 16 * (D * 2) + vf_off[mb];
        const pf_u32x2 lo = __builtin_bit_cast(pf_u32x2, __builtin_amdgcn_ds_read_tr16_b64_v4f16(
            (pf_fp16x4 __attribute__((address_space(3)))*)(base)));
        const pf_u32x2 hi = __builtin_bit_cast(pf_u32x2, __builtin_amdgcn_ds_read_tr16_b64_v4f16(
            (pf_fp16x4 __attribute__((address_space(3)))*)(base + 8 * (D * 2))));
        return __builtin_bit_cast(pf_half8, pf_u32x4{lo[0], lo[1], hi[0], hi[1]});
    };

    pf_float16 oacc[HALVES][MB];
    float m_run[HALVES], l_run[HALVES];
#pragma unroll
    for (int hb = 0; hb < HALVES; ++hb) {
        m_run[hb] = -1.0e30f;
        l_run[hb] = 0.f;
#pragma unroll
        for (int mb = 0; mb < MB; ++mb)
#pragma unroll
            for (int i = 0; i < 16; ++i) oacc[hb][mb][i] = 0.f;
    }
    // state carried from step to step
    pf_float16 s_cur[HALVES];   // raw scores of the tile whose weights are being computed
    pf_u32x4 pw_cur[HALVES][2]; // its P^T fragments (two fp16 weights per word), first E0 weights done
    pf_half8 kf[KSTEPS];        // K operand of the next S MFMAs
    float alpha_pend[HALVES];   // factor O still has to be multiplied with
    bool pend = false;          // ... if any

    auto lane_max = [&](const pf_float16& s) PF_INLINE {
        float m = s[0];
#pragma unroll
        for (int i = 1; i + 1 < 16; i += 2) m = fmaxf(fmaxf(m, s[i]), s[i + 1]);
        return fmaxf(m, s[15]);
    };
    auto needs_mask = [&](uint32_t tile) PF_INLINE {
        const uint32_t key0 = tile * kPfKeys;
        return key0 + kPfKeys > wg_limit || key0 + kPfKeys - 1u > qs + row0;
    };
    // causal / end-of-sequence mask of a tile's scores (diagonal and last tiles only)
    auto mask_scores = [&](pf_float16 (&sc)[HALVES], uint32_t tile) PF_INLINE {
        const uint32_t key0 = tile * kPfKeys;
#pragma unroll
        for (int hb = 0; hb < HALVES; ++hb)
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                const uint32_t key = key0 + (uint32_t)((i / 4) * 8 + half * 4 + (i % 4));
                if (key > my_pos[hb] || key >= seq_len) sc[hb][i] = -INFINITY;
            }
    };
    // Maxima of a tile (lane maxima of the raw scores in mpre) against the running row maxima.
    // A lane holds half of the keys of its row, so a row maximum grew by more than 2^8 exactly
    // when one of its two lanes exceeds the threshold thr = (m_run + 8) / scale: the common case
    // costs two compares.  When one did, the running maxima and sums move to the new scale at
    // once (every weight of the earlier tiles has been summed by now); O follows at the head of
    // the next step, after the last P.V MFMAs of the current tile.
    float thr[HALVES] = {-1.0e30f, -1.0e30f};
    auto decide = [&](const float (&mpre)[HALVES]) PF_INLINE {
        const bool grow = mpre[0] > thr[0] || mpre[1] > thr[1];
        if (__builtin_expect(__any(grow), 0)) {
#pragma unroll
            for (int hb = 0; hb < HALVES; ++hb) {
                const auto sw = __builtin_amdgcn_permlane32_swap(__float_as_uint(mpre[hb]), __float_as_uint(mpre[hb]), false, false);
                const float mx = fmaxf(__uint_as_float(sw[0]), __uint_as_float(sw[1])) * a.scale_log2e;
                const float m_new = fmaxf(m_run[hb], mx);
                const float alpha = __builtin_amdgcn_exp2f(m_run[hb] - m_new);
                m_run[hb] = m_new;
                thr[hb] = (m_new + 8.0f) / a.scale_log2e;
                l_run[hb] *= alpha;
                alpha_pend[hb] = alpha;
            }
            pend = true;
        }
    };
    auto rescale_o = [&]() PF_INLINE {
        if (__builtin_expect(pend, 0)) {
            // O lives in the accumulation registers, which vector instructions cannot address.
            // The wait states cover an MFMA of the previous step that may still be writing O.
            asm volatile("s_nop 7\n\ts_nop 7" ::: "memory");
#pragma unroll
            for (int hb = 0; hb < HALVES; ++hb)
#pragma unroll
                for (int mb = 0; mb < MB; ++mb)
#pragma unroll
                    for (int i = 0; i < 16; ++i) {
                        float t;
                        asm volatile("v_accvgpr_read_b32 %0, %1" : "=v"(t) : "a"(oacc[hb][mb][i]));
                        t *= alpha_pend[hb];
                        asm volatile("v_accvgpr_write_b32 %0, %1" : "=a"(oacc[hb][mb][i]) : "v"(t));
                    }
            pend = false;
        }
    };
    // Weight e (0 .. 31: half e / 16, key slot e % 16) of the tile with scores sc: one fma + exp2.
    // Every second one completes a pair; the pair is added to the row sum, rounded to fp16 and
    // stored in the P^T fragment one call later (finish_pair), so that no instruction needs the
    // result of the exp2 right behind it.
    float pe_a = 0.f, pe_b = 0.f;   // the pair in work
    auto finish_pair = [&](pf_u32x4 (&pwd)[HALVES][2], int pair) PF_INLINE {
        const int eh = pair / 8, i = (pair % 8) * 2;
        const pf_half2 ph = {(_Float16)pe_a, (_Float16)pe_b};
        // (plain adds: the dot-product instructions run on the matrix pipe and would wait for
        // the MFMA in flight)
        l_run[eh] += pe_a + pe_b;
        uint32_t w = __builtin_bit_cast(uint32_t, ph);
        pf_tie(w, l_run[eh]);
        pwd[eh][i / 8][(i % 8) / 2] = w;
    };
    auto element = [&](const pf_float16 (&sc)[HALVES], pf_u32x4 (&pwd)[HALVES][2], int e) PF_INLINE {
#ifdef MLC_PF_NO_WEIGHTS
        return;
#endif
        float x = sc[e / 16][e % 16];
        pf_tie(x);
        if (e % 2 == 0 && e >= 2) finish_pair(pwd, (e - 2) / 2);
        const float pv = __builtin_amdgcn_exp2f(fmaf(x, a.scale_log2e, -m_run[e / 16]));
        if (e % 2 == 0) {
            pe_a = pv;
            pf_tie(pe_a);
        } else {
            pe_b = pv;
            pf_tie(pe_b);
        }
    };

    // The MFMA slots of a step, in order: S(tile+1) [NS], P.V of tile, first half of the rows
    // [NP], second half [NP].  Slot DEC is where the maxima of tile+1 are settled: the weights
    // of tile are spread over the slots before it (E0 of them were done in the step before),
    // the first E0 weights of tile+1 over the slots behind it, so that no slot carries much
    // more vector work than one MFMA lasts.
    constexpr int NS = SLOTS_S, NP = SLOTS_PV, NSL = NS + 2 * NP;
    constexpr int LM = NS + 2;                 // lane maxima of S(tile+1) from slot LM on: two
                                               // whole slots after its last MFMA
    constexpr int LMQ = (NP >= 8) ? 4 : 2;     // ... spread over this many slots
    constexpr int DEC = LM + LMQ;
    constexpr int E0 = (NP >= 8) ? 8 : 6;
    constexpr int NLATE = NSL - 1 - DEC;       // slots behind DEC
    static_assert(DEC <= NS + NP && NLATE >= 1, "second half of P.V starts after the weights are complete");

    // One step: tile `tile` (scores in s_cur, K(tile+1) operand in kf) -> O; scores, maxima and
    // first weights of tile + 1; K(tile+2) operand; loads of tile + AHEAD.
    auto step = [&](auto sc, uint32_t tile) PF_INLINE {
        constexpr int S = decltype(sc)::value;
        constexpr int SNN = (S + 2) % NST;  // stage of tile + 2
        rescale_o();
        pf_half8 vf[MB][2];
        pf_float16 s_next[HALVES];
        pf_u32x4 pw_next[HALVES][2];
        float mnext[HALVES];
        const TileSrc ts = tile_src();
        pf_static_for<0, NSL>([&](auto sl) PF_INLINE {
            constexpr int slot = decltype(sl)::value;
            // ---- the MFMA of the slot
            if constexpr (slot < NS) {
                constexpr int ks = slot / 2, hb = slot % 2;
                if constexpr (ks == 0) pf_mfma_v_first(s_next[hb], kf[ks], qf[hb][ks]);
                else pf_mfma_v(s_next[hb], kf[ks], qf[hb][ks]);
            } else {
                constexpr int hb = (slot - NS) / NP, q = (slot - NS) % NP;
                pf_mfma_a(oacc[hb][q % MB], vf[q % MB][q / MB], pw_cur[hb][q / MB]);
            }
            // ---- LDS operand reads: V^T(tile) under the S MFMAs, K(tile+2) under the first P.V half
            if constexpr (slot < NS && slot % 2 == 0) {
                constexpr int c = slot / 2;
#ifdef MLC_PF_NO_LDS_READS
                vf[c % MB][c / MB] = qf[0][c];
#else
                vf[c % MB][c / MB] = read_vt(S, c % MB, c / MB);
#endif
            }
#ifndef MLC_PF_NO_LDS_READS
            if constexpr (slot >= NS && slot < NS + NP) kf[slot - NS] = read_k(SNN, slot - NS);
#endif
            // ---- weights of this tile
            if constexpr (slot < DEC)
                pf_static_for<E0 + (32 - E0) * slot / DEC, E0 + (32 - E0) * (slot + 1) / DEC>(
                    [&](auto ec) PF_INLINE { element(s_cur, pw_cur, decltype(ec)::value); });
            // ---- maxima of the next tile
            if constexpr (slot == LM) {
                pf_tie(s_next[0]);
                pf_tie(s_next[1]);
                if (__builtin_expect(needs_mask(tile + 1), 0)) mask_scores(s_next, tile + 1);
            }
#ifndef MLC_PF_NO_MAXIMA
            if constexpr (slot >= LM && slot < LM + LMQ) {
                // part (slot - LM) of LMQ of the 32 scores of this lane
                constexpr int per = 32 / LMQ, first = (slot - LM) * per, hb = first / 16;
                // (chains of three-operand maxima: per / 2 instructions)
                float m = (first % 16 == 0) ? s_next[hb][0] : mnext[hb];
#pragma unroll
                for (int i = first % 16 + (first % 16 == 0 ? 1 : 0); i + 1 < first % 16 + per; i += 2)
                    m = fmaxf(fmaxf(m, s_next[hb][i]), s_next[hb][i + 1]);
                if ((per - (first % 16 == 0 ? 1 : 0)) % 2 == 1) m = fmaxf(m, s_next[hb][first % 16 + per - 1]);
                mnext[hb] = m;
                pf_tie(mnext[hb]);
            }
            if constexpr (slot == DEC) {
                finish_pair(pw_cur, 15);   // the last weights of this tile
                decide(mnext);
                pf_tie(m_run[0], m_run[1]);
            }
#endif
            // ---- first weights of the next tile
            if constexpr (slot > DEC)
                pf_static_for<E0 * (slot - DEC - 1) / NLATE, E0 * (slot - DEC) / NLATE>(
                    [&](auto ec) PF_INLINE { element(s_next, pw_next, decltype(ec)::value); });
            // ---- loads of tile + AHEAD
            if constexpr (slot >= NS + NP && slot < NS + NP + 2 * LPT) {
#ifdef MLC_PF_NO_LOADS
                if (!(nx_tile >= AHEAD && nx_tile + 1u < n_tiles))
#endif
                tile_load(ts, (S + AHEAD) % NST, slot - NS - NP);
            }
        });
#pragma unroll
        for (int hb = 0; hb < HALVES; ++hb) {
            s_cur[hb] = s_next[hb];
#pragma unroll
            for (int t = 0; t < 2; ++t) pw_cur[hb][t] = pw_next[hb][t];
        }
        tile_advance();
        if constexpr (!B2 || S % 2 == 1) {
            pf_wait_vmcnt<KEEP>();
            pf_barrier();
        }
    };

    if (n_tiles > 0) {
        fetch_pages(0);
#pragma unroll
        for (int s = 0; s < AHEAD; ++s) {
            const TileSrc ts = tile_src();
#pragma unroll
            for (int l = 0; l < 2 * LPT; ++l) tile_load(ts, s, l);
            tile_advance();
        }
        pf_wait_vmcnt<KEEP>();   // this thread's part of tiles 0, 1 and 2 is in LDS
        pf_barrier();
#pragma unroll
        for (int ks = 0; ks < KSTEPS; ++ks) kf[ks] = read_k(0, ks);
#pragma unroll
        for (int ks = 0; ks < KSTEPS; ++ks)
#pragma unroll
            for (int hb = 0; hb < HALVES; ++hb) {
                if (ks == 0) pf_mfma_v_first(s_cur[hb], kf[ks], qf[hb][ks]);
                else pf_mfma_v(s_cur[hb], kf[ks], qf[hb][ks]);
            }
        asm volatile("s_nop 7\n\ts_nop 7" : "+v"(s_cur[0]), "+v"(s_cur[1]));
        {
            if (needs_mask(0)) mask_scores(s_cur, 0);
            float mpre[HALVES];
#pragma unroll
            for (int hb = 0; hb < HALVES; ++hb) mpre[hb] = lane_max(s_cur[hb]);
            decide(mpre);
            pf_static_for<0, E0>([&](auto ec) PF_INLINE { element(s_cur, pw_cur, decltype(ec)::value); });
        }
#pragma unroll
        for (int ks = 0; ks < KSTEPS; ++ks) kf[ks] = read_k(1 % NST, ks);

        for (uint32_t base = 0; base < n_tiles; base += NST) {
            step(std::integral_constant<int, 0>{}, base);
            if (base + 1 >= n_tiles) break;
            step(std::integral_constant<int, 1>{}, base + 1);
            if (base + 2 >= n_tiles) break;
            step(std::integral_constant<int, 2>{}, base + 2);
            if (base + 3 >= n_tiles) break;
            step(std::integral_constant<int, 3>{}, base + 3);
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
        pf_wait_vmcnt<0>();
        // the last MFMAs may still be writing O
        asm volatile("s_nop 7\n\ts_nop 7" ::: "memory");
#pragma unroll
        for (int hb = 0; hb < HALVES; ++hb)
#pragma unroll
            for (int mb = 0; mb < MB; ++mb) asm volatile("" : "+a"(oacc[hb][mb]));
    }
#undef PF_INLINE

#pragma unroll
    for (int hb = 0; hb < HALVES; ++hb) {
        if (row_ok[hb]) {
            const float l = l_run[hb] + __shfl_xor(l_run[hb], 32);
            const float inv = l > 0.f ? 1.0f / l : 0.f;
            float* orow = a.o + out_row[hb];
#pragma unroll
            for (int mb = 0; mb < MB; ++mb) {
#pragma unroll
                for (int g4 = 0; g4 < 4; ++g4) {
                    const float4 v = make_float4(oacc[hb][mb][g4 * 4 + 0] * inv, oacc[hb][mb][g4 * 4 + 1] * inv,
                                                 oacc[hb][mb][g4 * 4 + 2] * inv, oacc[hb][mb][g4 * 4 + 3] * inv);
                    *reinterpret_cast<float4*>(orow + mb * 32 + g4 * 8 + half * 4) = v;
                }
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
inline void launch_prefill_dg(PrefillArgs a, int stages, bool rows64, hipStream_t stream) {
    if constexpr (G <= 4) {
        if (rows64) {
            const uint32_t rows_per_wg = kPfRows * 2 * (4 / G);
            a.row_blocks = (a.chunk + rows_per_wg - 1) / rows_per_wg;
            const dim3 grid(a.row_blocks * a.kv_heads * a.batch), block(256);
            switch (stages) {
                case 2:
                case 4: hipLaunchKernelGGL((paged_prefill_mfma64_kernel<D, G, 4>), grid, block, 0, stream, a); break;
                case 8: hipLaunchKernelGGL((paged_prefill_mfma64_kernel<D, G, 8>), grid, block, 0, stream, a); break;
                default: hipLaunchKernelGGL((paged_prefill_mfma64_kernel<D, G, 6>), grid, block, 0, stream, a); break;
            }
            return;
        }
    }
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
inline void launch_prefill_d(const PrefillArgs& a, int stages, bool rows64, hipStream_t stream) {
    switch (a.num_heads / a.kv_heads) {
        case 8: launch_prefill_dg<D, 8>(a, stages, rows64, stream); break;
        case 4: launch_prefill_dg<D, 4>(a, stages, rows64, stream); break;
        case 2: launch_prefill_dg<D, 2>(a, stages, rows64, stream); break;
        default: launch_prefill_dg<D, 1>(a, stages, rows64, stream); break;
    }
}

// stages: LDS pipeline depth (2, 4, 6 or 8; anything else selects 6).  rows64: 64 chunk rows per
// wave (GQA ratios up to 4), else 32.
inline void launch_prefill(const PrefillArgs& a, size_t head_dim, int stages, bool rows64, hipStream_t stream) {
    if (head_dim == 64) launch_prefill_d<64>(a, stages, rows64, stream); else launch_prefill_d<128>(a, stages, rows64, stream);
}

}  // namespace mlc_hip
