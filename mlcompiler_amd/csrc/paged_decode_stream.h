// Tile-balanced paged flash-attention decode for gfx950 (MI355X), wave64.
//
// Same semantics as paged_decode_fast_kernel (MSL paged_flash_attention of the reference,
// compiler/runtime/metal_runtime.mm:2216-2335) and the same per-tile arithmetic; what differs
// is who decides the work.  Here the kernel does, from the caller's tables alone:
//
//   * The KV tiles of the whole batch are numbered in the order
//     [request][kv head][tile of the request]; with T tiles and W workgroups, workgroup w
//     takes T/W consecutive tiles (the first T%W workgroups one more): every workgroup gets
//     the same number of tiles (+-1) whatever the context lengths are, and the grid size does
//     not depend on the tables.
//   * A workgroup walks its range as one stream: tile k+1 is in flight while tile k is
//     consumed, also across the boundary between two (request, kv head) pairs; the running
//     softmax state is kept across the tiles of a pair and finalised when the pair (or the
//     range) ends.
//   * A pair that lies inside one range is written to O directly.  A pair cut by range
//     boundaries is summed up by the workgroup that holds its last tile, from the partials
//     the other workgroups that share it leave behind (one per workgroup: the pair that goes
//     on behind its range).  Which workgroups share a pair follows from the numbering, so
//     nobody needs a list.
//   * The per-request arrays (lengths, query positions, page-table offsets) either travel
//     inside the kernel arguments or are read from device memory, and so does the flat page
//     table.  Nothing is planned on the host.
#pragma once

#include <cstddef>

#include "paged_decode_kernels.h"

namespace mlc_hip {

static constexpr uint32_t kStreamSmallStride = 64;  // stride of the embedded arrays of up to 64 requests
static constexpr uint32_t kStreamEmbBatch = 256;    // requests whose arrays fit the kernel arguments
static constexpr uint32_t kStreamEmbWords = 960;    // words of the kernel arguments that carry tables
static constexpr uint32_t kStreamMaxBatch = 4096;   // 64-ary search over the tile prefix in two levels
static constexpr uint32_t kStreamMaxWgs = 2048;     // workgroups per launch, at most
static constexpr size_t kStreamPartBytes = 8u << 20;  // the partial buffer
static constexpr size_t kStreamProbeWord = kStreamPartBytes / 8;  // probe builds: time stamps behind the partials
// Words per lane of a workgroup's partial (see the kernel): NW waves x (OPL + 1) words.
constexpr size_t stream_partial_bytes(size_t G, size_t D, size_t NW) { return (G * D + 64 * NW) * 8; }

struct StreamArgs {
    const float* q;             // [B][H][D]
    const uint4* k_pages;       // fp16 pages, viewed as 16-byte chunks
    const uint4* v_pages;
    float* o;                   // [B][H][D]
    const uint32_t* pt_flat;    // device copy of page_tables_flat; null: the table is in emb, behind the arrays
    const uint32_t* meta;       // device [3][meta_stride]: seq_lens, q_positions, page_table_offsets;
                                // null: the arrays are in emb
    uint64_t* part;             // [n_wg][NW][OPL + 1][64] tagged words {value, launch tag}: one partial per
                                // workgroup (OPL = query heads per wave * D / 64)
    const uint32_t* tag_dev;    // null, or a device word that is added to `tag` (captured passes: the
                                // arguments are the same at every replay, the word is not)
    uint32_t* fault;            // host-visible word, set when a merge gave up waiting for a partial
    uint32_t batch;
    uint32_t num_heads;
    uint32_t kv_heads;
    uint32_t page_size;         // tokens per page
    uint32_t causal;
    uint32_t capacity_pages;    // page ids are clamped below this (0: not clamped)
    uint32_t meta_stride;
    float scale_log2e;          // log2(e) / sqrt(D)
    uint32_t pair_cost;         // units a pair's end counts for when the ranges are cut (0: tiles only)
    uint32_t tag;               // this launch's tag: differs from that of every earlier launch whose
                                // partials may still lie in `part`
    uint32_t spin_limit;        // rounds a merge polls for its partials before it gives up
    uint32_t test_flags;        // bit 0: partials are not published (tests of the give-up path)
    // The step's KV write done by this launch (null: none), as in DecodeArgs: the workgroup
    // that owns a pair's last tile writes that pair's slice of the new rows before it loads
    // anything.
    const uint4* new_k;
    const uint4* new_v;
    const uint32_t* new_ids;
    const uint32_t* new_slots;
    // The split of the output for the Q4_0 matmul that reads it (null: none): whoever writes a row
    // of o also writes it as hi + lo fp16 fragments in that matmul's B-operand layout
    // (q4_matmul_kernels.h), scaled by one power of two per (request, block of 32 columns), and the
    // exponents where the matmul's block-scale form looks for them.  Requests batch .. split_rows-1
    // are the padding of the last tile of 32 requests and are written as zeros.
    _Float16* split_frag;
    int8_t* split_exp;
    uint32_t split_rows;
    // seq_lens | q_positions | page_table_offsets (at a stride of 64 words for up to 64 requests,
    // of meta_stride words above) and, where it fits as well, the flat page table behind them: a
    // call whose tables travel here copies nothing to the device
    uint32_t emb[kStreamEmbWords];
};
static_assert(sizeof(StreamArgs) <= 4096, "kernel arguments are limited to 4 KiB");

// LDS of one workgroup: NBUF stages of one K tile and one V tile (8 KiB each), and in matrix-pipe
// mode (four waves, G query heads per KV head) the waves' results of a pair
constexpr size_t stream_static_lds_bytes(int NBUF, size_t G, size_t D, bool matrix_pipe) {
    return (size_t)NBUF * 2 * 8192 + (matrix_pipe ? (4 * G * D + 2 * 4 * G) * 4 : 24);
}
// dynamic LDS: tile prefix [B + 1], visible lengths [B], page-table offsets [B]
inline size_t stream_dynamic_lds_bytes(size_t batch) { return (4 * batch + 2) * 4; }

// Timing probes, compiled in only for experiments (results then are wrong or partly so):
//   -DMLC_STREAM_PROBE  thread 0 of every workgroup writes the 100 MHz counter at fixed points
//   -DMLC_NO_LOADS      the tile loads are not issued (what the arithmetic alone takes)
//   -DMLC_NO_COMPUTE    the tiles are loaded but not consumed (what the loads alone take)
//   -DMLC_NO_TAIL       partials are neither stored nor merged (what publication and merge take)
#ifdef MLC_STREAM_PROBE
#define MLC_PROBE(i)                                                                                   \
    do {                                                                                               \
        if (threadIdx.x == 0)                                                                          \
            (a.part + kStreamProbeWord)[blockIdx.x * 32 + (i)] = __builtin_amdgcn_s_memrealtime(); \
    } while (0)
#else
#define MLC_PROBE(i)
#endif
// (-DMLC_STREAM_PROBE_TILES adds three stamps per tile; each stamp costs about 0.2 us)
#ifdef MLC_STREAM_PROBE_TILES
#define MLC_PROBE_TILE(i) MLC_PROBE(i)
#else
#define MLC_PROBE_TILE(i)
#endif

// 16-byte global -> LDS load that bypasses the register file: lane i's 16 bytes land at LDS byte
// address lds_base + 16*i (lds_base wave-uniform).  Issued as inline assembly on purpose: the
// compiler then does not know of the load, so it neither waits for all loads in flight before
// LDS reads of another stage nor needs one array per stage; the ordering is explicit instead
// (sd_wait_vmcnt, sd_barrier).
// NT: non-temporal.  A K/V byte is read once per launch and need not stay in the L2, where it only
// pushes out what is read again (page tables, q, partials) and costs the allocation: measured
// 13.43 -> 12.88 us, 30.4 -> 27.7 us and 204.6 -> 192.2 us at configurations 2, 3 and 4 -- where one
// instruction fetches whole cache lines, as the matrix-pipe mode's loads do.  The vector mode's loads
// spread the 16-byte chunks of a row over eight instructions (the swizzle of its row groups), and
// non-temporal loads then fetch most lines more than once (FETCH_SIZE 1.6 times the bytes and
// 222 -> 521 us at configuration 4): it keeps the ordinary load.
template <bool NT>
__device__ __forceinline__ void sd_g2lds16(const void* g, uint32_t lds_base) {
#ifdef MLC_TILE_LOAD_PLAIN   // (timing experiments)
    constexpr bool kNt = false;
#else
    constexpr bool kNt = NT;
#endif
    if constexpr (kNt)
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off nt"
                     :
                     : "s"(lds_base), "v"(g)
                     : "memory", "m0");
    else
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off"
                     :
                     : "s"(lds_base), "v"(g)
                     : "memory", "m0");
}
__device__ __forceinline__ uint32_t sd_lds_addr(const void* p) {
    return (uint32_t)(uintptr_t)(const __attribute__((address_space(3))) void*)p;
}
// s_waitcnt vmcnt(N), other counters untouched; also a compiler barrier for memory accesses
// (the LDS reads behind it depend on loads the compiler does not know about).
template <int N>
__device__ __forceinline__ void sd_wait_vmcnt() {
    asm volatile("s_waitcnt vmcnt(%0)" : : "n"(N) : "memory");
}
// Workgroup barrier that orders LDS traffic only (global -> LDS loads stay in flight across it).
__device__ __forceinline__ void sd_barrier() {
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

// A word of a partial: {value, tag}, written and read whole (64-bit relaxed atomics at device
// scope: the store is written through to memory, the load bypasses the per-XCD L2 caches).
__device__ __forceinline__ void st_tagged(uint64_t* p, uint64_t v) {
    __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ uint64_t ld_tagged(const uint64_t* p) {
    return __hip_atomic_load(const_cast<uint64_t*>(p), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// exclusive-to-inclusive prefix sum over the 64 lanes in six DPP steps (no LDS traffic)
__device__ __forceinline__ uint32_t wave_inclusive_scan(uint32_t x) {
    x += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)x, 0x111, 0xF, 0xF, true);   // row_shr:1
    x += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)x, 0x112, 0xF, 0xF, true);   // row_shr:2
    x += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)x, 0x114, 0xF, 0xF, true);   // row_shr:4
    x += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)x, 0x118, 0xF, 0xF, true);   // row_shr:8
    x += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)x, 0x142, 0xA, 0xF, false);  // row_bcast:15 -> rows 1, 3
    x += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)x, 0x143, 0xC, 0xF, false);  // row_bcast:31 -> rows 2, 3
    return x;
}

// SMALL: at most 64 requests; lane r of every wave holds request r's figures in registers and
// nothing goes through LDS.  Otherwise they are kept in (dynamic) LDS.
// NBUF: tiles staged in LDS per workgroup; tile k + NBUF - 1 is requested while tile k is consumed.
// PVM: how a tile's arithmetic is done.  0: on the vector pipe with fp32 softmax weights; 1: on the
// vector pipe, weights rounded to fp16 for P.V (v_dot2); 2 and 3: on the matrix pipe (4 waves, at most
// 16 query heads per KV head): every wave takes a quarter of the tile's tokens for all heads of
// the group, S^T = K.q^T with v_mfma_f32_16x16x32_f16 (q as the sum of two fp16 numbers, so that
// the products are as exact as with fp32 q), O^T += V^T.P^T with v_mfma_f32_16x16x16_f16 (fp16
// weights as in mode 1; mode 3: the weight as the sum of two fp16 numbers, two MFMAs per V block,
// fp32-grade like mode 0), V^T through the transposing LDS read; the waves' results are combined
// through LDS where a pair of (request, KV head) ends.
// SPLIT: the launch also writes its output as the split-fp16 activations of the Q4_0 matmul that
// reads it (StreamArgs::split_frag).
template <int D, int HPW, int NW, int PVM, bool SMALL, int NBUF, bool SPLIT = false>
__global__ __launch_bounds__(64 * NW) void paged_decode_stream_kernel(const StreamArgs a) {
    constexpr bool PV16 = PVM == 1;
    constexpr bool MF = PVM == 2 || PVM == 3;
    constexpr bool MF_SPLIT_P = PVM == 3;
    static_assert(!MF || (NW == 4 && HPW * NW <= 16), "matrix-pipe mode: 4 waves, at most 16 heads per KV head");
    static_assert(NBUF >= 2 && NBUF <= 4, "2 to 4 stages");
    static_assert(D == 64 || D == 128, "head_dim 64 and 128");
    static_assert(NW == 1 || NW == 2 || NW == 4, "waves per GQA group");
    constexpr int CPR = D / 8;         // 16-byte chunks per row
    constexpr int RPI = 64 / CPR;      // rows fetched by one wave-wide load
    constexpr int TT = 8 * RPI;        // tokens per tile
    constexpr int OPL = HPW * D / 64;  // outputs per lane in the epilogue
    constexpr int HPK = D / 64;        // epilogue registers per head
    constexpr int G = HPW * NW;        // query heads per KV head
    constexpr int TILE_BYTES = TT * D * 2;  // one tensor, one KV head: 8 KiB
    constexpr int LPW = 16 / NW;            // tile-load instructions per wave and tile (8 K + 8 V in all)
    constexpr int STAGE_BYTES = 2 * TILE_BYTES;
    constexpr int TW = TT / NW;             // matrix-pipe mode: tokens of a tile per wave (16 or 8)
    constexpr int KST = D / 32;             // ... MFMA steps over head_dim for S^T
    constexpr int DB = D / 16;              // ... 16-row blocks of O^T
    __shared__ __attribute__((aligned(16))) unsigned char stages[NBUF * STAGE_BYTES];
    // matrix-pipe mode: the waves' (o, m, l) of a pair, combined where the pair ends
    __shared__ __attribute__((aligned(16))) float comb_o[MF ? NW * G * D : 4];
    __shared__ float comb_ml[MF ? 2 * NW * G : 2];
    extern __shared__ uint32_t s_meta[];
    const uint32_t B = a.batch;
    uint32_t* s_start = s_meta;            // [B + 1] tiles of the requests before r (one KV head)
    uint32_t* s_lim = s_meta + B + 1;      // [B] visible tokens
    uint32_t* s_off = s_lim + B;           // [B] offset of the request's page ids
    uint32_t* s_nzb = s_off + B;           // [B + 1] requests with tiles before r

    MLC_PROBE(0);
    // The embedded per-request arrays of a small batch are requested before anything else: their
    // address is the argument segment's, which a wave knows when it starts.
    uint32_t e_seq = 0, e_qp = 0, e_off = 0;
    if constexpr (SMALL) {
        const uint32_t l0 = threadIdx.x % 64;
        e_seq = a.emb[l0];
        e_qp = a.emb[kStreamSmallStride + l0];
        e_off = a.emb[2 * kStreamSmallStride + l0];
        __builtin_amdgcn_sched_barrier(0);
    }
    // Everything the prologue needs from the kernel arguments is requested now, in one go: left
    // to the compiler, each would be fetched where it is first used, one memory round trip after
    // the other on the way to the first tile load.
    {
        const uint64_t p0 = (uint64_t)a.q, p1 = (uint64_t)a.k_pages, p2 = (uint64_t)a.v_pages, p3 = (uint64_t)a.pt_flat,
                       p4 = (uint64_t)a.new_k, p5 = (uint64_t)a.meta, p6 = (uint64_t)a.tag_dev;
        asm volatile("" ::"s"(a.batch), "s"(a.num_heads), "s"(a.kv_heads), "s"(a.page_size), "s"(a.causal),
                     "s"(a.capacity_pages), "s"(a.scale_log2e), "s"(p0), "s"(p1), "s"(p2), "s"(p3), "s"(p4),
                     "s"(p5), "s"(p6), "s"(a.pair_cost), "s"(a.meta_stride), "s"(gridDim.x));
    }
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / 64);
    const int lane = threadIdx.x % 64;
    const int hg = wave;  // head group of this wave
    uint32_t tag_add = 0;   // (needed where the range ends; requested now)
    if (a.tag_dev) tag_add = *a.tag_dev;
    const int c = lane % CPR;
    const int r_l = lane / CPR;
    const int c7 = c & 7;
    const int gsw = c7 ^ ((c7 & 4) ? 3 : 0);  // row-group swizzle g(c)
    const uint32_t Hkv = a.kv_heads;
    const uint32_t row_u4 = Hkv * CPR;  // 16-byte chunks per token row (all KV heads)

    // ---- the per-request arrays: visible length, page-table offset, tile prefix
    uint32_t v_start = 0, v_tiles = 0, v_lim = 0, v_off = 0;  // SMALL: request `lane`
    uint32_t v_nzb = 0;                                        // SMALL: requests with tiles before `lane`
    uint32_t tiles_head;                                       // tiles of all requests (one KV head)
    uint32_t nz_head;                                          // requests with tiles
    if constexpr (SMALL) {
        // The arrays inside the kernel arguments are read before anything else is known (their
        // address is the argument segment's, no pointer has to be fetched first); lanes past
        // the batch read other arguments and are masked.
        // (embedded arrays of up to 64 requests sit at a stride of 64 words, so that these loads go
        // out before any argument has arrived)
        uint32_t seq = e_seq, qp = e_qp, off = e_off;
        if (a.meta != nullptr && (uint32_t)lane < B) {
            seq = a.meta[lane];
            qp = a.meta[a.meta_stride + lane];
            off = a.meta[2 * a.meta_stride + lane];
        }
        uint32_t lim = (a.causal && qp < seq) ? qp + 1u : seq;  // metal_runtime.mm:2286
        lim = (uint32_t)lane < B ? lim : 0u;
        v_lim = lim;
        v_off = off;
        v_tiles = (lim + TT - 1) / TT;
        const uint32_t incl = wave_inclusive_scan(v_tiles);
        v_start = incl - v_tiles;
        tiles_head = (uint32_t)__builtin_amdgcn_readlane((int)incl, 63);
        const uint64_t nz = __ballot(v_tiles != 0);
        v_nzb = (uint32_t)__builtin_popcountll(nz & ((1ull << lane) - 1ull));
        nz_head = (uint32_t)__builtin_popcountll(nz);
    } else {
        if (wave == 0) {
            const uint32_t* meta = a.meta ? a.meta : a.emb;
            const uint32_t stride = a.meta_stride;   // (more than 64 requests: the arrays are packed)
            uint32_t carry = 0, carry_nz = 0;
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
                const uint32_t x = wave_inclusive_scan(tiles);
                const uint64_t nz = __ballot(tiles != 0);
                if (i < B) {
                    s_start[i] = carry + x - tiles;
                    s_lim[i] = lim;
                    s_off[i] = off;
                    s_nzb[i] = carry_nz + (uint32_t)__builtin_popcountll(nz & ((1ull << lane) - 1ull));
                }
                carry += (uint32_t)__builtin_amdgcn_readlane((int)x, 63);
                carry_nz += (uint32_t)__builtin_popcountll(nz);
            }
            if (lane == 0) {
                s_start[B] = carry;
                s_nzb[B] = carry_nz;
            }
        }
        __syncthreads();
        tiles_head = s_start[B];
        nz_head = s_nzb[B];
    }
    MLC_PROBE(1);
    auto req_start = [&](uint32_t r) {
        if constexpr (SMALL) return (uint32_t)__builtin_amdgcn_readlane((int)v_start, (int)r);
        else return (uint32_t)__builtin_amdgcn_readfirstlane(s_start[r]);
    };
    auto req_tiles = [&](uint32_t r) {
        if constexpr (SMALL) return (uint32_t)__builtin_amdgcn_readlane((int)v_tiles, (int)r);
        else return (uint32_t)__builtin_amdgcn_readfirstlane(s_start[r + 1] - s_start[r]);
    };
    auto req_nzb = [&](uint32_t r) {
        if constexpr (SMALL) return (uint32_t)__builtin_amdgcn_readlane((int)v_nzb, (int)r);
        else return (uint32_t)__builtin_amdgcn_readfirstlane(s_nzb[r]);
    };
    auto req_lim = [&](uint32_t r) {
        if constexpr (SMALL) return (uint32_t)__builtin_amdgcn_readlane((int)v_lim, (int)r);
        else return (uint32_t)__builtin_amdgcn_readfirstlane(s_lim[r]);
    };
    auto req_off = [&](uint32_t r) {
        if constexpr (SMALL) return (uint32_t)__builtin_amdgcn_readlane((int)v_off, (int)r);
        else return (uint32_t)__builtin_amdgcn_readfirstlane(s_off[r]);
    };

    // ---- requests without visible tokens are in nobody's range: their rows are zero
    // (metal_runtime.mm:2254-2257)
    for (uint32_t rr = blockIdx.x; rr < B; rr += gridDim.x) {
        if (req_lim(rr) == 0) {
            float* orow = a.o + (size_t)rr * a.num_heads * D;
            for (uint32_t i = threadIdx.x; i < a.num_heads * D; i += 64 * NW) orow[i] = 0.f;
        }
    }
    if constexpr (SPLIT) {  // ... and so are their fragments, and those of the padding requests
        const uint32_t cols = a.num_heads * D;
        for (uint32_t rr = blockIdx.x; rr < a.split_rows; rr += gridDim.x) {
            if (rr < B && req_lim(rr) != 0) continue;
            const uint32_t t32 = rr / 32, n32 = rr % 32;
            for (uint32_t k8 = threadIdx.x; k8 < cols / 8; k8 += 64 * NW) {
                const size_t base = ((size_t)t32 * (cols / 16) + k8 / 2) * 2;
                const uint32_t fl = (k8 % 2) * 32 + n32;
                const uint4 z = make_uint4(0u, 0u, 0u, 0u);
                *reinterpret_cast<uint4*>(a.split_frag + ((base + 0) * 64 + fl) * 8) = z;
                *reinterpret_cast<uint4*>(a.split_frag + ((base + 1) * 64 + fl) * 8) = z;
            }
            for (uint32_t blk = threadIdx.x; blk < cols / 32; blk += 64 * NW)
                a.split_exp[((size_t)t32 * (cols / 32) + blk) * 32 + ((n32 % 8) / 4) * 16 + (n32 / 8) * 4 + n32 % 4] = 0;
        }
    }

    // The ranges are cut in units: a tile is one unit, and the end of a pair (the waves meet, the
    // pair's figures are put aside or published, q is fetched again) counts for PC more, so that a
    // workgroup whose range crosses from one pair into the next gets fewer tiles.  Unit numbering:
    // [request][kv head][the pair's tiles, then PC units that stand for its end].
    const uint32_t T = tiles_head * Hkv;                       // the host keeps this below 2^31
    // (nothing to balance where every tile gets a workgroup of its own)
    const uint32_t PC = T > gridDim.x ? a.pair_cost : 0u;
    const uint32_t UT = T + PC * nz_head * Hkv;                // ... and this
    const uint32_t W = gridDim.x < UT ? gridDim.x : UT;
    const uint32_t w = blockIdx.x;
    if (w >= W) return;
    // UT = W * tq + trem: the first trem workgroups take tq + 1 units, the others tq
    const uint32_t tq = __builtin_amdgcn_readfirstlane(UT / W), trem = UT - tq * W;
    auto unit_start = [&](uint32_t wg) { return wg * tq + (wg < trem ? wg : trem); };

    // Position in the tile stream: request, KV head, tile of the request, and the request's
    // figures.  All wave-uniform (kept in scalar registers).
    struct Cursor {
        uint32_t r, kvh, t, tiles, lim, off;
    };
    auto load_request = [&](Cursor& cu) {
        cu.tiles = req_tiles(cu.r);
        cu.lim = req_lim(cu.r);
        cu.off = req_off(cu.r);
    };
    // largest r with start[r] <= key (key below the total), starts counted in tiles (pc = 0) or
    // in units (pc = PC)
    auto find_request = [&](uint32_t key, uint32_t pc = 0) {
        if constexpr (SMALL) {
            // lanes past the batch hold the total, which is above any key
            return (uint32_t)__builtin_popcountll(__ballot(v_start + pc * v_nzb <= key)) - 1u;
        } else {
            uint32_t base = 0;
            if (B > 64) {  // 64-ary search, two levels
                const uint32_t idx = (uint32_t)lane * 64u;
                const uint32_t v = idx < B ? s_start[idx] + pc * s_nzb[idx] : 0xFFFFFFFFu;
                base = (uint32_t)(__builtin_popcountll(__ballot(v <= key)) - 1) * 64u;
            }
            const uint32_t idx = base + (uint32_t)lane;
            const uint32_t v = idx < B ? s_start[idx] + pc * s_nzb[idx] : 0xFFFFFFFFu;
            return (uint32_t)__builtin_amdgcn_readfirstlane(base + (uint32_t)__builtin_popcountll(__ballot(v <= key)) - 1u);
        }
    };
    // tiles in front of unit u
    auto tiles_before = [&](uint32_t u) {
        if (PC == 0) return u;
        if (u >= UT) return T;
        const uint32_t r = find_request(u / Hkv, PC);
        const uint32_t tiles = req_tiles(r), per = tiles + PC;
        const uint32_t rem = u - (req_start(r) + PC * req_nzb(r)) * Hkv;
        const uint32_t kvh = __builtin_amdgcn_readfirstlane(rem / per), x = rem - kvh * per;
        return req_start(r) * Hkv + kvh * tiles + (x < tiles ? x : tiles);
    };
    // This range in tiles: [g0, g1), n of them.  g0 comes with the cursor's start below; g1 and n
    // are worked out behind the first tile's request, off the way to it (before it only where the
    // range starts with a tile that holds a new row of the KV write, which needs them).
    const uint32_t u0 = unit_start(w), u1 = unit_start(w + 1u);
    uint32_t g0 = u0, g1 = 0, n = 0;
    auto seek = [&](Cursor& cu, uint32_t g) {
        cu.r = find_request(g / Hkv);
        load_request(cu);
        const uint32_t rem = g - req_start(cu.r) * Hkv;
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
        } while (req_tiles(cu.r) == 0);
        load_request(cu);
    };
    const uint32_t tpp = a.page_size / TT;  // tiles per page (page size is a multiple of the tile)

    Cursor ci, cc;  // issue side (one tile ahead) and consume side
    if (PC == 0) {
        seek(cc, g0);
    } else {
        // the cursor at unit u0, or, where that is one of the units of a pair's end, at the first
        // tile behind it
        cc.r = find_request(u0 / Hkv, PC);
        load_request(cc);
        const uint32_t per = cc.tiles + PC;
        const uint32_t rem = u0 - (req_start(cc.r) + PC * req_nzb(cc.r)) * Hkv;
        cc.kvh = __builtin_amdgcn_readfirstlane(rem / per);
        const uint32_t x = rem - cc.kvh * per;
        const uint32_t pair0 = req_start(cc.r) * Hkv + cc.kvh * cc.tiles;
        if (x < cc.tiles) {
            cc.t = x;
            g0 = pair0 + x;
        } else {
            if (u0 + (per - x) >= u1) return;  // nothing but units of a pair's end
            g0 = pair0 + cc.tiles;
            cc.t = cc.tiles - 1u;
            advance(cc);
        }
    }
    ci = cc;

    // (the embedded table is addressed as global memory, which the argument segment is: through
    // the constant address space the choice between the two would make every page-id load a flat
    // one, and the compiler waits for all loads in flight around those)
    typedef const __attribute__((address_space(1))) uint32_t* global_u32_ptr;
    const uint32_t* emb_table = (const uint32_t*)(global_u32_ptr)(uintptr_t)__builtin_amdgcn_kernarg_segment_ptr() +
                                offsetof(StreamArgs, emb) / 4 + 3u * (SMALL ? kStreamSmallStride : a.meta_stride);
    const uint32_t* pt_flat = a.pt_flat ? a.pt_flat : emb_table;
    // Page ids of the issue side's request, 64 tiles at a time: lane i holds the page of tile
    // pv_win + i.  Refetched when the issue side enters another request or another window.
    uint32_t pv = 0, pv_win = 0, pv_req = 0xFFFFFFFFu;
    // ... and of the first 64 tiles of the request behind it, requested when the issue side enters a
    // request, so that the step into the next request finds them in a register
    uint32_t pv_nx = 0, pv_nx_req = 0xFFFFFFFFu;
    auto prefetch_next_pages = [&](uint32_t r) {
        pv_nx_req = 0xFFFFFFFFu;
        do {
            ++r;
        } while (r < B && req_tiles(r) == 0);
        if (r >= B) return;
        pv_nx_req = r;
        const uint32_t idx = min((uint32_t)lane, req_tiles(r) - 1u) / tpp;   // (lanes past the end repeat the last id)
        pv_nx = pt_flat[req_off(r) + idx];
    };
    auto fetch_pages = [&](const Cursor& cu) {
        if (pv_nx_req == cu.r && cu.t < 64u) {
            pv = pv_nx;
            pv_req = cu.r;
            pv_win = 0;
        } else {
            pv_req = cu.r;
            pv_win = cu.t & ~63u;
            const uint32_t t = pv_win + (uint32_t)lane;
            pv = 0;
            if (t < cu.tiles) pv = pt_flat[cu.off + t / tpp];
        }
        // The ids are waited for here, inside whatever branch fetches them: left pending, the
        // compiler would wait at every later join of the control flow, and as it does not know
        // of the tile loads, that wait would be for all of them.
        asm volatile("" : "+v"(pv));
    };
    auto pages_ready = [&](const Cursor& cu) { return pv_req == cu.r && (cu.t & ~63u) == pv_win; };
    fetch_pages(ci);
    MLC_PROBE(2);

    // matrix-pipe mode: lane coordinates of the 16x16 MFMA layouts, the q operand (B of S^T =
    // K.q^T: column n16 = head of the group, dims 8*g4 .. +7 of every 32-dim step) as the sum of
    // two fp16 numbers, and the LDS offsets of this lane's K and V^T operand reads inside a tile.
    // K rows are stored with their 16-byte chunks permuted by chunk ^ ((row / (128 / D)) % CPR), V
    // rows by chunk ^ 2*((row % 4) / (128 / D)) (see issue_tile): the 16 lanes that the hardware
    // serves together then hit 16 different bank groups.
    const int n16 = lane % 16, g4 = lane / 16;
    typedef _Float16 sd_half4 __attribute__((ext_vector_type(4)));
    typedef float sd_f4 __attribute__((ext_vector_type(4)));
    half8_t qh[MF ? KST : 1], ql[MF ? KST : 1];
    uint32_t mf_k_off[MF ? KST : 1], mf_v_off[MF ? DB : 1];
    if constexpr (MF) {
        constexpr int RPB = 128 / D;   // rows per 256 bytes
        const uint32_t krow = (uint32_t)(wave * TW + n16 % TW);
#pragma unroll
        for (int ks = 0; ks < KST; ++ks)
            mf_k_off[ks] = krow * (D * 2) + ((((uint32_t)(ks * 4 + g4)) ^ ((krow / RPB) % CPR)) * 16);
        const uint32_t e4 = (uint32_t)n16 / 4, q4 = (uint32_t)n16 % 4;
        const uint32_t vrow = (uint32_t)(wave * TW + (4 * g4 + (int)e4) % TW);
        const uint32_t fv = 2u * ((vrow % 4u) / RPB);
#pragma unroll
        for (int b = 0; b < DB; ++b)
            mf_v_off[b] = TILE_BYTES + vrow * (D * 2) + (((uint32_t)(2 * b) + q4 / 2) ^ fv) * 16 + (q4 % 2) * 8;
    }
    // q of this wave's heads, dims c*8 .. c*8+7, scaled
    float qv[HPW][8];
    // matrix-pipe mode: q is fetched as it lies in memory (q_raw) and split into the two fp16
    // operands when the consume side reaches the pair.  With two stages the issue side is exactly
    // one tile ahead, so it fetches the next pair's q together with that pair's first tile and the
    // pair's end finds it in registers.
    constexpr bool Q_AHEAD = MF && NBUF == 2;
    float4 q_raw[MF ? 2 * KST : 1];
    auto fetch_q = [&](const Cursor& cu) {
        // (columns past the group: the loads are clamped onto the last head and the factor below is
        // zero; a select on the loaded value would put the load under a branch, and the wait for it
        // there would be for every load in flight)
        const int hcol = n16 < G ? n16 : G - 1;
        const float* qb = a.q + ((size_t)cu.r * a.num_heads + cu.kvh * G + hcol) * D + 8 * g4;
#pragma unroll
        for (int ks = 0; ks < (MF ? KST : 0); ++ks) {
            q_raw[2 * ks] = *reinterpret_cast<const float4*>(qb + 32 * ks);
            q_raw[2 * ks + 1] = *reinterpret_cast<const float4*>(qb + 32 * ks + 4);
        }
    };
    auto split_q = [&]() {
        const float q_factor = n16 < G ? a.scale_log2e : 0.f;
#pragma unroll
        for (int ks = 0; ks < (MF ? KST : 0); ++ks) {
            const float4 x0 = q_raw[2 * ks], x1 = q_raw[2 * ks + 1];
            const float x[8] = {x0.x, x0.y, x0.z, x0.w, x1.x, x1.y, x1.z, x1.w};
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const float v = x[i] * q_factor;
                const _Float16 hi = (_Float16)v;
                qh[ks][i] = hi;
                ql[ks][i] = (_Float16)(v - (float)hi);
            }
        }
    };
    auto load_q = [&](const Cursor& cu) {
        if constexpr (MF) {
            fetch_q(cu);
            split_q();
            return;
        }
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
    const uint32_t stages_lds = sd_lds_addr(stages);
    auto issue_tile = [&](const Cursor& cu, uint32_t slot) {
        uint32_t page_id = (uint32_t)__builtin_amdgcn_readlane((int)pv, (int)(cu.t & 63u));
        if (a.capacity_pages && page_id >= a.capacity_pages) page_id = a.capacity_pages - 1u;
        const uint32_t tile_start = cu.t * TT;
        const uint32_t slot0 = tile_start % a.page_size;
        const uint32_t last = cu.lim - 1u - tile_start;
        const size_t row0 = ((size_t)page_id * a.page_size + slot0) * row_u4 + cu.kvh * CPR + c;
        // (matrix-pipe mode: every wave loads exactly the rows it consumes, two loads of K and two
        // of V, so that no wave ever waits for another one's loads)
        constexpr int PARTS = (NW == 1 || MF) ? 2 : 1;
        constexpr int JN = MF ? 2 : (NW == 4) ? 4 : 8;
#pragma unroll
        for (int p = 0; p < PARTS; ++p) {
            const int tensor = (NW == 1 || MF) ? p : (NW == 2 ? hg : hg / 2);
            const int j0 = MF ? 2 * hg : (NW == 4) ? (hg % 2) * 4 : 0;
            const uint4* base = (tensor ? a.v_pages : a.k_pages) + row0;
            const uint32_t dst = (uint32_t)__builtin_amdgcn_readfirstlane((int)(stages_lds + slot * STAGE_BYTES + tensor * TILE_BYTES));
#pragma unroll
            for (int jj = 0; jj < JN; ++jj) {
                const int j = j0 + jj;
                uint32_t tr = (uint32_t)((j ^ gsw) * RPI + r_l);
                const uint4* src = base;
                if constexpr (MF) {
                    // rows in order, chunks permuted (see above): LDS chunk c of row tr holds the
                    // row's chunk c ^ f(tr)
                    constexpr int RPB = 128 / D;
                    tr = (uint32_t)(j * RPI + r_l);
                    const uint32_t f = tensor ? 2u * ((tr % 4u) / RPB) : (tr / RPB) % CPR;
                    src = base - c + ((uint32_t)c ^ f);
                }
                tr = tr < last ? tr : last;
#ifndef MLC_NO_LOADS
                sd_g2lds16<MF>(src + (size_t)tr * row_u4, dst + j * 1024);
#else
                asm volatile("" ::"v"(src + (size_t)tr * row_u4), "s"(dst + j * 1024));
#endif
            }
        }
    };
    // waits until this wave's loads of the oldest tile in flight have landed, given how many
    // tiles were issued after it (loads return in order; other loads issued in between only
    // make the wait longer, never shorter)
    auto wait_tile = [&](uint32_t younger) {
        if (younger == 0) sd_wait_vmcnt<0>();
        else if (younger == 1) sd_wait_vmcnt<LPW>();
        else if (younger == 2) sd_wait_vmcnt<(NBUF > 2 ? 2 * LPW : 0)>();
        else sd_wait_vmcnt<(NBUF > 3 ? 3 * LPW : 0)>();
    };

    float acc[HPW][8];
    float m_ref[HPW], l_sum[HPW];
    // matrix-pipe mode: O^T of this wave's tokens (lane: head n16, dims 16*b + 4*g4 .. +3), the
    // reference of column n16 (the same in its four lanes) and this lane's part of the row sum
    sd_f4 mf_o[MF ? DB : 1];
    float mf_m = kNegBig, mf_l = 0.f;
    auto reset_state = [&]() {
        if constexpr (MF) {
            mf_m = kNegBig;
            mf_l = 0.f;
#pragma unroll
            for (int b = 0; b < DB; ++b) mf_o[b] = sd_f4{0.f, 0.f, 0.f, 0.f};
            return;
        }
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
    auto consume_tile = [&](uint32_t slot, uint32_t t, uint32_t lim) {
        const unsigned char* cur = stages + (size_t)slot * STAGE_BYTES;
        const uint32_t tile_start = t * TT;
        if constexpr (MF) {
            typedef __fp16 sd_fp16x4 __attribute__((vector_size(8)));
            half8_t ka[KST];
#pragma unroll
            for (int ks = 0; ks < KST; ++ks) ka[ks] = *reinterpret_cast<const half8_t*>(cur + mf_k_off[ks]);
            sd_half4 va[DB];
#pragma unroll
            for (int b = 0; b < DB; ++b)
                va[b] = __builtin_bit_cast(sd_half4, __builtin_amdgcn_ds_read_tr16_b64_v4f16(
                    (sd_fp16x4 __attribute__((address_space(3)))*)(cur + mf_v_off[b])));
            sd_f4 s4 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int ks = 0; ks < KST; ++ks) {
                s4 = __builtin_amdgcn_mfma_f32_16x16x32_f16(ka[ks], qh[ks], s4, 0, 0, 0);
                s4 = __builtin_amdgcn_mfma_f32_16x16x32_f16(ka[ks], ql[ks], s4, 0, 0, 0);
            }
            // lane (n16, g4) holds the scores of head n16 for the wave's keys 4*g4 .. 4*g4+3
            const uint32_t key0 = tile_start + (uint32_t)(wave * TW + 4 * g4);
            float mloc = -INFINITY;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const bool visible = (4 * g4 + i < TW) && key0 + (uint32_t)i < lim;
                s4[i] = visible ? s4[i] : -INFINITY;
                mloc = max_nn(mloc, s4[i]);
            }
            if (__any(mloc > mf_m + kLazyTau)) {
                float mcol = max_nn(mloc, __shfl_xor(mloc, 16));
                mcol = max_nn(mcol, __shfl_xor(mcol, 32));
                const float m_new = max_nn(mf_m, mcol);
                const float alpha = fast_exp2(mf_m - m_new);
                mf_m = m_new;
                mf_l *= alpha;
#pragma unroll
                for (int b = 0; b < DB; ++b) mf_o[b] *= alpha;
            }
            sd_half4 pb;
            if constexpr (MF_SPLIT_P) {
                // the weight enters as the sum of two fp16 numbers, like q: the products with the
                // fp16 V are exact, only the order of the fp32 additions differs from the vector pipe
                sd_half4 pl;
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const float pf = fast_exp2(s4[i] - mf_m);
                    mf_l += pf;
                    pb[i] = (_Float16)pf;
                    pl[i] = (_Float16)(pf - (float)pb[i]);
                }
                if constexpr (TW == 8) {
                    // A wave has 8 tokens of the tile, the product sums over 16: the upper 8 places
                    // (lanes 32 .. 63, whose own weights are masked to zero and whose V^T operand
                    // repeats the rows of the lower ones, see mf_v_off) take the low parts of the 8
                    // weights, so that hi and lo go through one instruction per V block.
                    const uint2 lw = __builtin_bit_cast(uint2, pl);
                    const auto s0 = __builtin_amdgcn_permlane32_swap(lw.x, lw.x, false, false);
                    const auto s1 = __builtin_amdgcn_permlane32_swap(lw.y, lw.y, false, false);
                    const sd_half4 up = __builtin_bit_cast(sd_half4, make_uint2(s0[0], s1[0]));
                    const sd_half4 pboth = g4 < 2 ? pb : up;
#pragma unroll
                    for (int b = 0; b < DB; ++b) mf_o[b] = __builtin_amdgcn_mfma_f32_16x16x16f16(va[b], pboth, mf_o[b], 0, 0, 0);
                    return;
                }
#pragma unroll
                for (int b = 0; b < DB; ++b) {
                    mf_o[b] = __builtin_amdgcn_mfma_f32_16x16x16f16(va[b], pb, mf_o[b], 0, 0, 0);
                    mf_o[b] = __builtin_amdgcn_mfma_f32_16x16x16f16(va[b], pl, mf_o[b], 0, 0, 0);
                }
                return;
            }
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                pb[i] = (_Float16)fast_exp2(s4[i] - mf_m);
                mf_l += (float)pb[i];
            }
#pragma unroll
            for (int b = 0; b < DB; ++b) mf_o[b] = __builtin_amdgcn_mfma_f32_16x16x16f16(va[b], pb, mf_o[b], 0, 0, 0);
            return;
        }
        const uint4* kl = reinterpret_cast<const uint4*>(cur) + lane;
        const uint4* vl = kl + TILE_BYTES / 16;
        // All sixteen LDS reads of the tile are requested before anything is computed, K first
        // (64 registers): left to the compiler the reads sit next to their uses, two at a time,
        // and every pair exposes the LDS latency to a wave that has one other wave to hide behind.
        // The empty statements keep the reads from being moved back down.
        uint4 kreg[8], vreg[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) kreg[j] = kl[j * 64];
        asm volatile("" ::: "memory");
#pragma unroll
        for (int j = 0; j < 8; ++j) vreg[j] = vl[j * 64];
        asm volatile("" ::: "memory");
        float part[HPW][8];
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const uint4 kq = kreg[j];
            const half8_t kh = __builtin_bit_cast(half8_t, kq);
#pragma unroll
            for (int h = 0; h < HPW; ++h) {
                float s = 0.f;
#pragma unroll
                for (int i = 0; i < 8; ++i) s = fmaf(qv[h][i], (float)kh[i], s);  // v_fma_mix_f32 throughout
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
                const uint4 va4 = vreg[2 * k];
                const uint4 vb4 = vreg[2 * k + 1];
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
                const uint4 vq = vreg[j];
                const half8_t vh = __builtin_bit_cast(half8_t, vq);
#pragma unroll
                for (int h = 0; h < HPW; ++h)
#pragma unroll
                    for (int i = 0; i < 8; ++i) acc[h][i] = fmaf(pj[h][j], (float)vh[i], acc[h][i]);
            }
        }
    };

    // ---- end of a pair's tiles inside this range.  The rows of lanes are summed; a pair that lay
    // inside the range is written to O at once.  A pair cut by range boundaries is shared by
    // consecutive workgroups, and the one that holds its last tile (the highest-numbered sharer)
    // sums it up: every other sharer leaves its (o, m, l) in its own slot of the partial buffer --
    // a workgroup has one slot, because only the pair that goes on behind its range is published
    // -- and is done.  A partial is a set of 64-bit words {value, tag}: the tag is this launch's,
    // never seen in the buffer before, so every word says by itself whether it has been written
    // in this launch.  Nothing else is needed: no order among the stores, no acknowledgement, no
    // arrival counter.  The stores are relaxed device-scope atomics (written through to memory),
    // the summing workgroup reads with relaxed device-scope loads until every word of every
    // sharer's partial carries the tag, then folds them in workgroup order and its own part
    // last, so the result does not depend on timing (runs are bit-identical).  It waits only for
    // lower-numbered workgroups, which the hardware starts no later than itself; the wait is
    // bounded all the same (spin_limit rounds, then the fault word is set and the pass fails on
    // the host).  Nothing about a partial touches memory before the range has ended: a first
    // pair that ends in mid-range waits in registers, so the stream never stops for it.
    struct PairOut {
        uint32_t w_lo;   // first sharer
        float* orow;
    };
    // Brings the rows of lanes (the tokens a lane row owns) onto one reference and sums over
    // them by reduce-scatter across the lane bits above the chunk index: every step halves the
    // values a lane keeps (v_permlane32_swap / v_permlane16_swap hand the other half to the
    // partner, the last step of head_dim 64 goes over lane ^ 8).  Lane (r, c) ends up with
    // dims c*8 + r*HPK + kk (kk < HPK) of every head, summed over all tokens of the wave.
    auto reduce_rows = [&](float (&o_un)[OPL], float (&m_all)[HPW], float (&l_all)[HPW], bool last_of_range) {
        if constexpr (MF) {
            // every wave leaves its (o, m, l) of all heads of the group in LDS; wave hg then
            // combines the four for its own heads, in the lane layout the code below expects
            // (lane (r, c): dims c*8 + r*HPK + kk).  The sums run over the waves in a fixed
            // order in every lane, so l does not depend on the lane it is read from.
            float lt = mf_l + __shfl_xor(mf_l, 16);
            lt += __shfl_xor(lt, 32);
            if (n16 < G) {
#pragma unroll
                for (int b = 0; b < DB; ++b)
                    *reinterpret_cast<sd_f4*>(&comb_o[((size_t)wave * G + n16) * D + b * 16 + 4 * g4]) = mf_o[b];
                if (g4 == 0) {
                    comb_ml[wave * G + n16] = mf_m;
                    comb_ml[NW * G + wave * G + n16] = lt;
                }
            }
            sd_barrier();
#pragma unroll
            for (int h = 0; h < HPW; ++h) {
                const int hh = hg * HPW + h;
                float mw[NW], m = kNegBig;
#pragma unroll
                for (int w2 = 0; w2 < NW; ++w2) {
                    mw[w2] = comb_ml[w2 * G + hh];
                    m = max_nn(m, mw[w2]);
                }
                m_all[h] = m;
                float l = 0.f, o[HPK];
#pragma unroll
                for (int kk = 0; kk < HPK; ++kk) o[kk] = 0.f;
#pragma unroll
                for (int w2 = 0; w2 < NW; ++w2) {
                    const float wgt = fast_exp2(mw[w2] - m);
                    l += comb_ml[NW * G + w2 * G + hh] * wgt;
#pragma unroll
                    for (int kk = 0; kk < HPK; ++kk)
                        o[kk] += comb_o[((size_t)w2 * G + hh) * D + c * 8 + r_l * HPK + kk] * wgt;
                }
                l_all[h] = l;
#pragma unroll
                for (int kk = 0; kk < HPK; ++kk) o_un[h * HPK + kk] = o[kk];
            }
            // the waves run on their own between pairs: nobody writes the next pair's figures before
            // everybody has read these (at the range's end nobody writes them again)
            if (!last_of_range) sd_barrier();
            return;
        }
#pragma unroll
        for (int h = 0; h < HPW; ++h) {
            float m = m_ref[h];
#pragma unroll
            for (int off = CPR; off < 64; off <<= 1) m = max_nn(m, __shfl_xor(m, off));
            m_all[h] = m;
            const float wgt = fast_exp2(m_ref[h] - m);
            // with CPR == 16 every token's weight sits in two lanes (c and c^8): count it once
            // (one lane's sum for the whole wave: with the product fused into the first addition the
            // lanes' sums can differ in the last bit, and the partial's l must not depend on the
            // lane it is read from)
            l_all[h] = __builtin_bit_cast(float, __builtin_amdgcn_readfirstlane(__builtin_bit_cast(
                int, wave_sum((CPR == 16 && (c & 8)) ? 0.f : l_sum[h] * wgt))));
            float v4[4], v2[2];
#pragma unroll
            for (int i = 0; i < 4; ++i) {  // lane bit 5: keep dims i (lower half) or i + 4 (upper half)
                const auto sw = __builtin_amdgcn_permlane32_swap(__float_as_uint(acc[h][i] * wgt),
                                                                 __float_as_uint(acc[h][i + 4] * wgt), false, false);
                v4[i] = __uint_as_float(sw[0]) + __uint_as_float(sw[1]);
            }
#pragma unroll
            for (int i = 0; i < 2; ++i) {  // lane bit 4
                const auto sw = __builtin_amdgcn_permlane16_swap(__float_as_uint(v4[i]), __float_as_uint(v4[i + 2]),
                                                                 false, false);
                v2[i] = __uint_as_float(sw[0]) + __uint_as_float(sw[1]);
            }
            if constexpr (CPR == 8) {      // lane bit 3 (head_dim 64: eight rows of lanes)
                const bool up = (lane & 8) != 0;
                const float send = up ? v2[0] : v2[1];
                const float keep = up ? v2[1] : v2[0];
                o_un[h] = keep + dpp_f<kDppRowRor8>(send);
            } else {
                o_un[h * 2] = v2[0];
                o_un[h * 2 + 1] = v2[1];
            }
        }
    };
    // element (head k / HPK, dim) of output register k of this lane
    const int dim0 = c * 8 + r_l * HPK;
    // workgroup that holds unit u
    const uint32_t thr = trem * (tq + 1u);
    auto wg_of_unit = [&](uint32_t u) {
        return (uint32_t)__builtin_amdgcn_readfirstlane(u < thr ? u / (tq + 1u) : trem + (u - thr) / tq);
    };
    auto out_row = [&](const Cursor& cu) {
        return a.o + ((size_t)cu.r * a.num_heads + cu.kvh * G + hg * HPW) * D;
    };
    // who shares the pair whose first tile is ps
    auto pair_out = [&](const Cursor& cu, uint32_t ps) {
        PairOut po;
        // the pair's tiles are consecutive units; the PC units in front of them stand for the
        // end of the pair before
        po.w_lo = wg_of_unit(ps + PC * (Hkv * req_nzb(cu.r) + cu.kvh));
        po.orow = out_row(cu);
        return po;
    };
    auto store_direct = [&](float* orow, const float (&o_un)[OPL], const float (&l_all)[HPW]) {
        float val[OPL];
#pragma unroll
        for (int k = 0; k < OPL; ++k) {
            const float l = l_all[k / HPK];
            const float inv = l > 0.f ? 1.0f / l : 0.f;
            val[k] = o_un[k] * inv;
            orow[(k / HPK) * D + dim0 + (k % HPK)] = val[k];
        }
        if constexpr (SPLIT) {
            // A lane holds dims c*8 + r_l*HPK + kk of a head: a block of 32 columns is four values
            // of c, every r_l.  Its largest magnitude: over lane bits 0, 1 (c % 4) and the bits of r_l.
            // (the request and the head come from the row's address: nothing more to carry through
            // the stream for them)
            const uint32_t cols = a.num_heads * D;
            const uint32_t row_head = (uint32_t)__builtin_amdgcn_readfirstlane((int)((orow - a.o) / D));
            const uint32_t req = (uint32_t)__builtin_amdgcn_readfirstlane((int)(row_head / a.num_heads));
            const uint32_t head0 = row_head - req * a.num_heads;
            const uint32_t t32 = req / 32, n32 = req % 32;
#pragma unroll
            for (int h = 0; h < HPW; ++h) {
                float amax = 0.f;
#pragma unroll
                for (int kk = 0; kk < HPK; ++kk) amax = fmaxf(amax, fabsf(val[h * HPK + kk]));
                amax = fmaxf(amax, dpp_f<kDppQuadXor1>(amax));
                amax = fmaxf(amax, dpp_f<kDppQuadXor2>(amax));
                if constexpr (CPR == 8) amax = fmaxf(amax, dpp_f<kDppRowRor8>(amax));
                {
                    const auto sw = __builtin_amdgcn_permlane16_swap(__float_as_uint(amax), __float_as_uint(amax), false, false);
                    amax = fmaxf(__uint_as_float(sw[0]), __uint_as_float(sw[1]));
                }
                {
                    const auto sw = __builtin_amdgcn_permlane32_swap(__float_as_uint(amax), __float_as_uint(amax), false, false);
                    amax = fmaxf(__uint_as_float(sw[0]), __uint_as_float(sw[1]));
                }
                int e = 0;
                if (amax > 0.f && amax < INFINITY) (void)frexpf(amax, &e);   // q4_split_activations_kernel's scale
                int se = 14 - e;
                se = se > 100 ? 100 : (se < -100 ? -100 : se);
                const uint32_t col = (head0 + (uint32_t)h) * D + (uint32_t)dim0;   // this lane's first column
                const size_t base = ((size_t)t32 * (cols / 16) + col / 16) * 2;
                const uint32_t fl = ((col % 16) / 8) * 32 + n32;
                _Float16* f_hi = a.split_frag + ((base + 0) * 64 + fl) * 8 + col % 8;
                _Float16* f_lo = a.split_frag + ((base + 1) * 64 + fl) * 8 + col % 8;
                _Float16 hi[HPK], lo[HPK];
#pragma unroll
                for (int kk = 0; kk < HPK; ++kk) {
                    const float tv = __builtin_ldexpf(val[h * HPK + kk], se);
                    hi[kk] = (_Float16)tv;
                    lo[kk] = (_Float16)(tv - (float)hi[kk]);
                }
                if constexpr (HPK == 2) {   // (dim0 is even: the two are one aligned word)
                    typedef _Float16 sd_half2 __attribute__((ext_vector_type(2)));
                    *reinterpret_cast<sd_half2*>(f_hi) = sd_half2{hi[0], hi[1]};
                    *reinterpret_cast<sd_half2*>(f_lo) = sd_half2{lo[0], lo[1]};
                } else {
                    f_hi[0] = hi[0];
                    f_lo[0] = lo[0];
                }
                if (c % 4 == 0 && r_l == 0)
                    a.split_exp[((size_t)t32 * (cols / 32) + col / 32) * 32 + ((n32 % 8) / 4) * 16 + (n32 / 8) * 4 + n32 % 4] =
                        (int8_t)(-se);
            }
        }
    };
    // A wave's partial: PW tagged words per lane, word k of lane i at [k][i].  Words 0 .. OPL-1
    // are the lane's un-normalised outputs, word OPL carries m of head i in lane i < HPW and l of
    // head i - HPW in lanes HPW .. 2*HPW-1 (m in log2 units).
    constexpr int PW = OPL + 1;
    const uint32_t tag_sum = a.tag + tag_add;
    const uint32_t tag = tag_sum ? tag_sum : 0x9E3779B9u;   // (zero is what untouched memory holds)
    auto partial_of = [&](uint32_t wg) { return a.part + ((size_t)(wg * NW + (uint32_t)hg) * PW) * 64 + lane; };
    auto publish = [&](const float (&o_un)[OPL], const float (&m_all)[HPW], const float (&l_all)[HPW]) {
        uint64_t* dst = partial_of(w);
        const uint64_t hi = (uint64_t)tag << 32;
#pragma unroll
        for (int k = 0; k < OPL; ++k) st_tagged(dst + k * 64, hi | __float_as_uint(o_un[k]));
        float x = 0.f;
#pragma unroll
        for (int h = 0; h < HPW; ++h) x = lane == h ? m_all[h] : lane == HPW + h ? l_all[h] : x;
        st_tagged(dst + OPL * 64, hi | __float_as_uint(x));
    };
    // Sums up the pair this workgroup ends: the partials of workgroups po.w_lo .. w-1, eight at a
    // time, then this workgroup's own part.
    constexpr int MUNR = 8;
    auto merge_pair = [&](const PairOut& po, const float (&own_o)[OPL], const float (&own_m)[HPW],
                          const float (&own_l)[HPW]) {
        float acc_o[OPL], m_run[HPW], l_run[HPW];
#pragma unroll
        for (int k = 0; k < OPL; ++k) acc_o[k] = 0.f;
#pragma unroll
        for (int h = 0; h < HPW; ++h) {
            m_run[h] = kNegBig;
            l_run[h] = 0.f;
        }
        auto fold = [&](const float (&o)[OPL], const float (&m)[HPW], const float (&l)[HPW]) {
#pragma unroll
            for (int h = 0; h < HPW; ++h) {
                const float m_new = max_nn(m_run[h], m[h]);
                const float keep = fast_exp2(m_run[h] - m_new);
                const float wgt = fast_exp2(m[h] - m_new);
                l_run[h] = l_run[h] * keep + l[h] * wgt;
                m_run[h] = m_new;
#pragma unroll
                for (int kk = 0; kk < HPK; ++kk) acc_o[h * HPK + kk] = acc_o[h * HPK + kk] * keep + o[h * HPK + kk] * wgt;
            }
        };
        const uint32_t n_others = w - po.w_lo;
        uint32_t spins = 0;
        for (uint32_t s0 = 0; s0 < n_others; s0 += MUNR) {
            const uint32_t cnt = min((uint32_t)MUNR, n_others - s0);
            uint64_t wd[MUNR][PW];
            for (;;) {
                bool ok = true;
#pragma unroll
                for (int u = 0; u < MUNR; ++u) {
                    if ((uint32_t)u < cnt) {
                        const uint64_t* src = partial_of(po.w_lo + s0 + (uint32_t)u);
#pragma unroll
                        for (int k = 0; k < PW; ++k) wd[u][k] = ld_tagged(src + k * 64);
                    }
                }
#pragma unroll
                for (int u = 0; u < MUNR; ++u) {
                    if ((uint32_t)u < cnt) {
#pragma unroll
                        for (int k = 0; k < PW; ++k) ok = ok && (uint32_t)(wd[u][k] >> 32) == tag;
                    }
                }
                if (__all(ok)) break;
                if (++spins >= a.spin_limit) {   // a sharer never wrote: give up, tell the host
                    if (lane == 0) __hip_atomic_store(a.fault, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
                    break;
                }
            }
#pragma unroll
            for (int u = 0; u < MUNR; ++u) {
                if ((uint32_t)u < cnt) {
                    float o[OPL], m[HPW], l[HPW];
#pragma unroll
                    for (int k = 0; k < OPL; ++k) o[k] = __uint_as_float((uint32_t)wd[u][k]);
                    const int x = (int)(uint32_t)wd[u][OPL];
#pragma unroll
                    for (int h = 0; h < HPW; ++h) {
                        m[h] = __int_as_float(__builtin_amdgcn_readlane(x, h));
                        l[h] = __int_as_float(__builtin_amdgcn_readlane(x, HPW + h));
                    }
                    fold(o, m, l);
                }
            }
        }
        fold(own_o, own_m, own_l);
        store_direct(po.orow, acc_o, l_run);
    };

    // ---- the stream: the first NBUF tiles of the range go out together, then one tile per step
    // into the stage the step before has left
    // ---- the step's KV write: this workgroup owns the last tile of every pair that ends in
    // its range, so it writes those pairs' slices of the new rows before it loads the tiles
    // that hold them.  A new row is its request's newest position, so it lies in the pair's
    // last tile: where the range starts with another tile, that tile is requested first, the
    // rows are written behind it (their page ids and slots are a memory round trip of their
    // own), and the workgroup makes sure of the stores (every wave's memory counter at zero,
    // then a barrier) before the second tile goes out; where the range starts with a pair's
    // last tile, it writes and makes sure before it loads anything.  2 * CPR lanes move one
    // pair's K and V slice.
    bool kv_unsettled = false;
    auto write_new_rows = [&]() {
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
    };

    const bool kv_first = a.new_k != nullptr && cc.t + 1u == cc.tiles;
    if (kv_first) {
        g1 = tiles_before(u1);
        n = g1 - g0;
        write_new_rows();
        sd_wait_vmcnt<0>();  // the rows have left this wave before any wave of the workgroup loads them
        sd_barrier();
    }
    uint32_t issued = 1;
    issue_tile(ci, 0);
    load_q(cc);   // (behind the tile's request: q is a memory round trip of its own)
    if (pv_win == 0) prefetch_next_pages(ci.r);
    if (!kv_first) {
        g1 = tiles_before(u1);
        n = g1 - g0;
    }
    if (a.new_k != nullptr && !kv_first) {
        write_new_rows();
        kv_unsettled = true;
    }
    uint32_t seg_first = g0;  // first tile consumed for the pair under cc
    bool drain = false;       // stores are in flight: they do not complete in order with loads
    uint32_t slot = 0;        // stage of tile k
    bool kept = false;        // the range's first pair, which this workgroup sums up, waits in registers
                              // for the end of the range
    PairOut kept_po{};
    float kept_o[OPL], kept_m[HPW], kept_l[HPW];
    for (uint32_t k = 0; k < n; ++k) {
        // this wave's loads of tile k have landed ...
        if (k < 6) MLC_PROBE_TILE(8 + 3 * k);
        if (drain) sd_wait_vmcnt<0>(); else wait_tile(issued - k - 1u);
        drain = false;
        if (kv_unsettled) {  // first step only: nothing but the first tile was behind the stores, the
                             // counter has just been at zero in every wave that comes here
            kv_unsettled = false;
            sd_barrier();
        }
        // ... and everyone's; everyone has left tile k-1, whose stage is free (matrix-pipe mode: a
        // wave loads, reads and overwrites only its own rows of a stage, no barrier)
        if constexpr (!MF) sd_barrier();
        if (k < 6) MLC_PROBE_TILE(9 + 3 * k);
        if (k == 0) MLC_PROBE(3);
        // one tile went out up front; from the first step on the stream runs NBUF - 1 tiles ahead
        // (all stages requested at once would make every workgroup wait for the whole burst)
        while (issued < n && issued < k + (uint32_t)NBUF) {
            advance(ci);
            // (order: whatever the compiler waits for -- the page ids it takes over, registers of q it
            // believes busy -- comes while nothing is in flight; the next request's ids are asked for
            // last and are not waited for before the step into that request)
            const bool new_pages = !pages_ready(ci);
            if (new_pages) fetch_pages(ci);
            if constexpr (Q_AHEAD) {
                if (ci.t == 0) fetch_q(ci);   // first tile of the next pair: its q with it
            }
            issue_tile(ci, issued % (uint32_t)NBUF);
            ++issued;
            if (new_pages && pv_win == 0) prefetch_next_pages(ci.r);
        }
#ifndef MLC_NO_COMPUTE
        consume_tile(slot, cc.t, cc.lim);
#endif
        const bool pair_done = cc.t + 1u == cc.tiles;
        const bool range_done = k + 1 == n;
        if (k < 6) MLC_PROBE_TILE(10 + 3 * k);
        if (range_done) MLC_PROBE(4);
        if (pair_done || range_done) {
            float o_un[OPL], m_all[HPW], l_all[HPW];
            reduce_rows(o_un, m_all, l_all, range_done);
            const uint32_t ps = req_start(cc.r) * Hkv + cc.kvh * cc.tiles;  // pair's first tile
            const bool starts_here = seg_first == ps;                 // no workgroup before this one has tiles of the pair
            const bool ends_here = g0 + k + 1u == ps + cc.tiles;      // ... none behind it
            bool cur = false;  // this pair is summed up by this workgroup, now
            PairOut cur_po{};
            if (starts_here && ends_here) {
                store_direct(out_row(cc), o_un, l_all);
                drain = true;
            } else if (ends_here) {
                if (range_done) {
                    cur = true;
                    cur_po = pair_out(cc, ps);
                } else {
                    kept = true;
                    kept_po = pair_out(cc, ps);
#pragma unroll
                    for (int i = 0; i < OPL; ++i) kept_o[i] = o_un[i];
#pragma unroll
                    for (int h = 0; h < HPW; ++h) {
                        kept_m[h] = m_all[h];
                        kept_l[h] = l_all[h];
                    }
                }
            } else {
#ifndef MLC_NO_TAIL
                // (the pair goes on in the next workgroup: the range ends here)
                if (!(a.test_flags & 1u)) publish(o_un, m_all, l_all);
#endif
                MLC_PROBE(26);
            }
#ifndef MLC_NO_TAIL
            if (range_done && (kept || cur)) {
                MLC_PROBE(28);
                if (kept) merge_pair(kept_po, kept_o, kept_m, kept_l);
                else merge_pair(cur_po, o_un, m_all, l_all);
            }
#endif
            reset_state();
            seg_first = g0 + k + 1u;
        }
        if (!range_done) {
            advance(cc);
            if (pair_done) {
                if constexpr (Q_AHEAD) split_q();
                else load_q(cc);
            }
        }
        slot = slot + 1u == (uint32_t)NBUF ? 0u : slot + 1u;
    }
    MLC_PROBE(5);
#ifdef MLC_STREAM_PROBE
    if (threadIdx.x == 0) {
        (a.part + kStreamProbeWord)[blockIdx.x * 32 + 6] = n;
        const uint64_t hw = __builtin_amdgcn_s_getreg((31 << 11) | 4), xcc = __builtin_amdgcn_s_getreg((31 << 11) | 20);
        (a.part + kStreamProbeWord)[blockIdx.x * 32 + 7] = hw | (xcc << 32);
    }
#endif
}

}  // namespace mlc_hip
