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
// One workgroup = 32 consecutive chunk rows x the G query heads of one KV head
// (one wave per head when G >= 4), so a K/V tile is fetched from HBM once for the
// whole GQA group.  Per 32-key tile:
//   S^T = K . Q^T    A = K rows (32 keys x 16 dims per step) read from LDS,
//                    B = Q^T, resident in registers.  In the 32x32 accumulator layout
//                    lane l owns query row l%32, so every softmax statistic is
//                    lane-local (plus one exchange with lane l^32).
//   O^T += V^T . P^T A = V^T rows (32 dims x 16 keys per step) read from LDS,
//                    B = P^T, which is exactly what lane l already holds of S^T (keys
//                    of the 16-key group in the order 0-3, 8-11 | 4-7, 12-15); V^T is
//                    stored in LDS with that key order so no cross-lane traffic is needed.
// K tiles go global -> LDS directly (16-byte chunks XOR-swizzled by row to spread
// banks); V tiles go through registers and are written transposed.  Both are double
// buffered: the loads of tile t+1 are in flight while tile t is multiplied.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

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
    float scale_log2e;
};

typedef _Float16 pf_half8 __attribute__((ext_vector_type(8)));
typedef float pf_float16 __attribute__((ext_vector_type(16)));

static constexpr int kPfKeys = 32;  // keys per tile
static constexpr int kPfRows = 32;  // chunk rows per wave

__device__ __forceinline__ void pf_g2lds16(const void* g, void* lds_base) {
    __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)g,
                                     (__attribute__((address_space(3))) void*)lds_base, 16, 0, 0);
}

// D: head_dim (64 or 128); G: query heads per KV head; NWV: waves per workgroup (multiple of G
// or divisor arrangement: wave w handles head w % G and row block w / G).
template <int D, int G, int NWV>
__global__ __launch_bounds__(64 * NWV) void paged_prefill_mfma_kernel(const PrefillArgs a) {
    static_assert(D == 64 || D == 128, "head_dim 64 or 128");
    static_assert(NWV % G == 0, "waves cover whole GQA groups");
    constexpr int NT = 64 * NWV;
    constexpr int CPR = D / 8;            // 16-byte chunks per K/V row of one head
    constexpr int KSTEPS = D / 16;        // MFMA steps over head_dim for S^T
    constexpr int MB = D / 32;            // 32-row blocks of O^T
    constexpr int RB = NWV / G;           // row blocks per workgroup
    constexpr int K_TILE = kPfKeys * D * 2;          // bytes
    constexpr int VS = kPfKeys * 2 + 16;             // V^T row stride in bytes (padded)
    constexpr int V_TILE = D * VS;
    constexpr int CHUNKS = kPfKeys * CPR;            // 16-byte chunks per tile and tensor
    constexpr int LPT = (CHUNKS + NT - 1) / NT;      // chunks per thread
    static_assert(CHUNKS % NT == 0 || CHUNKS < NT, "tile chunks divide over the workgroup");

    __shared__ __attribute__((aligned(16))) unsigned char k_lds0[K_TILE];
    __shared__ __attribute__((aligned(16))) unsigned char k_lds1[K_TILE];
    __shared__ __attribute__((aligned(16))) unsigned char v_lds0[V_TILE];
    __shared__ __attribute__((aligned(16))) unsigned char v_lds1[V_TILE];

    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid / 64);
    const int lane = tid % 64;
    const int l32 = lane % 32;
    const int half = lane / 32;
    const uint32_t req = blockIdx.z;
    const uint32_t kvh = blockIdx.y;
    const uint32_t row0_wg = blockIdx.x * (kPfRows * RB);
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

    const size_t row_elems = (size_t)a.kv_heads * D;  // halves per token row (all KV heads)

    // ---- tile loaders
    // K: chunk position p of the tile (row = p / CPR, slot = p % CPR) is filled with global
    // chunk slot ^ (row % CPR) of key `row`: rows are 256 (or 128) bytes apart in LDS, the XOR
    // spreads the 32 rows an MFMA operand read touches over the banks.
    auto issue_k = [&](uint32_t tile, unsigned char* kbuf) {
        const uint32_t key0 = tile * kPfKeys;
        const uint32_t page_id = a.pt_flat[pt_base + key0 / a.page_size];
        const size_t tok0 = (size_t)page_id * a.page_size + key0 % a.page_size;
        const uint32_t last = wg_limit - 1u - key0;  // last valid row of the tile
#pragma unroll
        for (int i = 0; i < LPT; ++i) {
            const int p = i * NT + tid;
            if (CHUNKS < NT && p >= CHUNKS) break;
            uint32_t row = p / CPR;
            const int slot = p % CPR;
            const int chunk = slot ^ (row % CPR);
            row = row < last ? row : last;  // clamp: in bounds, masked later
            const _Float16* src = a.k_pages + (tok0 + row) * row_elems + (size_t)kvh * D + chunk * 8;
            pf_g2lds16(src, kbuf + (size_t)(i * NT + wave * 64) * 16);
        }
    };
    // V: thread loads chunk c of key k (k fastest over threads) into registers ...
    auto load_v = [&](uint32_t tile, uint4 (&vr)[LPT]) {
        const uint32_t key0 = tile * kPfKeys;
        const uint32_t page_id = a.pt_flat[pt_base + key0 / a.page_size];
        const size_t tok0 = (size_t)page_id * a.page_size + key0 % a.page_size;
        const uint32_t last = wg_limit - 1u - key0;
#pragma unroll
        for (int i = 0; i < LPT; ++i) {
            const int p = i * NT + tid;
            vr[i] = make_uint4(0, 0, 0, 0);
            if (CHUNKS < NT && p >= CHUNKS) break;
            uint32_t k = p % kPfKeys;
            const int c = p / kPfKeys;
            k = k < last ? k : last;
            vr[i] = *reinterpret_cast<const uint4*>(a.v_pages + (tok0 + k) * row_elems +
                                                    (size_t)kvh * D + c * 8);
        }
    };
    // ... and writes it transposed: V^T[dim][pos(k)], keys of each 16-key group ordered
    // 0-3, 8-11, 4-7, 12-15 (the order in which the S^T accumulators hold them).
    auto store_vt = [&](const uint4 (&vr)[LPT], unsigned char* vbuf) {
#pragma unroll
        for (int i = 0; i < LPT; ++i) {
            const int p = i * NT + tid;
            if (CHUNKS < NT && p >= CHUNKS) break;
            const int k = p % kPfKeys;
            const int c = p / kPfKeys;
            const int x = k & 15;
            const int pos = (k & 16) | (x & 3) | ((x & 8) >> 1) | ((x & 4) << 1);
            const _Float16* h8 = reinterpret_cast<const _Float16*>(&vr[i]);
#pragma unroll
            for (int e = 0; e < 8; ++e)
                *reinterpret_cast<_Float16*>(vbuf + (size_t)(c * 8 + e) * VS + pos * 2) = h8[e];
        }
    };

    pf_float16 oacc[MB];
#pragma unroll
    for (int mb = 0; mb < MB; ++mb)
#pragma unroll
        for (int i = 0; i < 16; ++i) oacc[mb][i] = 0.f;
    float m_run = -1.0e30f, l_run = 0.f;

    uint4 vr[LPT];
    if (n_tiles > 0) {
        issue_k(0, k_lds0);
        load_v(0, vr);
        store_vt(vr, v_lds0);
    }
    __builtin_amdgcn_s_waitcnt(0);
    __syncthreads();

    auto compute_tile = [&](uint32_t tile, const unsigned char* kbuf, const unsigned char* vbuf) {
        const uint32_t key0 = tile * kPfKeys;
        // ---- S^T = K . Q^T
        pf_float16 s;
#pragma unroll
        for (int i = 0; i < 16; ++i) s[i] = 0.f;
#pragma unroll
        for (int ks = 0; ks < KSTEPS; ++ks) {
            const int chunk = ks * 2 + half;
            const pf_half8 kf = *reinterpret_cast<const pf_half8*>(
                kbuf + (size_t)l32 * (D * 2) + ((chunk ^ (l32 % CPR)) * 16));
            s = __builtin_amdgcn_mfma_f32_32x32x16_f16(kf, qf[ks], s, 0, 0, 0);
        }
        // ---- mask + online softmax; register i holds key (i/4)*8 + half*4 + i%4 of the tile
        const bool need_mask = (key0 + kPfKeys > wg_limit) || (key0 + kPfKeys - 1u > qs + row0);
        float mx = -INFINITY;
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            float v = s[i] * a.scale_log2e;
            if (need_mask) {
                const uint32_t key = key0 + (uint32_t)((i / 4) * 8 + half * 4 + (i % 4));
                if (key > my_pos || key >= seq_len) v = -INFINITY;
            }
            s[i] = v;
            mx = fmaxf(mx, v);
        }
        mx = fmaxf(mx, __shfl_xor(mx, 32));
        const float m_new = fmaxf(m_run, mx);
        const float alpha = __builtin_amdgcn_exp2f(m_run - m_new);
        m_run = m_new;
        float rs = 0.f;
        pf_half8 pfrag[2];
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            const float p = __builtin_amdgcn_exp2f(s[i] - m_new);
            rs += p;
            pfrag[i / 8][i % 8] = (_Float16)p;
        }
        rs += __shfl_xor(rs, 32);
        l_run = l_run * alpha + rs;
#pragma unroll
        for (int mb = 0; mb < MB; ++mb)
#pragma unroll
            for (int i = 0; i < 16; ++i) oacc[mb][i] *= alpha;
        // ---- O^T += V^T . P^T
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) {
#pragma unroll
            for (int t = 0; t < 2; ++t) {
                const pf_half8 vf = *reinterpret_cast<const pf_half8*>(
                    vbuf + (size_t)(mb * 32 + l32) * VS + (t * 16 + half * 8) * 2);
                oacc[mb] = __builtin_amdgcn_mfma_f32_32x32x16_f16(vf, pfrag[t], oacc[mb], 0, 0, 0);
            }
        }
    };

    auto do_tile = [&](uint32_t tile, unsigned char* kcur, unsigned char* vcur, unsigned char* knxt,
                       unsigned char* vnxt) {
        const bool has_next = tile + 1 < n_tiles;
        if (has_next) {
            issue_k(tile + 1, knxt);
            load_v(tile + 1, vr);
        }
        compute_tile(tile, kcur, vcur);
        if (has_next) store_vt(vr, vnxt);
        __builtin_amdgcn_s_waitcnt(0);
        __syncthreads();
    };
    for (uint32_t tile = 0; tile < n_tiles; tile += 2) {
        do_tile(tile, k_lds0, v_lds0, k_lds1, v_lds1);
        if (tile + 1 < n_tiles) do_tile(tile + 1, k_lds1, v_lds1, k_lds0, v_lds0);
    }

    // ---- write O: lane owns row my_row; register i of block mb is dim mb*32 + (i/4)*8 + half*4 + i%4
    if (row_ok) {
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

template <int D>
inline void launch_prefill_d(const PrefillArgs& a, hipStream_t stream) {
    const uint32_t g = a.num_heads / a.kv_heads;
    auto grid = [&](int rb) { return dim3((a.chunk + kPfRows * rb - 1) / (kPfRows * rb), a.kv_heads, a.batch); };
    switch (g) {
        case 8: hipLaunchKernelGGL((paged_prefill_mfma_kernel<D, 8, 8>), grid(1), dim3(512), 0, stream, a); break;
        case 4: hipLaunchKernelGGL((paged_prefill_mfma_kernel<D, 4, 4>), grid(1), dim3(256), 0, stream, a); break;
        case 2: hipLaunchKernelGGL((paged_prefill_mfma_kernel<D, 2, 4>), grid(2), dim3(256), 0, stream, a); break;
        default: hipLaunchKernelGGL((paged_prefill_mfma_kernel<D, 1, 4>), grid(4), dim3(256), 0, stream, a); break;
    }
}

inline void launch_prefill(const PrefillArgs& a, size_t head_dim, hipStream_t stream) {
    if (head_dim == 64) launch_prefill_d<64>(a, stream); else launch_prefill_d<128>(a, stream);
}

}  // namespace mlc_hip
