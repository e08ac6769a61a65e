// Batched Q6_K matmul for gfx950 (the lm_head of the reference's batched decode step):
// out[b][r] = sum_c W[r][c] * x[b][c], W in Q6_K blocks of 256 weights (210 bytes: 128 bytes of
// low nibbles ql, 64 bytes of high bit pairs qh, 16 int8 scales of 16 weights each, fp16 d;
// value d * scale * (q - 32) with q in 0..63; compiler/runtime/quantization.cpp:142-147,
// 1469-1499), x and out fp32.
//
// Reference: MSL q6_k_matmul_v3_batched (compiler/runtime/metal_runtime.mm:1581-1655), one
// simdgroup per (4 rows, request), fp32 scalar arithmetic.  Here, like the Q4_0 matmul, the
// products run on the matrix cores with fp32-grade accuracy.  d * scale * (q - 32) has up to 24
// significant bits, too many for an fp16 pair, so the scale stays out of the matrix product:
// one MFMA k step covers exactly the 16 columns of one scale group, its operands are the
// exact small integers q - 32 (as fp16) and the activations split x * s = x_hi + x_lo (the
// same fragments as for Q4_0), and the group's sum S = (q-32).x_hi + (q-32).x_lo is added to
// the fp32 accumulator as (d * scale) * S.  The weights are the B operand (a lane holds weight
// row lane % 32), so d * scale is one number per lane, and the activations are the A operand.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "q4_matmul_kernels.h"

namespace mlc_hip {

// ---- generic path: any rows / cols / stride, raw Q6_K rows.  One wave per (row, request),
// lanes stride over the columns like the reference kernel; fp32 throughout.
__global__ __launch_bounds__(256) void q6_k_matmul_generic_kernel(
    const uint8_t* __restrict__ weights, const float* __restrict__ x, float* __restrict__ out,
    uint32_t batch, uint32_t rows, uint32_t cols, uint32_t row_stride) {
    const uint32_t wave = blockIdx.x * 4 + threadIdx.x / 64;
    const uint32_t lane = threadIdx.x % 64;
    if (wave >= batch * rows) return;
    const uint32_t b = wave / rows, r = wave - b * rows;
    const uint8_t* row = weights + (size_t)r * row_stride;
    const float* xv = x + (size_t)b * cols;
    float acc = 0.f;
    for (uint32_t c = lane; c < cols; c += 64) {
        const uint32_t blk = c / 256, off = c % 256;
        const uint32_t half = off / 128, quarter = (off % 128) / 32, l = off % 32;
        const uint8_t* p = row + (size_t)blk * 210;
        const uint8_t qlb = p[half * 64 + (quarter & 1u) * 32 + l];
        const uint32_t nib = quarter < 2 ? (qlb & 0xFu) : (qlb >> 4);
        const uint32_t hb = (p[128 + half * 32 + l] >> (quarter * 2)) & 3u;
        const int q = (int)(nib | (hb << 4)) - 32;
        const float scale = (float)(int8_t)p[192 + half * 8 + quarter * 2 + l / 16];
        const uint16_t dbits = (uint16_t)(p[208] | (p[209] << 8));
        const float d = (float)__builtin_bit_cast(_Float16, dbits);
        acc += d * scale * (float)q * xv[c];
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) acc += __shfl_xor(acc, off);
    if (lane == 0) out[(size_t)b * rows + r] = acc;
}

// Repacked weights (made on the host when the matrix enters the weight cache).  A *group* is
// the four k steps (quarters 0-3) of one (block, half, l0) with l0 in {0, 16}: 64 weights of a
// row, packed in 24 bytes that a lane half h reads as three 8-byte pieces:
//   piece 0: ql[half*64 +      l0 + 8h .. +7]   (low nibble: quarter 0, high nibble: quarter 2)
//   piece 1: ql[half*64 + 32 + l0 + 8h .. +7]   (quarters 1 and 3)
//   piece 2: qh[half*32 +      l0 + 8h .. +7]   (bit pair 2*quarter)
//   qa    [rows/32][groups][3][64 lanes] x 8 bytes     groups = cols/256 * 4, lane = h*32 + row%32
//   sc    [rows/32][groups][32 rows] x 4 int8           the group's scale for quarters 0..3
//   d     [rows/32][cols/256][32 rows] fp16
// Group number within a row: block*4 + half*2 + l0/16; its k step for quarter q is
// block*16 + half*8 + q*2 + l0/16 (columns block*256 + half*128 + q*32 + l0 .. +15).
struct Q6KArgs {
    const uint2* qa;
    const uint32_t* sc;
    const _Float16* d;
    const _Float16* xfrag;   // split activations, layout of q4_split_activations_kernel
    const float* inv_scale;  // [batch]
    float* out;              // [batch][rows]
    uint32_t batch, rows, nblocks;
};

// (0x6400 | v) is the half 1024 + v: two bytes -> half2 (v0 - 32, v1 - 32), exactly.
__device__ __forceinline__ q4_half2 q6_pair(uint32_t bytes, uint32_t sel) {
    const uint32_t m = __builtin_amdgcn_perm(0x64646464u, bytes, sel);
    const q4_half2 k1056 = {(_Float16)1056.0f, (_Float16)1056.0f};
    return __builtin_bit_cast(q4_half2, m) - k1056;
}

// One workgroup: RT tiles of 32 weight rows x NBT batch tiles of 32 x all of K; its 8 waves
// deal the groups out among themselves (group wave, wave + 8, ...), stream their pieces, scales
// and activation fragments into registers two groups ahead, and add their sums up in LDS.
template <int NBT, int RT>
__global__ __launch_bounds__(512) void q6_k_matmul_mfma_kernel(const Q6KArgs a) {
    constexpr int WAVES = 8, PF = 2;
    __shared__ float red[WAVES * RT * NBT * 16 * 64];
    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x / 64);
    const uint32_t lane = threadIdx.x % 64;
    const uint32_t l32 = lane % 32, half = lane / 32;
    const uint32_t tile0 = blockIdx.x * RT;
    const uint32_t groups = a.nblocks * 4;
    const uint32_t ksteps = a.nblocks * 16;

    q4_float16 acc[RT][NBT];
#pragma unroll
    for (int r = 0; r < RT; ++r)
#pragma unroll
        for (int t = 0; t < NBT; ++t)
#pragma unroll
            for (int i = 0; i < 16; ++i) acc[r][t][i] = 0.f;

    struct Group {
        uint2 p[RT][3];
        uint32_t sc[RT];
        _Float16 d[RT];
        q4_half8 x[NBT][4][2];  // [batch tile][quarter][hi, lo]
        bool real;               // false: a repeat past the end, multiplied with scale 0
    };
    auto load = [&](uint32_t g_raw, Group& k) __attribute__((always_inline)) {
        const uint32_t gi = min(g_raw, groups - 1u);
        k.real = g_raw < groups;
        const uint32_t blk = gi / 4, hi = (gi / 2) % 2, l0i = gi % 2;
#pragma unroll
        for (int r = 0; r < RT; ++r) {
            const size_t tg = (size_t)(tile0 + r) * groups + gi;
#pragma unroll
            // (non-temporal: a weight is read once per launch and need not stay in the L2)
            for (int pc = 0; pc < 3; ++pc) k.p[r][pc] = q4_stream_u2(a.qa + (tg * 3 + pc) * 64 + lane);
            k.sc[r] = __builtin_nontemporal_load(a.sc + tg * 32 + l32);
            k.d[r] = __builtin_nontemporal_load(a.d + ((size_t)(tile0 + r) * a.nblocks + blk) * 32 + l32);
        }
#pragma unroll
        for (int t = 0; t < NBT; ++t)
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const uint32_t kstep = blk * 16 + hi * 8 + q * 2 + l0i;
#pragma unroll
                for (int pt = 0; pt < 2; ++pt)
                    k.x[t][q][pt] = *reinterpret_cast<const q4_half8*>(
                        a.xfrag + ((((size_t)t * ksteps + kstep) * 2 + pt) * 64 + lane) * 8);
            }
    };
    auto multiply = [&](const Group& k) __attribute__((always_inline)) {
#pragma unroll
        for (int r = 0; r < RT; ++r) {
            const float d = k.real ? (float)k.d[r] : 0.0f;
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const uint2 ql = k.p[r][q & 1];
                const uint2 qh = k.p[r][2];
                // one byte per weight: low nibble | high bit pair << 4
                const uint32_t v0 = ((q >= 2 ? ql.x >> 4 : ql.x) & 0x0F0F0F0Fu) | (((qh.x >> (2 * q)) & 0x03030303u) << 4);
                const uint32_t v1 = ((q >= 2 ? ql.y >> 4 : ql.y) & 0x0F0F0F0Fu) | (((qh.y >> (2 * q)) & 0x03030303u) << 4);
                const q4_half2 n0 = q6_pair(v0, 0x04010400u), n1 = q6_pair(v0, 0x04030402u);
                const q4_half2 n2 = q6_pair(v1, 0x04010400u), n3 = q6_pair(v1, 0x04030402u);
                const q4_half8 w = {n0[0], n0[1], n1[0], n1[1], n2[0], n2[1], n3[0], n3[1]};
                const int s8 = (int)(int8_t)(k.sc[r] >> (8 * q));
                const float gscale = d * (float)s8;
#pragma unroll
                for (int t = 0; t < NBT; ++t) {
                    q4_float16 s;
#pragma unroll
                    for (int i = 0; i < 16; ++i) s[i] = 0.f;
                    s = __builtin_amdgcn_mfma_f32_32x32x16_f16(k.x[t][q][0], w, s, 0, 0, 0);
                    s = __builtin_amdgcn_mfma_f32_32x32x16_f16(k.x[t][q][1], w, s, 0, 0, 0);
#pragma unroll
                    for (int i = 0; i < 16; ++i) acc[r][t][i] = fmaf(gscale, s[i], acc[r][t][i]);
                }
            }
        }
    };

    // (the empty asm statements pin each group of loads where it is written, see the Q4_0 kernel)
    Group k[PF];
#pragma unroll
    for (int i = 0; i < PF; ++i) {
        load(wave + i * WAVES, k[i]);
        asm volatile("" ::: "memory");
    }
    for (uint32_t base = wave; base < groups; base += PF * WAVES) {
#pragma unroll
        for (int i = 0; i < PF; ++i) {
            multiply(k[i]);
            load(base + (i + PF) * WAVES, k[i]);
            asm volatile("" ::: "memory");
        }
    }

    // ---- the waves' sums meet in LDS.  Accumulator layout: lane holds weight row l32 of the
    // tile and, in register i, batch row (i/4)*8 + (lane/32)*4 + i%4 of the batch tile.
#pragma unroll
    for (int r = 0; r < RT; ++r)
#pragma unroll
        for (int t = 0; t < NBT; ++t)
#pragma unroll
            for (int i = 0; i < 16; ++i)
                red[(((wave * RT + r) * NBT + t) * 16 + i) * 64 + lane] = acc[r][t][i];
    __syncthreads();
    // wave w finishes the (r, t, i) combinations number w, w + 8, ...: 32 consecutive weight rows
    // of one request per half wave
    constexpr int COMBOS = RT * NBT * 16;
#pragma unroll
    for (int c = 0; c < COMBOS / WAVES; ++c) {
        const uint32_t combo = c * WAVES + wave;
        const uint32_t r = combo / (NBT * 16), t = (combo / 16) % NBT, i = combo % 16;
        const uint32_t b = t * 32 + (i / 4) * 8 + half * 4 + i % 4;
        float sum = 0.f;
#pragma unroll
        for (int w = 0; w < WAVES; ++w) sum += red[(((w * RT + r) * NBT + t) * 16 + i) * 64 + lane];
        if (b < a.batch) a.out[(size_t)b * a.rows + (tile0 + r) * 32 + l32] = sum * a.inv_scale[b];
    }
}

}  // namespace mlc_hip
