// Batched Q4_0 matmul for gfx950: out[b][r] = sum_c W[r][c] * x[b][c], W in Q4_0 blocks
// (32 weights: fp16 scale d, 16 bytes of nibbles; weight j in the low nibble of byte j,
// weight j+16 in the high nibble, value d * (nibble - 8)), x and out fp32.
//
// Reference: MSL q4_0_matmul_v3_batched (compiler/runtime/metal_runtime.mm:710-785), one
// simdgroup per (4 rows, request), fp32 scalar arithmetic.  With a decode batch of 32-64
// requests this is a GEMM (M = rows, N = batch, K = cols) that is bound by reading the
// weights once, so here it runs on the matrix cores (v_mfma_f32_32x32x16_f16, fp32
// accumulate) with fp32-grade accuracy:
//   * a weight d*(q-8) has at most 15 significant bits, so it is EXACTLY w_hi + w_lo with
//     w_hi = fp16(d*(q-8)) and w_lo = fma(d, q-8, -w_hi) (both fp16);
//   * an activation is split x*s = x_hi + x_lo (fp16 each, relative error 2^-22), s a power of
//     two per request that places the row's largest magnitude at 2^13..2^14;
//   * out = (W_hi.X_hi + W_hi.X_lo + W_lo.X_hi) / s -- three MFMAs per 16 columns; the dropped
//     W_lo.X_lo term is below 2^-22 of the products.
// The weights are repacked once, when they enter the library's weight cache, so that the A
// operand of a 32-row tile is one coalesced 8-byte load per lane and block; the activations
// are split by a small kernel into the B-operand layout, so that a fragment is one 16-byte
// load per lane.  K is split over workgroups when there are too few row tiles to fill the
// chip; the slices are summed in a fixed order by a second small kernel.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace mlc_hip {

typedef _Float16 q4_half2 __attribute__((ext_vector_type(2)));
typedef _Float16 q4_half8 __attribute__((ext_vector_type(8)));
typedef float q4_float16 __attribute__((ext_vector_type(16)));

// ---- generic path: any rows / cols / stride, raw Q4_0 rows.  One wave per (row, request),
// lanes stride over the columns like the reference kernel; fp32 throughout.
__global__ __launch_bounds__(256) void q4_0_matmul_generic_kernel(
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
        const uint32_t blk = c / 32, in_blk = c % 32;
        const uint8_t* p = row + (size_t)blk * 18;
        const uint16_t dbits = (uint16_t)(p[0] | (p[1] << 8));  // rows may start at odd addresses
        const _Float16 d = __builtin_bit_cast(_Float16, dbits);
        const uint8_t byte = p[2 + (in_blk & 15)];
        const int q = (int)(in_blk < 16 ? (byte & 0x0F) : (byte >> 4)) - 8;
        acc += (float)d * (float)q * xv[c];
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) acc += __shfl_xor(acc, off);
    if (lane == 0) out[(size_t)b * rows + r] = acc;
}

// ---- activations -> B-operand fragments.  One workgroup per (padded) request row:
// s = 2^(14 - exponent(max|x|)), then hi = fp16(x*s), lo = fp16(x*s - hi).  Element (n, k) of
// the padded batch goes to
//   frag[((n/32 * ksteps + k/16) * 2 + part) * 64 + ((k%16)/8)*32 + n%32][k%8],  part 0 hi, 1 lo
// so that lane l of a wave finds the 8 halves the MFMA wants from it (column n = l%32 of the
// batch tile, k group l/32) in 16 contiguous bytes.  Rows past `batch` are written as zeros.
__global__ __launch_bounds__(256) void q4_split_activations_kernel(
    const float* __restrict__ x, _Float16* __restrict__ frag, float* __restrict__ inv_scale,
    uint32_t batch, uint32_t cols) {
    __shared__ float red[4];
    constexpr int MAXV = 4;  // register-resident groups of 8 columns per thread: cols <= 8192
    const uint32_t n = blockIdx.x;
    const uint32_t ksteps = cols / 16;
    const uint32_t groups = cols / 8;
    const bool live = n < batch;
    const float4* xr = reinterpret_cast<const float4*>(x + (size_t)(live ? n : 0) * cols);
    const bool in_regs = groups <= 256 * MAXV;
    float4 v[MAXV][2];
    float amax = 0.f;
    if (live) {
        if (in_regs) {
#pragma unroll
            for (int j = 0; j < MAXV; ++j) {
                const uint32_t k8 = j * 256 + threadIdx.x;
                v[j][0] = v[j][1] = make_float4(0.f, 0.f, 0.f, 0.f);
                if (k8 < groups) { v[j][0] = xr[k8 * 2]; v[j][1] = xr[k8 * 2 + 1]; }
                amax = fmaxf(amax, fmaxf(fmaxf(fabsf(v[j][0].x), fabsf(v[j][0].y)), fmaxf(fabsf(v[j][0].z), fabsf(v[j][0].w))));
                amax = fmaxf(amax, fmaxf(fmaxf(fabsf(v[j][1].x), fabsf(v[j][1].y)), fmaxf(fabsf(v[j][1].z), fabsf(v[j][1].w))));
            }
        } else {
            for (uint32_t k4 = threadIdx.x; k4 < cols / 4; k4 += 256) {
                const float4 t = xr[k4];
                amax = fmaxf(amax, fmaxf(fmaxf(fabsf(t.x), fabsf(t.y)), fmaxf(fabsf(t.z), fabsf(t.w))));
            }
        }
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) amax = fmaxf(amax, __shfl_xor(amax, off));
    if (threadIdx.x % 64 == 0) red[threadIdx.x / 64] = amax;
    __syncthreads();
    amax = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
    int e = 0;
    if (amax > 0.f && amax < INFINITY) (void)frexpf(amax, &e);  // amax = m * 2^e, m in [0.5, 1)
    int se = 14 - e;
    se = se > 100 ? 100 : (se < -100 ? -100 : se);
    const float s = ldexpf(1.0f, se);
    if (threadIdx.x == 0 && live) inv_scale[n] = ldexpf(1.0f, -se);
    // 8 consecutive columns per thread and step: one 16-byte store to each part
    auto emit = [&](uint32_t k8, const float4& lo4, const float4& hi4) __attribute__((always_inline)) {
        const float in8[8] = {lo4.x, lo4.y, lo4.z, lo4.w, hi4.x, hi4.y, hi4.z, hi4.w};
        q4_half8 hi, lo;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const float t = live ? in8[i] * s : 0.f;
            hi[i] = (_Float16)t;
            lo[i] = (_Float16)(t - (float)hi[i]);
        }
        const uint32_t k = k8 * 8;
        const size_t base = ((size_t)(n / 32) * ksteps + k / 16) * 2;
        const uint32_t lane = ((k % 16) / 8) * 32 + n % 32;
        *reinterpret_cast<q4_half8*>(frag + ((base + 0) * 64 + lane) * 8) = hi;
        *reinterpret_cast<q4_half8*>(frag + ((base + 1) * 64 + lane) * 8) = lo;
    };
    if (in_regs) {
#pragma unroll
        for (int j = 0; j < MAXV; ++j) {
            const uint32_t k8 = j * 256 + threadIdx.x;
            if (k8 < groups) emit(k8, v[j][0], v[j][1]);
        }
    } else {
        for (uint32_t k8 = threadIdx.x; k8 < groups; k8 += 256) {
            const float4 z = make_float4(0.f, 0.f, 0.f, 0.f);
            emit(k8, live ? xr[k8 * 2] : z, live ? xr[k8 * 2 + 1] : z);
        }
    }
}

struct Q4Args {
    const uint2* qs;            // repacked nibbles [rows/32][nblocks][64 lanes] x 8 bytes
    const _Float16* d;          // repacked scales  [rows/32][nblocks][32 rows]
    const _Float16* xfrag;      // split activations, layout above
    const float* inv_scale;     // [batch]
    float* out;                 // [batch][rows], or the slice buffer [ksplit][batch][rows]
    uint32_t batch, rows, nblocks, blocks_per_slice, ksplit;
};

// (0x6400 | n) is the half 1024 + n: two nibbles -> half2 (n0 - 8, n1 - 8), exactly.
__device__ __forceinline__ q4_half2 q4_pair(uint32_t bytes, uint32_t sel) {
    const uint32_t m = __builtin_amdgcn_perm(0x64646464u, bytes, sel);
    const q4_half2 k1032 = {(_Float16)1032.0f, (_Float16)1032.0f};
    return __builtin_bit_cast(q4_half2, m) - k1032;
}

static constexpr int kQ4ChunkBlocks = 8;  // Q4_0 blocks (of 32 columns) staged in LDS at a time

// One workgroup: 256 weight rows x NBT batch tiles of 32 x one K slice, taken in chunks of 8
// blocks that are double buffered.  8 waves: wave w works on the 64 rows (two 32-row tiles) number w % 4 and on the
// blocks of parity w / 4, so every SIMD holds two waves whose unpacking (VALU) and MFMAs
// overlap; the two halves are added through LDS at the end.  Per chunk the waves copy the
// chunk's activation fragments into LDS (global -> LDS loads, shared by all waves) and their
// own nibbles and scales into registers, wait once, and then run unpack + MFMA.
template <int NBT>
__global__ __launch_bounds__(512) void q4_0_matmul_mfma_kernel(const Q4Args a) {
    constexpr int CB = kQ4ChunkBlocks;
    constexpr int FRAGS = CB * NBT * 4;  // 1 KiB fragments per chunk: [block][batch tile][k step][hi, lo]
    __shared__ __attribute__((aligned(16))) unsigned char xs[FRAGS * 1024];
    __shared__ __attribute__((aligned(16))) unsigned char xs1[FRAGS * 1024];
    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x / 64);
    const uint32_t lane = threadIdx.x % 64;
    const uint32_t l32 = lane % 32, half = lane / 32;
    const uint32_t pairs = a.rows / 64;
    const uint32_t khalf = wave / 4;                        // parity of the blocks this wave takes
    const uint32_t pair_raw = blockIdx.x * 4 + wave % 4;    // index of the 64-row pair of tiles
    const bool active = pair_raw < pairs;             // idle waves still take part in staging
    const uint32_t pair = active ? pair_raw : pairs - 1;
    const uint32_t slice = blockIdx.y;
    const uint32_t b0 = slice * a.blocks_per_slice;
    const uint32_t b1 = min(b0 + a.blocks_per_slice, a.nblocks);
    const uint32_t ksteps = a.nblocks * 2;

    q4_float16 acc[2][NBT];
#pragma unroll
    for (int r = 0; r < 2; ++r)
#pragma unroll
        for (int t = 0; t < NBT; ++t)
#pragma unroll
            for (int i = 0; i < 16; ++i) acc[r][t][i] = 0.f;

    // A chunk's loads: this wave's weights (blocks 2*jj + khalf of the chunk) -> registers, and
    // its share of the chunk's activation fragments -> LDS (fragment f by wave f % 8).
    struct Weights {
        uint2 q[CB / 2][2];
        _Float16 d[CB / 2][2];
    };
    auto issue = [&](uint32_t cb, unsigned char* xbuf, Weights& w) __attribute__((always_inline)) {
        const uint32_t nbk = min((uint32_t)CB, b1 - cb);
#pragma unroll
        for (int jj = 0; jj < CB / 2; ++jj)
#pragma unroll
            for (int r = 0; r < 2; ++r) {
                const uint32_t blk = cb + min(2u * jj + khalf, nbk - 1u);  // past the end: a repeat, unused
                const size_t tb = (size_t)(pair * 2 + r) * a.nblocks + blk;
                w.q[jj][r] = a.qs[tb * 64 + lane];
                w.d[jj][r] = a.d[tb * 32 + l32];
            }
#pragma unroll
        for (int i = 0; i < FRAGS / 8; ++i) {
            const uint32_t f = i * 8 + wave;
            const uint32_t p = f % 2, ks = (f / 2) % 2, t = (f / 4) % NBT;
            const uint32_t j = min(f / (4 * NBT), nbk - 1u);
            const _Float16* src =
                a.xfrag + ((((size_t)t * ksteps + (cb + j) * 2 + ks) * 2 + p) * 64 + lane) * 8;
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)src,
                                             (__attribute__((address_space(3))) void*)(xbuf + f * 1024), 16, 0, 0);
        }
    };
    // unpack + MFMA over the chunk's blocks of this wave
    auto compute = [&](uint32_t cb, const unsigned char* xbuf, const Weights& w) __attribute__((always_inline)) {
        const uint32_t nbk = min((uint32_t)CB, b1 - cb);
#pragma unroll
        for (int jj = 0; jj < CB / 2; ++jj) {
            const uint32_t j = 2u * jj + khalf;
            if (j >= nbk) break;
            q4_half8 xf[NBT][2][2];
#pragma unroll
            for (int t = 0; t < NBT; ++t)
#pragma unroll
                for (int ks = 0; ks < 2; ++ks)
#pragma unroll
                    for (int p = 0; p < 2; ++p)
                        xf[t][ks][p] = *reinterpret_cast<const q4_half8*>(
                            xbuf + (size_t)((((j * NBT + t) * 2 + ks) * 2 + p) * 1024) + lane * 16);
#pragma unroll
            for (int r = 0; r < 2; ++r) {
                const q4_half2 d2 = {w.d[jj][r], w.d[jj][r]};
                // k step 0: low nibbles of this lane's 8 bytes, k step 1: high nibbles
#pragma unroll
                for (int ks = 0; ks < 2; ++ks) {
                    const uint32_t w0 = (ks ? (w.q[jj][r].x >> 4) : w.q[jj][r].x) & 0x0F0F0F0Fu;
                    const uint32_t w1 = (ks ? (w.q[jj][r].y >> 4) : w.q[jj][r].y) & 0x0F0F0F0Fu;
                    q4_half2 n[4] = {q4_pair(w0, 0x04010400u), q4_pair(w0, 0x04030402u),
                                     q4_pair(w1, 0x04010400u), q4_pair(w1, 0x04030402u)};
                    q4_half8 whi, wlo;
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const q4_half2 h = d2 * n[e];
                        const q4_half2 l = __builtin_elementwise_fma(d2, n[e], -h);
                        whi[2 * e] = h[0]; whi[2 * e + 1] = h[1];
                        wlo[2 * e] = l[0]; wlo[2 * e + 1] = l[1];
                    }
#pragma unroll
                    for (int t = 0; t < NBT; ++t) {
                        acc[r][t] = __builtin_amdgcn_mfma_f32_32x32x16_f16(whi, xf[t][ks][0], acc[r][t], 0, 0, 0);
                        acc[r][t] = __builtin_amdgcn_mfma_f32_32x32x16_f16(whi, xf[t][ks][1], acc[r][t], 0, 0, 0);
                        acc[r][t] = __builtin_amdgcn_mfma_f32_32x32x16_f16(wlo, xf[t][ks][0], acc[r][t], 0, 0, 0);
                    }
                }
            }
        }
    };
    // Two staging buffers and two register sets: the loads of chunk c+1 are in flight while
    // chunk c is multiplied.  One barrier per chunk: it says that everybody's loads of chunk c
    // have landed and that everybody has left chunk c-1, whose buffer chunk c+1 overwrites.
    Weights wa, wb;
    issue(b0, xs, wa);
    for (uint32_t cb = b0; cb < b1; cb += 2 * CB) {
        __builtin_amdgcn_s_waitcnt(0);
        __syncthreads();
        if (cb + CB < b1) issue(cb + CB, xs1, wb);
        compute(cb, xs, wa);
        if (cb + CB >= b1) break;
        __builtin_amdgcn_s_waitcnt(0);
        __syncthreads();
        if (cb + 2 * CB < b1) issue(cb + 2 * CB, xs, wa);
        compute(cb + CB, xs1, wb);
    }
    __syncthreads();  // everyone is done with the staging memory: the steps below reuse it

    // ---- the odd-block waves hand their sums to the even-block waves (staging memory is free:
    // the loop ended with a barrier)
    static_assert(4 * 2 * NBT * 16 * 64 * 4 <= FRAGS * 1024, "partial sums fit the staging buffer");
    float* red = reinterpret_cast<float*>(xs) + (size_t)(wave % 4) * (2 * NBT * 16 * 64);
    if (khalf == 1) {
#pragma unroll
        for (int r = 0; r < 2; ++r)
#pragma unroll
            for (int t = 0; t < NBT; ++t)
#pragma unroll
                for (int i = 0; i < 16; ++i) red[((r * NBT + t) * 16 + i) * 64 + lane] = acc[r][t][i];
    }
    __syncthreads();
    if (khalf == 0) {
#pragma unroll
        for (int r = 0; r < 2; ++r)
#pragma unroll
            for (int t = 0; t < NBT; ++t)
#pragma unroll
                for (int i = 0; i < 16; ++i) acc[r][t][i] += red[((r * NBT + t) * 16 + i) * 64 + lane];
    }
    __syncthreads();  // the epilogue below reuses the same memory
    if (!active || khalf == 1) return;

    // Accumulator layout: lane holds batch column l32 of the tile and, in register i, weight
    // row (i/4)*8 + half*4 + i%4 of the 32-row tile.  The tile goes through this wave's part of
    // the (now free) staging memory so that every store instruction writes whole 128-byte runs
    // of out[b][row..].
    static_assert(4 * 32 * 33 * 4 <= FRAGS * 1024, "epilogue tiles fit the staging buffer");
    float (*tl)[33] = reinterpret_cast<float (*)[33]>(xs + (wave % 4) * (32 * 33 * 4));
    float* out = a.out + (size_t)slice * a.batch * a.rows;
#pragma unroll
    for (int t = 0; t < NBT; ++t) {
        const uint32_t b = t * 32 + l32;
        const float inv = b < a.batch ? a.inv_scale[b] : 0.f;
#pragma unroll
        for (int r = 0; r < 2; ++r) {
#pragma unroll
            for (int i = 0; i < 16; ++i) tl[l32][(i / 4) * 8 + half * 4 + (i % 4)] = acc[r][t][i] * inv;
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
            // lane -> (batch row bb = pass*2 + half, weight row l32): 32 consecutive floats per half wave
#pragma unroll
            for (int pass = 0; pass < 16; ++pass) {
                const uint32_t bl = pass * 2 + half;
                const uint32_t bb = t * 32 + bl;
                if (bb < a.batch) out[(size_t)bb * a.rows + (pair * 2 + r) * 32 + l32] = tl[bl][l32];
            }
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        }
    }
}

// out[i] = slice 0 + slice 1 + ... in that order.
__global__ __launch_bounds__(256) void q4_sum_slices_kernel(const float* __restrict__ slices,
                                                            float* __restrict__ out, uint32_t n,
                                                            uint32_t ksplit) {
    const uint32_t i = blockIdx.x * 256 + threadIdx.x;
    if (i >= n) return;
    float s = slices[i];
    for (uint32_t k = 1; k < ksplit; ++k) s += slices[(size_t)k * n + i];
    out[i] = s;
}

}  // namespace mlc_hip
