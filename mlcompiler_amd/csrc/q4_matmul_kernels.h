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
// The default arithmetic (IOP) instead takes the integers q - 8 as operand, exact in fp16, and adds
// every block's sum (q-8).x_hi + (q-8).x_lo to the result as d * sum: nothing is dropped.  There
// the activations may also come with one power-of-two scale per (request, block of 32 columns)
// (BS), which a kernel that produces 32 neighbouring columns of a request can compute on its own:
// the epilogues below (gate/up split + SiLU * up; residual add + RMSNorm) and the decode attention
// write the next matmul's fragments that way.
// The weights are repacked once, when they enter the library's weight cache, so that the A
// operand of a 32-row tile is one coalesced 8-byte load per lane and block; the activations
// are split by a small kernel into the B-operand layout, so that a fragment is one 16-byte
// load per lane.  K is split over workgroups only when there are too few row tiles to fill the
// chip and K is long; the slices are then summed in a fixed order (q4_sum_slices_kernel, or
// the fused row kernel of walker_kernels.h).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "paged_decode_kernels.h"
#include "paged_rope_kernels.h"

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
    // 2 (one batch tile, kernels without the SiLU epilogue): the grid's z dimension halves the
    // batch; workgroup z takes requests 16 z .. 16 z + 15 of the tile and fetches only their
    // activation fragments (the other 16 lanes of a half wave repeat those addresses and their
    // results are dropped).  The fragments are the largest stream of a workgroup that has all of
    // K, 4 bytes per request and column through one CU's memory path; this halves it where the
    // grid would otherwise leave half of the CUs idle anyway (quarters of the batch on four
    // workgroups were measured as well and gain nothing more).  0 or 1: the whole tile.
    uint32_t bsplit;
    // When rope_on is set (ksplit == 1, out is a fused qkv row of rope.qkv_rows = rows floats per
    // request): the epilogue also does what qkv_split_rope_cast_kernel would do with that row.
    uint32_t rope_on;
    RopeArgs rope;
    // Kernels built with BS: the activations were split with one power-of-two scale per (request,
    // block of 32 columns) instead of one per request: x = (hi + lo) * 2^e.  blk_exp holds the
    // exponents e as [batch tile of 32][nblocks][32 bytes], request c of the tile at byte
    // ((c % 8) / 4) * 16 + (c / 8) * 4 + c % 4 -- the order in which a lane's 16 accumulator
    // registers hold the requests, so that one 16-byte load per block brings a lane's 16 exponents;
    // inv_scale is not read.
    const int8_t* blk_exp;
    // Kernels built with SILU (two row tiles per workgroup, ksplit == 1, rows = 2 * ffn_inner): the
    // output is a fused gate/up row; workgroup j takes tile j of the gate half and tile j of the up
    // half (tile_stride = ffn_inner / 32 apart) and its epilogue also does the gate/up split and
    // SiLU(gate) * up of those 32 columns -> gate, up, silu_out ([batch][ffn_inner] each).  With
    // split_frag set it goes on to split the 32 products of every request into the B-operand
    // fragments of the matmul that consumes them (K = ffn_inner), scaled per (request, block):
    // block j of that matmul is exactly this workgroup's 32 columns.
    uint32_t tile_stride, ffn_inner;
    float* gate;
    float* up;
    float* silu_out;
    _Float16* split_frag;
    int8_t* split_blk_exp;
    // One row tile per workgroup, ksplit == 1, no RoPE epilogue, add_resid set: the epilogue also
    // does the residual add that follows the matmul (add_out = out + add_resid, [batch][rows]), leaves
    // every request's sum of squares over the workgroup's 32 columns in ssq_out[tile][64] (the
    // RMSNorm that follows is finished by the matmul that reads it, see ssq_in) and writes
    // add_out * gamma as the split-fp16 fragments of that matmul (split_frag / split_blk_exp,
    // K = rows).  gamma[c] for c < n_gamma, 1 beyond.
    const float* add_resid;
    float* add_out;
    const float* gamma;
    uint32_t n_gamma;
    float* ssq_out;
    // ssq_in set (BS kernels): the activations are h * gamma of an RMSNorm whose per-request factor
    // 1 / sqrt(mean(h^2) + eps) is still missing: it is computed here from the ssq_tiles partial
    // sums of squares per request (ssq_in[tile][64], summed in a fixed order) and multiplied into the
    // result, and the workgroups also write the RMSNorm's own output rms_out = h * factor * gamma
    // ([batch][rms_len], h = rms_src), 1024 elements per workgroup of the grid.
    const float* ssq_in;
    uint32_t ssq_tiles, rms_len;
    float rms_eps;
    const float* rms_src;
    float* rms_out;
};

// Maximum / sum over the 32 lanes of a half wave, every lane gets the result.
__device__ __forceinline__ float q4_half_wave_max(float v) {
    v = fmaxf(v, dpp_f<kDppQuadXor1>(v));
    v = fmaxf(v, dpp_f<kDppQuadXor2>(v));
    v = fmaxf(v, dpp_f<kDppHalfMirror>(v));
    v = fmaxf(v, dpp_f<kDppRowRor8>(v));
    const auto sw = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    return fmaxf(__uint_as_float(sw[0]), __uint_as_float(sw[1]));
}
__device__ __forceinline__ float q4_half_wave_sum(float v) {
    v += dpp_f<kDppQuadXor1>(v);
    v += dpp_f<kDppQuadXor2>(v);
    v += dpp_f<kDppHalfMirror>(v);
    v += dpp_f<kDppRowRor8>(v);
    const auto sw = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    return __uint_as_float(sw[0]) + __uint_as_float(sw[1]);
}

// One value per lane, the 32 lanes of a half wave holding columns col0 .. col0+31 (one Q4_0 block)
// of request b: writes them as hi + lo fp16 fragments of a matmul with K = k_cols, scaled by the
// block's own power of two, and the exponent (q4_split_activations_kernel's scale, per block).
__device__ __forceinline__ void q4_emit_block(float v, uint32_t b, uint32_t col, uint32_t k_cols, _Float16* frag,
                                              int8_t* blk_exp) {
    const float amax = q4_half_wave_max(fabsf(v));
    int e = 0;
    if (amax > 0.f && amax < INFINITY) (void)frexpf(amax, &e);
    int se = 14 - e;
    se = se > 100 ? 100 : (se < -100 ? -100 : se);
    const float tv = __builtin_ldexpf(v, se);
    const _Float16 hi = (_Float16)tv;
    const _Float16 lo = (_Float16)(tv - (float)hi);
    const uint32_t t = b / 32, c = b % 32;
    const size_t base = ((size_t)t * (k_cols / 16) + col / 16) * 2;
    const uint32_t fl = ((col % 16) / 8) * 32 + c;
    frag[((base + 0) * 64 + fl) * 8 + col % 8] = hi;
    frag[((base + 1) * 64 + fl) * 8 + col % 8] = lo;
    if (col % 32 == 0)
        blk_exp[((size_t)t * (k_cols / 32) + col / 32) * 32 + ((c % 8) / 4) * 16 + (c / 8) * 4 + c % 4] = (int8_t)(-se);
}

// The split + RoPE + cast (+ paged write) of one element of a request's fused qkv row, by the
// thread that just produced it; the partner of its (even, odd) pair sits in the neighbouring
// lane.  Same arithmetic, element for element, as qkv_split_rope_cast_kernel.  What the thread
// needs from memory for it (its cos / sin pair, its request's page row) is fetched before the
// matmul's main loop, so that the epilogue adds no memory round trip to the kernel's tail.
struct Q4RopeFetch {
    float c, s;        // rotation of this element's pair (1, 0 where none applies)
    uint32_t page_row; // page_ids[req] * page_size + slots[req]
};

__device__ __forceinline__ Q4RopeFetch q4_rope_prefetch(const RopeArgs& p, uint32_t req, uint32_t feat) {
    Q4RopeFetch f = {1.0f, 0.0f, 0u};
    if (req >= p.batch || feat >= p.q_rows + p.k_rows + p.v_rows) return f;
    const bool is_q = feat < p.q_rows;
    const bool is_k = !is_q && feat < p.q_rows + p.k_rows;
    const uint32_t local = is_q ? feat : (is_k ? feat - p.q_rows : feat - p.q_rows - p.k_rows);
    if (is_q || is_k) {
        const uint32_t d = (local & ~1u) % p.head_dim;
        if (d < p.rotary_dim) {
            const uint32_t ci = req * (p.rotary_dim / 2) + d / 2;
            f.c = p.cos_table[ci];
            f.s = p.sin_table[ci];
        }
    }
    if (!is_q && (is_k ? p.k_pages : p.v_pages)) f.page_row = p.page_ids[req] * p.page_size + p.slots[req];
    return f;
}

__device__ __forceinline__ void q4_rope_epilogue(const RopeArgs& p, const Q4RopeFetch& f, uint32_t req,
                                                 uint32_t feat, float val) {
    const float other = __shfl_xor(val, 1);
    const bool odd = (feat & 1u) != 0;
    const float2 x = odd ? make_float2(other, val) : make_float2(val, other);
    if (feat >= p.q_rows + p.k_rows + p.v_rows) return;
    const bool is_q = feat < p.q_rows;
    const bool is_k = !is_q && feat < p.q_rows + p.k_rows;
    const uint32_t local = is_q ? feat : (is_k ? feat - p.q_rows : feat - p.q_rows - p.k_rows);
    float2 y = x;
    if ((is_q || is_k) && (local & ~1u) % p.head_dim < p.rotary_dim) y = rope_rotate(x, f.c, f.s);
    const float mine = odd ? y.y : y.x;
    if (is_q) {
        p.q[(size_t)req * p.q_rows + local] = mine;
        return;
    }
    float* f32 = is_k ? p.k : p.v;
    const uint32_t rows = is_k ? p.k_rows : p.v_rows;
    if (f32) f32[(size_t)req * rows + local] = mine;
    const _Float16 h = (_Float16)mine;
    _Float16* f16 = is_k ? p.k_f16 : p.v_f16;
    if (f16) f16[(size_t)req * rows + local] = h;
    _Float16* pool = is_k ? p.k_pages : p.v_pages;
    if (pool) pool[(size_t)f.page_row * rows + local] = h;
}

// 8-byte non-temporal load (data that is read once and need not displace anything in the L2).
__device__ __forceinline__ uint2 q4_stream_u2(const uint2* p) {
    typedef uint32_t q4_u32x2 __attribute__((ext_vector_type(2)));
    const q4_u32x2 v = __builtin_nontemporal_load(reinterpret_cast<const q4_u32x2*>(p));
    return make_uint2(v[0], v[1]);
}

// (0x6400 | n) is the half 1024 + n: two nibbles -> half2 (n0 - 8, n1 - 8), exactly.
__device__ __forceinline__ q4_half2 q4_pair(uint32_t bytes, uint32_t sel) {
    const uint32_t m = __builtin_amdgcn_perm(0x64646464u, bytes, sel);
    const q4_half2 k1032 = {(_Float16)1032.0f, (_Float16)1032.0f};
    return __builtin_bit_cast(q4_half2, m) - k1032;
}

// One workgroup: RT tiles of 32 weight rows x NBT batch tiles of 32 x one K slice.  The
// slice's blocks are dealt out to the WAVES waves (block b0 + wave, + WAVES, ...); a wave streams
// its blocks' nibbles, scales and activation fragments straight from memory into registers, PF
// blocks ahead, unpacks and multiplies; there is no staging memory and no barrier until the
// waves' sums meet in LDS at the end.  With the whole K range in one workgroup (ksplit = 1) the
// result goes straight to the output; K slices are only worth it when there are too few row
// tiles to fill the chip and K is long.
//
// IOP (integer operand): the matrix product runs over the exact integers q - 8 and the block
// scale d is applied to each block's sum in fp32, acc += d * ((q-8).x_hi + (q-8).x_lo): four
// MFMAs and 16 multiply-adds per (block, tile) instead of six MFMAs and the exact hi + lo split
// of d * (q - 8).  The weights are then the B operand (a lane holds weight row lane % 32, so d
// is one number per lane) and the activations the A operand; both fragment layouts serve either
// role unchanged.  No product is rounded and no term is dropped: what remains is the fp32
// rounding of the additions and of one multiply per block.
__device__ __forceinline__ float q4_silu_times(float g, float u) {  // walker_kernels.h: silu_times
    const float silu = g / (1.0f + expf(-g));
    return silu * u;
}

template <int NBT, int RT, int WAVES, bool IOP, bool BS = false, bool SILU = false>
__global__ __launch_bounds__(WAVES * 64) void q4_0_matmul_mfma_kernel(const Q4Args a) {
    static_assert(!BS || IOP, "per-block activation scales: integer-operand arithmetic only");
    static_assert(!SILU || (IOP && RT == 2), "SiLU epilogue: gate tile and up tile, integer-operand arithmetic");
    constexpr int PF = WAVES >= 16 ? 2 : 4;  // blocks in flight per wave
    constexpr int PITCH = 65;                // floats per accumulator register in LDS (bank spread)
    __shared__ float red[WAVES * RT * NBT * 16 * PITCH];
    __shared__ float rms_scale[BS ? 32 * NBT : 1];   // BS with ssq_in: every request's RMSNorm factor
    constexpr int SSQ_P = WAVES * 64 / (32 * NBT);   // threads per request that share the sum over the partials
    constexpr int SSQ_NL = 128 / SSQ_P < 8 ? 128 / SSQ_P : 8;   // partials per thread, at most: up to 128 tiles (rows of
                                                                // 4096), 64 with two batch tiles (the host checks)
    __shared__ float ssq_lds[BS ? SSQ_P * 32 * NBT : 1];
    constexpr int RMS_NE = WAVES >= 16 ? 1 : 2;   // elements of the norm's output per thread: 1024 per workgroup
    __shared__ float rms_h_lds[BS ? RMS_NE * WAVES * 64 : 1];   // ... parked here through the main loop
    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x / 64);
    const uint32_t lane = threadIdx.x % 64;
    const uint32_t l32 = lane % 32;
    const uint32_t tile0 = SILU ? blockIdx.x : blockIdx.x * RT;
    const uint32_t tile_step = SILU ? a.tile_stride : 1u;   // row tile r of the workgroup: tile0 + r * tile_step
    const uint32_t slice = blockIdx.y;
    const uint32_t bz = blockIdx.z;   // (batch half, with bsplit == 2)
    const uint32_t lane_x = (a.bsplit < 2 || (lane % 32) / 16 == bz) ? lane : (lane ^ 16u);
    const uint32_t b0 = slice * a.blocks_per_slice;
    const uint32_t b1 = min(b0 + a.blocks_per_slice, a.nblocks);
    const uint32_t ksteps = a.nblocks * 2;

    q4_float16 acc[RT][NBT];
#pragma unroll
    for (int r = 0; r < RT; ++r)
#pragma unroll
        for (int t = 0; t < NBT; ++t)
#pragma unroll
            for (int i = 0; i < 16; ++i) acc[r][t][i] = 0.f;

    // epilogue mapping, thread -> (weight row, batch column): consecutive threads write
    // consecutive rows of out[b][..]
    constexpr uint32_t ROWS = 32 * RT, COLS_PER_PASS = WAVES * 64 / ROWS, PASSES = 32 * NBT / COLS_PER_PASS;
    const uint32_t row = threadIdx.x % ROWS, bsub = threadIdx.x / ROWS;
    // (fetched ahead only where a thread has one or two outputs: more would cost the loop registers)
    constexpr bool ROPE_AHEAD = PASSES <= 2;
    Q4RopeFetch rope_pre[ROPE_AHEAD ? PASSES : 1];
    if (ROPE_AHEAD && a.rope_on) {
#pragma unroll
        for (uint32_t pass = 0; pass < PASSES; ++pass)
            rope_pre[pass] = q4_rope_prefetch(a.rope, pass * COLS_PER_PASS + bsub, tile0 * 32 + row);
    }

    // (the fused residual add: the residual and gamma of this thread's outputs, fetched ahead like the
    // RoPE operands)
    constexpr bool ADD_AHEAD = IOP && RT == 1 && PASSES <= 2;
    float resid_pre[ADD_AHEAD ? PASSES : 1] = {};
    float gamma_pre = 1.0f;
    if constexpr (ADD_AHEAD) {
        if (a.add_resid) {
#pragma unroll
            for (uint32_t pass = 0; pass < PASSES; ++pass) {
                const uint32_t b = pass * COLS_PER_PASS + bsub;
                if (b < a.batch) resid_pre[pass] = a.add_resid[(size_t)b * a.rows + tile0 * 32 + row];
            }
            if (tile0 * 32 + row < a.n_gamma) gamma_pre = a.gamma[tile0 * 32 + row];
        }
    }

    // A block's weights (3 registers per row tile, from HBM) and its activations (16 per batch tile,
    // from the L2) are fetched separately: the weights further ahead, PFW blocks, where the registers
    // allow it.  A wave of the TinyLlama shapes has four blocks in all, so all of its weights are on
    // the way from the start instead of in two rounds of a memory latency each.
    constexpr int PFW = (IOP && WAVES >= 16 && (RT == 1 || (SILU && !BS))) ? 4 : PF;
    static_assert(PFW % PF == 0, "a block's activations sit in slot (block number) % PF");
    struct BlockW {
        uint2 q[RT];
        _Float16 d[RT];
        bool real;               // false: a repeat past the end of the slice, multiplied with scale 0
    };
    struct BlockX {
        q4_half8 x[NBT][2][2];  // [batch tile][k step][hi, lo]
        uint4 ex[BS ? NBT : 1];   // BS: scale exponents of the 16 batch columns in this lane's registers, a byte each
    };
    auto load_w = [&](uint32_t blk_raw, BlockW& k) __attribute__((always_inline)) {
        // Past the end of the slice: a repeat of its last block, multiplied with the scale set to
        // zero, so that the multiply needs no branch (a branch lets the compiler sink these loads
        // into it, next to their use, which undoes the prefetch).
        const uint32_t blk = min(blk_raw, b1 - 1u);
        k.real = blk_raw < b1;
#pragma unroll
        for (int r = 0; r < RT; ++r) {
            const size_t tb = (size_t)(tile0 + r * tile_step) * a.nblocks + blk;
            // (non-temporal: a weight is read once per launch and need not stay in the L2)
            k.q[r] = q4_stream_u2(a.qs + tb * 64 + lane);
            k.d[r] = __builtin_nontemporal_load(a.d + tb * 32 + l32);
        }
    };
    auto load_x = [&](uint32_t blk_raw, BlockX& k) __attribute__((always_inline)) {
        const uint32_t blk = min(blk_raw, b1 - 1u);
#pragma unroll
        for (int t = 0; t < NBT; ++t)
#pragma unroll
            for (int ks = 0; ks < 2; ++ks)
#pragma unroll
                for (int p = 0; p < 2; ++p)
                    k.x[t][ks][p] = *reinterpret_cast<const q4_half8*>(
                        a.xfrag + ((((size_t)t * ksteps + blk * 2 + ks) * 2 + p) * 64 + lane_x) * 8);
        if constexpr (BS) {
            // register i of the accumulator is batch column (i/4)*8 + (lane/32)*4 + i%4
#pragma unroll
            for (int t = 0; t < NBT; ++t)
                k.ex[t] = *reinterpret_cast<const uint4*>(a.blk_exp + ((size_t)t * a.nblocks + blk) * 32 + (lane / 32) * 16);
        }
    };
    auto multiply = [&](const BlockW& k, const BlockX& kx) __attribute__((always_inline)) {
        if constexpr (IOP) {
#pragma unroll
            for (int r = 0; r < RT; ++r) {
                // (SILU: one row tile's products after the other, or the scheduler keeps three
                // sets of 16 in flight and the loop no longer fits the 128 registers a wave has)
                if constexpr (SILU && WAVES == 16) { if (r) __builtin_amdgcn_sched_barrier(0); }
                const float d = k.real ? (float)k.d[r] : 0.0f;
                q4_half8 w[2];
#pragma unroll
                for (int ks = 0; ks < 2; ++ks) {
                    const uint32_t w0 = (ks ? (k.q[r].x >> 4) : k.q[r].x) & 0x0F0F0F0Fu;
                    const uint32_t w1 = (ks ? (k.q[r].y >> 4) : k.q[r].y) & 0x0F0F0F0Fu;
                    const q4_half2 n0 = q4_pair(w0, 0x04010400u), n1 = q4_pair(w0, 0x04030402u);
                    const q4_half2 n2 = q4_pair(w1, 0x04010400u), n3 = q4_pair(w1, 0x04030402u);
                    w[ks] = q4_half8{n0[0], n0[1], n1[0], n1[1], n2[0], n2[1], n3[0], n3[1]};
                }
#pragma unroll
                for (int t = 0; t < NBT; ++t) {
                    q4_float16 sblk;
#pragma unroll
                    for (int i = 0; i < 16; ++i) sblk[i] = 0.f;
#pragma unroll
                    for (int ks = 0; ks < 2; ++ks) {
                        sblk = __builtin_amdgcn_mfma_f32_32x32x16_f16(kx.x[t][ks][0], w[ks], sblk, 0, 0, 0);
                        sblk = __builtin_amdgcn_mfma_f32_32x32x16_f16(kx.x[t][ks][1], w[ks], sblk, 0, 0, 0);
                    }
                    if constexpr (BS) {
#pragma unroll
                        for (int j = 0; j < 4; ++j) {
                            const uint32_t e4 = j == 0 ? kx.ex[t].x : j == 1 ? kx.ex[t].y : j == 2 ? kx.ex[t].z : kx.ex[t].w;
#pragma unroll
                            for (int e = 0; e < 4; ++e) {
                                const int ex = (int)(e4 << (24 - 8 * e)) >> 24;   // signed byte e
                                acc[r][t][j * 4 + e] = fmaf(__builtin_ldexpf(d, ex), sblk[j * 4 + e], acc[r][t][j * 4 + e]);
                            }
                            // (16 waves with two row tiles: four scaled values of d at a time, not sixteen,
                            // or the loop does not fit the 128 registers a wave has)
                            if constexpr (SILU && WAVES == 16) __builtin_amdgcn_sched_barrier(0);
                        }
                    } else {
#pragma unroll
                        for (int i = 0; i < 16; ++i) acc[r][t][i] = fmaf(d, sblk[i], acc[r][t][i]);
                    }
                }
            }
            return;
        }
#pragma unroll
        for (int r = 0; r < RT; ++r) {
            const _Float16 d = k.real ? k.d[r] : (_Float16)0.0f;
            const q4_half2 d2 = {d, d};
            // k step 0: low nibbles of this lane's 8 bytes, k step 1: high nibbles
#pragma unroll
            for (int ks = 0; ks < 2; ++ks) {
                const uint32_t w0 = (ks ? (k.q[r].x >> 4) : k.q[r].x) & 0x0F0F0F0Fu;
                const uint32_t w1 = (ks ? (k.q[r].y >> 4) : k.q[r].y) & 0x0F0F0F0Fu;
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
                    acc[r][t] = __builtin_amdgcn_mfma_f32_32x32x16_f16(whi, kx.x[t][ks][0], acc[r][t], 0, 0, 0);
                    acc[r][t] = __builtin_amdgcn_mfma_f32_32x32x16_f16(whi, kx.x[t][ks][1], acc[r][t], 0, 0, 0);
                    acc[r][t] = __builtin_amdgcn_mfma_f32_32x32x16_f16(wlo, kx.x[t][ks][0], acc[r][t], 0, 0, 0);
                }
            }
        }
    };

    // The empty asm statements (they claim to touch memory) pin every group of loads where it
    // is written: without them the compiler moves the loads for a later block down to just
    // before their use, across the loop's back edge too, and the prefetch is gone.
    // The RMSNorm that the producer of the activations left unfinished (ssq_in): the requests'
    // sums of squares, for the factors in the epilogue, and this thread's elements of the norm's own
    // output, which is written at the end.  Thread (request b, part p) takes the partials of tiles
    // p, p + SSQ_P, ...; their loads go out first, so that they are back and summed up while the
    // first blocks' are on the way, and take no registers through the main loop.
    float rms_h[BS ? RMS_NE : 1] = {};
    float ssq_part[BS ? SSQ_NL : 1] = {};
    if constexpr (BS) {
        if (a.ssq_in) {
            const uint32_t sb = threadIdx.x % (32 * NBT), sp = threadIdx.x / (32 * NBT);
#pragma unroll
            for (int j = 0; j < SSQ_NL; ++j) {
                const uint32_t tl = sp + j * SSQ_P;
                if (tl < a.ssq_tiles && sb < a.batch) ssq_part[j] = a.ssq_in[tl * 64 + sb];
            }
            const uint32_t n_el = a.batch * a.rms_len, n_thr = gridDim.x * (WAVES * 64);
#pragma unroll
            for (int j = 0; j < RMS_NE; ++j) {
                const uint32_t el = j * n_thr + blockIdx.x * (WAVES * 64) + threadIdx.x;
                if (el < n_el) rms_h[j] = a.rms_src[el];
            }
            asm volatile("" ::: "memory");
        }
    }
    BlockW k[PFW];
    BlockX kx[PF];
#pragma unroll
    for (int i = 0; i < PFW; ++i) {
        load_w(b0 + wave + i * WAVES, k[i]);
        asm volatile("" ::: "memory");
    }
#pragma unroll
    for (int i = 0; i < PF; ++i) {
        load_x(b0 + wave + i * WAVES, kx[i]);
        asm volatile("" ::: "memory");
    }
    if constexpr (BS) {
        if (a.ssq_in) {
            float part = 0.f;
#pragma unroll
            for (int j = 0; j < SSQ_NL; ++j) part += ssq_part[j];
            ssq_lds[threadIdx.x] = part;   // [part][request]; read behind the barrier that follows the main loop
#pragma unroll
            for (int j = 0; j < RMS_NE; ++j) rms_h_lds[j * WAVES * 64 + threadIdx.x] = rms_h[j];
            asm volatile("" ::: "memory");
        }
    }
    for (uint32_t base = b0 + wave; base < b1; base += PFW * WAVES) {
#pragma unroll
        for (int i = 0; i < PFW; ++i) {
            multiply(k[i], kx[i % PF]);
            load_w(base + (i + PFW) * WAVES, k[i]);
            load_x(base + (i + PF) * WAVES, kx[i % PF]);
            asm volatile("" ::: "memory");
        }
    }

    // ---- the waves' sums meet in LDS.  Accumulator layout: lane holds batch column l32 of the
    // tile and, in register i, weight row (i/4)*8 + (lane/32)*4 + i%4 of the 32-row tile (IOP:
    // the other way round, lane holds the weight row and the register the batch column).
#pragma unroll
    for (int r = 0; r < RT; ++r)
#pragma unroll
        for (int t = 0; t < NBT; ++t)
#pragma unroll
            for (int i = 0; i < 16; ++i)
                red[(((wave * RT + r) * NBT + t) * 16 + i) * PITCH + lane] = acc[r][t][i];
    __syncthreads();
    if constexpr (BS) {
        if (a.ssq_in) {
            if (threadIdx.x < 32 * NBT) {
                float total = 0.f;
#pragma unroll
                for (int sp = 0; sp < SSQ_P; ++sp) total += ssq_lds[sp * 32 * NBT + threadIdx.x];
                rms_scale[threadIdx.x] = 1.0f / sqrtf(total / (float)a.rms_len + a.rms_eps);
            }
            __syncthreads();
            // the norm's own output: h * factor * gamma, the arithmetic of rms_norm_batched_kernel
            const uint32_t n_el = a.batch * a.rms_len, n_thr = gridDim.x * (WAVES * 64);
#pragma unroll
            for (int j = 0; j < RMS_NE; ++j) {
                const uint32_t el = j * n_thr + blockIdx.x * (WAVES * 64) + threadIdx.x;
                if (el < n_el) {
                    const uint32_t rb = el / a.rms_len, rc = el - rb * a.rms_len;
                    const float gm = rc < a.n_gamma ? a.gamma[rc] : 1.0f;
                    a.rms_out[el] = rms_h_lds[j * WAVES * 64 + threadIdx.x] * rms_scale[rb] * gm;
                }
            }
        }
    }
    if constexpr (SILU) {
        // thread -> (column rr of the workgroup's 32 ffn columns, request b); the 32 lanes of a half
        // wave hold one request's 32 columns, which are one block of the consuming matmul's K
        constexpr uint32_t B_PER_PASS = WAVES * 2, S_PASSES = 32 * NBT / B_PER_PASS;
        const uint32_t rr = threadIdx.x % 32, bs = threadIdx.x / 32;
        const uint32_t col = tile0 * 32 + rr;            // column of gate / up / silu_out
#pragma unroll
        for (uint32_t pass = 0; pass < S_PASSES; ++pass) {
            const uint32_t b = pass * B_PER_PASS + bs;
            const bool live = b < a.batch;
            const uint32_t t = b / 32, in_reg = b % 32;
            const uint32_t i = (in_reg / 8) * 4 + in_reg % 4, ln = ((in_reg % 8) / 4) * 32 + rr;
            float sg = 0.f, su = 0.f;
#pragma unroll
            for (int w = 0; w < WAVES; ++w) {
                sg += red[(((w * RT + 0) * NBT + t) * 16 + i) * PITCH + ln];
                su += red[(((w * RT + 1) * NBT + t) * 16 + i) * PITCH + ln];
            }
            float prod = 0.f;
            if (live) {
                const float inv = BS ? (a.ssq_in ? rms_scale[b] : 1.0f) : a.inv_scale[b];
                const float gv = sg * inv, uv = su * inv;
                prod = q4_silu_times(gv, uv);
                a.out[(size_t)b * a.rows + col] = gv;
                a.out[(size_t)b * a.rows + a.ffn_inner + col] = uv;
                a.gate[(size_t)b * a.ffn_inner + col] = gv;
                a.up[(size_t)b * a.ffn_inner + col] = uv;
                a.silu_out[(size_t)b * a.ffn_inner + col] = prod;
            }
            // (uniform; requests past the batch are written as zeros)
            if (a.split_frag) q4_emit_block(prod, b, col, a.ffn_inner, a.split_frag, a.split_blk_exp);
        }
        return;
    }
    const uint32_t r = row / 32, rr = row % 32;
    float* out = a.out + (size_t)slice * a.batch * a.rows;
#pragma unroll
    for (uint32_t pass = 0; pass < PASSES; ++pass) {
        const uint32_t b = pass * COLS_PER_PASS + bsub;
        const bool fused_add = IOP && RT == 1 && a.add_resid;   // (uniform; then a half wave is one request's 32 columns)
        if (b >= a.batch && !fused_add) continue;
        if (a.bsplit == 2 && (b % 32) / 16 != bz) continue;   // the other half's workgroup has these requests
        const bool live = b < a.batch;
        const uint32_t t = b / 32;
        const uint32_t in_reg = IOP ? b % 32 : rr, in_lane = IOP ? rr : b % 32;
        const uint32_t i = (in_reg / 8) * 4 + in_reg % 4, ln = ((in_reg % 8) / 4) * 32 + in_lane;
        float sum = 0.f;
#pragma unroll
        for (int w = 0; w < WAVES; ++w) sum += red[(((w * RT + r) * NBT + t) * 16 + i) * PITCH + ln];
        float val;
        if constexpr (BS) val = a.ssq_in ? sum * rms_scale[b % (32 * NBT)] : sum;
        else val = live ? sum * a.inv_scale[b] : 0.f;
        const uint32_t col = tile0 * 32 + row;
        if (live) out[(size_t)b * a.rows + col] = val;
        if (a.rope_on)  // (the lanes of a pair share b)
            q4_rope_epilogue(a.rope, ROPE_AHEAD ? rope_pre[ROPE_AHEAD ? pass : 0] : q4_rope_prefetch(a.rope, b, col), b, col, val);
        if constexpr (IOP && RT == 1) {
            if (fused_add) {
                // residual add, this request's sum of squares over the 32 columns, and h * gamma as the
                // next matmul's fragments (requests past the batch: zeros)
                float hv = 0.f;
                if (live) {
                    hv = val + (ADD_AHEAD ? resid_pre[ADD_AHEAD ? pass : 0] : a.add_resid[(size_t)b * a.rows + col]);
                    a.add_out[(size_t)b * a.rows + col] = hv;
                }
                const float ssq = q4_half_wave_sum(hv * hv);
                if (row == 0 && live) a.ssq_out[(size_t)tile0 * 64 + b] = ssq;
                const float gm = ADD_AHEAD ? gamma_pre : (col < a.n_gamma ? a.gamma[col] : 1.0f);
                q4_emit_block(hv * gm, b, col, a.rows, a.split_frag, a.split_blk_exp);
            }
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
