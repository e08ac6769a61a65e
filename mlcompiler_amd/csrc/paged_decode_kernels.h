// Helpers shared by the paged flash-attention decode kernels for gfx950 (MI355X), wave64:
// fp16 vector types, DPP lane exchanges, wave reductions, the softmax constants.
//
// Semantics of the kernels that use them: MSL kernel paged_flash_attention of the reference
// (compiler/runtime/metal_runtime.mm:2216-2335): for each (request, query head)
//   O = softmax(q . K^T / sqrt(D), causal: kv_pos <= q_pos) . V
// with K/V rows read through the request's page table from fp16 pages laid out
// [page][slot][kv_head][dim], fp32 accumulation and fp32 output.
//
// Lane layout of the vector-pipe arithmetic (D = 64 or 128):
//   a K (or V) row of one KV head is D halves = D/8 16-byte chunks; lane
//   (r, c) = (lane / CPR, lane % CPR), CPR = D/8, holds chunk c of row r of a
//   "row group" of RPI = 64/CPR consecutive tokens, so one wave-wide 16-byte load
//   reads RPI whole rows, fully coalesced.  A tile is 8 row groups
//   (64 tokens for D=64, 32 for D=128).
//   QK: every lane forms the partial dot over its 8 dims for 8 row groups, then a
//   3-step reduce-scatter over the 8 c-lanes (DPP half-mirror, quad xor 2, quad
//   xor 1 fused into v_add_f32) leaves lane (r, c) holding the complete scores of
//   ONE token for all its heads.  To keep that exchange free of selects, register
//   j' of lane c holds row group j' ^ g(c), g(c) = c ^ ((c & 4) ? 3 : 0): the
//   swizzle is applied to the load address, which costs nothing.
//   Softmax: exp2 with log2(e)/sqrt(D) folded into q; the running reference
//   maximum is only raised when a tile exceeds it by more than 2^8 (exact math,
//   any reference works; this removes almost all accumulator rescales).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace mlc_hip {

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

}  // namespace mlc_hip
