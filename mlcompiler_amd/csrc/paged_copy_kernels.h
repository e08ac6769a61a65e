// Paged KV write / read kernels for gfx950: the batched one-row-per-request
// scatter of the decode step and the single-request multi-token scatter / gather
// that sit either side of it.  All of them are pure copies (bit-exact by
// construction); the only design point is that a token row of all KV heads is
// contiguous in a page, so rows move as 16-byte chunks with coalesced stores.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace mlc_hip {

// MSL scatter_kv_paged_batched_f16 (compiler/runtime/metal_runtime.mm:405-424):
//   page[page_ids[r]][slots[r]][kv][d] = src[r][kv][d].
// src row r (n_kv_heads*head_dim halves) and its destination row are both
// contiguous, so the copy runs in units of UNIT bytes (16 when everything is
// 16-byte aligned, else 2).
template <typename UnitT>
__global__ void scatter_kv_paged_batched_kernel(const UnitT* __restrict__ src,
                                                UnitT* __restrict__ page_storage,
                                                const uint32_t* __restrict__ page_ids,
                                                const uint32_t* __restrict__ slots,
                                                uint32_t batch, uint32_t row_units,
                                                uint32_t page_size) {
    const uint32_t gid = blockIdx.x * blockDim.x + threadIdx.x;
    if (gid >= batch * row_units) return;
    const uint32_t req = gid / row_units;
    const uint32_t u = gid - req * row_units;
    const size_t dst_row = (size_t)page_ids[req] * page_size + slots[req];
    page_storage[dst_row * row_units + u] = src[gid];
}

// The K row and the V row of a decode step in one launch: two scatter_kv_paged_batched copies
// with the same (page id, slot) per request.  The batched step encodes them back to back
// (compiler/runtime/batched_walker.cpp:304-307); each on its own costs a launch for 32 KiB.
template <typename UnitT>
__global__ void scatter_kv_pair_kernel(const UnitT* __restrict__ src0, UnitT* __restrict__ pages0,
                                       const UnitT* __restrict__ src1, UnitT* __restrict__ pages1,
                                       const uint32_t* __restrict__ page_ids,
                                       const uint32_t* __restrict__ slots, uint32_t batch,
                                       uint32_t row_units, uint32_t page_size, uint32_t n_tensors) {
    // n_tensors = 1: only the first copy exists (src1 / pages1 are null and must not be touched)
    const uint32_t gid = blockIdx.x * blockDim.x + threadIdx.x;
    const uint32_t per = batch * row_units;
    if (gid >= n_tensors * per) return;
    const uint32_t which = gid / per, e = gid - which * per;
    const uint32_t req = e / row_units;
    const uint32_t u = e - req * row_units;
    const size_t dst_row = (size_t)page_ids[req] * page_size + slots[req];
    if (which == 0) pages0[dst_row * row_units + u] = src0[e];
    else pages1[dst_row * row_units + u] = src1[e];
}

// MSL scatter_kv_paged_f16/f32 (metal_runtime.mm:468-512): src is
// [kv][token][dim]; token t goes to absolute slot start_slot + t of the page
// table.  One thread per UNIT of a (kv, token) row of head_dim elements.
template <typename UnitT>
__global__ void scatter_kv_paged_kernel(const UnitT* __restrict__ src,
                                        UnitT* __restrict__ page_storage,
                                        const uint32_t* __restrict__ page_table,
                                        uint32_t n_kv_heads, uint32_t tokens, uint32_t head_units,
                                        uint32_t page_size, uint32_t start_slot) {
    const size_t gid = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t total = (size_t)n_kv_heads * tokens * head_units;
    if (gid >= total) return;
    const uint32_t u = (uint32_t)(gid % head_units);
    const size_t tmp = gid / head_units;
    const uint32_t token = (uint32_t)(tmp % tokens);
    const uint32_t kv = (uint32_t)(tmp / tokens);
    const uint32_t abs_slot = start_slot + token;
    const uint32_t page_idx = abs_slot / page_size;
    const uint32_t slot = abs_slot - page_idx * page_size;
    const size_t dst = (((size_t)page_table[page_idx] * page_size + slot) * n_kv_heads + kv) *
                           head_units + u;
    page_storage[dst] = src[gid];
}

// MSL gather_kv_pages_f16/f32 (metal_runtime.mm:328-370): the inverse, into
// dst [kv][token][dim].
template <typename UnitT>
__global__ void gather_kv_pages_kernel(const UnitT* __restrict__ page_storage,
                                       UnitT* __restrict__ dst,
                                       const uint32_t* __restrict__ page_table,
                                       uint32_t n_kv_heads, uint32_t num_tokens,
                                       uint32_t head_units, uint32_t page_size) {
    const size_t gid = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t total = (size_t)n_kv_heads * num_tokens * head_units;
    if (gid >= total) return;
    const uint32_t u = (uint32_t)(gid % head_units);
    const size_t tmp = gid / head_units;
    const uint32_t tok = (uint32_t)(tmp % num_tokens);
    const uint32_t kv = (uint32_t)(tmp / num_tokens);
    const uint32_t page_idx = tok / page_size;
    const uint32_t slot = tok - page_idx * page_size;
    const size_t s = (((size_t)page_table[page_idx] * page_size + slot) * n_kv_heads + kv) *
                         head_units + u;
    dst[gid] = page_storage[s];
}

}  // namespace mlc_hip
