// Chunked-prefill paged attention (MFMA path) for gfx950 -- placeholder until the
// kernel lands: every shape is reported unsupported, so the C ABI entry fails loudly.
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

inline bool prefill_shape_supported(size_t, size_t) { return false; }
inline void launch_prefill(const PrefillArgs&, size_t, hipStream_t) {}

}  // namespace mlc_hip
