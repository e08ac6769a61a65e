// HipExecutor: the C++ host side above the C ABI (include/mlc_hip.h).
//
// It serves, with identical names, argument order, ownership and bool-return
// conventions, the methods of the reference's mlc::runtime::MetalExecutor that
// the paged-KV path uses (compiler/runtime/metal_runtime.hpp:27, 181-183,
// 510-533, 619-703).  A HIP build of the reference runtime defines those
// MetalExecutor methods as one-line forwards to this class (or straight to the
// C ABI), which lets paged_kv.cpp, batched_walker.cpp and the scheduler compile
// and run unchanged.
#pragma once

#include <cstddef>
#include <cstdint>
#include <string>
#include <vector>

namespace mlc_amd {

class HipExecutor {
public:
    static HipExecutor& Instance();

    bool isAvailable() const;
    const char* lastError() const;

    // metal_runtime.hpp:181-183
    bool beginForwardPassCB() const;
    bool flushForwardPassCB() const;
    bool hasForwardPassCB() const;

    // metal_runtime.hpp:510-523
    bool encodePagedFlashAttention(void* q_buf, void* k_pages_buf, void* v_pages_buf, void* o_buf,
                                   const std::vector<uint32_t>& page_tables_flat,
                                   const std::vector<uint32_t>& page_table_offsets,
                                   const std::vector<uint32_t>& seq_lens,
                                   const std::vector<uint32_t>& q_positions,
                                   size_t batch, size_t num_heads, size_t kv_heads,
                                   size_t head_dim, size_t page_size_tokens,
                                   bool apply_causal) const;

    // metal_runtime.hpp:526-533
    bool encodeScatterKVPagedBatched(void* page_storage_buffer,
                                     const std::vector<uint32_t>& page_ids,
                                     const std::vector<uint32_t>& slots_in_page,
                                     size_t page_size_tokens, size_t n_kv_heads, size_t head_dim,
                                     size_t batch, const void* src_buffer) const;

    // metal_runtime.hpp:619-626
    bool gatherKVPages(void* page_storage_buffer, const std::vector<uint32_t>& page_table,
                       size_t page_size_tokens, size_t n_kv_heads, size_t head_dim,
                       size_t num_tokens, void* dst_buffer, size_t dtype_bytes) const;

    // metal_runtime.hpp:645-658
    bool runPagedFlashAttention(void* q_buffer, void* k_pages_buffer, void* v_pages_buffer,
                                void* o_buffer,
                                const std::vector<uint32_t>& page_tables_flat,
                                const std::vector<uint32_t>& page_table_offsets,
                                const std::vector<uint32_t>& seq_lens,
                                const std::vector<uint32_t>& q_positions,
                                size_t batch, size_t num_heads, size_t kv_heads, size_t head_dim,
                                size_t page_size_tokens, bool apply_causal) const;

    // metal_runtime.hpp:666-674
    bool scatterKVPaged(void* page_storage_buffer, const std::vector<uint32_t>& page_table,
                        size_t page_size_tokens, size_t n_kv_heads, size_t head_dim,
                        size_t tokens, size_t start_slot, const void* src_buffer,
                        size_t dtype_bytes) const;

    // metal_runtime.hpp:680-687
    bool scatterKVPagedBatched(void* page_storage_buffer, const std::vector<uint32_t>& page_ids,
                               const std::vector<uint32_t>& slots_in_page,
                               size_t page_size_tokens, size_t n_kv_heads, size_t head_dim,
                               size_t batch, const void* src_buffer) const;

    // metal_runtime.hpp:540-547 (needs an open pass, like every encode* method)
    bool encodeQkvSplitRopeCast(void* qkv_buf, void* q_buf, void* k_buf, void* v_buf,
                                void* k_f16_buf, void* v_f16_buf, void* cos_buf, void* sin_buf,
                                size_t batch, size_t num_heads, size_t kv_heads, size_t head_dim,
                                size_t qkv_rows, size_t q_rows, size_t k_rows, size_t v_rows,
                                size_t rotary_dim) const;

    // The same step fused with the two batched KV scatters that follow it in the walker
    // (batched_walker.cpp:287-331); k_f32_buf / v_f32_buf may be null.  No reference method.
    bool encodeQkvSplitRopeScatter(void* qkv_buf, void* q_buf, void* k_pages_buffer,
                                   void* v_pages_buffer, void* k_f32_buf, void* v_f32_buf,
                                   void* cos_buf, void* sin_buf,
                                   const std::vector<uint32_t>& page_ids,
                                   const std::vector<uint32_t>& slots_in_page,
                                   size_t page_size_tokens, size_t batch, size_t num_heads,
                                   size_t kv_heads, size_t head_dim, size_t qkv_rows, size_t q_rows,
                                   size_t k_rows, size_t v_rows, size_t rotary_dim) const;

    // metal_runtime.hpp:474-479, 501-506, 549-552: the walker's small per-layer operators
    bool encodeRmsNormBatched(void* in_buf, const std::vector<float>& weight, float epsilon,
                              size_t batch, size_t length, void* out_buf) const;
    bool encodeAddBatched(void* a_buf, void* b_buf, void* out_buf, size_t total_elements) const;
    bool encodeSiluMulBatched(void* gate_buf, void* up_buf, void* out_buf,
                              size_t total_elements) const;
    bool encodeGateUpSplitSiluMul(void* gate_up_buf, void* gate_buf, void* up_buf, void* out_buf,
                                  size_t batch, size_t ffn_inner, size_t ffn_gate_up_rows) const;

    // metal_runtime.hpp:481-489
    bool encodeMatMulQ4_0Batched(const std::string& weight_name, const std::vector<uint8_t>& weights,
                                 void* in_buf, size_t batch, size_t rows, size_t cols,
                                 size_t row_stride, uint32_t quant_version, void* out_buf) const;

    // metal_runtime.hpp:491-498 (lm_head of the batched step) and :452-459 (the waiting form)
    bool encodeMatMulQ6KBatched(const std::string& weight_name, const std::vector<uint8_t>& weights,
                                void* in_buf, size_t batch, size_t rows, size_t cols,
                                size_t row_stride, void* out_buf) const;
    bool runMatMulQ6KBatched(const std::string& weight_name, const std::vector<uint8_t>& weights,
                             void* in_buf, size_t batch, size_t rows, size_t cols,
                             size_t row_stride, void* out_buf) const;

    // Chunked prefill over paged KV: no reference method (the reference loops its
    // decode path per prompt token, batched_executor.cpp:454-466).
    bool runPagedPrefillAttention(void* q_f16_buffer, void* k_pages_buffer, void* v_pages_buffer,
                                  void* o_buffer,
                                  const std::vector<uint32_t>& page_tables_flat,
                                  const std::vector<uint32_t>& page_table_offsets,
                                  const std::vector<uint32_t>& seq_lens,
                                  const std::vector<uint32_t>& q_start,
                                  size_t batch, size_t chunk, size_t num_heads, size_t kv_heads,
                                  size_t head_dim, size_t page_size_tokens) const;

    // metal_runtime.hpp:693-703
    void* allocateScratchBuffer(size_t bytes) const;
    void releaseScratchBuffer(void* buffer) const;
    void uploadToBuffer(void* buffer, const void* src, size_t bytes, size_t dst_offset = 0) const;
    void downloadFromBuffer(const void* buffer, void* dst, size_t bytes,
                            size_t src_offset = 0) const;
    void* getOrAllocCachedBuffer(const char* name, size_t bytes) const;

private:
    HipExecutor() = default;
};

}  // namespace mlc_amd
