// HipExecutor: vector-taking C++ methods forwarded to the C ABI.  The length
// checks the reference makes on its std::vector arguments
// (compiler/runtime/metal_runtime.mm:7241-7243, 7747-7749) live here, because
// the C ABI only sees pointers.
#include "hip_executor.hpp"

#include "../../include/mlc_hip.h"

namespace mlc_amd {

namespace {
const uint32_t kNoIds[1] = {0};
const uint32_t* data_or_dummy(const std::vector<uint32_t>& v) {
    return v.empty() ? kNoIds : v.data();
}
}  // namespace

HipExecutor& HipExecutor::Instance() {
    static HipExecutor inst;
    return inst;
}

bool HipExecutor::isAvailable() const { return mlc_hip_available() != 0; }
const char* HipExecutor::lastError() const { return mlc_hip_last_error(); }

bool HipExecutor::beginForwardPassCB() const { return mlc_hip_begin() != 0; }
bool HipExecutor::flushForwardPassCB() const { return mlc_hip_flush() != 0; }
bool HipExecutor::hasForwardPassCB() const { return mlc_hip_has_open_pass() != 0; }

bool HipExecutor::encodePagedFlashAttention(void* q_buf, void* k_pages_buf, void* v_pages_buf,
                                            void* o_buf,
                                            const std::vector<uint32_t>& page_tables_flat,
                                            const std::vector<uint32_t>& page_table_offsets,
                                            const std::vector<uint32_t>& seq_lens,
                                            const std::vector<uint32_t>& q_positions,
                                            size_t batch, size_t num_heads, size_t kv_heads,
                                            size_t head_dim, size_t page_size_tokens,
                                            bool apply_causal) const {
    // The reference's encode variant trusts its caller; vectors that are too short
    // would be read out of bounds here, so they are refused instead.
    if (page_table_offsets.size() < batch + 1 || seq_lens.size() < batch ||
        q_positions.size() < batch)
        return false;
    return mlc_hip_paged_attn_decode(q_buf, k_pages_buf, v_pages_buf, o_buf,
                                     data_or_dummy(page_tables_flat), page_tables_flat.size(),
                                     page_table_offsets.data(), seq_lens.data(),
                                     q_positions.data(), batch, num_heads, kv_heads, head_dim,
                                     page_size_tokens, apply_causal ? 1 : 0, /*sync=*/0) != 0;
}

bool HipExecutor::runPagedFlashAttention(void* q_buffer, void* k_pages_buffer,
                                         void* v_pages_buffer, void* o_buffer,
                                         const std::vector<uint32_t>& page_tables_flat,
                                         const std::vector<uint32_t>& page_table_offsets,
                                         const std::vector<uint32_t>& seq_lens,
                                         const std::vector<uint32_t>& q_positions,
                                         size_t batch, size_t num_heads, size_t kv_heads,
                                         size_t head_dim, size_t page_size_tokens,
                                         bool apply_causal) const {
    if (page_table_offsets.size() != batch + 1) return false;                 // :7747
    if (seq_lens.size() != batch || q_positions.size() != batch) return false;  // :7748
    return mlc_hip_paged_attn_decode(q_buffer, k_pages_buffer, v_pages_buffer, o_buffer,
                                     data_or_dummy(page_tables_flat), page_tables_flat.size(),
                                     page_table_offsets.data(), seq_lens.data(),
                                     q_positions.data(), batch, num_heads, kv_heads, head_dim,
                                     page_size_tokens, apply_causal ? 1 : 0, /*sync=*/1) != 0;
}

bool HipExecutor::encodeScatterKVPagedBatched(void* page_storage_buffer,
                                              const std::vector<uint32_t>& page_ids,
                                              const std::vector<uint32_t>& slots_in_page,
                                              size_t page_size_tokens, size_t n_kv_heads,
                                              size_t head_dim, size_t batch,
                                              const void* src_buffer) const {
    if (page_ids.size() < batch || slots_in_page.size() < batch) return false;
    return mlc_hip_scatter_kv_paged_batched_f16(page_storage_buffer, page_ids.data(),
                                                slots_in_page.data(), page_size_tokens,
                                                n_kv_heads, head_dim, batch, src_buffer,
                                                /*sync=*/0) != 0;
}

bool HipExecutor::scatterKVPagedBatched(void* page_storage_buffer,
                                        const std::vector<uint32_t>& page_ids,
                                        const std::vector<uint32_t>& slots_in_page,
                                        size_t page_size_tokens, size_t n_kv_heads,
                                        size_t head_dim, size_t batch,
                                        const void* src_buffer) const {
    if (page_ids.size() != batch || slots_in_page.size() != batch) return false;  // :7243
    return mlc_hip_scatter_kv_paged_batched_f16(page_storage_buffer, page_ids.data(),
                                                slots_in_page.data(), page_size_tokens,
                                                n_kv_heads, head_dim, batch, src_buffer,
                                                /*sync=*/1) != 0;
}

bool HipExecutor::scatterKVPaged(void* page_storage_buffer, const std::vector<uint32_t>& page_table,
                                 size_t page_size_tokens, size_t n_kv_heads, size_t head_dim,
                                 size_t tokens, size_t start_slot, const void* src_buffer,
                                 size_t dtype_bytes) const {
    return mlc_hip_scatter_kv_paged(page_storage_buffer, data_or_dummy(page_table),
                                    page_table.size(), page_size_tokens, n_kv_heads, head_dim,
                                    tokens, start_slot, src_buffer, dtype_bytes) != 0;
}

bool HipExecutor::gatherKVPages(void* page_storage_buffer, const std::vector<uint32_t>& page_table,
                                size_t page_size_tokens, size_t n_kv_heads, size_t head_dim,
                                size_t num_tokens, void* dst_buffer, size_t dtype_bytes) const {
    return mlc_hip_gather_kv_pages(page_storage_buffer, data_or_dummy(page_table),
                                   page_table.size(), page_size_tokens, n_kv_heads, head_dim,
                                   num_tokens, dst_buffer, dtype_bytes) != 0;
}

bool HipExecutor::encodeQkvSplitRopeCast(void* qkv_buf, void* q_buf, void* k_buf, void* v_buf,
                                         void* k_f16_buf, void* v_f16_buf, void* cos_buf,
                                         void* sin_buf, size_t batch, size_t num_heads,
                                         size_t kv_heads, size_t head_dim, size_t qkv_rows,
                                         size_t q_rows, size_t k_rows, size_t v_rows,
                                         size_t rotary_dim) const {
    return mlc_hip_qkv_split_rope_cast(qkv_buf, q_buf, k_buf, v_buf, k_f16_buf, v_f16_buf, cos_buf,
                                       sin_buf, batch, num_heads, kv_heads, head_dim, qkv_rows,
                                       q_rows, k_rows, v_rows, rotary_dim, /*sync=*/0) != 0;
}

bool HipExecutor::encodeQkvSplitRopeScatter(void* qkv_buf, void* q_buf, void* k_pages_buffer,
                                            void* v_pages_buffer, void* k_f32_buf, void* v_f32_buf,
                                            void* cos_buf, void* sin_buf,
                                            const std::vector<uint32_t>& page_ids,
                                            const std::vector<uint32_t>& slots_in_page,
                                            size_t page_size_tokens, size_t batch, size_t num_heads,
                                            size_t kv_heads, size_t head_dim, size_t qkv_rows,
                                            size_t q_rows, size_t k_rows, size_t v_rows,
                                            size_t rotary_dim) const {
    if (page_ids.size() < batch || slots_in_page.size() < batch) return false;
    return mlc_hip_qkv_split_rope_scatter(qkv_buf, q_buf, k_pages_buffer, v_pages_buffer, k_f32_buf,
                                          v_f32_buf, cos_buf, sin_buf, page_ids.data(),
                                          slots_in_page.data(), page_size_tokens, batch, num_heads,
                                          kv_heads, head_dim, qkv_rows, q_rows, k_rows, v_rows,
                                          rotary_dim, /*sync=*/0) != 0;
}

bool HipExecutor::encodeRmsNormBatched(void* in_buf, const std::vector<float>& weight, float epsilon,
                                       size_t batch, size_t length, void* out_buf) const {
    return mlc_hip_rms_norm_batched(in_buf, weight.data(), weight.size(), epsilon, batch, length,
                                    out_buf, /*sync=*/0) != 0;
}

bool HipExecutor::encodeAddBatched(void* a_buf, void* b_buf, void* out_buf,
                                   size_t total_elements) const {
    return mlc_hip_add_batched(a_buf, b_buf, out_buf, total_elements, /*sync=*/0) != 0;
}

bool HipExecutor::encodeSiluMulBatched(void* gate_buf, void* up_buf, void* out_buf,
                                       size_t total_elements) const {
    return mlc_hip_silu_mul_batched(gate_buf, up_buf, out_buf, total_elements, /*sync=*/0) != 0;
}

bool HipExecutor::encodeGateUpSplitSiluMul(void* gate_up_buf, void* gate_buf, void* up_buf,
                                           void* out_buf, size_t batch, size_t ffn_inner,
                                           size_t ffn_gate_up_rows) const {
    return mlc_hip_gate_up_split_silu_mul(gate_up_buf, gate_buf, up_buf, out_buf, batch, ffn_inner,
                                          ffn_gate_up_rows, /*sync=*/0) != 0;
}

bool HipExecutor::encodeMatMulQ4_0Batched(const std::string& weight_name,
                                          const std::vector<uint8_t>& weights, void* in_buf,
                                          size_t batch, size_t rows, size_t cols, size_t row_stride,
                                          uint32_t quant_version, void* out_buf) const {
    return mlc_hip_matmul_q4_0_batched(weight_name.c_str(), weights.data(), weights.size(), in_buf,
                                       batch, rows, cols, row_stride, quant_version, out_buf,
                                       /*sync=*/0) != 0;
}

bool HipExecutor::encodeMatMulQ6KBatched(const std::string& weight_name,
                                         const std::vector<uint8_t>& weights, void* in_buf,
                                         size_t batch, size_t rows, size_t cols, size_t row_stride,
                                         void* out_buf) const {
    return mlc_hip_matmul_q6_k_batched(weight_name.c_str(), weights.data(), weights.size(), in_buf,
                                       batch, rows, cols, row_stride, out_buf, /*sync=*/0) != 0;
}

bool HipExecutor::runMatMulQ6KBatched(const std::string& weight_name,
                                      const std::vector<uint8_t>& weights, void* in_buf, size_t batch,
                                      size_t rows, size_t cols, size_t row_stride,
                                      void* out_buf) const {
    return mlc_hip_matmul_q6_k_batched(weight_name.c_str(), weights.data(), weights.size(), in_buf,
                                       batch, rows, cols, row_stride, out_buf, /*sync=*/1) != 0;
}

bool HipExecutor::runPagedPrefillAttention(void* q_f16_buffer, void* k_pages_buffer,
                                           void* v_pages_buffer, void* o_buffer,
                                           const std::vector<uint32_t>& page_tables_flat,
                                           const std::vector<uint32_t>& page_table_offsets,
                                           const std::vector<uint32_t>& seq_lens,
                                           const std::vector<uint32_t>& q_start,
                                           size_t batch, size_t chunk, size_t num_heads,
                                           size_t kv_heads, size_t head_dim,
                                           size_t page_size_tokens) const {
    if (page_table_offsets.size() != batch + 1) return false;
    if (seq_lens.size() != batch || q_start.size() != batch) return false;
    return mlc_hip_paged_attn_prefill(q_f16_buffer, k_pages_buffer, v_pages_buffer, o_buffer,
                                      data_or_dummy(page_tables_flat), page_tables_flat.size(),
                                      page_table_offsets.data(), seq_lens.data(), q_start.data(),
                                      batch, chunk, num_heads, kv_heads, head_dim,
                                      page_size_tokens, /*sync=*/1) != 0;
}

void* HipExecutor::allocateScratchBuffer(size_t bytes) const { return mlc_hip_alloc(bytes); }
void HipExecutor::releaseScratchBuffer(void* buffer) const { mlc_hip_free(buffer); }
void HipExecutor::uploadToBuffer(void* buffer, const void* src, size_t bytes,
                                 size_t dst_offset) const {
    (void)mlc_hip_upload(buffer, src, bytes, dst_offset);
}
void HipExecutor::downloadFromBuffer(const void* buffer, void* dst, size_t bytes,
                                     size_t src_offset) const {
    (void)mlc_hip_download(buffer, dst, bytes, src_offset);
}
void* HipExecutor::getOrAllocCachedBuffer(const char* name, size_t bytes) const {
    return mlc_hip_cached(name, bytes);
}

}  // namespace mlc_amd
