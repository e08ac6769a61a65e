// The translation unit a HIP build of the reference adds in place of metal_runtime.mm: the
// paged-path methods of mlc::runtime::MetalExecutor (compiler/runtime/metal_runtime.hpp:23-711)
// forwarded to the C ABI of libmlc_hip.so (include/mlc_hip.h).  It is compiled against the
// reference's own header where that lies (tests/integration/Makefile); nothing of the
// reference is part of this file.
//
// Defined here: every MetalExecutor method that compiler/runtime/paged_kv.cpp and
// compiler/runtime/batched_walker.cpp call, plus the paged-path test entry points
// (tests/test_paged_kv.cpp, tests/test_paged_flash.cpp).  Buffer handles are device pointers;
// std::vector metadata is borrowed for the call (copied inside), as in the reference.
#include "runtime/metal_runtime.hpp"

#include <stdexcept>

#include "mlc_hip.h"

namespace mlc {
namespace runtime {

struct MetalExecutor::Impl {};

MetalExecutor::MetalExecutor() = default;
MetalExecutor::~MetalExecutor() = default;

MetalExecutor& MetalExecutor::Instance() {  // metal_runtime.mm:5774-5777
    static MetalExecutor instance;
    return instance;
}

bool MetalExecutor::isAvailable() const { return mlc_hip_available() != 0; }

void MetalExecutor::requireAvailable() const {  // metal_runtime.mm:5786-5790
    if (!isAvailable()) throw std::runtime_error(std::string("MI355X (gfx950) device unavailable: ") + mlc_hip_last_error());
}

// ---- buffers: metal_runtime.mm:8218-8297
void* MetalExecutor::allocateScratchBuffer(size_t bytes) const { return mlc_hip_alloc(bytes); }
void MetalExecutor::releaseScratchBuffer(void* buffer) const { mlc_hip_free(buffer); }
void* MetalExecutor::getOrAllocCachedBuffer(const char* name, size_t bytes) const { return mlc_hip_cached(name, bytes); }
void MetalExecutor::uploadToBuffer(void* buffer, const void* src, size_t bytes, size_t dst_offset) const {
    (void)mlc_hip_upload(buffer, src, bytes, dst_offset);
}
void MetalExecutor::downloadFromBuffer(const void* buffer, void* dst, size_t bytes, size_t src_offset) const {
    (void)mlc_hip_download(buffer, dst, bytes, src_offset);
}

// ---- the per-pass command buffer: metal_runtime.mm:6000-6064
bool MetalExecutor::beginForwardPassCB() const { return mlc_hip_begin() != 0; }
bool MetalExecutor::flushForwardPassCB() const { return mlc_hip_flush() != 0; }
bool MetalExecutor::hasForwardPassCB() const { return mlc_hip_has_open_pass() != 0; }

// ---- paged attention: metal_runtime.mm:7074-7166 (encode) and :7727-7826 (run)
bool MetalExecutor::encodePagedFlashAttention(void* q_buf, void* k_pages_buf, void* v_pages_buf, void* o_buf,
                                              const std::vector<uint32_t>& page_tables_flat,
                                              const std::vector<uint32_t>& page_table_offsets,
                                              const std::vector<uint32_t>& seq_lens,
                                              const std::vector<uint32_t>& q_positions, size_t batch,
                                              size_t num_heads, size_t kv_heads, size_t head_dim,
                                              size_t page_size_tokens, bool apply_causal) const {
    // the reference's encode variant validates nothing; the vectors must at least hold what is read
    if (page_table_offsets.size() < batch + 1 || seq_lens.size() < batch || q_positions.size() < batch) return false;
    return mlc_hip_paged_attn_decode(q_buf, k_pages_buf, v_pages_buf, o_buf, page_tables_flat.data(),
                                     page_tables_flat.size(), page_table_offsets.data(), seq_lens.data(),
                                     q_positions.data(), batch, num_heads, kv_heads, head_dim, page_size_tokens,
                                     apply_causal ? 1 : 0, /*sync=*/0) != 0;
}

bool MetalExecutor::runPagedFlashAttention(void* q_buffer, void* k_pages_buffer, void* v_pages_buffer,
                                           void* o_buffer, const std::vector<uint32_t>& page_tables_flat,
                                           const std::vector<uint32_t>& page_table_offsets,
                                           const std::vector<uint32_t>& seq_lens,
                                           const std::vector<uint32_t>& q_positions, size_t batch,
                                           size_t num_heads, size_t kv_heads, size_t head_dim,
                                           size_t page_size_tokens, bool apply_causal) const {
    if (page_table_offsets.size() != batch + 1 || seq_lens.size() != batch || q_positions.size() != batch)
        return false;  // metal_runtime.mm:7747-7748
    return mlc_hip_paged_attn_decode(q_buffer, k_pages_buffer, v_pages_buffer, o_buffer, page_tables_flat.data(),
                                     page_tables_flat.size(), page_table_offsets.data(), seq_lens.data(),
                                     q_positions.data(), batch, num_heads, kv_heads, head_dim, page_size_tokens,
                                     apply_causal ? 1 : 0, /*sync=*/1) != 0;
}

// ---- KV writes and reads: metal_runtime.mm:7168-7294, :7828-7906, :7647-7721
bool MetalExecutor::encodeScatterKVPagedBatched(void* page_storage_buffer, const std::vector<uint32_t>& page_ids,
                                                const std::vector<uint32_t>& slots_in_page,
                                                size_t page_size_tokens, size_t n_kv_heads, size_t head_dim,
                                                size_t batch, const void* src_buffer) const {
    if (page_ids.size() < batch || slots_in_page.size() < batch) return false;
    return mlc_hip_scatter_kv_paged_batched_f16(page_storage_buffer, page_ids.data(), slots_in_page.data(),
                                                page_size_tokens, n_kv_heads, head_dim, batch, src_buffer, 0) != 0;
}

bool MetalExecutor::scatterKVPagedBatched(void* page_storage_buffer, const std::vector<uint32_t>& page_ids,
                                          const std::vector<uint32_t>& slots_in_page, size_t page_size_tokens,
                                          size_t n_kv_heads, size_t head_dim, size_t batch,
                                          const void* src_buffer) const {
    if (page_ids.size() != batch || slots_in_page.size() != batch) return false;  // metal_runtime.mm:7243
    return mlc_hip_scatter_kv_paged_batched_f16(page_storage_buffer, page_ids.data(), slots_in_page.data(),
                                                page_size_tokens, n_kv_heads, head_dim, batch, src_buffer, 1) != 0;
}

bool MetalExecutor::scatterKVPaged(void* page_storage_buffer, const std::vector<uint32_t>& page_table,
                                   size_t page_size_tokens, size_t n_kv_heads, size_t head_dim, size_t tokens,
                                   size_t start_slot, const void* src_buffer, size_t dtype_bytes) const {
    return mlc_hip_scatter_kv_paged(page_storage_buffer, page_table.data(), page_table.size(), page_size_tokens,
                                    n_kv_heads, head_dim, tokens, start_slot, src_buffer, dtype_bytes) != 0;
}

bool MetalExecutor::gatherKVPages(void* page_storage_buffer, const std::vector<uint32_t>& page_table,
                                  size_t page_size_tokens, size_t n_kv_heads, size_t head_dim, size_t num_tokens,
                                  void* dst_buffer, size_t dtype_bytes) const {
    return mlc_hip_gather_kv_pages(page_storage_buffer, page_table.data(), page_table.size(), page_size_tokens,
                                   n_kv_heads, head_dim, num_tokens, dst_buffer, dtype_bytes) != 0;
}

// ---- the walker's layer loop: metal_runtime.mm:7915-8025, :6887-7072, :8029-8091
bool MetalExecutor::encodeQkvSplitRopeCast(void* qkv_buf, void* q_buf, void* k_buf, void* v_buf, void* k_f16_buf,
                                           void* v_f16_buf, void* cos_buf, void* sin_buf, size_t batch,
                                           size_t num_heads, size_t kv_heads, size_t head_dim, size_t qkv_rows,
                                           size_t q_rows, size_t k_rows, size_t v_rows, size_t rotary_dim) const {
    return mlc_hip_qkv_split_rope_cast(qkv_buf, q_buf, k_buf, v_buf, k_f16_buf, v_f16_buf, cos_buf, sin_buf, batch,
                                       num_heads, kv_heads, head_dim, qkv_rows, q_rows, k_rows, v_rows, rotary_dim,
                                       /*sync=*/0) != 0;
}

bool MetalExecutor::encodeRmsNormBatched(void* in_buf, const std::vector<float>& weight, float epsilon, size_t batch,
                                         size_t length, void* out_buf) const {
    return mlc_hip_rms_norm_batched(in_buf, weight.data(), weight.size(), epsilon, batch, length, out_buf, 0) != 0;
}

bool MetalExecutor::encodeMatMulQ4_0Batched(const std::string& weight_name, const std::vector<uint8_t>& weights,
                                            void* in_buf, size_t batch, size_t rows, size_t cols, size_t row_stride,
                                            uint32_t quant_version, void* out_buf) const {
    return mlc_hip_matmul_q4_0_batched(weight_name.c_str(), weights.data(), weights.size(), in_buf, batch, rows,
                                       cols, row_stride, quant_version, out_buf, 0) != 0;
}

bool MetalExecutor::encodeMatMulQ6KBatched(const std::string& weight_name, const std::vector<uint8_t>& weights,
                                           void* in_buf, size_t batch, size_t rows, size_t cols, size_t row_stride,
                                           void* out_buf) const {
    return mlc_hip_matmul_q6_k_batched(weight_name.c_str(), weights.data(), weights.size(), in_buf, batch, rows,
                                       cols, row_stride, out_buf, 0) != 0;
}

bool MetalExecutor::encodeAddBatched(void* a_buf, void* b_buf, void* out_buf, size_t total_elements) const {
    return mlc_hip_add_batched(a_buf, b_buf, out_buf, total_elements, 0) != 0;
}

bool MetalExecutor::encodeSiluMulBatched(void* gate_buf, void* up_buf, void* out_buf, size_t total_elements) const {
    return mlc_hip_silu_mul_batched(gate_buf, up_buf, out_buf, total_elements, 0) != 0;
}

bool MetalExecutor::encodeGateUpSplitSiluMul(void* gate_up_buf, void* gate_buf, void* up_buf, void* out_buf,
                                             size_t batch, size_t ffn_inner, size_t ffn_gate_up_rows) const {
    return mlc_hip_gate_up_split_silu_mul(gate_up_buf, gate_buf, up_buf, out_buf, batch, ffn_inner,
                                          ffn_gate_up_rows, 0) != 0;
}

// ---- the walker's lm_head fallback for a head it cannot encode (batched_walker.cpp:436-453):
// one row at a time through host vectors.  Served by the batched kernels with batch 1.
namespace {
bool host_matvec(bool q6k, const std::string& name, const std::vector<uint8_t>& weights,
                 const std::vector<float>& input, size_t rows, size_t cols, size_t row_stride,
                 uint32_t quant_version, std::vector<float>& output, const std::vector<float>* bias) {
    if (input.size() < cols) return false;
    void* in = mlc_hip_alloc(cols * sizeof(float));
    void* out = mlc_hip_alloc(rows * sizeof(float));
    bool ok = in && out && mlc_hip_upload(in, input.data(), cols * sizeof(float), 0) != 0;
    if (ok)
        ok = q6k ? mlc_hip_matmul_q6_k_batched(name.c_str(), weights.data(), weights.size(), in, 1, rows, cols,
                                               row_stride, out, /*sync=*/1) != 0
                 : mlc_hip_matmul_q4_0_batched(name.c_str(), weights.data(), weights.size(), in, 1, rows, cols,
                                               row_stride, quant_version, out, /*sync=*/1) != 0;
    if (ok) {
        output.resize(rows);
        ok = mlc_hip_download(out, output.data(), rows * sizeof(float), 0) != 0;
    }
    if (ok && bias) {
        if (bias->size() < rows) ok = false;
        else for (size_t r = 0; r < rows; ++r) output[r] += (*bias)[r];
    }
    if (in) mlc_hip_free(in);
    if (out) mlc_hip_free(out);
    return ok;
}
}  // namespace

bool MetalExecutor::runMatMulQ4_0(const std::string& weight_name, const std::vector<uint8_t>& weights,
                                  const std::vector<float>& input, size_t rows, size_t cols, size_t row_stride,
                                  uint32_t quant_version, std::vector<float>& output,
                                  const std::vector<float>* bias) const {
    return host_matvec(false, weight_name, weights, input, rows, cols, row_stride, quant_version, output, bias);
}

bool MetalExecutor::runMatMulQ6K(const std::string& weight_name, const std::vector<uint8_t>& weights,
                                 const std::vector<float>& input, size_t rows, size_t cols, size_t row_stride,
                                 std::vector<float>& output, const std::vector<float>* bias) const {
    return host_matvec(true, weight_name, weights, input, rows, cols, row_stride, 0, output, bias);
}

// Every other MetalExecutor method belongs to paths outside the paged decode step (single-stream
// MPS attention, the other quantisation formats, fusion windows); a full HIP build of the
// reference gives each the body its non-Apple build has: return false / nullptr
// (metal_runtime.mm:7161-7165), so that callers take their CPU branch.

}  // namespace runtime
}  // namespace mlc
