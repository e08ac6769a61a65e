// Driver around the REAL reference code, compiled from the sources where they
// lie under /root/reference (see oracle/Makefile, target _ref).  TEST
// INFRASTRUCTURE ONLY: it exists to pin oracle/paged_oracle.c against the
// reference's own executor-CPU attention and fp16 conversions.  Nothing of the
// reference is copied here: this file only includes its headers and calls
//   mlc::runtime::RunAttentionCPU         compiler/runtime/attention_cpu.cpp:272-478
//   mlc::runtime::fp16ToFloat/floatToFp16 compiler/runtime/float_convert.hpp:14-76
//   mlc::runtime::applyRotaryEmbedding / computeRotaryCoefficients
//                                         compiler/runtime/quantization.cpp:772-823
//   mlc::runtime::quantizeRowQ4_0 / dotProductRowQ4_0 / dequantizeRowQ4_0
//   mlc::runtime::quantizeRowQ6_K / dotProductRowQ6_K / dequantizeRowQ6_K
//                                         compiler/runtime/quantization.cpp:235-311
// the way the reference's own test does (tests/test_runtime.cpp:1659-1690):
// an ExecutionGraph with one Attention node, state tensors {Hkv, ctx, D}
// tagged role=kv_cache so ExecutionContext stores them as F16
// (compiler/runtime/execution_context.cpp:145-157), rotary_dim 0 (no RoPE).
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <string>
#include <unistd.h>
#include <vector>

#include "frontends/ggml_types.hpp"
#include "runtime/attention_cpu.hpp"
#include "runtime/execution_context.hpp"
#include "runtime/execution_graph.hpp"
#include "runtime/float_convert.hpp"
#include "runtime/operator_backend.hpp"
#include "runtime/quantization.hpp"
#include "runtime/session.hpp"

namespace {

// A Session needs a GGUF file to open; an empty one (no tensors, no metadata)
// is enough because the Attention node never touches weights.
std::string write_empty_gguf() {
    std::string path = "/tmp/paged_oracle_ref_" + std::to_string(getpid()) + ".gguf";
    FILE* f = std::fopen(path.c_str(), "wb");
    if (!f) return std::string();
    const uint32_t magic = 0x46554747u;  // "GGUF"
    const uint32_t version = 3;
    const uint64_t zero = 0;
    std::fwrite(&magic, 4, 1, f);
    std::fwrite(&version, 4, 1, f);
    std::fwrite(&zero, 8, 1, f);  // n_tensors
    std::fwrite(&zero, 8, 1, f);  // n_kv
    std::fclose(f);
    return path;
}

}  // namespace

extern "C" {

float ref_fp16_to_float(uint16_t h) { return mlc::runtime::fp16ToFloat(h); }
uint16_t ref_float_to_fp16(float v) { return mlc::runtime::floatToFp16(v); }
void ref_fp16_to_float_n(const uint16_t* src, float* dst, size_t n) {
    mlc::runtime::castF16toF32(src, dst, n);
}
void ref_float_to_fp16_n(const float* src, uint16_t* dst, size_t n) {
    mlc::runtime::castF32toF16(src, dst, n);
}

// One decode step of the reference's executor-CPU attention for ONE request.
//   q        fp32 [heads][head_dim]
//   k_cache  fp16 [kv_heads][ctx_len][head_dim]   (the reference's contiguous cache layout)
//   v_cache  same
//   position the sequence position of the query; rows [0, position] are attended.
//   k_new/v_new fp32 [kv_heads][head_dim]: the row RunAttentionCPU writes at `position`
//            before attending (attention_cpu.cpp:398-418).
// out fp32 [heads][head_dim].  Returns 1 on success.
int ref_run_attention_cpu(const float* q, const uint16_t* k_cache, const uint16_t* v_cache,
                          size_t heads, size_t kv_heads, size_t head_dim, size_t ctx_len,
                          size_t position, const float* k_new, const float* v_new, float* out) {
    using namespace mlc::runtime;
    try {
        std::string path = write_empty_gguf();
        if (path.empty()) return 0;
        Session session(path);
        ::unlink(path.c_str());

        ExecutionGraph graph;
        graph.addTensor("q", {static_cast<int64_t>(heads * head_dim)}, mlc::ir::DataType::F32);
        graph.addTensor("k_in", {static_cast<int64_t>(kv_heads * head_dim)}, mlc::ir::DataType::F32);
        graph.addTensor("v_in", {static_cast<int64_t>(kv_heads * head_dim)}, mlc::ir::DataType::F32);
        std::vector<int64_t> cache_shape{static_cast<int64_t>(kv_heads),
                                         static_cast<int64_t>(ctx_len),
                                         static_cast<int64_t>(head_dim)};
        auto& kc = graph.addTensor("kv_k", cache_shape, mlc::ir::DataType::F32);
        kc.is_state = true;
        kc.metadata["role"] = "kv_cache";
        auto& vc = graph.addTensor("kv_v", cache_shape, mlc::ir::DataType::F32);
        vc.is_state = true;
        vc.metadata["role"] = "kv_cache";
        graph.addTensor("attn_out", {static_cast<int64_t>(heads * head_dim)}, mlc::ir::DataType::F32);
        auto& node = graph.addNode("attention", ExecOpType::Attention, {"q", "k_in", "v_in"},
                                   {"attn_out", "kv_k", "kv_v"}, BackendKind::CPU);
        node.attributes["heads"] = static_cast<float>(heads);
        node.attributes["kv_heads"] = static_cast<float>(kv_heads);
        node.attributes["head_dim"] = static_cast<float>(head_dim);
        node.annotations["kv_cache_k"] = "kv_k";
        node.annotations["kv_cache_v"] = "kv_v";

        ExecutionContext context(session, &graph);
        context.setSequencePosition(position);
        context.ensureStateTensor(*graph.getTensor("kv_k"));
        context.ensureStateTensor(*graph.getTensor("kv_v"));
        TensorStorage* ks = context.tensorStorage("kv_k");
        TensorStorage* vs = context.tensorStorage("kv_v");
        if (!ks || !vs) return 0;
        if (ks->dtype != mlc::frontend::GGML_TYPE_F16) return 0;  // F16 KV cache is the default
        const size_t bytes = kv_heads * ctx_len * head_dim * sizeof(uint16_t);
        if (ks->raw_data.size() != bytes || vs->raw_data.size() != bytes) return 0;
        std::memcpy(ks->raw_data.data(), k_cache, bytes);
        std::memcpy(vs->raw_data.data(), v_cache, bytes);

        std::vector<float> qv(q, q + heads * head_dim);
        std::vector<float> kn(k_new, k_new + kv_heads * head_dim);
        std::vector<float> vn(v_new, v_new + kv_heads * head_dim);
        const ExecutionNode& n = graph.nodes().front();
        BackendExecutionResult res = RunAttentionCPU(n, &context, qv, kn, vn);
        if (!res.success) return 0;
        const std::vector<float>* o = context.getTensor("attn_out");
        if (!o || o->size() != heads * head_dim) return 0;
        std::memcpy(out, o->data(), o->size() * sizeof(float));
        return 1;
    } catch (...) {
        return 0;
    }
}

// applyRotaryEmbedding on one head vector (in place); n_pairs entries of cos/sin.
void ref_apply_rotary(float* data, const float* cos, const float* sin, size_t n_pairs,
                      size_t head_dim, size_t rotary_dim) {
    std::vector<float> c(cos, cos + n_pairs), s(sin, sin + n_pairs);
    mlc::runtime::applyRotaryEmbedding(data, c, s, head_dim, rotary_dim);
}

// computeRotaryCoefficients; cos/sin must hold rotary_dim / 2 floats.  Returns the pair count.
size_t ref_rotary_coefficients(size_t position, size_t rotary_dim, float freq_base, float freq_scale,
                               float* cos, float* sin) {
    std::vector<float> c, s;
    mlc::runtime::computeRotaryCoefficients(position, rotary_dim, freq_base, freq_scale, c, s);
    std::memcpy(cos, c.data(), c.size() * sizeof(float));
    std::memcpy(sin, s.data(), s.size() * sizeof(float));
    return c.size();
}

// quantizeRowQ4_0 / dotProductRowQ4_0 / dequantizeRowQ4_0 (compiler/runtime/quantization.cpp:235-311)
size_t ref_quantize_row_q4_0(const float* src, size_t cols, uint8_t* dst, size_t dst_cap) {
    std::vector<uint8_t> out;
    mlc::runtime::quantizeRowQ4_0(src, cols, 1, out);
    if (out.size() > dst_cap) return 0;
    std::memcpy(dst, out.data(), out.size());
    return out.size();
}
float ref_dot_q4_0(const uint8_t* row, size_t cols, const float* vec) {
    return mlc::runtime::dotProductRowQ4_0(row, cols, 1, vec);
}
void ref_dequantize_row_q4_0(const uint8_t* row, size_t cols, float* dst) {
    mlc::runtime::dequantizeRowQ4_0(row, cols, 1, dst);
}

// dequantizeRowQ6_K / dotProductRowQ6_K / quantizeRowQ6_K (compiler/runtime/quantization.cpp:1469-1663)
void ref_dequantize_row_q6_k(const uint8_t* row, size_t cols, float* dst) {
    mlc::runtime::dequantizeRowQ6_K(row, cols, dst);
}
float ref_dot_q6_k(const uint8_t* row, size_t cols, const float* vec) {
    return mlc::runtime::dotProductRowQ6_K(row, cols, vec);
}
size_t ref_quantize_row_q6_k(const float* src, size_t cols, uint8_t* dst, size_t dst_cap) {
    std::vector<uint8_t> out;
    mlc::runtime::quantizeRowQ6_K(src, cols, out);
    if (out.size() <= dst_cap) std::memcpy(dst, out.data(), out.size());
    return out.size();
}

}  // extern "C"
