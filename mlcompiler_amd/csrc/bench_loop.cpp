// Native benchmark loop around the C ABI: the role tools/paged_flash_bench.cpp plays in
// the reference (compiler-side harness that calls the executor in a tight loop), so that
// the measured rate is the GPU's and not the Python interpreter's call overhead.
// It only calls entry points of include/mlc_hip.h; it adds no kernels of its own.
#include <chrono>
#include <cstddef>
#include <cstdint>

#include <hip/hip_runtime.h>

#include "../../include/mlc_hip.h"

// Plain streaming copy of known size: the yardstick the FETCH_SIZE / WRITE_SIZE counters are
// scaled by, and the practical HBM ceiling quoted beside the decode kernel.
__global__ __launch_bounds__(256) void mlc_bench_copy_kernel(const uint4* __restrict__ src,
                                                             uint4* __restrict__ dst, size_t n) {
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (size_t)gridDim.x * 256)
        dst[i] = src[i];
}

extern "C" {

// Enqueues `steps` decode-attention layer calls (encode variant, one open pass), layer i
// reading K/V pool i % n_layers, and reports the HIP-event time of the whole region
// (milliseconds) and the wall time from first enqueue to completion (seconds).
// Returns 1 on success.
int mlc_bench_decode_loop(const void* q, void* const* k_pools, void* const* v_pools,
                          size_t n_layers, void* o,
                          const uint32_t* page_tables_flat, size_t n_flat,
                          const uint32_t* page_table_offsets, const uint32_t* seq_lens,
                          const uint32_t* q_positions, size_t batch, size_t num_heads,
                          size_t kv_heads, size_t head_dim, size_t page_size_tokens,
                          int apply_causal, size_t steps, float* event_ms, double* wall_s) {
    if (!mlc_hip_begin()) return 0;
    const auto t0 = std::chrono::steady_clock::now();
    if (!mlc_hip_timer_start()) return 0;
    for (size_t i = 0; i < steps; ++i) {
        const size_t l = i % n_layers;
        if (!mlc_hip_paged_attn_decode(q, k_pools[l], v_pools[l], o, page_tables_flat, n_flat,
                                       page_table_offsets, seq_lens, q_positions, batch,
                                       num_heads, kv_heads, head_dim, page_size_tokens,
                                       apply_causal, /*sync=*/0))
            return 0;
    }
    const float ms = mlc_hip_timer_stop();
    if (ms < 0.f) return 0;
    if (!mlc_hip_flush()) return 0;
    const auto t1 = std::chrono::steady_clock::now();
    if (event_ms) *event_ms = ms;
    if (wall_s) *wall_s = std::chrono::duration<double>(t1 - t0).count();
    return 1;
}

// One decode step with KV write per layer call: scatter K row, scatter V row, attention
// (compiler/runtime/batched_walker.cpp:304-331).
int mlc_bench_decode_step_loop(const void* q, void* const* k_pools, void* const* v_pools,
                               size_t n_layers, void* o, const void* new_k, const void* new_v,
                               const uint32_t* page_ids, const uint32_t* slots,
                               const uint32_t* page_tables_flat, size_t n_flat,
                               const uint32_t* page_table_offsets, const uint32_t* seq_lens,
                               const uint32_t* q_positions, size_t batch, size_t num_heads,
                               size_t kv_heads, size_t head_dim, size_t page_size_tokens,
                               size_t steps, float* event_ms, double* wall_s) {
    if (!mlc_hip_begin()) return 0;
    const auto t0 = std::chrono::steady_clock::now();
    if (!mlc_hip_timer_start()) return 0;
    for (size_t i = 0; i < steps; ++i) {
        const size_t l = i % n_layers;
        if (!mlc_hip_scatter_kv_paged_batched_f16(k_pools[l], page_ids, slots, page_size_tokens,
                                                  kv_heads, head_dim, batch, new_k, 0))
            return 0;
        if (!mlc_hip_scatter_kv_paged_batched_f16(v_pools[l], page_ids, slots, page_size_tokens,
                                                  kv_heads, head_dim, batch, new_v, 0))
            return 0;
        if (!mlc_hip_paged_attn_decode(q, k_pools[l], v_pools[l], o, page_tables_flat, n_flat,
                                       page_table_offsets, seq_lens, q_positions, batch,
                                       num_heads, kv_heads, head_dim, page_size_tokens, 1, 0))
            return 0;
    }
    const float ms = mlc_hip_timer_stop();
    if (ms < 0.f) return 0;
    if (!mlc_hip_flush()) return 0;
    const auto t1 = std::chrono::steady_clock::now();
    if (event_ms) *event_ms = ms;
    if (wall_s) *wall_s = std::chrono::duration<double>(t1 - t0).count();
    return 1;
}

// Chunked prefill: `steps` calls of the MFMA kernel on the same inputs.
int mlc_bench_prefill_loop(const void* q_f16, const void* k_pages, const void* v_pages, void* o,
                           const uint32_t* page_tables_flat, size_t n_flat,
                           const uint32_t* page_table_offsets, const uint32_t* seq_lens,
                           const uint32_t* q_start, size_t batch, size_t chunk, size_t num_heads,
                           size_t kv_heads, size_t head_dim, size_t page_size_tokens, size_t steps,
                           float* event_ms, double* wall_s) {
    if (!mlc_hip_begin()) return 0;
    const auto t0 = std::chrono::steady_clock::now();
    if (!mlc_hip_timer_start()) return 0;
    for (size_t i = 0; i < steps; ++i) {
        if (!mlc_hip_paged_attn_prefill(q_f16, k_pages, v_pages, o, page_tables_flat, n_flat,
                                        page_table_offsets, seq_lens, q_start, batch, chunk,
                                        num_heads, kv_heads, head_dim, page_size_tokens, 0))
            return 0;
    }
    const float ms = mlc_hip_timer_stop();
    if (ms < 0.f) return 0;
    if (!mlc_hip_flush()) return 0;
    const auto t1 = std::chrono::steady_clock::now();
    if (event_ms) *event_ms = ms;
    if (wall_s) *wall_s = std::chrono::duration<double>(t1 - t0).count();
    return 1;
}

// `steps` launches of the copy kernel over `bytes` bytes (src and dst are device buffers of
// that size), on the library's stream; reports the HIP-event time in milliseconds.
int mlc_bench_copy_loop(const void* src, void* dst, size_t bytes, size_t steps, float* event_ms) {
    hipStream_t stream = static_cast<hipStream_t>(mlc_hip_stream());
    if (!stream || !src || !dst) return 0;
    const size_t n = bytes / 16;
    const unsigned grid = (unsigned)((n + 255) / 256 < 65536 * 4 ? (n + 255) / 256 : 65536 * 4);
    if (!mlc_hip_timer_start()) return 0;
    for (size_t i = 0; i < steps; ++i)
        hipLaunchKernelGGL(mlc_bench_copy_kernel, dim3(grid), dim3(256), 0, stream,
                           static_cast<const uint4*>(src), static_cast<uint4*>(dst), n);
    const float ms = mlc_hip_timer_stop();
    if (ms < 0.f) return 0;
    if (event_ms) *event_ms = ms;
    return 1;
}

}  // extern "C"
