// Native benchmark loop around the C ABI: the role tools/paged_flash_bench.cpp plays in
// the reference (compiler-side harness that calls the executor in a tight loop), so that
// the measured rate is the GPU's and not the Python interpreter's call overhead.
// It only calls entry points of include/mlc_hip.h; it adds no kernels of its own.
#include <algorithm>
#include <chrono>
#include <string>
#include <vector>
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

// Plain streaming read: every thread loads 16-byte units with a grid stride and folds them into
// one word that is stored only if it has a value it never has.  The same number of bytes as a
// decode launch, read contiguously with nothing else to do.
__global__ __launch_bounds__(256) void mlc_bench_read_kernel(const uint4* __restrict__ a, const uint4* __restrict__ b,
                                                             size_t n_each, uint32_t* sink) {
    uint32_t acc = 0;
    const size_t stride = (size_t)gridDim.x * 256;
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n_each; i += stride) {
        const uint4 x = a[i], y = b[i];
        acc ^= x.x ^ x.y ^ x.z ^ x.w ^ y.x ^ y.y ^ y.z ^ y.w;
    }
    if (acc == 0x9E3779B9u && sink) sink[0] = acc;
}

// 16-byte load, ordinary or non-temporal.
template <bool NT>
__device__ __forceinline__ uint4 load16(const uint4* p) {
    if constexpr (NT) {
        typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
        const u32x4 v = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p));
        return make_uint4(v[0], v[1], v[2], v[3]);
    } else {
        return *p;
    }
}

// Tuned streaming read, into registers: a workgroup takes 256 * U consecutive 16-byte units of each
// tensor per trip, so every lane has 2 * U independent 16-byte loads in flight before it folds
// any of them (the plain kernel above has two).  The grid is persistent (a few workgroups per CU)
// and swept by the caller.  This is the yardstick for what the memory system delivers to a launch
// of a given size with nothing else to do.  NT: non-temporal loads (the data is read once: it need
// not stay in the L2).
template <int U, bool NT>
__global__ __launch_bounds__(256) void mlc_bench_read_unrolled_kernel(const uint4* __restrict__ a,
                                                                      const uint4* __restrict__ b, size_t n_each,
                                                                      uint32_t* sink) {
    uint32_t acc = 0;
    const size_t stride = (size_t)gridDim.x * 256 * U;
    size_t i = (size_t)blockIdx.x * 256 * U + threadIdx.x;
    for (; i + (size_t)(U - 1) * 256 < n_each; i += stride) {
        uint4 x[U], y[U];
#pragma unroll
        for (int u = 0; u < U; ++u) x[u] = load16<NT>(&a[i + (size_t)u * 256]);
#pragma unroll
        for (int u = 0; u < U; ++u) y[u] = load16<NT>(&b[i + (size_t)u * 256]);
#pragma unroll
        for (int u = 0; u < U; ++u) acc ^= x[u].x ^ x[u].y ^ x[u].z ^ x[u].w ^ y[u].x ^ y[u].y ^ y[u].z ^ y[u].w;
    }
    for (int u = 0; u < U; ++u) {   // the ragged end of the last trip
        const size_t j = i + (size_t)u * 256;
        if (j < n_each) {
            const uint4 x = a[j], y = b[j];
            acc ^= x.x ^ x.y ^ x.z ^ x.w ^ y.x ^ y.y ^ y.z ^ y.w;
        }
    }
    if (acc == 0x9E3779B9u && sink) sink[0] = acc;
}

// Tuned streaming read, global -> LDS, shaped like the decode kernel's tile loads: every wave
// moves 1 KiB per instruction straight into LDS (no registers), U instructions per tensor and
// trip, two trips in flight (the next trip is requested before the current one is waited for).
// Units past the end are clamped onto the last one (in bounds, read twice).
template <int U, bool NT>
__global__ __launch_bounds__(256) void mlc_bench_read_lds_kernel(const uint4* __restrict__ a, const uint4* __restrict__ b,
                                                                 size_t n_each, uint32_t* sink) {
    __shared__ __attribute__((aligned(16))) unsigned char stage[2][2 * U * 4096];
    const uint32_t wave = threadIdx.x / 64, lane = threadIdx.x % 64;
    const uint32_t base = (uint32_t)(uintptr_t)(const __attribute__((address_space(3))) void*)&stage[0][0];
    const size_t stride = (size_t)gridDim.x * 256 * U;
    const size_t first = (size_t)blockIdx.x * 256 * U + threadIdx.x;
    auto issue = [&](size_t i, uint32_t buf) {
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            const uint4* src = t ? b : a;
#pragma unroll
            for (int u = 0; u < U; ++u) {
                size_t j = i + (size_t)u * 256;
                j = j < n_each ? j : n_each - 1;
                const uint32_t dst = __builtin_amdgcn_readfirstlane(base + buf * (2 * U * 4096) + (t * U + u) * 4096 + wave * 1024);
                if constexpr (NT)
                    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off nt" : : "s"(dst), "v"(src + j) : "memory", "m0");
                else
                    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off" : : "s"(dst), "v"(src + j) : "memory", "m0");
            }
        }
    };
    if (first >= n_each) return;
    uint32_t buf = 0;
    issue(first, 0);
    for (size_t i = first; i < n_each; i += stride) {
        const bool more = i + stride < n_each;
        if (more) {
            issue(i + stride, buf ^ 1u);
            asm volatile("s_waitcnt vmcnt(%0)" : : "n"(2 * U) : "memory");
        } else {
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        }
        buf ^= 1u;
    }
    // one word of what landed, so that the loads have a consumer
    const uint32_t w = reinterpret_cast<const uint32_t*>(&stage[0][0])[lane];
    if (w == 0x9E3779B9u && sink) sink[0] = w;
}

extern "C" {

// `steps` launches of the streaming-read kernel, launch i reading the first bytes_each bytes of
// K pool and V pool i % n_layers (device buffers of at least that size) on the library's stream;
// reports the HIP-event time of the region in milliseconds.
int mlc_bench_read_loop(void* const* k_pools, void* const* v_pools, size_t n_layers, size_t bytes_each,
                        size_t steps, float* event_ms) {
    hipStream_t stream = static_cast<hipStream_t>(mlc_hip_stream());
    if (!stream || !k_pools || !v_pools || !n_layers) return 0;
    const size_t n = bytes_each / 16;
    const size_t want = (n + 255) / 256;
    const unsigned grid = (unsigned)(want < 256 * 8 ? (want ? want : 1) : 256 * 8);
    if (!mlc_hip_timer_start()) return 0;
    for (size_t i = 0; i < steps; ++i)
        hipLaunchKernelGGL(mlc_bench_read_kernel, dim3(grid), dim3(256), 0, stream,
                           static_cast<const uint4*>(k_pools[i % n_layers]),
                           static_cast<const uint4*>(v_pools[i % n_layers]), n, static_cast<uint32_t*>(nullptr));
    const float ms = mlc_hip_timer_stop();
    if (ms < 0.f) return 0;
    if (event_ms) *event_ms = ms;
    return 1;
}

// The tuned reads: kind 0 = into registers, 1 = global -> LDS, 2 and 3 = the same with non-temporal
// loads; unroll = 16-byte loads per tensor
// and trip (1, 2, 4 or 8); grid = workgroups of 256 threads.  Same rotation over the pools and the
// same timing as mlc_bench_read_loop.  Returns 0 for a combination that is not built.
int mlc_bench_read_tuned_loop(void* const* k_pools, void* const* v_pools, size_t n_layers, size_t bytes_each,
                              size_t steps, int kind, int unroll, unsigned grid, float* event_ms) {
    hipStream_t stream = static_cast<hipStream_t>(mlc_hip_stream());
    if (!stream || !k_pools || !v_pools || !n_layers || !grid) return 0;
    const size_t n = bytes_each / 16;
    if (!n) return 0;
    void (*kern)(const uint4*, const uint4*, size_t, uint32_t*) = nullptr;
    if (kind == 0) {
        kern = unroll == 1 ? mlc_bench_read_unrolled_kernel<1, false> : unroll == 2 ? mlc_bench_read_unrolled_kernel<2, false>
             : unroll == 4 ? mlc_bench_read_unrolled_kernel<4, false> : unroll == 8 ? mlc_bench_read_unrolled_kernel<8, false> : nullptr;
    } else if (kind == 1) {
        kern = unroll == 1 ? mlc_bench_read_lds_kernel<1, false> : unroll == 2 ? mlc_bench_read_lds_kernel<2, false>
             : unroll == 4 ? mlc_bench_read_lds_kernel<4, false> : nullptr;
    } else if (kind == 2) {
        kern = unroll == 1 ? mlc_bench_read_unrolled_kernel<1, true> : unroll == 2 ? mlc_bench_read_unrolled_kernel<2, true>
             : unroll == 4 ? mlc_bench_read_unrolled_kernel<4, true> : unroll == 8 ? mlc_bench_read_unrolled_kernel<8, true> : nullptr;
    } else if (kind == 3) {
        kern = unroll == 1 ? mlc_bench_read_lds_kernel<1, true> : unroll == 2 ? mlc_bench_read_lds_kernel<2, true>
             : unroll == 4 ? mlc_bench_read_lds_kernel<4, true> : nullptr;
    }
    if (!kern) return 0;
    if (!mlc_hip_timer_start()) return 0;
    for (size_t i = 0; i < steps; ++i)
        hipLaunchKernelGGL(kern, dim3(grid), dim3(256), 0, stream, static_cast<const uint4*>(k_pools[i % n_layers]),
                           static_cast<const uint4*>(v_pools[i % n_layers]), n, static_cast<uint32_t*>(nullptr));
    const float ms = mlc_hip_timer_stop();
    if (ms < 0.f) return 0;
    if (event_ms) *event_ms = ms;
    return 1;
}

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

// One whole decoder layer per step, in the order of the reference's layer loop
// (compiler/runtime/batched_walker.cpp:246-405): RMSNorm, qkv matmul, split + RoPE + KV write,
// paged attention, out-projection, add, RMSNorm, gate/up matmul, SiLU gate, down-projection,
// add.  Layer i uses K/V pool i % n_layers and its own device copy of the weights (the host
// data is the same, the weight names differ), so that neither sits in the Infinity Cache from
// the step before.
struct MlcBenchLayer {
    const void* x;            // [batch][hidden] fp32 input of the layer
    void* norm; void* qkv; void* q; void* attn; void* o; void* resid; void* gate_up;
    void* gate; void* up; void* mix; void* down; void* out;
    void* out2;               // when set: step i reads step i-1's output (out, out2 alternate), like
                              // consecutive layers of a model; otherwise every step reads x
    const void* cos; const void* sin;
    const float* attn_norm_w; const float* ffn_norm_w;
    const void* w_qkv; size_t w_qkv_bytes;
    const void* w_o; size_t w_o_bytes;
    const void* w_gate_up; size_t w_gate_up_bytes;
    const void* w_down; size_t w_down_bytes;
    size_t hidden, ffn_inner, num_heads, kv_heads, head_dim, page_size_tokens, batch;
    const uint32_t* page_ids; const uint32_t* slots;
    const uint32_t* page_tables_flat; size_t n_flat;
    const uint32_t* page_table_offsets; const uint32_t* seq_lens; const uint32_t* q_positions;
    // when head_w is set: after every n_layers-th layer the final RMSNorm and the Q6_K lm_head
    // (batched_walker.cpp:415-431), i.e. n_layers steps are one decode step of the model
    const float* head_norm_w; const void* head_w; size_t head_bytes; size_t head_rows; void* logits;
    double* enqueue_s;        // when set: receives the host time spent encoding (before the wait),
                              // measured over the first 256 steps and scaled to the loop's steps
};

// Weight-cache names of layer l's four matrices.
static std::vector<std::string> layer_weight_names(size_t n_layers) {
    std::vector<std::string> names(n_layers * 4);
    for (size_t l = 0; l < n_layers; ++l) {
        const char* kinds[4] = {"attn_qkv", "attn_output", "ffn_gate_up", "ffn_down"};
        for (int k = 0; k < 4; ++k) names[l * 4 + k] = "bench.l" + std::to_string(l) + "." + kinds[k];
    }
    return names;
}

// Encodes step i of the layer loop (layer i % n_layers, input = the step before's output).
static int encode_layer_step(const MlcBenchLayer* L, const std::vector<std::string>& names,
                             void* const* k_pools, void* const* v_pools, size_t n_layers, size_t i) {
    const size_t B = L->batch, HID = L->hidden, FFN = L->ffn_inner;
    const size_t q_rows = L->num_heads * L->head_dim, kv_rows = L->kv_heads * L->head_dim;
    const size_t qkv_rows = q_rows + 2 * kv_rows;
    const size_t s_hid = HID / 32 * 18, s_ffn = FFN / 32 * 18;
    const size_t l = i % n_layers;
    const void* x = (L->out2 && i > 0) ? ((i - 1) % 2 ? L->out2 : L->out) : L->x;
    void* out = (L->out2 && i % 2) ? L->out2 : L->out;
    int ok = mlc_hip_rms_norm_batched(x, L->attn_norm_w, HID, 1e-5f, B, HID, L->norm, 0);
    ok = ok && mlc_hip_matmul_q4_0_batched(names[l * 4 + 0].c_str(), L->w_qkv, L->w_qkv_bytes, L->norm, B,
                                           qkv_rows, HID, s_hid, 1, L->qkv, 0);
    ok = ok && mlc_hip_qkv_split_rope_scatter(L->qkv, L->q, k_pools[l], v_pools[l], nullptr, nullptr,
                                              L->cos, L->sin, L->page_ids, L->slots,
                                              L->page_size_tokens, B, L->num_heads, L->kv_heads,
                                              L->head_dim, qkv_rows, q_rows, kv_rows, kv_rows,
                                              L->head_dim, 0);
    ok = ok && mlc_hip_paged_attn_decode(L->q, k_pools[l], v_pools[l], L->attn, L->page_tables_flat,
                                         L->n_flat, L->page_table_offsets, L->seq_lens,
                                         L->q_positions, B, L->num_heads, L->kv_heads, L->head_dim,
                                         L->page_size_tokens, 1, 0);
    ok = ok && mlc_hip_matmul_q4_0_batched(names[l * 4 + 1].c_str(), L->w_o, L->w_o_bytes, L->attn, B, HID,
                                           HID, s_hid, 1, L->o, 0);
    ok = ok && mlc_hip_add_batched(x, L->o, L->resid, B * HID, 0);
    ok = ok && mlc_hip_rms_norm_batched(L->resid, L->ffn_norm_w, HID, 1e-5f, B, HID, L->norm, 0);
    ok = ok && mlc_hip_matmul_q4_0_batched(names[l * 4 + 2].c_str(), L->w_gate_up, L->w_gate_up_bytes,
                                           L->norm, B, 2 * FFN, HID, s_hid, 1, L->gate_up, 0);
    ok = ok && mlc_hip_gate_up_split_silu_mul(L->gate_up, L->gate, L->up, L->mix, B, FFN, 2 * FFN, 0);
    ok = ok && mlc_hip_matmul_q4_0_batched(names[l * 4 + 3].c_str(), L->w_down, L->w_down_bytes, L->mix, B,
                                           HID, FFN, s_ffn, 1, L->down, 0);
    ok = ok && mlc_hip_add_batched(L->resid, L->down, out, B * HID, 0);
    if (ok && L->head_w && l == n_layers - 1) {
        ok = mlc_hip_rms_norm_batched(out, L->head_norm_w, HID, 1e-5f, B, HID, L->norm, 0);
        ok = ok && mlc_hip_matmul_q6_k_batched("bench.lm_head", L->head_w, L->head_bytes, L->norm, B,
                                               L->head_rows, HID, HID / 256 * 210, L->logits, 0);
    }
    return ok;
}

int mlc_bench_layer_loop(const MlcBenchLayer* L, void* const* k_pools, void* const* v_pools,
                         size_t n_layers, size_t steps, float* event_ms, double* wall_s) {
    const std::vector<std::string> names = layer_weight_names(n_layers);
    if (!mlc_hip_begin()) return 0;
    const auto t0 = std::chrono::steady_clock::now();
    if (!mlc_hip_timer_start()) return 0;
    // (host time of encoding: taken over the first 256 steps and scaled to all of them -- further on
    // the host is so far ahead of the GPU that the queue is full and encode calls wait for room)
    const size_t enq_steps = std::min<size_t>(steps, 256);
    double enq_s = 0.0;
    for (size_t i = 0; i < steps; ++i) {
        if (!encode_layer_step(L, names, k_pools, v_pools, n_layers, i)) return 0;
        if (i + 1 == enq_steps) enq_s = std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count();
    }
    if (L->enqueue_s) *L->enqueue_s = enq_s * (double)steps / (double)enq_steps;
    const float ms = mlc_hip_timer_stop();
    if (ms < 0.f) return 0;
    if (!mlc_hip_flush()) return 0;
    const auto t1 = std::chrono::steady_clock::now();
    if (event_ms) *event_ms = ms;
    if (wall_s) *wall_s = std::chrono::duration<double>(t1 - t0).count();
    return 1;
}

// The same loop with one pass over the n_layers layers (n_layers even, so that a pass ends in
// the buffer the next one starts from) captured into a HIP graph through the library's capture
// calls and replayed `replays` times: measures what replaying prebuilt launches saves over
// encoding them call by call.  The pass is run once uncaptured first, so that every weight, norm
// vector, page table and scratch buffer is already on the device (a capture holds kernel launches
// only).  event_ms receives the time of all replays.  Returns 1 on success, 0 on failure.
int mlc_bench_layer_loop_graph(const MlcBenchLayer* L, void* const* k_pools, void* const* v_pools,
                               size_t n_layers, size_t replays, float* event_ms, size_t* n_nodes) {
    if (n_layers == 0 || n_layers % 2 != 0) return 0;
    const std::vector<std::string> names = layer_weight_names(n_layers);
    if (!mlc_hip_begin()) return 0;
    for (size_t i = 0; i < n_layers; ++i)
        if (!encode_layer_step(L, names, k_pools, v_pools, n_layers, i)) return 0;
    if (!mlc_hip_flush() || !mlc_hip_begin()) return 0;
    if (!mlc_hip_capture_begin()) return 0;
    int ok = 1;
    for (size_t i = 0; ok && i < n_layers; ++i) ok = encode_layer_step(L, names, k_pools, v_pools, n_layers, i);
    const int handle = mlc_hip_capture_end();
    if (!ok || handle <= 0) return 0;
    if (n_nodes) *n_nodes = mlc_hip_captured_launches(handle);
    int rc = mlc_hip_replay(handle) && mlc_hip_flush() && mlc_hip_begin();   // one replay to warm up
    rc = rc && mlc_hip_timer_start();
    for (size_t i = 0; rc && i < replays; ++i) rc = mlc_hip_replay(handle);
    const float ms = rc ? mlc_hip_timer_stop() : -1.f;
    if (ms < 0.f) rc = 0;
    if (event_ms) *event_ms = ms;
    if (!mlc_hip_flush()) rc = 0;
    mlc_hip_capture_release(handle);
    return rc;
}

}  // extern "C"
