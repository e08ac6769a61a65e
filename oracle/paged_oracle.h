/*
 * CPU oracle for the paged-KV attention path.  TEST INFRASTRUCTURE ONLY:
 * nothing in the shipped library links or loads this file; it is the checker
 * the GPU kernels are compared with, and the CPU baseline that is timed
 * beside them.
 *
 * Every function restates, in plain C, one piece of the reference
 * (G-Krishna-chandra/MLcompiler); the citation next to each prototype names
 * the reference file and lines it follows.
 *
 * Pinning status (what each function has been checked against):
 *   oracle_fp16_to_float, oracle_float_to_fp16_ref
 *       - all 65536 halves / a float sweep against the reference's own inline
 *         functions compiled from compiler/runtime/float_convert.hpp
 *         (oracle/_ref), and against numpy's IEEE binary16.
 *   oracle_paged_attention_executor
 *       - bit-for-bit against the reference's RunAttentionCPU compiled from
 *         its own sources (oracle/_ref), on gathered-contiguous copies of the
 *         same paged cache; known answers tests/test_runtime.cpp:1692-1705,
 *         compiler/main.cpp:4026-4031; closed forms (S=1, equal keys,
 *         constant V, page-permutation invariance) and a float64 brute force.
 *   oracle_paged_attention_flashref
 *       - same known answers and closed forms; agreement with the executor
 *         ordering to float rounding; float64 brute force.
 *   oracle_scatter_*, oracle_gather_*
 *       - closed-form index pattern of tests/test_paged_kv.cpp:219-267 and
 *         scatter->gather identity; untouched-bytes invariant.
 *   oracle_pool_*, oracle_req_*
 *       - the allocator sequences asserted in tests/test_paged_kv.cpp:34-207.
 *   oracle_paged_attention_prefill
 *       - PARITY UNPINNED against the reference: the reference has no
 *         multi-query paged attention.  It is defined row-wise through
 *         oracle_paged_attention_executor (a query at absolute position p
 *         sees kv positions <= p, metal_runtime.mm:2286) and checked against
 *         a float64 brute force only.
 */
#ifndef PAGED_ORACLE_H
#define PAGED_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* compiler/runtime/float_convert.hpp:14-48 -- IEEE binary16 -> binary32. */
float oracle_fp16_to_float(uint16_t h);

/* compiler/runtime/float_convert.hpp:57-76 -- the reference's own
 * binary32 -> binary16: round-half-up on the magnitude, NaN becomes Inf,
 * |x| < 2^-25 flushes to signed zero.  NOT round-to-nearest-even. */
uint16_t oracle_float_to_fp16_ref(float value);

/* IEEE round-to-nearest-even binary32 -> binary16 (what the GPU's convert
 * instruction and numpy do); used to build inputs shared by both sides. */
uint16_t oracle_float_to_fp16_rne(float value);

/* Bulk forms of the three conversions above (float_convert.hpp:80-104 are the
 * reference's bulk loops: element-wise calls of the scalar functions). */
void oracle_fp16_to_float_n(const uint16_t* src, float* dst, size_t n);
void oracle_float_to_fp16_ref_n(const float* src, uint16_t* dst, size_t n);
void oracle_float_to_fp16_rne_n(const float* src, uint16_t* dst, size_t n);

/* compiler/runtime/metal_runtime.mm:405-424 (kernel) and :7231-7294 (host
 * argument checks).  src is [batch][n_kv_heads][head_dim] halves; row r goes
 * to page page_ids[r], slot slots_in_page[r].  Returns 1 on success, 0 on the
 * argument errors the reference rejects. */
int oracle_scatter_kv_paged_batched_f16(uint16_t* page_storage,
                                        const uint32_t* page_ids,
                                        const uint32_t* slots_in_page,
                                        size_t page_size_tokens,
                                        size_t n_kv_heads,
                                        size_t head_dim,
                                        size_t batch,
                                        const uint16_t* src);

/* compiler/runtime/metal_runtime.mm:468-512 (kernels), :7828-7906 (host).
 * src is [n_kv_heads][tokens][head_dim]; token t lands at absolute slot
 * start_slot + t of the request's page table.  dtype_bytes is 2 or 4. */
int oracle_scatter_kv_paged(void* page_storage,
                            const uint32_t* page_table, size_t n_page_table,
                            size_t page_size_tokens, size_t n_kv_heads,
                            size_t head_dim, size_t tokens, size_t start_slot,
                            const void* src, size_t dtype_bytes);

/* compiler/runtime/metal_runtime.mm:328-370 (kernels), :7647-7721 (host).
 * dst is [n_kv_heads][num_tokens][head_dim]. */
int oracle_gather_kv_pages(const void* page_storage,
                           const uint32_t* page_table, size_t n_page_table,
                           size_t page_size_tokens, size_t n_kv_heads,
                           size_t head_dim, size_t num_tokens,
                           void* dst, size_t dtype_bytes);

/* The step before the KV write: split one fused qkv row per request into q, k, v
 * (strided_copy_f32, compiler/runtime/metal_runtime.mm:447-455), rotate q and k
 * in place (batched_rope :287-314; same arithmetic as the CPU
 * applyRotaryEmbedding, compiler/runtime/quantization.cpp:772-793: pair
 * (2p, 2p+1) -> (x0*c - x1*s, x0*s + x1*c), every product and sum rounded to
 * fp32 on its own), and cast k and v to fp16 with round-to-nearest-even
 * (cast_f32_to_f16 :457-464, `half(x)`), in the order of
 * MetalExecutor::encodeQkvSplitRopeCast (:7915-8025).
 *   qkv [batch][qkv_rows]; q [batch][q_rows]; k [batch][k_rows]; v [batch][v_rows];
 *   cos, sin [batch][rotary_dim/2]; k_f16, v_f16 like k, v.
 * rotary_dim == 0 skips the rotation (cos/sin may be NULL).  Returns 0 when a
 * buffer is missing or the row counts do not fit (q_rows + k_rows + v_rows >
 * qkv_rows, q_rows != num_heads*head_dim, k_rows != kv_heads*head_dim,
 * rotary_dim > head_dim or odd). */
int oracle_qkv_split_rope_cast(const float* qkv, float* q, float* k, float* v,
                               uint16_t* k_f16, uint16_t* v_f16,
                               const float* cos_table, const float* sin_table,
                               size_t batch, size_t num_heads, size_t kv_heads, size_t head_dim,
                               size_t qkv_rows, size_t q_rows, size_t k_rows, size_t v_rows,
                               size_t rotary_dim);

/* compiler/runtime/quantization.cpp:795-823: cos/sin of position * base^(-2i/rotary_dim) * scale
 * for i < rotary_dim/2, all in fp32 (powf, cosf, sinf).  base <= 0 -> 10000, scale == 0 -> 1.
 * Returns the number of pairs written. */
size_t oracle_rotary_coefficients(size_t position, size_t rotary_dim, float freq_base,
                                  float freq_scale, float* cos_out, float* sin_out);

/* ---- the walker's other per-layer operators (compiler/runtime/batched_walker.cpp:246-405) ----
 *
 * RMSNorm over `batch` rows of `length` floats with one shared weight vector: the CPU rmsNorm
 * of compiler/runtime/operator_backend.cpp:186-203 per row (sequential fp32 sum of squares,
 * mean, inv = 1/sqrtf(mean + eps), out = in * inv * gamma; gamma = 1 past the end of weight),
 * which the kernel rms_norm_kernel_v2_batched (metal_runtime.mm:166-208) follows up to the
 * order of its sum.  Returns 0 when a buffer is missing or batch/length is 0
 * (metal_runtime.mm:6895). */
int oracle_rms_norm_batched(const float* in, const float* weight, size_t n_weight, float epsilon,
                            size_t batch, size_t length, float* out);

/* add_vectors (metal_runtime.mm:44-52) over a flat range: encodeAddBatched (:7014-7042). */
int oracle_add(const float* a, const float* b, float* out, size_t n);

/* feedforward_silu_mul (metal_runtime.mm:32-42): out = gate / (1 + expf(-gate)) * up. */
int oracle_silu_mul(const float* gate, const float* up, float* out, size_t n);

/* encodeGateUpSplitSiluMul (metal_runtime.mm:8029-8091): gate = gate_up[:, 0:inner],
 * up = gate_up[:, inner:2*inner] (rows of gate_up_rows floats), out = silu(gate) * up. */
int oracle_gate_up_split_silu_mul(const float* gate_up, float* gate, float* up, float* out,
                                  size_t batch, size_t ffn_inner, size_t gate_up_rows);

/* Q4_0 rows: 18-byte blocks of 32 weights (fp16 scale d, then 16 bytes; byte j holds weight j
 * in its low nibble and weight j+16 in its high nibble, value = d * (nibble - 8)),
 * compiler/runtime/quantization.cpp:70-74, 191-214.  out[b][r] = the CPU dotProductRowQ4_0
 * (quantization.cpp:240-269: one fp32 accumulator, blocks in order, within a block the pairs
 * (j, j+16) in order, each term d * q * x rounded as written) of weight row r (row_stride bytes
 * apart) with input row b.  Same result layout and constraints as q4_0_matmul_v3_batched
 * (metal_runtime.mm:710-785; host :6930-6990: cols >= 64, rows % 4 == 0). */
int oracle_matmul_q4_0_batched(const uint8_t* weights, const float* in, size_t batch, size_t rows,
                               size_t cols, size_t row_stride, float* out, int n_threads);

/* quantizeRowQ4_0 (quantization.cpp:271-311), used to make test weights: scale = (value of
 * largest magnitude) / -8, q = clamp((int)(x / scale + 8.5), 0, 15), scale stored through the
 * reference's floatToFp16.  dst must hold ceil(cols/32)*18 bytes. */
void oracle_quantize_row_q4_0(const float* src, size_t cols, uint8_t* dst);

/* Q6_K rows: 210-byte blocks of 256 weights (128 bytes of low nibbles, 64 bytes of high bit
 * pairs, 16 int8 scales of 16 weights each, fp16 d; value d * scale * (q - 32)),
 * compiler/runtime/quantization.cpp:142-147.
 * oracle_dequantize_row_q6_k = dequantizeRowQ6_K (quantization.cpp:1469-1499);
 * oracle_matmul_q6_k_batched: out[b][r] = the CPU dotProductRowQ6_K (quantization.cpp:1570-1586,
 * the row dequantized block by block, then summed left to right in fp32) of weight row r with
 * input row b; result layout and constraints of q6_k_matmul_v3_batched
 * (compiler/runtime/metal_runtime.mm:1581-1655, host :6973-7012: cols >= 64, rows % 4 == 0);
 * oracle_quantize_row_q6_k = quantizeRowQ6_K (quantization.cpp:1588-1663), used to make test
 * weights.  All three are checked against the reference's own build of these functions. */
void oracle_dequantize_row_q6_k(const uint8_t* src, size_t cols, float* dst);
int oracle_matmul_q6_k_batched(const uint8_t* weights, const float* in, size_t batch, size_t rows,
                               size_t cols, size_t row_stride, float* out, int n_threads);
void oracle_quantize_row_q6_k(const float* src, size_t cols, uint8_t* dst);

/* The executor-CPU attention, compiler/runtime/attention_cpu.cpp:437-470
 * (per head: left-to-right dot over every cached row :99-105, softmax that
 * subtracts the max, exponentiates and divides each weight by the sum :21-33,
 * then V axpy :166-170), reading rows through the page layout of
 * compiler/runtime/metal_runtime.mm:2266-2276 and applying that kernel's
 * causal rule :2286 and empty-sequence rule :2254-2257,2333.  GQA map
 * kv = head*kv_heads/heads (attention_cpu.cpp:443).  fp32 throughout.
 * n_threads > 1 spreads (request, head) pairs over OpenMP threads; the
 * arithmetic of each pair is unchanged.  Returns 1, or 0 on the argument
 * errors of metal_runtime.mm:7742-7750. */
int oracle_paged_attention_executor(const float* q,
                                    const uint16_t* k_pages,
                                    const uint16_t* v_pages,
                                    float* out,
                                    const uint32_t* page_tables_flat, size_t n_page_tables_flat,
                                    const uint32_t* page_table_offsets,
                                    const uint32_t* seq_lens,
                                    const uint32_t* q_positions,
                                    size_t batch, size_t num_heads, size_t kv_heads,
                                    size_t head_dim, size_t page_size_tokens,
                                    int apply_causal, int n_threads);

/* The kernel's in-test CPU twin, tests/test_paged_flash.cpp:17-91: same
 * semantics, but weights stay un-normalised and the accumulated output is
 * multiplied by 1/sum at the end. */
int oracle_paged_attention_flashref(const float* q,
                                    const uint16_t* k_pages,
                                    const uint16_t* v_pages,
                                    float* out,
                                    const uint32_t* page_tables_flat, size_t n_page_tables_flat,
                                    const uint32_t* page_table_offsets,
                                    const uint32_t* seq_lens,
                                    const uint32_t* q_positions,
                                    size_t batch, size_t num_heads, size_t kv_heads,
                                    size_t head_dim, size_t page_size_tokens,
                                    int apply_causal);

/* Chunked prefill over paged KV.  q is fp16 [batch][chunk][num_heads][head_dim];
 * request r's chunk row i sits at absolute position q_start[r] + i and sees
 * kv positions <= that (metal_runtime.mm:2286 applied per row; the reference
 * reaches the same result by looping its decode path once per token,
 * compiler/runtime/batched_executor.cpp:454-466).  out is fp32, same shape. */
int oracle_paged_attention_prefill(const uint16_t* q_f16,
                                   const uint16_t* k_pages,
                                   const uint16_t* v_pages,
                                   float* out,
                                   const uint32_t* page_tables_flat, size_t n_page_tables_flat,
                                   const uint32_t* page_table_offsets,
                                   const uint32_t* seq_lens,
                                   const uint32_t* q_start,
                                   size_t batch, size_t chunk, size_t num_heads,
                                   size_t kv_heads, size_t head_dim,
                                   size_t page_size_tokens, int n_threads);

/* compiler/runtime/parity_harness.cpp:214-255 -- max|a-b|, mean|a-b|, rms and
 * cosine, all accumulated in double.  cosine is NaN when either norm is 0. */
void oracle_metrics(const float* a, const float* b, size_t n,
                    double* max_abs, double* mean_abs, double* rms, double* cosine);

/* tests/test_paged_flash.cpp:93-102 -- cosine that returns 0 for a zero norm. */
double oracle_cosine(const float* a, const float* b, size_t n);

/* compiler/runtime/paged_kv.cpp:10-42 -- LIFO free list of page ids; a fresh
 * pool hands out 0,1,2,...  The caller owns `pool` (oracle_pool_free). */
typedef struct oracle_page_pool oracle_page_pool;
oracle_page_pool* oracle_pool_new(uint32_t capacity);
void oracle_pool_free(oracle_page_pool* pool);
int oracle_pool_allocate(oracle_page_pool* pool, uint32_t* id_out);          /* 0 = exhausted */
int oracle_pool_allocate_n(oracle_page_pool* pool, size_t n, uint32_t* out); /* all or nothing */
void oracle_pool_release(oracle_page_pool* pool, uint32_t page_id);
size_t oracle_pool_in_use(const oracle_page_pool* pool);
size_t oracle_pool_free_count(const oracle_page_pool* pool);

/* compiler/runtime/paged_kv.hpp:65-97, paged_kv.cpp:44-81 -- one request's
 * page chain.  page_table is caller storage of page_table_cap entries. */
typedef struct {
    uint32_t page_size_tokens;
    uint32_t* page_table;
    size_t page_table_cap;
    size_t n_pages;
    uint32_t tokens_in_last_page;
} oracle_request_kv;
size_t oracle_req_total_tokens(const oracle_request_kv* st);
int oracle_req_reserve(oracle_request_kv* st, oracle_page_pool* pool, size_t target_tokens);
int oracle_req_extend_one_token(oracle_request_kv* st, oracle_page_pool* pool,
                                uint32_t* page_id, uint32_t* slot);
int oracle_req_locate(const oracle_request_kv* st, size_t pos, uint32_t* page_id, uint32_t* slot);
void oracle_req_release_all(oracle_request_kv* st, oracle_page_pool* pool);

#ifdef __cplusplus
}
#endif
#endif
