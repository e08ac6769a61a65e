/*
 * mlc_hip.h -- C ABI of the MI355X (gfx950) implementation of MLcompiler's
 * paged-KV attention hot path.
 *
 * Every entry point is what a HIP-backed mlc::runtime::MetalExecutor method
 * forwards to; the comment above each one names the reference method (or
 * kernel) it replaces.  All pointers named *_buf / page_storage / q / o are
 * DEVICE pointers obtained from mlc_hip_alloc / mlc_hip_cached (or any other
 * hipMalloc'ed memory of the current device); pointers to uint32_t metadata
 * are HOST pointers, borrowed for the duration of the call only (they are
 * copied before the call returns), exactly like the std::vector arguments of
 * the reference.
 *
 * Return convention mirrors the reference's `bool`: 1 = success, 0 = failure
 * (GPU unavailable, bad arguments, no open pass for an encode variant, or a
 * HIP error).  mlc_hip_last_error() describes the most recent failure of the
 * calling thread.  Nothing here throws.
 *
 * Threading: single-threaded by contract, like the reference
 * (compiler/runtime/paged_kv.hpp:25-27).  All work is ordered on one HIP
 * stream; "encode" variants enqueue and return, "run"/sync variants also wait.
 */
#ifndef MLC_HIP_H
#define MLC_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* MetalExecutor::isAvailable  (compiler/runtime/metal_runtime.hpp:27).
 * 1 when a gfx950 device is usable; initialises the library on first call. */
int mlc_hip_available(void);

/* Text of the last failure on this thread ("" if none). Never NULL. */
const char* mlc_hip_last_error(void);

/* ---- device buffers -------------------------------------------------------
 * MetalExecutor::allocateScratchBuffer / releaseScratchBuffer
 * (metal_runtime.hpp:693-694, metal_runtime.mm:8248-8271).  Caller owns. */
void* mlc_hip_alloc(size_t bytes);
void  mlc_hip_free(void* buffer);

/* MetalExecutor::getOrAllocCachedBuffer (metal_runtime.hpp:703,
 * metal_runtime.mm:8218-8246): name-keyed, library-owned, grow-only; a larger
 * request reallocates and invalidates the pointer handed out before. */
void* mlc_hip_cached(const char* name, size_t bytes);

/* MetalExecutor::uploadToBuffer / downloadFromBuffer (metal_runtime.hpp:695-696,
 * metal_runtime.mm:8273-8297).  Ordered after all work already enqueued on the
 * library's stream; both return when the copy is complete. */
int mlc_hip_upload(void* buffer, const void* src, size_t bytes, size_t dst_offset);
int mlc_hip_download(const void* buffer, void* dst, size_t bytes, size_t src_offset);

/* Fill `bytes` bytes with zero on the stream (PagedKVStorage::initialize
 * zero-fills its pools through uploadToBuffer, paged_kv.cpp:113-117; this is
 * the same result without the host staging copy). */
int mlc_hip_zero(void* buffer, size_t bytes);

/* ---- forward pass ("command buffer") --------------------------------------
 * MetalExecutor::beginForwardPassCB / flushForwardPassCB / hasForwardPassCB
 * (metal_runtime.hpp:181-183, metal_runtime.mm:6000-6064).  begin is
 * idempotent; flush waits for everything enqueued since begin and closes the
 * pass (returns 0 if a kernel failed). */
int mlc_hip_begin(void);
int mlc_hip_flush(void);
int mlc_hip_has_open_pass(void);

/* ---- the hot path ----------------------------------------------------------
 * Batched paged flash-attention decode: one query token per request.
 *   sync = 0: MetalExecutor::encodePagedFlashAttention
 *             (metal_runtime.hpp:510-523, metal_runtime.mm:7074-7166) --
 *             requires an open pass, enqueues, no argument validation beyond
 *             what keeps the kernel in bounds of the metadata.
 *   sync = 1: MetalExecutor::runPagedFlashAttention
 *             (metal_runtime.hpp:645-658, metal_runtime.mm:7727-7826) --
 *             validates like :7742-7750, runs, waits.
 * Kernel semantics: MSL paged_flash_attention, metal_runtime.mm:2216-2335.
 *   q  fp32 [batch][num_heads][head_dim]           o  fp32, same shape
 *   k_pages, v_pages  fp16 [pool pages][page_size_tokens][kv_heads][head_dim]
 *   page_tables_flat  all requests' page ids, concatenated (n_page_tables_flat)
 *   page_table_offsets [batch+1]; seq_lens [batch]; q_positions [batch]
 * Softmax scale is 1/sqrt(head_dim), derived inside as the reference does
 * (metal_runtime.mm:7133).  Query head h reads KV head h*kv_heads/num_heads. */
int mlc_hip_paged_attn_decode(const void* q, const void* k_pages, const void* v_pages, void* o,
                              const uint32_t* page_tables_flat, size_t n_page_tables_flat,
                              const uint32_t* page_table_offsets,
                              const uint32_t* seq_lens,
                              const uint32_t* q_positions,
                              size_t batch, size_t num_heads, size_t kv_heads,
                              size_t head_dim, size_t page_size_tokens,
                              int apply_causal, int sync);

/* Batched paged KV write: one new fp16 K (or V) row per request.
 *   sync = 0: MetalExecutor::encodeScatterKVPagedBatched
 *             (metal_runtime.hpp:526-533, metal_runtime.mm:7168-7225)
 *   sync = 1: MetalExecutor::scatterKVPagedBatched
 *             (metal_runtime.hpp:680-687, metal_runtime.mm:7231-7294)
 * Kernel: MSL scatter_kv_paged_batched_f16, metal_runtime.mm:405-424.
 *   src  fp16 [batch][n_kv_heads][head_dim]; row r -> page page_ids[r],
 *   slot slots_in_page[r] of page_storage. */
int mlc_hip_scatter_kv_paged_batched_f16(void* page_storage,
                                         const uint32_t* page_ids,
                                         const uint32_t* slots_in_page,
                                         size_t page_size_tokens, size_t n_kv_heads,
                                         size_t head_dim, size_t batch,
                                         const void* src, int sync);

/* ---- the callers' data formats either side of the path --------------------
 * MetalExecutor::scatterKVPaged (metal_runtime.hpp:666-674,
 * metal_runtime.mm:7828-7906; kernels :468-512): multi-token write for one
 * request, src [n_kv_heads][tokens][head_dim], dtype_bytes 2 or 4.  Waits. */
int mlc_hip_scatter_kv_paged(void* page_storage,
                             const uint32_t* page_table, size_t n_page_table,
                             size_t page_size_tokens, size_t n_kv_heads, size_t head_dim,
                             size_t tokens, size_t start_slot,
                             const void* src, size_t dtype_bytes);

/* MetalExecutor::gatherKVPages (metal_runtime.hpp:619-626,
 * metal_runtime.mm:7647-7721; kernels :328-370): pages -> contiguous
 * [n_kv_heads][num_tokens][head_dim].  Waits. */
int mlc_hip_gather_kv_pages(const void* page_storage,
                            const uint32_t* page_table, size_t n_page_table,
                            size_t page_size_tokens, size_t n_kv_heads, size_t head_dim,
                            size_t num_tokens, void* dst, size_t dtype_bytes);

/* The step before the KV write.  MetalExecutor::encodeQkvSplitRopeCast
 * (metal_runtime.hpp:540-547, metal_runtime.mm:7915-8025; kernels
 * strided_copy_f32 :447-455, batched_rope :287-314, cast_f32_to_f16 :457-464):
 *   q[r][:]  = rope(qkv[r][0 : q_rows])                    fp32 [batch][q_rows]
 *   k[r][:]  = rope(qkv[r][q_rows : q_rows+k_rows])        fp32 [batch][k_rows]
 *   v[r][:]  =      qkv[r][q_rows+k_rows : ... + v_rows]   fp32 [batch][v_rows]
 *   k_f16 = half(k), v_f16 = half(v)   (round to nearest even, as MSL half())
 * rope rotates pairs (2p, 2p+1), p < rotary_dim/2, of every head with
 * cos_buf/sin_buf [batch][rotary_dim/2] (fp32, device): x0*c - x1*s, x0*s + x1*c,
 * each product and sum rounded on its own as in the CPU
 * applyRotaryEmbedding (compiler/runtime/quantization.cpp:772-793).
 * rotary_dim == 0 skips it.  sync = 0 needs an open pass (the reference form),
 * sync = 1 waits.  One launch instead of the reference's seven dispatches. */
int mlc_hip_qkv_split_rope_cast(const void* qkv, void* q, void* k, void* v,
                                void* k_f16, void* v_f16,
                                const void* cos_buf, const void* sin_buf,
                                size_t batch, size_t num_heads, size_t kv_heads, size_t head_dim,
                                size_t qkv_rows, size_t q_rows, size_t k_rows, size_t v_rows,
                                size_t rotary_dim, int sync);

/* The same step fused with the two scatter_kv_paged_batched_f16 calls that
 * follow it in the walker (compiler/runtime/batched_walker.cpp:287-331): the
 * fp16 K and V rows go straight to page page_ids[r], slot slots_in_page[r] of
 * k_pages / v_pages (layout and index formula of metal_runtime.mm:405-424), so
 * the fp16 staging buffers and two launches disappear.  k_f32 / v_f32 may be
 * NULL when the caller does not need the fp32 copies.  No single counterpart
 * in the reference; results are bit-identical to
 * mlc_hip_qkv_split_rope_cast followed by two batched scatters. */
int mlc_hip_qkv_split_rope_scatter(const void* qkv, void* q, void* k_pages, void* v_pages,
                                   void* k_f32, void* v_f32,
                                   const void* cos_buf, const void* sin_buf,
                                   const uint32_t* page_ids, const uint32_t* slots_in_page,
                                   size_t page_size_tokens,
                                   size_t batch, size_t num_heads, size_t kv_heads, size_t head_dim,
                                   size_t qkv_rows, size_t q_rows, size_t k_rows, size_t v_rows,
                                   size_t rotary_dim, int sync);

/* ---- the other per-layer operators of the batched decode step ---------------
 * (compiler/runtime/batched_walker.cpp:246-405).  sync = 0 needs an open pass
 * like every encode* method of the reference; sync = 1 also waits.
 *
 * MetalExecutor::encodeRmsNormBatched (metal_runtime.hpp:474-479,
 * metal_runtime.mm:6887-6926; kernel rms_norm_kernel_v2_batched :166-208):
 * out[r][i] = in[r][i] * (1 / sqrt(mean(in[r]^2) + epsilon)) * weight[i] for
 * `batch` rows of `length` floats.  weight is a HOST vector borrowed for the
 * call (the reference copies it into its "norm_w" buffer per call); entries
 * past n_weight count as 1. */
int mlc_hip_rms_norm_batched(const void* in, const float* weight, size_t n_weight, float epsilon,
                             size_t batch, size_t length, void* out, int sync);

/* MetalExecutor::encodeAddBatched (metal_runtime.hpp:501-502,
 * metal_runtime.mm:7014-7042; kernel add_vectors :44-52): out = a + b. */
int mlc_hip_add_batched(const void* a, const void* b, void* out, size_t total_elements, int sync);

/* MetalExecutor::encodeSiluMulBatched (metal_runtime.hpp:505-506,
 * metal_runtime.mm:7044-7072; kernel feedforward_silu_mul :32-42):
 * out = gate / (1 + exp(-gate)) * up. */
int mlc_hip_silu_mul_batched(const void* gate, const void* up, void* out, size_t total_elements,
                             int sync);

/* MetalExecutor::encodeGateUpSplitSiluMul (metal_runtime.hpp:549-552,
 * metal_runtime.mm:8029-8091): gate = gate_up[:, 0:ffn_inner],
 * up = gate_up[:, ffn_inner:2*ffn_inner] (rows of ffn_gate_up_rows floats),
 * out = silu(gate) * up; one launch instead of three dispatches. */
int mlc_hip_gate_up_split_silu_mul(const void* gate_up, void* gate, void* up, void* out,
                                   size_t batch, size_t ffn_inner, size_t ffn_gate_up_rows,
                                   int sync);

/* MetalExecutor::encodeMatMulQ4_0Batched (metal_runtime.hpp:481-489,
 * metal_runtime.mm:6928-6990; kernel q4_0_matmul_v3_batched :710-785):
 * out[b][r] = sum_c W[r][c] * in[b][c] for `batch` requests; W is `rows` Q4_0
 * rows of `cols` weights, row_stride bytes apart (18-byte blocks of 32:
 * fp16 scale, 16 nibble bytes; compiler/runtime/quantization.cpp:70-74,
 * 191-214).  `weights` is the HOST copy, uploaded the first time a
 * weight_name is seen and kept on the device (getOrCacheWeight); in/out are
 * device fp32 [batch][cols] / [batch][rows].  Same constraints as the
 * reference (cols >= 64, rows % 4 == 0).  Shapes with rows % 64 == 0 and
 * cols % 32 == 0 run on the matrix cores with split-fp16 operands (relative
 * error about 2^-22 per product, fp32 accumulation); others on a scalar
 * kernel.  Uses library-owned scratch buffers: calls are stream-ordered and
 * must not overlap from several threads (single-threaded contract above). */
int mlc_hip_matmul_q4_0_batched(const char* weight_name, const void* weights, size_t weight_bytes,
                                const void* in, size_t batch, size_t rows, size_t cols,
                                size_t row_stride, uint32_t quant_version, void* out, int sync);

/* MetalExecutor::encodeMatMulQ6KBatched (metal_runtime.hpp:491-498,
 * metal_runtime.mm:6973-7012; kernel q6_k_matmul_v3_batched :1581-1655), the
 * lm_head of the batched decode step (batched_walker.cpp:429-431), and with
 * sync = 1 MetalExecutor::runMatMulQ6KBatched (metal_runtime.hpp:452-459):
 * out[b][r] = sum_c W[r][c] * in[b][c]; W is `rows` Q6_K rows of `cols`
 * weights, row_stride bytes apart (210-byte blocks of 256: 128 bytes of low
 * nibbles, 64 bytes of high bit pairs, 16 int8 scales, fp16 d;
 * compiler/runtime/quantization.cpp:142-147, 1469-1499).  `weights` is the
 * HOST copy, uploaded the first time a weight_name is seen and kept on the
 * device; in/out are device fp32 [batch][cols] / [batch][rows].  Same
 * constraints as the reference (cols >= 64, rows % 4 == 0).  Shapes with
 * rows % 32 == 0 and cols % 256 == 0 run on the matrix cores with fp32-grade
 * accuracy, others on a scalar kernel. */
int mlc_hip_matmul_q6_k_batched(const char* weight_name, const void* weights, size_t weight_bytes,
                                const void* in, size_t batch, size_t rows, size_t cols,
                                size_t row_stride, void* out, int sync);

/* Chunked prefill over paged KV (MFMA path).  No counterpart in the reference,
 * which prefills by looping the decode path once per prompt token
 * (compiler/runtime/batched_executor.cpp:454-466); semantics are the decode
 * kernel's causal rule (metal_runtime.mm:2286) applied per query row:
 *   q  fp16 [batch][chunk][num_heads][head_dim]; row i of request r sits at
 *      absolute position q_start[r] + i and attends kv positions <= that and
 *      < seq_lens[r].   o  fp32, same shape as q.
 * page_table_offsets has batch + 1 entries (the last one is the number of page ids in use, as
 * in the decode call, metal_runtime.mm:7747); request r's table holds at least
 * ceil(seq_lens[r] / page_size_tokens) page ids from page_table_offsets[r] on.
 * sync as above (0 needs an open pass). */
int mlc_hip_paged_attn_prefill(const void* q_f16, const void* k_pages, const void* v_pages,
                               void* o,
                               const uint32_t* page_tables_flat, size_t n_page_tables_flat,
                               const uint32_t* page_table_offsets,
                               const uint32_t* seq_lens,
                               const uint32_t* q_start,
                               size_t batch, size_t chunk, size_t num_heads, size_t kv_heads,
                               size_t head_dim, size_t page_size_tokens, int sync);

/* Decode attention for callers that cannot allocate (code under HIP graph capture, tight
 * serving loops, harnesses that forbid hipMalloc).  It has no counterpart in the reference.
 * Same result as mlc_hip_paged_attn_decode (same kernel), but the call itself allocates no device
 * or pinned memory and creates no stream or event: the kernel's scratch memory (the split-K partial
 * results, 8.5 MiB) is a static device array that every GPU the library runs on holds until the
 * process ends; seq_lens [batch], q_positions [batch] and page_table_offsets [batch + 1] (HOST
 * arrays, as in the decode call) travel inside the kernel arguments; the flat page table is read
 * where the caller keeps it:
 *   page_tables_flat_device  DEVICE pointer to n_page_tables_flat uint32 page ids (4-byte aligned)
 *   stream                   hipStream_t to launch on; NULL = the library's stream
 * Limits, refused with an error otherwise: batch <= 256; head_dim 64 or 128; GQA ratio 1, 2, 4, 8,
 * 16 or 32; page size a multiple of 64 (head_dim 64) or 32 (head_dim 128) tokens; q, o and the
 * pools 16-byte aligned.  mlc_hip_available() must have returned 1 before (set-up creates the
 * library's stream and looks up the scratch array's device address).  The call returns when the
 * kernel is enqueued (no synchronisation).  Every decode launch of this library on one GPU
 * uses the same scratch array, so they must follow each other: the library remembers the stream
 * of the last one and puts a launch on another stream behind what that stream held at the time
 * (events created at set-up); what the caller enqueues on its own streams by other means is the
 * caller's to order.  Operators that earlier encode calls held back are launched first, on the
 * library's stream, and a caller's stream is put behind them.  Not possible while a pass is
 * being captured.  The page ids cannot be checked on the host; for pools obtained from
 * mlc_hip_alloc the kernel clamps them below the pool's size. */
int mlc_hip_paged_attn_decode_noalloc(const void* q, const void* k_pages, const void* v_pages, void* o,
                                      const uint32_t* page_tables_flat_device, size_t n_page_tables_flat,
                                      const uint32_t* page_table_offsets,
                                      const uint32_t* seq_lens,
                                      const uint32_t* q_positions,
                                      size_t batch, size_t num_heads, size_t kv_heads,
                                      size_t head_dim, size_t page_size_tokens, int apply_causal,
                                      void* stream);

/* ---- a whole pass replayed from a HIP graph (no reference counterpart; the closest thing in
 * the reference is its single command buffer per forward pass, metal_runtime.mm:6000-6064).
 * The launches of a decode step are the same from step to step: what changes is the content of
 * the page tables, the per-request lengths and positions, the (page, slot) of the new K / V rows
 * and the caller's own buffers.  A captured pass keeps the launches and reads all of that from
 * device memory at fixed addresses, so that a step costs one graph launch instead of the encode
 * calls:
 *
 *   mlc_hip_begin(); <encode the step once, uncaptured>; mlc_hip_flush();     // everything resident
 *   mlc_hip_begin(); mlc_hip_capture_begin(); <the same encode calls>; h = mlc_hip_capture_end();
 *   per step: upload the step's inputs into the same buffers (mlc_hip_upload);
 *             mlc_hip_replay_update(h, <the step's tables>); mlc_hip_replay(h); mlc_hip_flush();
 *
 * While a pass is being captured the encode calls record their launches instead of running them;
 * a call that would have to allocate, copy metadata or wait fails (and the capture with it): run
 * the pass once uncaptured first, which puts weights, norm vectors and tables on the device.  The
 * decode attention of a captured pass must be served by the tile-balanced kernel (head_dim 64 or
 * 128, page size a multiple of its tile, 16-byte aligned buffers).  mlc_hip_capture_end returns a
 * handle > 0, or 0 (then nothing was kept; encode the pass uncaptured).  mlc_hip_captured_launches
 * counts the launches of the encode calls; the pass holds one more, the library's own first launch,
 * which moves a device word on by which the decode launches of one replay tell their split-K
 * partials from those of the replay before.
 *
 * mlc_hip_replay_update copies the step's tables (seq_lens [batch], q_positions [batch],
 * page_table_offsets [batch + 1], the flat table; page_ids / slots_in_page [batch]) over the
 * device copies the captured launches read (same addresses, ordered on the library's stream) and
 * checks what the capture took for granted: the same batch size; tables that cover their
 * seq_lens; that no device buffer of the library which the pass may read (weights, norm vectors,
 * named buffers, the tables' copy) was freed or moved since the capture; if the attention launch of the
 * captured pass does the step's KV write, that (page_ids, slots_in_page) are every request's newest
 * position on pages no two requests share.  It returns 0 when the step cannot be replayed (encode
 * it uncaptured; capture again if it said the copies had to move).  page_ids / slots_in_page may
 * be NULL for a pass without KV write.  The replay reads whatever the tables' device copy holds
 * when it runs: call mlc_hip_replay_update right before mlc_hip_replay. */
int    mlc_hip_capture_begin(void);
int    mlc_hip_capture_end(void);
size_t mlc_hip_captured_launches(int handle);
int    mlc_hip_replay_update(int handle, const uint32_t* page_tables_flat, size_t n_page_tables_flat,
                             const uint32_t* page_table_offsets, const uint32_t* seq_lens,
                             const uint32_t* q_positions, const uint32_t* page_ids,
                             const uint32_t* slots_in_page, size_t batch);
int    mlc_hip_replay(int handle);
void   mlc_hip_capture_release(int handle);

/* ---- measurement helpers (no reference counterpart) ------------------------
 * The library's stream as a hipStream_t, for callers that need to order their
 * own work or events with it. */
void* mlc_hip_stream(void);

/* hipEvent pair on the library's stream: start records, stop records, waits
 * and returns the elapsed milliseconds (negative on error). */
int   mlc_hip_timer_start(void);
float mlc_hip_timer_stop(void);

/* Number of kernels the last mlc_hip_paged_attn_decode call launched and the
 * number of workgroups that took part of the work (for benchmarks and tests). */
int mlc_hip_last_decode_launches(void);
int mlc_hip_last_decode_work_items(void);
/* Name of the kernel variant the last decode call launched, with its template arguments, e.g.
 * "stream<64,2,4,mfma-p32,regs,2>" (head_dim, query heads per wave, waves per group, arithmetic mode,
 * where the per-request figures live, LDS stages) or "generic". */
const char* mlc_hip_last_decode_kernel(void);
/* Number of KV writes so far that went out fused with a neighbour: a batched K scatter with its
 * V twin, or split + RoPE + cast with the scatters of its fp16 rows (for tests). */
long mlc_hip_fused_kv_write_launches(void);
/* Number of Q4_0 matmuls so far that went out with the split + RoPE + cast (and KV write) of
 * their output as epilogue (for tests). */
long mlc_hip_fused_matmul_rope_launches(void);
/* Number of Q4_0 matmuls so far that went out with the gate/up split + SiLU * up of their output
 * as epilogue, and how many of those also wrote the activation fragments of the Q4_0 matmul
 * that reads the products (for tests). */
long mlc_hip_fused_matmul_silu_launches(void);
long mlc_hip_fused_matmul_silu_split_launches(void);
/* Number of decode attention launches so far that also wrote their output as the activation
 * fragments of the Q4_0 matmul that reads it (for tests). */
long mlc_hip_fused_decode_split_launches(void);
/* Number of Q4_0 matmuls so far that went out with the residual add behind them, the sums of
 * squares of the RMSNorm behind that and the split-fp16 input of the Q4_0 matmul that reads the
 * norm as epilogue (that matmul finishes the norm; for tests). */
long mlc_hip_fused_matmul_norm_launches(void);
/* Number of decode attention launches so far that carried the step's KV write (a pair of
 * batched K / V scatters of every request's newest position encoded just before it). */
long mlc_hip_kv_writes_in_decode_launches(void);
/* Number of fused row-operator launches so far (for tests of "fuse_row_ops"). */
long mlc_hip_row_program_launches(void);
/* Number of times so far the decode path copied a page table to the device: the copy is
 * reused while the table's content stays the same (for tests and benchmarks). */
long mlc_hip_decode_table_uploads(void);

/* Tunables (0 selects the automatic choice where noted):
 *   "decode_wgs_per_cu"     workgroups per CU of the tile-balanced kernel's grid (0 = automatic)
 *   "decode_stages"         2, 3 or 4 K/V tiles staged in LDS per workgroup of the tile-balanced kernel
 *                           (0 = automatic: 2; batches above 64 requests take 3 at most)
 *   "decode_grid_wgs"       exact grid size of the tile-balanced kernel (0 = from the above; for tests)
 *   "decode_heads_per_wave" 1, 2, 4 or 8: the most query heads one wavefront handles;
 *                           the GQA group is spread over group/that many waves (0 = automatic)
 *   "decode_spin_limit"     rounds a workgroup that sums up a split pair polls for the other workgroups'
 *                           partials before it gives up and the pass fails (default 200000, about 0.1 s)
 *   "decode_test_flags"     bit 0: partials are not published (tests of the give-up path)
 *   "decode_pv_fp16"        0 (default) = fp32-grade softmax weights: fp32 on the vector pipe, the sum
 *                           of two fp16 numbers on the matrix pipe; 1 = weights rounded to fp16
 *                           for the P.V product (fp32 accumulate)
 *   "decode_force_generic"  1 = always use the shape-agnostic kernel
 *   "q4_force_generic"      1 = Q4_0 matmul always on the scalar kernel
 *   "q4_ksplit"             K slices of the Q4_0 MFMA matmul (0 = automatic)
 *   "q4_int_operand"        1 (default) = the Q4_0 MFMA matmul multiplies the integers q - 8 and
 *                           applies the block scale to each block's sum in fp32; 0 = it
 *                           multiplies d * (q - 8) as an exact pair of fp16 numbers
 *   "fuse_row_ops"          1 (default) = row-local operators encoded back to back in a pass
 *                           (sum of matmul K slices, add, RMSNorm, gate/up SiLU, the fp16 split
 *                           of the next matmul's input) are collected and launched as one
 *                           kernel when something else is encoded, the pass is flushed or a
 *                           call has sync = 1; every output buffer is still written.  The
 *                           same holds for the KV write: split + RoPE + cast and the two
 *                           batched scatters of its fp16 rows (or two batched scatters with
 *                           the same page ids) become one launch.  A Q4_0 matmul and a decode
 *                           attention call may be held back for a call or two as well, and
 *                           take on the work of the operators encoded right behind them
 *                           (split + RoPE + cast + KV write; gate/up split + SiLU * up; residual
 *                           add + RMSNorm; the fp16 split of the matmul that reads their output):
 *                           see the mlc_hip_fused_* counters above.
 *                           0 = each operator is launched when it is encoded
 *   "decode_pair_cost"      0..64: the tile-balanced decode kernel gives every workgroup the same
 *                           number of units, a KV tile counting one and the end of a (request,
 *                           KV head) pair this many; 0 = the same number of tiles; -1 (default) =
 *                           2 for GQA ratios of 4 and more (workgroups of four waves), 0 below
 *   "decode_mfma"           1 (default) = the tile-balanced decode kernel does a tile's arithmetic
 *                           on the matrix pipe where the shape allows it (4 to 16 query heads per
 *                           KV head in 4 waves); 0 = on the vector pipe
 *   "prefill_stages"        2, 4, 6 or 8 K/V tiles staged in LDS by the prefill kernel (0 = automatic:
 *                           6); with 8 the kernel with 64 rows per wave lets its waves meet only
 *                           after every second tile;
 *                           the kernel with 64 rows per wave has no 2-stage build and runs 4
 *                           stages when 2 is asked for
 *   "prefill_rows64"        1 (default) = heads/kv_heads up to 4 run the prefill kernel with 64
 *                           chunk rows per wave; 0 = the kernel with 32 rows per wave for every
 *                           ratio (ratio 8 always runs it)
 * Returns 0 for an unknown name or value. */
int mlc_hip_set_option(const char* name, long value);

#ifdef __cplusplus
}
#endif
#endif /* MLC_HIP_H */
