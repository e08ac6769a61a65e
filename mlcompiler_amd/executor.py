"""HipExecutor: the Python face of the C ABI, with the method names, argument
order and bool-return conventions of the reference's MetalExecutor paged path
(compiler/runtime/metal_runtime.hpp:181-183, 510-533, 619-703), so that tests
read like tests/test_paged_flash.cpp and tests/test_paged_kv.cpp.

Buffers are opaque device pointers (ints), metadata are sequences of uint32.
Nothing here computes: every method is one call into csrc/libmlc_hip.so.
"""
from __future__ import annotations

import ctypes as C

import numpy as np

from ._lib import NativeLibraryError, load

_u32p = C.POINTER(C.c_uint32)


def _u32(seq) -> np.ndarray:
    return np.ascontiguousarray(seq, dtype=np.uint32)


def _ptr(a: np.ndarray):
    return a.ctypes.data_as(_u32p)


class HipExecutor:
    """Singleton, like MetalExecutor::Instance() (metal_runtime.mm:5774-5777)."""

    _instance = None

    @classmethod
    def Instance(cls) -> "HipExecutor":
        if cls._instance is None:
            cls._instance = cls()
        return cls._instance

    def __init__(self):
        self._lib = load()

    # -- availability / errors
    def isAvailable(self) -> bool:
        return bool(self._lib.mlc_hip_available())

    def requireAvailable(self) -> None:
        if not self.isAvailable():
            raise NativeLibraryError("no gfx950 device: " + self.lastError())

    def lastError(self) -> str:
        return self._lib.mlc_hip_last_error().decode()

    # -- buffers (metal_runtime.hpp:693-703)
    def allocateScratchBuffer(self, nbytes: int) -> int:
        return self._lib.mlc_hip_alloc(nbytes) or 0

    def releaseScratchBuffer(self, buffer: int) -> None:
        self._lib.mlc_hip_free(buffer)

    def getOrAllocCachedBuffer(self, name: str, nbytes: int) -> int:
        return self._lib.mlc_hip_cached(name.encode(), nbytes) or 0

    def uploadToBuffer(self, buffer: int, src: np.ndarray, nbytes: int | None = None,
                       dst_offset: int = 0) -> bool:
        src = np.ascontiguousarray(src)
        n = src.nbytes if nbytes is None else nbytes
        return bool(self._lib.mlc_hip_upload(buffer, src.ctypes.data, n, dst_offset))

    def downloadFromBuffer(self, buffer: int, dst: np.ndarray, nbytes: int | None = None,
                           src_offset: int = 0) -> bool:
        assert dst.flags.c_contiguous and dst.flags.writeable
        n = dst.nbytes if nbytes is None else nbytes
        return bool(self._lib.mlc_hip_download(buffer, dst.ctypes.data, n, src_offset))

    def zeroBuffer(self, buffer: int, nbytes: int) -> bool:
        return bool(self._lib.mlc_hip_zero(buffer, nbytes))

    # -- forward pass (metal_runtime.hpp:181-183)
    def beginForwardPassCB(self) -> bool:
        return bool(self._lib.mlc_hip_begin())

    def flushForwardPassCB(self) -> bool:
        return bool(self._lib.mlc_hip_flush())

    def hasForwardPassCB(self) -> bool:
        return bool(self._lib.mlc_hip_has_open_pass())

    # -- paged flash attention (metal_runtime.hpp:510-523, 645-658)
    def _attn(self, q, k_pages, v_pages, o, page_tables_flat, page_table_offsets, seq_lens,
              q_positions, batch, num_heads, kv_heads, head_dim, page_size_tokens, apply_causal,
              sync) -> bool:
        flat = _u32(page_tables_flat)
        off = _u32(page_table_offsets)
        sl = _u32(seq_lens)
        qp = _u32(q_positions)
        # the reference rejects vectors of the wrong length (metal_runtime.mm:7747-7748)
        if off.size != batch + 1 or sl.size != batch or qp.size != batch:
            return False
        flat_arg = flat if flat.size else np.zeros(1, np.uint32)
        return bool(self._lib.mlc_hip_paged_attn_decode(
            q, k_pages, v_pages, o, _ptr(flat_arg), flat.size, _ptr(off), _ptr(sl), _ptr(qp),
            batch, num_heads, kv_heads, head_dim, page_size_tokens, int(bool(apply_causal)), sync))

    def runPagedFlashAttention(self, q_buffer, k_pages_buffer, v_pages_buffer, o_buffer,
                               page_tables_flat, page_table_offsets, seq_lens, q_positions,
                               batch, num_heads, kv_heads, head_dim, page_size_tokens,
                               apply_causal) -> bool:
        return self._attn(q_buffer, k_pages_buffer, v_pages_buffer, o_buffer, page_tables_flat,
                          page_table_offsets, seq_lens, q_positions, batch, num_heads, kv_heads,
                          head_dim, page_size_tokens, apply_causal, 1)

    def encodePagedFlashAttention(self, q_buf, k_pages_buf, v_pages_buf, o_buf, page_tables_flat,
                                  page_table_offsets, seq_lens, q_positions, batch, num_heads,
                                  kv_heads, head_dim, page_size_tokens, apply_causal) -> bool:
        return self._attn(q_buf, k_pages_buf, v_pages_buf, o_buf, page_tables_flat,
                          page_table_offsets, seq_lens, q_positions, batch, num_heads, kv_heads,
                          head_dim, page_size_tokens, apply_causal, 0)

    # -- batched paged KV write (metal_runtime.hpp:526-533, 680-687)
    def _scatter_batched(self, page_storage, page_ids, slots_in_page, page_size_tokens,
                         n_kv_heads, head_dim, batch, src, sync) -> bool:
        pid = _u32(page_ids)
        sl = _u32(slots_in_page)
        if sync and (pid.size != batch or sl.size != batch):  # metal_runtime.mm:7243
            return False
        if pid.size < batch or sl.size < batch:
            return False
        return bool(self._lib.mlc_hip_scatter_kv_paged_batched_f16(
            page_storage, _ptr(pid), _ptr(sl), page_size_tokens, n_kv_heads, head_dim, batch, src,
            sync))

    def scatterKVPagedBatched(self, page_storage_buffer, page_ids, slots_in_page,
                              page_size_tokens, n_kv_heads, head_dim, batch, src_buffer) -> bool:
        return self._scatter_batched(page_storage_buffer, page_ids, slots_in_page,
                                     page_size_tokens, n_kv_heads, head_dim, batch, src_buffer, 1)

    def encodeScatterKVPagedBatched(self, page_storage_buffer, page_ids, slots_in_page,
                                    page_size_tokens, n_kv_heads, head_dim, batch,
                                    src_buffer) -> bool:
        return self._scatter_batched(page_storage_buffer, page_ids, slots_in_page,
                                     page_size_tokens, n_kv_heads, head_dim, batch, src_buffer, 0)

    # -- single-request scatter / gather (metal_runtime.hpp:619-626, 666-674)
    def scatterKVPaged(self, page_storage_buffer, page_table, page_size_tokens, n_kv_heads,
                       head_dim, tokens, start_slot, src_buffer, dtype_bytes) -> bool:
        pt = _u32(page_table)
        pt_arg = pt if pt.size else np.zeros(1, np.uint32)
        return bool(self._lib.mlc_hip_scatter_kv_paged(
            page_storage_buffer, _ptr(pt_arg), pt.size, page_size_tokens, n_kv_heads, head_dim,
            tokens, start_slot, src_buffer, dtype_bytes))

    def gatherKVPages(self, page_storage_buffer, page_table, page_size_tokens, n_kv_heads,
                      head_dim, num_tokens, dst_buffer, dtype_bytes) -> bool:
        pt = _u32(page_table)
        pt_arg = pt if pt.size else np.zeros(1, np.uint32)
        return bool(self._lib.mlc_hip_gather_kv_pages(
            page_storage_buffer, _ptr(pt_arg), pt.size, page_size_tokens, n_kv_heads, head_dim,
            num_tokens, dst_buffer, dtype_bytes))

    # -- the step before the KV write (metal_runtime.hpp:540-547, metal_runtime.mm:7915-8025)
    def encodeQkvSplitRopeCast(self, qkv_buf, q_buf, k_buf, v_buf, k_f16_buf, v_f16_buf, cos_buf,
                               sin_buf, batch, num_heads, kv_heads, head_dim, qkv_rows, q_rows,
                               k_rows, v_rows, rotary_dim, sync: bool = False) -> bool:
        return bool(self._lib.mlc_hip_qkv_split_rope_cast(
            qkv_buf, q_buf, k_buf, v_buf, k_f16_buf, v_f16_buf, cos_buf, sin_buf, batch, num_heads,
            kv_heads, head_dim, qkv_rows, q_rows, k_rows, v_rows, rotary_dim, int(bool(sync))))

    # the same step fused with the two batched scatters that follow it in the walker
    # (batched_walker.cpp:287-331); no single reference method
    def encodeQkvSplitRopeScatter(self, qkv_buf, q_buf, k_pages_buffer, v_pages_buffer, cos_buf,
                                  sin_buf, page_ids, slots_in_page, page_size_tokens, batch,
                                  num_heads, kv_heads, head_dim, qkv_rows, q_rows, k_rows, v_rows,
                                  rotary_dim, k_f32_buf=None, v_f32_buf=None,
                                  sync: bool = False) -> bool:
        ids = _u32(page_ids)
        sl = _u32(slots_in_page)
        if ids.size != batch or sl.size != batch:
            return False
        return bool(self._lib.mlc_hip_qkv_split_rope_scatter(
            qkv_buf, q_buf, k_pages_buffer, v_pages_buffer, k_f32_buf, v_f32_buf, cos_buf, sin_buf,
            _ptr(ids), _ptr(sl), page_size_tokens, batch, num_heads, kv_heads, head_dim, qkv_rows,
            q_rows, k_rows, v_rows, rotary_dim, int(bool(sync))))

    # -- the other per-layer operators of the batched decode step
    def encodeRmsNormBatched(self, in_buf, weight, epsilon, batch, length, out_buf,
                             sync: bool = False) -> bool:  # metal_runtime.hpp:474-479
        w = np.ascontiguousarray(weight, np.float32)
        return bool(self._lib.mlc_hip_rms_norm_batched(
            in_buf, w.ctypes.data if w.size else None, w.size, float(epsilon), batch, length, out_buf,
            int(bool(sync))))

    def encodeAddBatched(self, a_buf, b_buf, out_buf, total_elements, sync: bool = False) -> bool:
        return bool(self._lib.mlc_hip_add_batched(a_buf, b_buf, out_buf, total_elements,
                                                  int(bool(sync))))  # metal_runtime.hpp:501-502

    def encodeSiluMulBatched(self, gate_buf, up_buf, out_buf, total_elements,
                             sync: bool = False) -> bool:  # metal_runtime.hpp:505-506
        return bool(self._lib.mlc_hip_silu_mul_batched(gate_buf, up_buf, out_buf, total_elements,
                                                       int(bool(sync))))

    def encodeGateUpSplitSiluMul(self, gate_up_buf, gate_buf, up_buf, out_buf, batch, ffn_inner,
                                 ffn_gate_up_rows, sync: bool = False) -> bool:  # :549-552
        return bool(self._lib.mlc_hip_gate_up_split_silu_mul(
            gate_up_buf, gate_buf, up_buf, out_buf, batch, ffn_inner, ffn_gate_up_rows,
            int(bool(sync))))

    def encodeMatMulQ4_0Batched(self, weight_name, weights, in_buf, batch, rows, cols, row_stride,
                                quant_version, out_buf, sync: bool = False) -> bool:
        """metal_runtime.hpp:481-489; `weights` is the host byte array of the Q4_0 rows."""
        w = np.ascontiguousarray(weights, np.uint8)
        return bool(self._lib.mlc_hip_matmul_q4_0_batched(
            weight_name.encode(), w.ctypes.data, w.size, in_buf, batch, rows, cols, row_stride,
            quant_version, out_buf, int(bool(sync))))

    # -- chunked prefill (no reference method; see include/mlc_hip.h)

    def encodeMatMulQ6KBatched(self, weight_name, weights, in_buf, batch, rows, cols, row_stride,
                               out_buf, sync: bool = False) -> bool:
        """metal_runtime.hpp:491-498 (sync=True: runMatMulQ6KBatched, :452-459); `weights` is the
        host byte array of the Q6_K rows."""
        w = np.ascontiguousarray(weights, np.uint8)
        return bool(self._lib.mlc_hip_matmul_q6_k_batched(
            weight_name.encode(), w.ctypes.data, w.size, in_buf, batch, rows, cols, row_stride,
            out_buf, int(bool(sync))))
    def runPagedPrefillAttention(self, q_f16_buffer, k_pages_buffer, v_pages_buffer, o_buffer,
                                 page_tables_flat, page_table_offsets, seq_lens, q_start, batch,
                                 chunk, num_heads, kv_heads, head_dim, page_size_tokens,
                                 sync: bool = True) -> bool:
        flat = _u32(page_tables_flat)
        off = _u32(page_table_offsets)
        sl = _u32(seq_lens)
        qs = _u32(q_start)
        if off.size != batch + 1 or sl.size != batch or qs.size != batch:
            return False
        flat_arg = flat if flat.size else np.zeros(1, np.uint32)
        return bool(self._lib.mlc_hip_paged_attn_prefill(
            q_f16_buffer, k_pages_buffer, v_pages_buffer, o_buffer, _ptr(flat_arg), flat.size,
            _ptr(off), _ptr(sl), _ptr(qs), batch, chunk, num_heads, kv_heads, head_dim,
            page_size_tokens, int(bool(sync))))

    # -- a pass replayed from a HIP graph
    def captureBegin(self) -> bool:
        return bool(self._lib.mlc_hip_capture_begin())

    def captureEnd(self) -> int:
        """Handle > 0 of the captured pass, or 0 (see lastError)."""
        return int(self._lib.mlc_hip_capture_end())

    def capturedLaunches(self, handle: int) -> int:
        return int(self._lib.mlc_hip_captured_launches(handle))

    def replayUpdate(self, handle, page_tables_flat, page_table_offsets, seq_lens, q_positions,
                     page_ids=None, slots_in_page=None) -> bool:
        flat, off, seq, pos = (_u32(x) for x in (page_tables_flat, page_table_offsets, seq_lens, q_positions))
        ids = _u32(page_ids) if page_ids is not None else None
        slots = _u32(slots_in_page) if slots_in_page is not None else None
        return bool(self._lib.mlc_hip_replay_update(handle, _ptr(flat), flat.size, _ptr(off), _ptr(seq), _ptr(pos),
                                                    _ptr(ids) if ids is not None else None,
                                                    _ptr(slots) if slots is not None else None, seq.size))

    def replay(self, handle: int) -> bool:
        return bool(self._lib.mlc_hip_replay(handle))

    def captureRelease(self, handle: int) -> None:
        self._lib.mlc_hip_capture_release(handle)

    # -- measurement helpers
    def timerStart(self) -> bool:
        return bool(self._lib.mlc_hip_timer_start())

    def timerStopMs(self) -> float:
        return float(self._lib.mlc_hip_timer_stop())

    def lastDecodeLaunches(self) -> int:
        return int(self._lib.mlc_hip_last_decode_launches())

    def lastDecodeWorkItems(self) -> int:
        return int(self._lib.mlc_hip_last_decode_work_items())

    def lastDecodeKernel(self) -> str:
        return (self._lib.mlc_hip_last_decode_kernel() or b"").decode()

    def tableUploads(self) -> int:
        """Times so far the decode path copied a page table to the device."""
        return int(self._lib.mlc_hip_decode_table_uploads())

    def fusedKvWriteLaunches(self) -> int:
        """KV writes so far that went out fused with a neighbour (option "fuse_row_ops")."""
        return int(self._lib.mlc_hip_fused_kv_write_launches())

    def kvWritesInDecodeLaunches(self) -> int:
        """Decode attention launches so far that carried the step's KV write."""
        return int(self._lib.mlc_hip_kv_writes_in_decode_launches())

    def fusedMatmulRopeLaunches(self) -> int:
        """Q4_0 matmuls so far launched with the split + RoPE + cast of their output as epilogue."""
        return int(self._lib.mlc_hip_fused_matmul_rope_launches())

    def fusedMatmulSiluLaunches(self) -> int:
        """Q4_0 matmuls so far launched with the gate/up split + SiLU * up of their output as epilogue."""
        return int(self._lib.mlc_hip_fused_matmul_silu_launches())

    def fusedMatmulSiluSplitLaunches(self) -> int:
        """... of which also wrote the activation fragments of the matmul that reads the products."""
        return int(self._lib.mlc_hip_fused_matmul_silu_split_launches())

    def fusedDecodeSplitLaunches(self) -> int:
        """Decode attention launches so far that also wrote the next Q4_0 matmul's activation fragments."""
        return int(self._lib.mlc_hip_fused_decode_split_launches())

    def fusedMatmulNormLaunches(self) -> int:
        """Q4_0 matmuls so far launched with the residual add, the RMSNorm's sums and the next matmul's
        input as epilogue."""
        return int(self._lib.mlc_hip_fused_matmul_norm_launches())

    def rowProgramLaunches(self) -> int:
        """Fused row-operator launches so far (option "fuse_row_ops")."""
        return int(self._lib.mlc_hip_row_program_launches())

    def setOption(self, name: str, value: int) -> bool:
        return bool(self._lib.mlc_hip_set_option(name.encode(), int(value)))

    def stream(self) -> int:
        return self._lib.mlc_hip_stream() or 0
