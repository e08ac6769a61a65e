"""Seeded synthetic workloads of the paged attention path: the reference's own test scenarios
(tests/test_paged_flash.cpp:214-275), the benchmark configurations, chunked-prefill inputs, one
decoder layer's Q4_0 / Q6_K weights (block formats of compiler/runtime/quantization.cpp) and a
helper that pushes a decode workload through the HIP executor.  Everything here is numpy and the
executor: the benchmark and the parity tests build their inputs from this one module."""
from __future__ import annotations

from dataclasses import dataclass, field

import numpy as np


@dataclass
class DecodeCase:
    name: str
    batch: int
    num_heads: int
    kv_heads: int
    head_dim: int
    page_size: int
    capacity_pages: int
    seq_lens: np.ndarray
    q_positions: np.ndarray
    page_tables_flat: np.ndarray
    page_table_offsets: np.ndarray
    apply_causal: bool
    q: np.ndarray = field(repr=False, default=None)          # fp32 [B,H,D]
    k_pages: np.ndarray = field(repr=False, default=None)    # uint16 view of fp16 pool
    v_pages: np.ndarray = field(repr=False, default=None)

    @property
    def kv_bytes(self) -> int:
        """Algorithmic KV bytes of one decode call: sum_r 2 * S_r * Hkv * D * 2."""
        lim = np.minimum(self.seq_lens, self.q_positions + 1) if self.apply_causal else self.seq_lens
        return int(lim.astype(np.int64).sum()) * 4 * self.kv_heads * self.head_dim


def _f16_bits(rng: np.random.Generator, n: int, dist: str) -> np.ndarray:
    out = np.empty(n, np.uint16)
    step = 1 << 24
    for i in range(0, n, step):
        m = min(step, n - i)
        if dist == "normal":
            x = rng.standard_normal(m, dtype=np.float32)
        else:
            x = rng.random(m, dtype=np.float32) - 0.5
        out[i:i + m] = x.astype(np.float16).view(np.uint16)
    return out


def make_case(name, batch, num_heads, kv_heads, head_dim, page_size, seq_lens, *, capacity_pages=None,
              causal=True, q_positions=None, permute=True, seed=0, dist="normal",
              scale_k_rows=0.0) -> DecodeCase:
    rng = np.random.default_rng(seed)
    seq_lens = np.asarray(seq_lens, np.uint32)
    pages_needed = (seq_lens.astype(np.int64) + page_size - 1) // page_size
    total_pages = int(pages_needed.sum())
    if capacity_pages is None:
        capacity_pages = max(total_pages, 1)
    assert total_pages <= capacity_pages
    ids = rng.permutation(capacity_pages).astype(np.uint32) if permute else np.arange(capacity_pages, dtype=np.uint32)
    flat = ids[:total_pages].copy()
    off = np.zeros(batch + 1, np.uint32)
    off[1:] = np.cumsum(pages_needed)
    if q_positions is None:
        q_positions = np.where(seq_lens > 0, seq_lens - 1, 0).astype(np.uint32)
    q_positions = np.asarray(q_positions, np.uint32)
    n_el = capacity_pages * page_size * kv_heads * head_dim
    q = (rng.standard_normal((batch, num_heads, head_dim), dtype=np.float32) if dist == "normal"
         else (rng.random((batch, num_heads, head_dim), dtype=np.float32) - 0.5))
    k = _f16_bits(rng, n_el, dist)
    v = _f16_bits(rng, n_el, dist)
    if scale_k_rows > 0:
        # a fraction of K token rows (all heads) scaled x8 to stress max tracking
        rows = capacity_pages * page_size
        pick = rng.random(rows) < scale_k_rows
        kk = k.view(np.float16).reshape(rows, kv_heads * head_dim)
        kk[pick] = (kk[pick].astype(np.float32) * 8.0).astype(np.float16)
    return DecodeCase(name, batch, num_heads, kv_heads, head_dim, page_size, capacity_pages,
                      seq_lens, q_positions, flat, off, causal, q, k, v)


def reference_scenarios():
    """The seven scenarios of tests/test_paged_flash.cpp:214-275 (uniform(-0.5, 0.5) inputs,
    ascending page ids, q at the last token)."""
    S = []
    mk = lambda *a, **k: S.append(make_case(*a, permute=False, dist="uniform", seed=0xBEEF, **k))
    mk("SingleRequestSmall", 1, 2, 2, 64, 4, [8], capacity_pages=8)
    mk("TwoRequestsDisjointPages", 2, 2, 2, 64, 4, [10, 12], capacity_pages=16)
    mk("FourRequestsGQA", 4, 8, 2, 64, 4, [20, 14, 8, 18], capacity_pages=32)
    mk("EightRequestsVariableLength", 8, 8, 2, 64, 8, [4, 12, 20, 32, 7, 16, 28, 11], capacity_pages=64)
    mk("MultiplePagesPerRequest", 4, 4, 2, 64, 16, [64, 50, 40, 32], capacity_pages=32)
    mk("TinyLlamaLikeShape", 4, 32, 4, 64, 64, [32, 48, 64, 96], capacity_pages=8)
    mk("NoCausal", 2, 4, 2, 64, 8, [16, 24], capacity_pages=16, causal=False)
    return S


def baseline_config(idx: int, *, batch=None, seed=1234) -> DecodeCase:
    """Decode configurations 1-4 of the benchmark definition."""
    rng = np.random.default_rng(seed + idx)
    if idx == 1:
        return make_case("cfg1_single", 1, 32, 4, 64, 64, [512], capacity_pages=8, permute=False, seed=seed)
    if idx == 2:
        b = batch or 32
        sl = rng.integers(128, 2049, size=b)
        cap = 1024 if b == 32 else int(((sl + 63) // 64).sum()) + 64
        return make_case(f"cfg2_tinyllama_b{b}", b, 32, 4, 64, 64, sl, capacity_pages=cap, seed=seed)
    if idx == 3:
        b = batch or 64
        sl = rng.integers(256, 4097, size=b)
        cap = int(((sl + 63) // 64).sum()) + 64
        return make_case("cfg3_decode_step_b64", b, 32, 4, 64, 64, sl, capacity_pages=max(cap, 4096 if b == 64 else cap), seed=seed)
    if idx == 4:
        b = batch or 64
        sl = rng.integers(1024, 8193, size=b)
        cap = 16384 if b == 64 else int(((sl + 63) // 64).sum()) + 16
        return make_case("cfg4_llama3_8b", b, 32, 8, 128, 64, sl, capacity_pages=cap, seed=seed, scale_k_rows=0.01)
    raise ValueError(idx)


class DeviceCase:
    """Uploads a DecodeCase through the executor's buffer calls (like
    tests/test_paged_flash.cpp:171-186) and runs the decode entry points."""

    def __init__(self, exe, case: DecodeCase):
        self.exe, self.case = exe, case
        c = case
        self.q_buf = exe.allocateScratchBuffer(c.q.nbytes)
        self.k_buf = exe.allocateScratchBuffer(c.k_pages.nbytes)
        self.v_buf = exe.allocateScratchBuffer(c.v_pages.nbytes)
        self.o_buf = exe.allocateScratchBuffer(c.q.nbytes)
        assert self.q_buf and self.k_buf and self.v_buf and self.o_buf
        assert exe.uploadToBuffer(self.q_buf, c.q)
        assert exe.uploadToBuffer(self.k_buf, c.k_pages)
        assert exe.uploadToBuffer(self.v_buf, c.v_pages)
        # poison the output so a kernel that writes nothing is caught
        assert exe.uploadToBuffer(self.o_buf, np.full(c.q.shape, np.nan, np.float32))

    def run(self, sync=True) -> np.ndarray:
        c, e = self.case, self.exe
        args = (self.q_buf, self.k_buf, self.v_buf, self.o_buf, c.page_tables_flat,
                c.page_table_offsets, c.seq_lens, c.q_positions, c.batch, c.num_heads,
                c.kv_heads, c.head_dim, c.page_size, c.apply_causal)
        if sync:
            assert e.runPagedFlashAttention(*args), e.lastError()
        else:
            assert e.beginForwardPassCB()
            assert e.encodePagedFlashAttention(*args), e.lastError()
            assert e.flushForwardPassCB(), e.lastError()
        out = np.empty(c.q.shape, np.float32)
        assert e.downloadFromBuffer(self.o_buf, out)
        return out

    def free(self):
        for b in (self.q_buf, self.k_buf, self.v_buf, self.o_buf):
            self.exe.releaseScratchBuffer(b)


def make_prefill(B, C, H, Hkv, D, P, ctx, seed=0, scale_k=0.0):
    """Chunked-prefill input: ctx[r] cached tokens, then a chunk of C new tokens (already written
    to the cache); q is fp16 [B][C][H][D], the pools and tables are laid out as for decode."""
    rng = np.random.default_rng(seed)
    ctx = np.asarray(ctx, np.int64)
    seq = (ctx + C).astype(np.uint32)
    pages = (seq.astype(np.int64) + P - 1) // P
    cap = int(pages.sum()) + 3
    ids = rng.permutation(cap).astype(np.uint32)
    flat = ids[:int(pages.sum())]
    off = np.zeros(B + 1, np.uint32)
    off[1:] = np.cumsum(pages)
    q = rng.standard_normal((B, C, H, D), dtype=np.float32).astype(np.float16)
    k = rng.standard_normal(cap * P * Hkv * D, dtype=np.float32).astype(np.float16)
    v = rng.standard_normal(cap * P * Hkv * D, dtype=np.float32).astype(np.float16)
    return dict(B=B, C=C, H=H, Hkv=Hkv, D=D, P=P, seq=seq, q_start=ctx.astype(np.uint32), flat=flat,
                off=off, q=q.view(np.uint16), k=k.view(np.uint16), v=v.view(np.uint16))


# ---------------------------------------------------------------------------------------------
# GGUF block formats, as numpy encoders (the operators only ever decode them)
# ---------------------------------------------------------------------------------------------

def q4_0_row_bytes(cols: int) -> int:
    return cols // 32 * 18


def quantize_q4_0(w) -> np.ndarray:
    """Rows of floats -> Q4_0 rows, uint8 [rows][cols/32*18]: per block of 32 an fp16 scale
    d = (value of largest magnitude) / -8 and 32 four-bit codes min(15, trunc(x/d + 8.5)), element j in
    the low and element j+16 in the high nibble of byte j (quantizeRowQ4_0,
    compiler/runtime/quantization.cpp)."""
    w = np.ascontiguousarray(w, np.float32)
    rows, cols = w.shape
    assert cols % 32 == 0
    x = w.reshape(rows, cols // 32, 32)
    pick = np.argmax(np.abs(x), axis=2)
    mx = np.take_along_axis(x, pick[..., None], axis=2)[..., 0]
    d = (mx / np.float32(-8.0)).astype(np.float32)
    inv = np.where(d != 0, np.float32(1.0) / np.where(d != 0, d, np.float32(1.0)), np.float32(0.0)).astype(np.float32)
    codes = np.minimum(15, (x * inv[..., None] + np.float32(8.5)).astype(np.int32)).astype(np.uint8)
    out = np.empty((rows, cols // 32, 18), np.uint8)
    out[..., :2] = d.astype(np.float16).view(np.uint8).reshape(rows, cols // 32, 2)
    out[..., 2:] = codes[..., :16] | (codes[..., 16:] << 4)
    return out.reshape(rows, q4_0_row_bytes(cols))


def q6_k_row_bytes(cols: int) -> int:
    return cols // 256 * 210


def quantize_q6_k(w) -> np.ndarray:
    """Rows of floats -> Q6_K rows, uint8 [rows][cols/256*210]: per super-block of 256, low nibbles
    ql[128], high bit pairs qh[64], sixteen int8 sub-block scales and one fp16 scale; element i
    decodes to d * scales[i/16] * (code_i - 32) (dequantizeRowQ6_K, compiler/runtime/
    quantization.cpp).  A plain round-to-nearest encoder: the scales are not searched the way the
    reference's quantiser searches them, which the operators that read the format cannot tell."""
    w = np.ascontiguousarray(w, np.float32)
    rows, cols = w.shape
    assert cols % 256 == 0
    nb = cols // 256
    x = w.reshape(rows, nb, 16, 16)
    sub = np.abs(x).max(axis=3) / np.float32(31.0)                   # [rows, nb, 16]
    top = sub.max(axis=2)
    d = (top / np.float32(127.0)).astype(np.float16)
    d32 = d.astype(np.float32)
    safe = np.where(d32 > 0, d32, np.float32(1.0))
    sc = np.clip(np.rint(sub / safe[..., None]), 1, 127).astype(np.int8)
    step = d32[..., None] * sc.astype(np.float32)
    codes = np.where(step[..., None] > 0, np.rint(x / np.where(step > 0, step, 1.0)[..., None]), 0.0)
    codes = (np.clip(codes, -32, 31) + 32).astype(np.uint8).reshape(rows, nb, 2, 4, 32)   # half, quarter, l
    lo, hi = codes & 0xF, codes >> 4
    out = np.empty((rows, nb, 210), np.uint8)
    ql = out[..., :128].reshape(rows, nb, 2, 64)
    ql[..., :32] = lo[..., 0, :] | (lo[..., 2, :] << 4)
    ql[..., 32:] = lo[..., 1, :] | (lo[..., 3, :] << 4)
    out[..., 128:192] = (hi[..., 0, :] | (hi[..., 1, :] << 2) | (hi[..., 2, :] << 4)
                         | (hi[..., 3, :] << 6)).reshape(rows, nb, 64)
    out[..., 192:208] = sc.view(np.uint8)
    out[..., 208:] = d.view(np.uint8).reshape(rows, nb, 2)
    return out.reshape(rows, q6_k_row_bytes(cols))


# ---------------------------------------------------------------------------------------------
# One TinyLlama-shape decoder layer of the reference's batched decode step
# (compiler/runtime/batched_walker.cpp:246-405) as data
# ---------------------------------------------------------------------------------------------

HID, H, HKV, D, FFN, P = 2048, 32, 4, 64, 5632, 64
Q_ROWS, KV_ROWS = H * D, HKV * D
QKV_ROWS = Q_ROWS + 2 * KV_ROWS
VOCAB = 32000


def q4_weights(rng, rows, cols, scale):
    return quantize_q4_0((rng.standard_normal((rows, cols)) * scale).astype(np.float32))


def make_layer_weights(seed):
    rng = np.random.default_rng(seed)
    return {
        "w_qkv": q4_weights(rng, QKV_ROWS, HID, 0.03),
        "w_o": q4_weights(rng, HID, HID, 0.03),
        "w_gu": q4_weights(rng, 2 * FFN, HID, 0.03),
        "w_down": q4_weights(rng, HID, FFN, 0.02),
        "g_attn": rng.uniform(0.5, 1.5, HID).astype(np.float32),
        "g_ffn": rng.uniform(0.5, 1.5, HID).astype(np.float32),
    }


def make_head_weights(rng):
    """Final norm vector and the Q6_K output matrix of the model (32000 x 2048)."""
    head_norm = rng.uniform(0.5, 1.5, HID).astype(np.float32)
    return head_norm, quantize_q6_k((rng.standard_normal((VOCAB, HID)) * 0.03).astype(np.float32))


def weight_bytes(w):
    return sum(w[k].nbytes for k in ("w_qkv", "w_o", "w_gu", "w_down"))


def rotary_tables(q_positions, head_dim=D, theta=10000.0):
    """cos/sin [batch][head_dim/2] of angle position * theta^(-2i/head_dim) in single precision
    (the reference's rotary coefficients, compiler/runtime/quantization.cpp:795-823)."""
    i = np.arange(head_dim // 2, dtype=np.float32)
    inv_freq = np.power(np.float32(theta), -(np.float32(2.0) * i / np.float32(head_dim))).astype(np.float32)
    ang = (np.asarray(q_positions, np.float32)[:, None] * inv_freq).astype(np.float32)
    return np.cos(ang).astype(np.float32), np.sin(ang).astype(np.float32)
