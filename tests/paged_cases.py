"""Seeded synthetic workloads for the paged attention path and helpers that push
them through the HIP executor.  The shapes are the reference's own test scenarios
(tests/test_paged_flash.cpp:214-275) and the five benchmark configurations."""
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
        return make_case("cfg2_tinyllama_b32", b, 32, 4, 64, 64, sl, capacity_pages=1024, seed=seed)
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


def oracle_decode(case: DecodeCase, n_threads=8):
    from oracle import paged_oracle as po
    c = case
    return po.paged_attention_executor(c.q, c.k_pages, c.v_pages, c.page_tables_flat,
                                       c.page_table_offsets, c.seq_lens, c.q_positions, c.batch,
                                       c.num_heads, c.kv_heads, c.head_dim, c.page_size,
                                       c.apply_causal, n_threads)


# acceptance bar of the benchmark definition: per (request, head)
MIN_COSINE = 0.9999
MAX_ABS = 2e-3


def assert_parity(got, want, head_dim, what=""):
    from oracle import paged_oracle as po
    assert np.all(np.isfinite(got)), f"{what}: non-finite output"
    rep = po.per_head_report(got, want, head_dim)
    assert rep["min_cosine"] >= MIN_COSINE, f"{what}: {rep}"
    assert rep["max_abs"] <= MAX_ABS, f"{what}: {rep}"
    return rep
