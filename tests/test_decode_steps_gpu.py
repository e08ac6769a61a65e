"""Decode as the batched walker drives it (compiler/runtime/batched_walker.cpp:128-142, 304-331):
every step extends each request by one token, scatters the new K row and the new V row to the
(page, slot) the allocator handed out, and attends over the updated cache.

* configuration 3 at its full size (batch 64, contexts 256..4096) as one such step, all 64
  requests against the oracle, both pools bit-exact;
* 130 consecutive steps of a small batch: requests cross tile and page boundaries (a fresh page is
  opened whenever a request's last page is full), the attention launch carries the write at every
  step, and the device copy of the page table is refreshed only at the steps where some table
  actually grew."""
from dataclasses import replace

import numpy as np
import pytest

from oracle import paged_oracle as po
from paged_cases import DeviceCase, assert_parity, baseline_config, make_case, oracle_decode
from test_kv_write_in_decode_gpu import _expect, _newest, _rows, _step

pytestmark = pytest.mark.gpu


def test_config3_full_size_step_every_request(exe):
    case = baseline_config(3)
    assert case.batch == 64
    ids, slots = _newest(case)                 # (page_table.back(), (S - 1) % 64), some at slot 0 of a fresh page
    new_k, new_v = _rows(case, 303)
    want_k, want_v, want_o = _expect(case, ids, slots, new_k, new_v)
    print(f"[case] config 3 full step, KV bytes {case.kv_bytes}", flush=True)
    out, kp, vp, carried = _step(exe, case, ids, slots, new_k, new_v, 1)
    assert carried == 1
    assert np.array_equal(kp, want_k) and np.array_equal(vp, want_v)
    rep = assert_parity(out, want_o, case.head_dim, "config 3 step")
    print("[case] config 3 step:", rep, flush=True)


def test_130_consecutive_decode_steps(exe):
    H, HKV, D, P, STEPS = 32, 4, 64, 64, 130
    start = [0, 59, 63, 64, 120, 500, 1000]           # tokens already cached per request
    B = len(start)
    cap = sum((s + STEPS + P - 1) // P for s in start) + 2
    rng = np.random.default_rng(130)
    free = list(rng.permutation(cap).astype(np.uint32))    # page ids in the order they are handed out
    tables = []
    for s in start:
        tables.append([free.pop() for _ in range((s + P - 1) // P)])
    row = HKV * D
    k_pool = rng.standard_normal(cap * P * row, dtype=np.float32).astype(np.float16).view(np.uint16)
    v_pool = rng.standard_normal(cap * P * row, dtype=np.float32).astype(np.float16).view(np.uint16)
    q_all = rng.standard_normal((STEPS, B, H, D), dtype=np.float32)

    k_buf, v_buf = exe.allocateScratchBuffer(k_pool.nbytes), exe.allocateScratchBuffer(v_pool.nbytes)
    q_buf, o_buf = exe.allocateScratchBuffer(B * H * D * 4), exe.allocateScratchBuffer(B * H * D * 4)
    nk_buf, nv_buf = exe.allocateScratchBuffer(B * row * 2), exe.allocateScratchBuffer(B * row * 2)
    lens = list(start)
    uploads0, carried0 = exe.tableUploads(), exe.kvWritesInDecodeLaunches()
    grew_steps = 0
    try:
        assert exe.uploadToBuffer(k_buf, k_pool) and exe.uploadToBuffer(v_buf, v_pool)
        for step in range(STEPS):
            # the allocator's part (RequestKVState::extend_one_token, paged_kv.cpp:52-66)
            ids, slots, grew = [], [], False
            for r in range(B):
                if lens[r] % P == 0:
                    tables[r].append(free.pop())
                    grew = True
                ids.append(tables[r][-1])
                slots.append(lens[r] % P)
                lens[r] += 1
            grew_steps += grew or step == 0
            flat = np.array([p for t in tables for p in t], np.uint32)
            off = np.zeros(B + 1, np.uint32)
            off[1:] = np.cumsum([len(t) for t in tables])
            seq = np.array(lens, np.uint32)
            qpos = seq - 1
            new_k = rng.standard_normal((B, row), dtype=np.float32).astype(np.float16).view(np.uint16)
            new_v = rng.standard_normal((B, row), dtype=np.float32).astype(np.float16).view(np.uint16)
            assert exe.uploadToBuffer(q_buf, q_all[step]) and exe.uploadToBuffer(nk_buf, new_k)
            assert exe.uploadToBuffer(nv_buf, new_v)
            assert exe.beginForwardPassCB()
            assert exe.encodeScatterKVPagedBatched(k_buf, ids, slots, P, HKV, D, B, nk_buf), exe.lastError()
            assert exe.encodeScatterKVPagedBatched(v_buf, ids, slots, P, HKV, D, B, nv_buf), exe.lastError()
            assert exe.encodePagedFlashAttention(q_buf, k_buf, v_buf, o_buf, flat, off, seq, qpos, B, H, HKV, D, P,
                                                 True), exe.lastError()
            assert exe.flushForwardPassCB(), exe.lastError()
            got = np.empty((B, H, D), np.float32)
            assert exe.downloadFromBuffer(o_buf, got)
            # the same step on the host copy of the pools
            assert po.scatter_kv_paged_batched_f16(k_pool, ids, slots, P, HKV, D, B, new_k)
            assert po.scatter_kv_paged_batched_f16(v_pool, ids, slots, P, HKV, D, B, new_v)
            want = po.paged_attention_executor(q_all[step], k_pool, v_pool, flat, off, seq, qpos, B, H, HKV, D, P,
                                               True, 4)
            assert_parity(got, want, D, f"step {step} lens {lens}")
        kp, vp = np.empty_like(k_pool), np.empty_like(v_pool)
        assert exe.downloadFromBuffer(k_buf, kp) and exe.downloadFromBuffer(v_buf, vp)
        assert np.array_equal(kp, k_pool) and np.array_equal(vp, v_pool)
    finally:
        for b in (k_buf, v_buf, q_buf, o_buf, nk_buf, nv_buf):
            exe.releaseScratchBuffer(b)
    assert exe.kvWritesInDecodeLaunches() - carried0 == STEPS       # the attention launch took every write
    # tables of this size travel inside the kernel arguments: nothing was copied to the device,
    # although the table changed at every step where some request opened a page
    assert exe.tableUploads() - uploads0 == 0
    assert 0 < grew_steps < STEPS // 4


def test_large_page_table_is_uploaded_only_when_it_changes(exe):
    H, HKV, D, P = 32, 4, 64, 64
    lens = [30000 - 2, 29000, 64 * 300 - 1]       # 1 240 pages: more than the kernel arguments hold
    B = len(lens)
    cap = sum((s + 8 + P - 1) // P for s in lens) + 2
    rng = np.random.default_rng(31)
    free = list(rng.permutation(cap).astype(np.uint32))
    tables = [[free.pop() for _ in range((s + P - 1) // P)] for s in lens]
    row = HKV * D
    k_pool = rng.standard_normal(cap * P * row, dtype=np.float32).astype(np.float16).view(np.uint16)
    v_pool = rng.standard_normal(cap * P * row, dtype=np.float32).astype(np.float16).view(np.uint16)
    k_buf, v_buf = exe.allocateScratchBuffer(k_pool.nbytes), exe.allocateScratchBuffer(v_pool.nbytes)
    q_buf, o_buf = exe.allocateScratchBuffer(B * H * D * 4), exe.allocateScratchBuffer(B * H * D * 4)
    uploads = []
    try:
        assert exe.uploadToBuffer(k_buf, k_pool) and exe.uploadToBuffer(v_buf, v_pool)
        for step in range(4):
            grew = False
            for r in range(B):
                if lens[r] % P == 0:
                    tables[r].append(free.pop())
                    grew = True
                lens[r] += 1
            flat = np.array([p for t in tables for p in t], np.uint32)
            off = np.zeros(B + 1, np.uint32)
            off[1:] = np.cumsum([len(t) for t in tables])
            seq = np.array(lens, np.uint32)
            q = rng.standard_normal((B, H, D), dtype=np.float32)
            assert exe.uploadToBuffer(q_buf, q)
            before = exe.tableUploads()
            for _layer in range(3):        # the layers of a step pass the same tables
                assert exe.runPagedFlashAttention(q_buf, k_buf, v_buf, o_buf, flat, off, seq, seq - 1, B, H, HKV, D, P,
                                                  True), exe.lastError()
            uploads.append((grew or step == 0, exe.tableUploads() - before))
            got = np.empty((B, H, D), np.float32)
            assert exe.downloadFromBuffer(o_buf, got)
            want = po.paged_attention_executor(q, k_pool, v_pool, flat, off, seq, seq - 1, B, H, HKV, D, P, True, 8)
            assert_parity(got, want, D, f"long requests, step {step}")
    finally:
        for b in (k_buf, v_buf, q_buf, o_buf):
            exe.releaseScratchBuffer(b)
    assert [n for _, n in uploads] == [1 if changed else 0 for changed, _ in uploads], uploads
    assert sum(changed for changed, _ in uploads) in (2, 3)     # the first step and where a request opened a page
