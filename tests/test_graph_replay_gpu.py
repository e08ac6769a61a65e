"""A decode step captured once into a HIP graph (mlc_hip_capture_begin / _end) and replayed for
the following steps with the tables refreshed in place (mlc_hip_replay_update / mlc_hip_replay).

The captured pass is what the batched walker encodes around the attention of one layer
(compiler/runtime/batched_walker.cpp:304-349): scatter the new K row, scatter the new V row,
paged attention, residual add.  Every replayed step is compared bit for bit with the same step
encoded call by call on a second set of buffers, and with the oracle; requests cross tile and
page boundaries on the way (tables grow), with no launch re-recorded."""
import numpy as np
import pytest

from oracle import paged_oracle as po
from paged_cases import assert_parity

pytestmark = pytest.mark.gpu

H, HKV, D, P = 32, 4, 64, 64
ROW = HKV * D


class _Buffers:
    def __init__(self, exe, k_pool, v_pool, B):
        self.exe = exe
        self.k = exe.allocateScratchBuffer(k_pool.nbytes)
        self.v = exe.allocateScratchBuffer(v_pool.nbytes)
        self.q = exe.allocateScratchBuffer(B * H * D * 4)
        self.o = exe.allocateScratchBuffer(B * H * D * 4)
        self.y = exe.allocateScratchBuffer(B * H * D * 4)
        self.nk = exe.allocateScratchBuffer(B * ROW * 2)
        self.nv = exe.allocateScratchBuffer(B * ROW * 2)
        assert exe.uploadToBuffer(self.k, k_pool) and exe.uploadToBuffer(self.v, v_pool)

    def inputs(self, q, new_k, new_v):
        e = self.exe
        assert e.uploadToBuffer(self.q, q) and e.uploadToBuffer(self.nk, new_k) and e.uploadToBuffer(self.nv, new_v)

    def encode(self, t, B):
        e = self.exe
        assert e.encodeScatterKVPagedBatched(self.k, t["ids"], t["slots"], P, HKV, D, B, self.nk), e.lastError()
        assert e.encodeScatterKVPagedBatched(self.v, t["ids"], t["slots"], P, HKV, D, B, self.nv), e.lastError()
        assert e.encodePagedFlashAttention(self.q, self.k, self.v, self.o, t["flat"], t["off"], t["seq"], t["qpos"],
                                           B, H, HKV, D, P, True), e.lastError()
        assert e.encodeAddBatched(self.o, self.q, self.y, B * H * D), e.lastError()

    def outputs(self, B):
        o, y = np.empty((B, H, D), np.float32), np.empty((B, H, D), np.float32)
        assert self.exe.downloadFromBuffer(self.o, o) and self.exe.downloadFromBuffer(self.y, y)
        return o, y

    def pools(self, like):
        k, v = np.empty_like(like), np.empty_like(like)
        assert self.exe.downloadFromBuffer(self.k, k) and self.exe.downloadFromBuffer(self.v, v)
        return k, v

    def free(self):
        for b in (self.k, self.v, self.q, self.o, self.y, self.nk, self.nv):
            self.exe.releaseScratchBuffer(b)


class _Requests:
    """The allocator's part of a step (RequestKVState::extend_one_token, paged_kv.cpp:52-66)."""

    def __init__(self, start, cap, rng):
        self.free = list(rng.permutation(cap).astype(np.uint32))
        self.tables = [[self.free.pop() for _ in range((s + P - 1) // P)] for s in start]
        self.lens = list(start)

    def step(self):
        ids, slots = [], []
        for r in range(len(self.lens)):
            if self.lens[r] % P == 0:
                self.tables[r].append(self.free.pop())
            ids.append(self.tables[r][-1])
            slots.append(self.lens[r] % P)
            self.lens[r] += 1
        off = np.zeros(len(self.lens) + 1, np.uint32)
        off[1:] = np.cumsum([len(t) for t in self.tables])
        seq = np.array(self.lens, np.uint32)
        return dict(ids=np.array(ids, np.uint32), slots=np.array(slots, np.uint32),
                    flat=np.array([p for t in self.tables for p in t], np.uint32), off=off, seq=seq, qpos=seq - 1)


def test_replayed_steps_equal_encoded_steps(exe):
    start, steps = [63, 64, 130, 700, 1, 0], 70
    B = len(start)
    cap = sum((s + steps + P - 1) // P for s in start) + 2
    rng = np.random.default_rng(2024)
    reqs = _Requests(start, cap, rng)
    k_pool = rng.standard_normal(cap * P * ROW, dtype=np.float32).astype(np.float16).view(np.uint16)
    v_pool = rng.standard_normal(cap * P * ROW, dtype=np.float32).astype(np.float16).view(np.uint16)
    eager, graph = _Buffers(exe, k_pool, v_pool, B), _Buffers(exe, k_pool, v_pool, B)
    handle = 0
    carried0 = exe.kvWritesInDecodeLaunches()
    try:
        for step in range(steps):
            t = reqs.step()
            q = rng.standard_normal((B, H, D), dtype=np.float32)
            new_k = rng.standard_normal((B, ROW), dtype=np.float32).astype(np.float16).view(np.uint16)
            new_v = rng.standard_normal((B, ROW), dtype=np.float32).astype(np.float16).view(np.uint16)
            for bufs in (eager, graph):
                bufs.inputs(q, new_k, new_v)
            # the step encoded call by call
            assert exe.beginForwardPassCB()
            eager.encode(t, B)
            assert exe.flushForwardPassCB(), exe.lastError()
            if step == 0:
                # once uncaptured on the other buffers too (this is the execution of step 0 there),
                # then the same calls recorded
                assert exe.beginForwardPassCB()
                graph.encode(t, B)
                assert exe.flushForwardPassCB(), exe.lastError()
                assert exe.beginForwardPassCB()
                assert exe.captureBegin(), exe.lastError()
                graph.encode(t, B)
                handle = exe.captureEnd()
                assert handle > 0, exe.lastError()
                assert exe.flushForwardPassCB()
                assert exe.capturedLaunches(handle) == 2      # attention (carrying the KV write) and the add
            else:
                assert exe.replayUpdate(handle, t["flat"], t["off"], t["seq"], t["qpos"], t["ids"], t["slots"]), \
                    exe.lastError()
                assert exe.beginForwardPassCB()
                assert exe.replay(handle), exe.lastError()
                assert exe.flushForwardPassCB(), exe.lastError()
            o_e, y_e = eager.outputs(B)
            o_g, y_g = graph.outputs(B)
            assert np.array_equal(o_e, o_g) and np.array_equal(y_e, y_g), f"step {step}"
            assert po.scatter_kv_paged_batched_f16(k_pool, t["ids"], t["slots"], P, HKV, D, B, new_k)
            assert po.scatter_kv_paged_batched_f16(v_pool, t["ids"], t["slots"], P, HKV, D, B, new_v)
            want = po.paged_attention_executor(q, k_pool, v_pool, t["flat"], t["off"], t["seq"], t["qpos"], B, H, HKV,
                                               D, P, True, 4)
            assert_parity(o_g, want, D, f"replayed step {step}")
            assert np.array_equal(y_g, o_g + q)
        for bufs in (eager, graph):
            kp, vp = bufs.pools(k_pool)
            assert np.array_equal(kp, k_pool) and np.array_equal(vp, v_pool)
        # one launch per encoded step carried the write (+ the warm-up pass); replays encode nothing
        assert exe.kvWritesInDecodeLaunches() - carried0 == steps + 2
    finally:
        if handle:
            exe.captureRelease(handle)
        eager.free()
        graph.free()


def test_what_a_capture_and_a_replay_refuse(exe):
    B = 3
    rng = np.random.default_rng(7)
    reqs = _Requests([10, 70, 200], 16, rng)
    pool = rng.standard_normal(16 * P * ROW, dtype=np.float32).astype(np.float16).view(np.uint16)
    bufs = _Buffers(exe, pool, pool, B)
    handle = 0
    try:
        t = reqs.step()
        bufs.inputs(rng.standard_normal((B, H, D), dtype=np.float32), pool[:B * ROW], pool[:B * ROW])
        # tables the library has not seen yet cannot be captured: the copy to the device is not a launch
        assert exe.beginForwardPassCB()
        assert exe.captureBegin(), exe.lastError()
        ok = exe.encodePagedFlashAttention(bufs.q, bufs.k, bufs.v, bufs.o, t["flat"], t["off"], t["seq"], t["qpos"], B,
                                           H, HKV, D, P, True)
        assert not ok and "captured" in exe.lastError()
        assert exe.captureEnd() == 0
        assert not exe.captureBegin() or exe.captureEnd() == 0      # an empty capture is refused as well
        assert exe.flushForwardPassCB()
        # uploads, downloads and waits are refused while capturing, and leave the capture unusable
        assert exe.beginForwardPassCB() and exe.captureBegin()
        assert not exe.uploadToBuffer(bufs.q, np.zeros(4, np.float32))
        assert exe.captureEnd() == 0
        assert exe.flushForwardPassCB()
        # after one uncaptured pass the same calls can be captured
        assert exe.beginForwardPassCB()
        bufs.encode(t, B)
        assert exe.flushForwardPassCB()
        assert exe.beginForwardPassCB() and exe.captureBegin()
        bufs.encode(t, B)
        handle = exe.captureEnd()
        assert handle > 0, exe.lastError()
        assert exe.flushForwardPassCB()
        t2 = reqs.step()
        # another batch size, rows that are not the newest positions, a table that does not cover its length
        assert not exe.replayUpdate(handle, t2["flat"], t2["off"][:-1], t2["seq"][:-1], t2["qpos"][:-1], t2["ids"][:-1],
                                    t2["slots"][:-1])
        stale = t2["slots"].copy()
        stale[1] = (stale[1] + 63) % 64
        assert not exe.replayUpdate(handle, t2["flat"], t2["off"], t2["seq"], t2["qpos"], t2["ids"], stale)
        assert "newest" in exe.lastError()
        long_seq = t2["seq"].copy()
        long_seq[0] += 500
        assert not exe.replayUpdate(handle, t2["flat"], t2["off"], long_seq, long_seq - 1, t2["ids"], t2["slots"])
        assert exe.replayUpdate(handle, t2["flat"], t2["off"], t2["seq"], t2["qpos"], t2["ids"], t2["slots"]), exe.lastError()
        assert not exe.replay(handle + 1000)
    finally:
        if handle:
            exe.captureRelease(handle)
        bufs.free()


def test_capture_in_a_process_that_only_saw_small_tables():
    """Small tables travel inside the kernel arguments and are never copied to the device by an
    ordinary call; a capture must still find them there (capture_begin sends them).  Run in a
    process of its own, so that no earlier test has put tables on the device."""
    import os
    import subprocess
    import sys
    code = r"""
import sys, numpy as np
sys.path.insert(0, %r); sys.path.insert(0, %r)
import test_graph_replay_gpu as t
from mlcompiler_amd import HipExecutor
exe = HipExecutor.Instance(); exe.requireAvailable()
rng = np.random.default_rng(3)
reqs = t._Requests([5, 70], 8, rng)
pool = rng.standard_normal(8 * t.P * t.ROW, dtype=np.float32).astype(np.float16).view(np.uint16)
bufs = t._Buffers(exe, pool, pool, 2)
tab = reqs.step()
bufs.inputs(rng.standard_normal((2, t.H, t.D), dtype=np.float32), pool[:2 * t.ROW], pool[:2 * t.ROW])
assert exe.beginForwardPassCB(); bufs.encode(tab, 2); assert exe.flushForwardPassCB()
assert exe.tableUploads() == 0
assert exe.beginForwardPassCB() and exe.captureBegin(), exe.lastError()
bufs.encode(tab, 2)
h = exe.captureEnd()
assert h > 0, exe.lastError()
assert exe.flushForwardPassCB()
a = bufs.outputs(2)[0]
assert exe.replayUpdate(h, tab["flat"], tab["off"], tab["seq"], tab["qpos"], tab["ids"], tab["slots"]), exe.lastError()
assert exe.beginForwardPassCB() and exe.replay(h) and exe.flushForwardPassCB()
assert np.array_equal(a, bufs.outputs(2)[0])
print("ok")
""" % (os.path.dirname(os.path.dirname(os.path.abspath(__file__))), os.path.dirname(os.path.abspath(__file__)))
    proc = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, timeout=240)
    assert proc.returncode == 0 and "ok" in proc.stdout, proc.stdout + proc.stderr
