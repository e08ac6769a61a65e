"""The decode entry point that allocates nothing, against the ordinary decode entry point.

Both run the same tile-balanced kernel; the one under test takes the flat page table as a device
pointer, the per-request arrays inside the kernel arguments and its scratch memory from the
library's static device array.  Called twice in a row, the second time with a smaller batch, so
that whatever the first call left in the shared scratch array (the partials) must not leak into
the second.  Also on a stream of the caller's own, between launches on the library's stream (the
library orders the launches that share its scratch array), and with the device's free memory
read before and after the calls."""
import ctypes as C

import numpy as np
import pytest

from mlcompiler_amd import HipExecutor
from mlcompiler_amd._lib import load
from paged_cases import baseline_config, make_case

pytestmark = pytest.mark.gpu


def _u32p(a):
    return a.ctypes.data_as(C.POINTER(C.c_uint32))


def _run_both(exe, lib, c):
    """Returns (output of mlc_hip_paged_attn_decode, output of ..._noalloc) for case c."""
    nbytes = c.q.nbytes
    q = exe.allocateScratchBuffer(nbytes)
    o_ref = exe.allocateScratchBuffer(nbytes)
    o_new = exe.allocateScratchBuffer(nbytes)
    k = exe.allocateScratchBuffer(c.k_pages.nbytes)
    v = exe.allocateScratchBuffer(c.v_pages.nbytes)
    flat = np.ascontiguousarray(c.page_tables_flat, dtype=np.uint32)
    d_flat = exe.allocateScratchBuffer(max(flat.nbytes, 4))
    try:
        exe.uploadToBuffer(q, c.q)
        exe.uploadToBuffer(k, c.k_pages)
        exe.uploadToBuffer(v, c.v_pages)
        if flat.nbytes:
            exe.uploadToBuffer(d_flat, flat)
        exe.zeroBuffer(o_ref, nbytes)
        exe.zeroBuffer(o_new, nbytes)
        assert exe.runPagedFlashAttention(q, k, v, o_ref, c.page_tables_flat, c.page_table_offsets, c.seq_lens,
                                          c.q_positions, c.batch, c.num_heads, c.kv_heads, c.head_dim,
                                          c.page_size, c.apply_causal), exe.lastError()
        off = np.ascontiguousarray(c.page_table_offsets, dtype=np.uint32)
        seq = np.ascontiguousarray(c.seq_lens, dtype=np.uint32)
        qpos = np.ascontiguousarray(c.q_positions, dtype=np.uint32)
        ok = lib.mlc_hip_paged_attn_decode_noalloc(q, k, v, o_new, d_flat, flat.size, _u32p(off), _u32p(seq),
                                                   _u32p(qpos), c.batch, c.num_heads, c.kv_heads, c.head_dim,
                                                   c.page_size, int(c.apply_causal), None)
        assert ok, exe.lastError()
        a = np.empty_like(c.q)
        b = np.empty_like(c.q)
        exe.downloadFromBuffer(o_ref, a)   # synchronises the library's stream, which both launches used
        exe.downloadFromBuffer(o_new, b)
        return a, b
    finally:
        for buf in (q, o_ref, o_new, k, v, d_flat):
            exe.releaseScratchBuffer(buf)


def test_noalloc_matches_decode_twice_second_smaller():
    exe = HipExecutor.Instance()
    exe.requireAvailable()
    lib = load()
    big = baseline_config(2)                     # batch 32, contexts up to 2048: split requests, merges
    small = make_case("small", 5, 32, 4, 64, 64, [1, 700, 130, 64, 65], capacity_pages=96, seed=77)
    for c in (big, small):
        assert exe.lastDecodeLaunches() >= 0
        ref, new = _run_both(exe, lib, c)
        assert np.isfinite(new).all()
        # same kernel, same split of the work, partials merged in slot order: bit-identical
        assert np.array_equal(ref, new), float(np.abs(ref - new).max())


def test_noalloc_refuses_what_it_cannot_serve():
    exe = HipExecutor.Instance()
    exe.requireAvailable()
    lib = load()
    c = make_case("tiny", 2, 8, 2, 64, 64, [5, 100], capacity_pages=8, seed=3)
    off = np.ascontiguousarray(c.page_table_offsets, dtype=np.uint32)
    seq = np.ascontiguousarray(c.seq_lens, dtype=np.uint32)
    qpos = np.ascontiguousarray(c.q_positions, dtype=np.uint32)
    buf = exe.allocateScratchBuffer(1 << 20)
    try:
        # head_dim 96 is the generic kernel's, which plans on the host
        assert not lib.mlc_hip_paged_attn_decode_noalloc(buf, buf, buf, buf, buf, len(c.page_tables_flat), _u32p(off),
                                                         _u32p(seq), _u32p(qpos), 2, 8, 2, 96, 64, 0, None)
        assert b"head_dim" in lib.mlc_hip_last_error()
        # more requests than the kernel arguments hold
        n = 300
        off_b = np.arange(n + 1, dtype=np.uint32)
        ones = np.ones(n, dtype=np.uint32)
        assert not lib.mlc_hip_paged_attn_decode_noalloc(buf, buf, buf, buf, buf, n, _u32p(off_b), _u32p(ones),
                                                         _u32p(ones), n, 8, 2, 64, 64, 0, None)
        assert b"256" in lib.mlc_hip_last_error()
    finally:
        exe.releaseScratchBuffer(buf)


def _hip():
    hip = C.CDLL("libamdhip64.so")
    hip.hipStreamCreate.argtypes = [C.POINTER(C.c_void_p)]
    hip.hipStreamSynchronize.argtypes = [C.c_void_p]
    hip.hipStreamDestroy.argtypes = [C.c_void_p]
    hip.hipMemGetInfo.argtypes = [C.POINTER(C.c_size_t), C.POINTER(C.c_size_t)]
    return hip


def test_noalloc_on_a_second_stream_between_launches_on_the_library_stream():
    """Launches on the library's stream and on a stream of the caller's alternate, all of them using
    the one scratch array, none of them waited for in between: every output must be what the
    ordinary entry point gives, and the no-allocation calls must leave the device's free memory
    as it was."""
    exe = HipExecutor.Instance()
    exe.requireAvailable()
    lib = load()
    hip = _hip()
    stream = C.c_void_p()
    assert hip.hipStreamCreate(C.byref(stream)) == 0
    c = baseline_config(2)
    rounds = 6
    nbytes = c.q.nbytes
    q, k, v = (exe.allocateScratchBuffer(n) for n in (nbytes, c.k_pages.nbytes, c.v_pages.nbytes))
    outs_lib = [exe.allocateScratchBuffer(nbytes) for _ in range(rounds)]
    outs_own = [exe.allocateScratchBuffer(nbytes) for _ in range(rounds)]
    flat = np.ascontiguousarray(c.page_tables_flat, dtype=np.uint32)
    d_flat = exe.allocateScratchBuffer(flat.nbytes)
    off, seq, qpos = (np.ascontiguousarray(a, dtype=np.uint32) for a in (c.page_table_offsets, c.seq_lens, c.q_positions))
    try:
        exe.uploadToBuffer(q, c.q)
        exe.uploadToBuffer(k, c.k_pages)
        exe.uploadToBuffer(v, c.v_pages)
        exe.uploadToBuffer(d_flat, flat)
        want = np.empty_like(c.q)
        assert exe.runPagedFlashAttention(q, k, v, outs_lib[0], c.page_tables_flat, c.page_table_offsets, c.seq_lens,
                                          c.q_positions, c.batch, c.num_heads, c.kv_heads, c.head_dim, c.page_size,
                                          c.apply_causal), exe.lastError()
        exe.downloadFromBuffer(outs_lib[0], want)
        for o in outs_lib + outs_own:
            exe.zeroBuffer(o, nbytes)
        assert exe.flushForwardPassCB()
        free0, total = C.c_size_t(), C.c_size_t()
        assert hip.hipMemGetInfo(C.byref(free0), C.byref(total)) == 0
        assert exe.beginForwardPassCB()
        for i in range(rounds):
            assert exe.encodePagedFlashAttention(q, k, v, outs_lib[i], c.page_tables_flat, c.page_table_offsets, c.seq_lens,
                                                 c.q_positions, c.batch, c.num_heads, c.kv_heads, c.head_dim, c.page_size,
                                                 c.apply_causal), exe.lastError()
            assert lib.mlc_hip_paged_attn_decode_noalloc(q, k, v, outs_own[i], d_flat, flat.size, _u32p(off), _u32p(seq),
                                                         _u32p(qpos), c.batch, c.num_heads, c.kv_heads, c.head_dim,
                                                         c.page_size, int(c.apply_causal), stream), exe.lastError()
        assert hip.hipStreamSynchronize(stream) == 0
        assert exe.flushForwardPassCB(), exe.lastError()
        free1 = C.c_size_t()
        assert hip.hipMemGetInfo(C.byref(free1), C.byref(total)) == 0
        assert free1.value == free0.value, (free0.value, free1.value)
        got = np.empty_like(c.q)
        for o in outs_lib + outs_own:
            exe.downloadFromBuffer(o, got)
            assert np.array_equal(got, want), float(np.abs(got - want).max())
    finally:
        for buf in [q, k, v, d_flat] + outs_lib + outs_own:
            exe.releaseScratchBuffer(buf)
        hip.hipStreamDestroy(stream)
