"""Bit-exact checks of the paged KV write / read kernels against the CPU oracle,
through the C ABI.  Layout patterns follow tests/test_paged_kv.cpp of the reference."""
import numpy as np
import pytest

from oracle import paged_oracle as po
from paged_cases import DeviceCase, assert_parity, baseline_config, oracle_decode

pytestmark = pytest.mark.gpu


def _pool(exe, host: np.ndarray) -> int:
    buf = exe.allocateScratchBuffer(host.nbytes)
    assert buf and exe.uploadToBuffer(buf, host)
    return buf


def _read(exe, buf, like: np.ndarray) -> np.ndarray:
    out = np.empty_like(like)
    assert exe.downloadFromBuffer(buf, out)
    return out


@pytest.mark.parametrize("B,Hkv,D,P", [(1, 4, 64, 64), (32, 4, 64, 64), (64, 4, 64, 64),
                                       (64, 8, 128, 64), (5, 2, 64, 4), (7, 3, 20, 8), (3, 1, 2, 4)])
@pytest.mark.parametrize("sync", [True, False])
def test_scatter_batched_bit_exact(exe, B, Hkv, D, P, sync):
    print(f"[scatter] B={B} Hkv={Hkv} D={D} P={P} sync={sync}", flush=True)
    rng = np.random.default_rng(B * 1000 + D)
    cap = max(2 * B, 8)
    pool = rng.integers(0, 65536, size=cap * P * Hkv * D, dtype=np.uint16)
    src = rng.integers(0, 65536, size=B * Hkv * D, dtype=np.uint16)
    page_ids = rng.permutation(cap)[:B].astype(np.uint32)   # distinct pages: no write collisions
    slots = rng.integers(0, P, size=B).astype(np.uint32)
    want = pool.copy()
    assert po.scatter_kv_paged_batched_f16(want, page_ids, slots, P, Hkv, D, B, src)
    d_pool, d_src = _pool(exe, pool), _pool(exe, src)
    try:
        if sync:
            assert exe.scatterKVPagedBatched(d_pool, page_ids, slots, P, Hkv, D, B, d_src), exe.lastError()
        else:
            assert exe.beginForwardPassCB()
            assert exe.encodeScatterKVPagedBatched(d_pool, page_ids, slots, P, Hkv, D, B, d_src), exe.lastError()
            assert exe.flushForwardPassCB()
        got = _read(exe, d_pool, pool)
    finally:
        exe.releaseScratchBuffer(d_pool)
        exe.releaseScratchBuffer(d_src)
    assert np.array_equal(got, want)
    # only B*Hkv*D halves may differ from the pool before the call
    assert int((got != pool).sum()) <= B * Hkv * D


def test_scatter_same_page_different_slots(exe):
    # several requests of a batch never share a page in production, but two K rows may
    # target one page through different slots in tests: both must land
    P, Hkv, D = 64, 4, 64
    pool = np.zeros(4 * P * Hkv * D, np.uint16)
    src = np.arange(3 * Hkv * D, dtype=np.uint16) + 1
    page_ids, slots = [2, 2, 0], [0, 63, 5]
    want = pool.copy()
    assert po.scatter_kv_paged_batched_f16(want, page_ids, slots, P, Hkv, D, 3, src)
    d_pool, d_src = _pool(exe, pool), _pool(exe, src)
    try:
        assert exe.scatterKVPagedBatched(d_pool, page_ids, slots, P, Hkv, D, 3, d_src)
        got = _read(exe, d_pool, pool)
    finally:
        exe.releaseScratchBuffer(d_pool)
        exe.releaseScratchBuffer(d_src)
    assert np.array_equal(got, want)


def test_scatter_rejects_bad_arguments(exe):
    P, Hkv, D, B = 64, 4, 64, 2
    pool = np.zeros(4 * P * Hkv * D, np.uint16)
    src = np.zeros(B * Hkv * D, np.uint16)
    d_pool, d_src = _pool(exe, pool), _pool(exe, src)
    try:
        ok = lambda **k: exe.scatterKVPagedBatched(k.get("pool", d_pool), k.get("ids", [0, 1]),
                                                   k.get("slots", [0, 0]), k.get("P", P),
                                                   k.get("Hkv", Hkv), k.get("D", D), k.get("B", B),
                                                   k.get("src", d_src))
        assert ok()
        # metal_runtime.mm:7241-7243
        assert not ok(pool=0)
        assert not ok(src=0)
        assert not ok(B=0)
        assert not ok(Hkv=0)
        assert not ok(D=0)
        assert not ok(P=0)
        assert not ok(ids=[0])
        assert not ok(slots=[0, 0, 0])
        # beyond the reference
        assert not ok(slots=[0, 64])
        assert not ok(ids=[0, 4])
        # encode variant without an open pass (metal_runtime.mm:7178)
        assert not exe.hasForwardPassCB()
        assert not exe.encodeScatterKVPagedBatched(d_pool, [0, 1], [0, 0], P, Hkv, D, B, d_src)
    finally:
        exe.releaseScratchBuffer(d_pool)
        exe.releaseScratchBuffer(d_src)


def test_decode_step_with_kv_write(exe):
    """Benchmark configuration 3 at reduced batch: every request appends one K and one V
    row through the allocator's (page, slot) -- some open a fresh page -- then attends
    over the updated cache (compiler/runtime/batched_walker.cpp:128-142, 299-331)."""
    B, H, Hkv, D, P = 16, 32, 4, 64, 64
    rng = np.random.default_rng(33)
    prev = rng.integers(255, 1500, size=B)
    prev[:4] = [64, 128, 640, 1024]  # these appends open a fresh page
    cap = int(((prev + 1 + P - 1) // P).sum()) + 8
    # token-by-token growth through the allocator, requests interleaved so that their
    # page chains are non-contiguous
    pool_alloc = po.PagePool(cap)
    states = [po.RequestKVState(P, max_pages=64) for _ in range(B)]
    for t in range(int(prev.max())):
        for r in range(B):
            if t < int(prev[r]):
                assert states[r].extend_one_token(pool_alloc) is not None
    k_pool = rng.standard_normal(cap * P * Hkv * D, dtype=np.float32).astype(np.float16).view(np.uint16)
    v_pool = rng.standard_normal(cap * P * Hkv * D, dtype=np.float32).astype(np.float16).view(np.uint16)
    new_k = rng.standard_normal(B * Hkv * D, dtype=np.float32).astype(np.float16).view(np.uint16)
    new_v = rng.standard_normal(B * Hkv * D, dtype=np.float32).astype(np.float16).view(np.uint16)
    q = rng.standard_normal((B, H, D), dtype=np.float32)

    page_ids, slots = [], []
    for st in states:
        pid, slot = st.extend_one_token(pool_alloc)
        page_ids.append(pid)
        slots.append(slot)
    assert slots[:4] == [0, 0, 0, 0] and all(s == int(p) % P for s, p in zip(slots, prev))
    flat, off, seq = [], [0], []
    for st in states:
        flat += st.page_table
        off.append(len(flat))
        seq.append(st.total_tokens())
    qpos = [s - 1 for s in seq]

    d_k, d_v = _pool(exe, k_pool), _pool(exe, v_pool)
    d_nk, d_nv, d_q = _pool(exe, new_k), _pool(exe, new_v), _pool(exe, q)
    d_o = exe.allocateScratchBuffer(q.nbytes)
    try:
        assert exe.beginForwardPassCB()
        assert exe.encodeScatterKVPagedBatched(d_k, page_ids, slots, P, Hkv, D, B, d_nk)
        assert exe.encodeScatterKVPagedBatched(d_v, page_ids, slots, P, Hkv, D, B, d_nv)
        assert exe.encodePagedFlashAttention(d_q, d_k, d_v, d_o, flat, off, seq, qpos, B, H, Hkv, D,
                                             P, True), exe.lastError()
        assert exe.flushForwardPassCB()
        got_k, got_v = _read(exe, d_k, k_pool), _read(exe, d_v, v_pool)
        got_o = _read(exe, d_o, q)
    finally:
        for b in (d_k, d_v, d_nk, d_nv, d_q, d_o):
            exe.releaseScratchBuffer(b)
    assert po.scatter_kv_paged_batched_f16(k_pool, page_ids, slots, P, Hkv, D, B, new_k)
    assert po.scatter_kv_paged_batched_f16(v_pool, page_ids, slots, P, Hkv, D, B, new_v)
    assert np.array_equal(got_k, k_pool) and np.array_equal(got_v, v_pool)  # bit-exact
    want = po.paged_attention_executor(q, k_pool, v_pool, flat, off, seq, qpos, B, H, Hkv, D, P, True, 8)
    assert_parity(got_o, want, D, "decode step")


# ---- single-request scatter / gather: tests/test_paged_kv.cpp:219-267 pattern

def _pattern(pages, P, Hkv, D, dtype):
    p, s, h, d = np.meshgrid(np.arange(pages), np.arange(P), np.arange(Hkv), np.arange(D), indexing="ij")
    return (p * 1e5 + s * 1e3 + h * 10 + d).astype(dtype)


@pytest.mark.parametrize("dtype", [np.float32, np.float16])
def test_gather_out_of_order_page_table(exe, dtype):
    P, Hkv, D, pages = 4, 2, 8, 12
    # fp16 cannot hold the pattern exactly; use a reduced pattern that it can
    pool = _pattern(pages, P, Hkv, D, np.float32)
    if dtype == np.float16:
        pool = (pool % 2048).astype(np.float16)
    table = [7, 2, 11]   # tests/test_paged_kv.cpp:292
    ntok = 10            # last page partially read
    nbytes = np.dtype(dtype).itemsize
    want = np.zeros((Hkv, ntok, D), dtype)
    assert po.gather_kv_pages(pool, table, P, Hkv, D, ntok, want, nbytes)
    for h in range(Hkv):
        for t in range(ntok):
            assert np.array_equal(want[h, t], pool[table[t // P], t % P, h])  # closed form
    d_pool = _pool(exe, pool)
    d_dst = exe.allocateScratchBuffer(want.nbytes)
    try:
        assert exe.gatherKVPages(d_pool, table, P, Hkv, D, ntok, d_dst, nbytes), exe.lastError()
        got = _read(exe, d_dst, want)
    finally:
        exe.releaseScratchBuffer(d_pool)
        exe.releaseScratchBuffer(d_dst)
    assert np.array_equal(got.view(np.uint8), want.view(np.uint8))


@pytest.mark.parametrize("dtype,D", [(np.float32, 8), (np.float16, 8), (np.float16, 64), (np.float32, 6)])
def test_scatter_then_gather_roundtrip(exe, dtype, D):
    # scatter(start_slot=3, 11 tokens, pages {5, 1, 8}) then gather = identity
    # (tests/test_paged_kv.cpp:404-474)
    P, Hkv, pages = 4, 2, 10
    tokens, start = 11, 3
    table = [5, 1, 8, 3]
    nbytes = np.dtype(dtype).itemsize
    rng = np.random.default_rng(D)
    src = rng.standard_normal((Hkv, tokens, D)).astype(dtype)
    pool0 = rng.standard_normal(pages * P * Hkv * D).astype(dtype)
    want_pool = pool0.copy()
    assert po.scatter_kv_paged(want_pool, table, P, Hkv, D, tokens, start, src, nbytes)
    d_pool, d_src = _pool(exe, pool0), _pool(exe, src)
    d_dst = exe.allocateScratchBuffer((start + tokens) * Hkv * D * nbytes)
    try:
        assert exe.scatterKVPaged(d_pool, table, P, Hkv, D, tokens, start, d_src, nbytes), exe.lastError()
        got_pool = _read(exe, d_pool, pool0)
        assert np.array_equal(got_pool.view(np.uint8), want_pool.view(np.uint8))
        full = np.zeros((Hkv, start + tokens, D), dtype)
        assert exe.gatherKVPages(d_pool, table, P, Hkv, D, start + tokens, d_dst, nbytes)
        full = _read(exe, d_dst, full)
    finally:
        for b in (d_pool, d_src, d_dst):
            exe.releaseScratchBuffer(b)
    assert np.array_equal(full[:, start:, :].view(np.uint8), src.view(np.uint8))


def test_scatter_gather_reject_bad_arguments(exe):
    # tests/test_paged_kv.cpp:541-595
    P, Hkv, D = 4, 2, 8
    pool = np.zeros(8 * P * Hkv * D, np.float32)
    d_pool = _pool(exe, pool)
    d_buf = exe.allocateScratchBuffer(pool.nbytes)
    try:
        assert not exe.gatherKVPages(0, [0], P, Hkv, D, 4, d_buf, 4)
        assert not exe.gatherKVPages(d_pool, [0], P, Hkv, D, 4, 0, 4)
        assert not exe.gatherKVPages(d_pool, [0], P, Hkv, D, 4, d_buf, 3)
        assert not exe.gatherKVPages(d_pool, [0], P, Hkv, D, 5, d_buf, 4)   # table too short
        assert not exe.gatherKVPages(d_pool, [0], P, Hkv, D, 0, d_buf, 4)
        assert not exe.gatherKVPages(d_pool, [0], 0, Hkv, D, 4, d_buf, 4)
        assert not exe.scatterKVPaged(d_pool, [0], P, Hkv, D, 4, 4, d_buf, 4)  # start_slot >= P
        assert not exe.scatterKVPaged(d_pool, [0], P, Hkv, D, 5, 0, d_buf, 4)  # table too short
        assert not exe.scatterKVPaged(d_pool, [0], P, Hkv, D, 4, 0, d_buf, 8)
        assert not exe.scatterKVPaged(d_pool, [0], P, Hkv, D, 0, 0, d_buf, 4)
        assert exe.scatterKVPaged(d_pool, [0], P, Hkv, D, 4, 0, d_buf, 4)
    finally:
        exe.releaseScratchBuffer(d_pool)
        exe.releaseScratchBuffer(d_buf)


def test_cached_buffers_and_offsets(exe):
    # name-keyed grow-only cache (metal_runtime.mm:8218-8246) and offset copies (:8273-8297)
    a = exe.getOrAllocCachedBuffer("t_cache_a", 1024)
    assert a and exe.getOrAllocCachedBuffer("t_cache_a", 512) == a
    b = exe.getOrAllocCachedBuffer("t_cache_a", 4096)
    assert b
    data = np.arange(256, dtype=np.uint32)
    assert exe.uploadToBuffer(b, data, dst_offset=1024)
    back = np.zeros(64, np.uint32)
    assert exe.downloadFromBuffer(b, back, src_offset=1024 + 64 * 4)
    assert np.array_equal(back, data[64:128])
    assert not exe.uploadToBuffer(b, data, dst_offset=4096)   # beyond the buffer


# ---- the KV write of a step encoded call by call goes out as one launch: same bytes --------------

@pytest.mark.parametrize("B,Hkv,D,P", [(32, 4, 64, 64), (5, 2, 64, 4), (7, 3, 20, 8)])
@pytest.mark.parametrize("fuse", [1, 0])
def test_k_and_v_scatter_pair_in_one_pass(exe, B, Hkv, D, P, fuse):
    """encodeScatterKVPagedBatched for K, then for V with the same page ids (the two calls of
    batched_walker.cpp:304-307): one launch with fusion on; a third scatter with other ids, and a
    scatter into the pool the first one wrote, must not join."""
    print(f"[scatter pair] B={B} Hkv={Hkv} D={D} P={P} fuse={fuse}", flush=True)
    rng = np.random.default_rng(B + D)
    cap = 2 * B + 4
    n = cap * P * Hkv * D
    k_pool, v_pool = (rng.integers(0, 65536, n, dtype=np.uint16) for _ in range(2))
    nk, nv, nk2 = (rng.integers(0, 65536, B * Hkv * D, dtype=np.uint16) for _ in range(3))
    ids = rng.permutation(cap)[:B].astype(np.uint32)
    slots = rng.integers(0, P, B).astype(np.uint32)
    ids2 = ((ids + 1) % cap).astype(np.uint32)
    want_k, want_v = k_pool.copy(), v_pool.copy()
    assert po.scatter_kv_paged_batched_f16(want_k, ids, slots, P, Hkv, D, B, nk)
    assert po.scatter_kv_paged_batched_f16(want_v, ids, slots, P, Hkv, D, B, nv)
    assert po.scatter_kv_paged_batched_f16(want_k, ids2, slots, P, Hkv, D, B, nk2)   # third call
    assert po.scatter_kv_paged_batched_f16(want_k, ids2, slots, P, Hkv, D, B, nv)    # fourth: same pool again
    bufs = [_pool(exe, a) for a in (k_pool, v_pool, nk, nv, nk2)]
    d_k, d_v, d_nk, d_nv, d_nk2 = bufs
    assert exe.setOption("fuse_row_ops", fuse)
    before = exe.fusedKvWriteLaunches()
    try:
        assert exe.beginForwardPassCB()
        assert exe.encodeScatterKVPagedBatched(d_k, ids, slots, P, Hkv, D, B, d_nk)
        assert exe.encodeScatterKVPagedBatched(d_v, ids, slots, P, Hkv, D, B, d_nv)     # joins
        assert exe.encodeScatterKVPagedBatched(d_k, ids2, slots, P, Hkv, D, B, d_nk2)   # other ids: on its own
        assert exe.encodeScatterKVPagedBatched(d_k, ids2, slots, P, Hkv, D, B, d_nv)    # same pool: on its own, later
        assert exe.flushForwardPassCB(), exe.lastError()
        got_k, got_v = _read(exe, d_k, k_pool), _read(exe, d_v, v_pool)
    finally:
        exe.setOption("fuse_row_ops", 1)
        for b in bufs:
            exe.releaseScratchBuffer(b)
    assert np.array_equal(got_k, want_k) and np.array_equal(got_v, want_v)
    assert exe.fusedKvWriteLaunches() - before == (1 if fuse else 0)


@pytest.mark.parametrize("fuse", [1, 0])
@pytest.mark.parametrize("only_k", [False, True])
def test_rope_cast_then_scatters_in_one_pass(exe, fuse, only_k):
    """encodeQkvSplitRopeCast, then the batched scatters of its fp16 K and V rows
    (batched_walker.cpp:287-307): one launch with fusion on, every buffer of the three calls
    written, bit-identical to the calls on their own."""
    B, H, Hkv, D, P = 9, 8, 2, 64, 16
    q_rows, kv_rows = H * D, Hkv * D
    qkv_rows = q_rows + 2 * kv_rows
    rng = np.random.default_rng(31 + only_k)
    qkv = rng.standard_normal((B, qkv_rows)).astype(np.float32)
    pos = rng.integers(0, 500, B)
    cos = np.zeros((B, D // 2), np.float32)
    sin = np.zeros((B, D // 2), np.float32)
    for r in range(B):
        cos[r], sin[r] = po.rotary_coefficients(int(pos[r]), D)
    cap = 2 * B
    k_pool, v_pool = (rng.integers(0, 65536, cap * P * kv_rows, dtype=np.uint16) for _ in range(2))
    ids = rng.permutation(cap)[:B].astype(np.uint32)
    slots = rng.integers(0, P, B).astype(np.uint32)
    wq, wk, wv, wk16, wv16 = po.qkv_split_rope_cast(qkv, cos, sin, B, H, Hkv, D, qkv_rows, q_rows, kv_rows, kv_rows, D)
    want_k, want_v = k_pool.copy(), v_pool.copy()
    assert po.scatter_kv_paged_batched_f16(want_k, ids, slots, P, Hkv, D, B, wk16)
    if not only_k:
        assert po.scatter_kv_paged_batched_f16(want_v, ids, slots, P, Hkv, D, B, wv16)
    d_qkv, d_cos, d_sin, d_kp, d_vp = (_pool(exe, a) for a in (qkv, cos, sin, k_pool, v_pool))
    d_q = exe.allocateScratchBuffer(B * q_rows * 4)
    d_k, d_v = (exe.allocateScratchBuffer(B * kv_rows * 4) for _ in range(2))
    d_k16, d_v16 = (exe.allocateScratchBuffer(B * kv_rows * 2) for _ in range(2))
    bufs = [d_qkv, d_cos, d_sin, d_kp, d_vp, d_q, d_k, d_v, d_k16, d_v16]
    assert exe.setOption("fuse_row_ops", fuse)
    before = exe.fusedKvWriteLaunches()
    try:
        assert exe.beginForwardPassCB()
        assert exe.encodeQkvSplitRopeCast(d_qkv, d_q, d_k, d_v, d_k16, d_v16, d_cos, d_sin, B, H, Hkv, D, qkv_rows,
                                          q_rows, kv_rows, kv_rows, D), exe.lastError()
        assert exe.encodeScatterKVPagedBatched(d_kp, ids, slots, P, Hkv, D, B, d_k16)
        if not only_k:
            assert exe.encodeScatterKVPagedBatched(d_vp, ids, slots, P, Hkv, D, B, d_v16)
        assert exe.flushForwardPassCB(), exe.lastError()
        got = {n: _read(exe, b, like) for n, b, like in
               (("q", d_q, wq), ("k", d_k, wk), ("v", d_v, wv), ("k16", d_k16, wk16), ("v16", d_v16, wv16),
                ("kp", d_kp, k_pool), ("vp", d_vp, v_pool))}
    finally:
        exe.setOption("fuse_row_ops", 1)
        for b in bufs:
            exe.releaseScratchBuffer(b)
    for name, want in (("q", wq), ("k", wk), ("v", wv), ("k16", wk16), ("v16", wv16), ("kp", want_k), ("vp", want_v)):
        assert np.array_equal(got[name].view(np.uint8), np.ascontiguousarray(want).view(np.uint8)), name
    assert exe.fusedKvWriteLaunches() - before == (1 if fuse else 0)
