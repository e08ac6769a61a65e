"""A decode step as the batched walker encodes it (compiler/runtime/batched_walker.cpp:304-331):
the batched scatter of every request's new K row, the same for V, then the attention over the
pages.  When the two scatters write every request's newest position into the pools the
attention reads, the attention launch does the write itself.  Pools and outputs must come out
exactly as from the three launches, and when the rows are not the newest positions (or only one
scatter is pending, or causality hides the position) the calls run one after the other."""
from dataclasses import replace

import numpy as np
import pytest

from oracle import paged_oracle as po
from paged_cases import DeviceCase, assert_parity, make_case, oracle_decode

pytestmark = pytest.mark.gpu


def _newest(case):
    last = case.seq_lens.astype(np.int64) - 1
    ids = np.array([case.page_tables_flat[case.page_table_offsets[r] + last[r] // case.page_size]
                    for r in range(case.batch)], np.uint32)
    return ids, (last % case.page_size).astype(np.uint32)


def _step(exe, case, ids, slots, new_k, new_v, fuse, *, only_k=False, target=0):
    """scatter K, scatter V, attention in one open pass -> (output, K pool, V pool, launches that carried the write)"""
    dev = DeviceCase(exe, case)
    nk, nv = (exe.allocateScratchBuffer(a.nbytes) for a in (new_k, new_v))
    assert exe.uploadToBuffer(nk, new_k) and exe.uploadToBuffer(nv, new_v)
    split = "decode_grid_wgs"
    assert exe.setOption("fuse_row_ops", fuse) and exe.setOption(split, target)
    before = exe.kvWritesInDecodeLaunches()
    c = case
    try:
        assert exe.beginForwardPassCB()
        assert exe.encodeScatterKVPagedBatched(dev.k_buf, ids, slots, c.page_size, c.kv_heads, c.head_dim, c.batch, nk)
        if not only_k:
            assert exe.encodeScatterKVPagedBatched(dev.v_buf, ids, slots, c.page_size, c.kv_heads, c.head_dim, c.batch, nv)
        assert exe.encodePagedFlashAttention(dev.q_buf, dev.k_buf, dev.v_buf, dev.o_buf, c.page_tables_flat,
                                             c.page_table_offsets, c.seq_lens, c.q_positions, c.batch, c.num_heads,
                                             c.kv_heads, c.head_dim, c.page_size, c.apply_causal), exe.lastError()
        assert exe.flushForwardPassCB(), exe.lastError()
        out = np.empty(c.q.shape, np.float32)
        kp, vp = np.empty_like(c.k_pages), np.empty_like(c.v_pages)
        assert exe.downloadFromBuffer(dev.o_buf, out)
        assert exe.downloadFromBuffer(dev.k_buf, kp) and exe.downloadFromBuffer(dev.v_buf, vp)
    finally:
        exe.setOption("fuse_row_ops", 1)
        exe.setOption(split, 0)
        dev.free()
        exe.releaseScratchBuffer(nk)
        exe.releaseScratchBuffer(nv)
    return out, kp, vp, exe.kvWritesInDecodeLaunches() - before


def _expect(case, ids, slots, new_k, new_v, only_k=False):
    kp, vp = case.k_pages.copy(), case.v_pages.copy()
    assert po.scatter_kv_paged_batched_f16(kp, ids, slots, case.page_size, case.kv_heads, case.head_dim, case.batch, new_k)
    if not only_k:
        assert po.scatter_kv_paged_batched_f16(vp, ids, slots, case.page_size, case.kv_heads, case.head_dim, case.batch, new_v)
    return kp, vp, oracle_decode(replace(case, k_pages=kp, v_pages=vp))


def _rows(case, seed):
    rng = np.random.default_rng(seed)
    row = case.kv_heads * case.head_dim
    return tuple(rng.standard_normal((case.batch, row)).astype(np.float16).view(np.uint16) for _ in range(2))


@pytest.mark.parametrize("shape", [(8, 2, 64), (32, 4, 64), (32, 8, 128), (8, 8, 64)], ids=["g4d64", "g8d64", "g4d128", "mha"])
@pytest.mark.parametrize("target", [0, 2048, 1, 5],
                         ids=["balanced_auto", "balanced_many_splits", "balanced_one_workgroup", "balanced_five_workgroups"])
def test_attention_launch_carries_the_kv_write(exe, shape, target):
    h, hkv, d = shape
    lens = [1, 64, 65, 130, 700, 2000, 63, 128]     # newest position at page starts, page ends, mid-page
    case = make_case("kvstep", len(lens), h, hkv, d, 64, lens, seed=3 + d, capacity_pages=64)
    ids, slots = _newest(case)
    new_k, new_v = _rows(case, 17)
    want_k, want_v, want_o = _expect(case, ids, slots, new_k, new_v)
    print(f"[case] kv write in decode {shape} target={target}", flush=True)
    plain = _step(exe, case, ids, slots, new_k, new_v, 0, target=target)
    fused = _step(exe, case, ids, slots, new_k, new_v, 1, target=target)
    assert plain[3] == 0 and fused[3] == 1
    for got in (plain, fused):
        assert np.array_equal(got[1], want_k) and np.array_equal(got[2], want_v)
        assert_parity(got[0], want_o, d, "kv step")
    assert np.array_equal(plain[0], fused[0])      # the same kernel did the arithmetic


def test_other_rows_are_written_by_their_own_launch(exe):
    case = make_case("kvstep_other", 4, 8, 2, 64, 64, [70, 200, 64, 129], seed=9, capacity_pages=16)
    ids, slots = _newest(case)
    new_k, new_v = _rows(case, 5)
    # (a) rows of an older position of request 1
    slots_a = slots.copy()
    slots_a[1] -= 1
    # (b) causality hides the newest position of request 2
    case_b = replace(case, q_positions=np.array([69, 199, 10, 128], np.uint32))
    for c, sl, only_k in ((case, slots_a, False), (case_b, slots, False), (case, slots, True)):
        want_k, want_v, want_o = _expect(c, ids, sl, new_k, new_v, only_k)
        out, kp, vp, carried = _step(exe, c, ids, sl, new_k, new_v, 1, only_k=only_k)
        assert carried == 0
        assert np.array_equal(kp, want_k) and np.array_equal(vp, want_v)
        assert_parity(out, want_o, 64, "kv step, separate launches")


@pytest.mark.parametrize("opts", [{"decode_heads_per_wave": 8}, {"decode_heads_per_wave": 1}, {"decode_stages": 3},
                                  {"decode_mfma": 0}, {"decode_grid_wgs": 2048}],
                         ids=lambda o: ",".join(f"{k[7:]}={v}" for k, v in o.items()))
def test_kv_write_and_many_splits_in_every_kernel_variant(exe, opts):
    """The same step through the other shapes of the tile-balanced kernel (other head groupings,
    three LDS stages, vector pipe, one tile per workgroup), with one request long enough to be
    cut into more partials than one round of the merge loads."""
    lens = [1, 65, 700, 9000, 128]
    case = make_case("kvstep_variants", len(lens), 32, 8, 64, 64, lens, seed=21, capacity_pages=160)
    ids, slots = _newest(case)
    new_k, new_v = _rows(case, 23)
    want_k, want_v, want_o = _expect(case, ids, slots, new_k, new_v)
    for name, value in opts.items():
        if name != "decode_grid_wgs":
            assert exe.setOption(name, value)
    try:
        out, kp, vp, carried = _step(exe, case, ids, slots, new_k, new_v, 1, target=opts.get("decode_grid_wgs", 0))
    finally:
        for name in opts:
            exe.setOption(name, 1 if name == "decode_mfma" else 0)
    assert carried == 1
    assert np.array_equal(kp, want_k) and np.array_equal(vp, want_v)
    assert_parity(out, want_o, 64, f"kv step {opts}")


def test_a_shared_page_keeps_the_launches_apart(exe):
    """Two requests whose tables name the same physical page (the reference's allocator never
    does that, the interface does not forbid it): the row written for one request is then also
    read for the other, so the attention launch must not take the write; the three launches run
    one after the other and give what the calls in their order give."""
    case = make_case("kvstep_shared", 3, 8, 2, 64, 64, [130, 100, 70], seed=31, capacity_pages=16)
    flat = case.page_tables_flat.copy()
    off = case.page_table_offsets
    flat[off[1] + 1] = flat[off[0] + 2]       # request 1's last page is request 0's last page
    case = replace(case, page_tables_flat=flat)
    ids, slots = _newest(case)
    new_k, new_v = _rows(case, 41)
    want_k, want_v, want_o = _expect(case, ids, slots, new_k, new_v)
    out, kp, vp, carried = _step(exe, case, ids, slots, new_k, new_v, 1)
    assert carried == 0
    assert np.array_equal(kp, want_k) and np.array_equal(vp, want_v)
    assert_parity(out, want_o, 64, "kv step, shared page")
    # the same tables without the repeated page: the attention launch takes the write again
    case2 = make_case("kvstep_unshared", 3, 8, 2, 64, 64, [130, 100, 70], seed=31, capacity_pages=16)
    ids2, slots2 = _newest(case2)
    assert _step(exe, case2, ids2, slots2, new_k, new_v, 1)[3] == 1
