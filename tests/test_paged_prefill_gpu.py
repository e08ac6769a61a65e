"""Chunked prefill over paged KV (MFMA kernel) against the CPU oracle, through the C ABI.
The oracle applies the decode path's causal rule row by row (the reference has no
multi-query paged kernel; it prefills by looping its decode path per token)."""
import numpy as np
import pytest

from oracle import paged_oracle as po
from mlcompiler_amd.workloads import make_prefill
from paged_cases import MAX_ABS, MIN_COSINE

pytestmark = pytest.mark.gpu


def run_gpu(exe, w, sync=True):
    bufs = [exe.allocateScratchBuffer(w[n].nbytes) for n in ("q", "k", "v")]
    o_bytes = w["B"] * w["C"] * w["H"] * w["D"] * 4
    o_buf = exe.allocateScratchBuffer(o_bytes)
    try:
        for b, n in zip(bufs, ("q", "k", "v")):
            assert exe.uploadToBuffer(b, w[n])
        assert exe.uploadToBuffer(o_buf, np.full(o_bytes // 4, np.nan, np.float32))
        if not sync:
            assert exe.beginForwardPassCB()
        ok = exe.runPagedPrefillAttention(bufs[0], bufs[1], bufs[2], o_buf, w["flat"], w["off"],
                                          w["seq"], w["q_start"], w["B"], w["C"], w["H"], w["Hkv"],
                                          w["D"], w["P"], sync=sync)
        assert ok, exe.lastError()
        if not sync:
            assert exe.flushForwardPassCB()
        out = np.empty((w["B"], w["C"], w["H"], w["D"]), np.float32)
        assert exe.downloadFromBuffer(o_buf, out)
    finally:
        for b in bufs + [o_buf]:
            exe.releaseScratchBuffer(b)
    return out


def oracle(w, n_threads=8):
    return po.paged_attention_prefill(w["q"], w["k"], w["v"], w["flat"], w["off"], w["seq"],
                                      w["q_start"], w["B"], w["C"], w["H"], w["Hkv"], w["D"], w["P"],
                                      n_threads)


def check(exe, w, what):
    print(f"[prefill] {what} B={w['B']} C={w['C']} H={w['H']}/{w['Hkv']} D={w['D']} P={w['P']} "
          f"seq={w['seq'].tolist()}", flush=True)
    got = run_gpu(exe, w)
    want = oracle(w)
    assert np.all(np.isfinite(got)), what
    rep = po.per_head_report(got, want, w["D"])
    assert rep["min_cosine"] >= MIN_COSINE and rep["max_abs"] <= MAX_ABS, (what, rep)
    return rep, got, want


@pytest.mark.parametrize("H,Hkv", [(8, 2), (8, 8), (8, 4), (8, 1), (32, 8)])
@pytest.mark.parametrize("D", [128, 64])
def test_prefill_small(exe, H, Hkv, D):
    w = make_prefill(2, 40, H, Hkv, D, 64, [100, 0], seed=H + D)
    check(exe, w, "small")


def test_prefill_chunk_not_multiple_of_32_and_pages(exe):
    w = make_prefill(3, 70, 8, 2, 128, 32, [5, 64, 31], seed=4)
    check(exe, w, "ragged")
    w = make_prefill(2, 33, 8, 2, 64, 128, [130, 1], seed=5)
    check(exe, w, "page128")


def test_prefill_first_rows_see_only_the_prefix(exe):
    # ctx = 0: row i of the chunk sees keys 0..i only; row 0 must equal V[0] exactly-ish
    w = make_prefill(1, 64, 8, 2, 128, 64, [0], seed=6)
    rep, got, want = check(exe, w, "from scratch")
    v = w["v"].view(np.float16).reshape(-1, 64, 2, 128)
    pid = int(w["flat"][0])
    for h in range(8):
        assert np.allclose(got[0, 0, h], v[pid, 0, h // 4].astype(np.float32), atol=1e-3)


def test_prefill_matches_decode_row_by_row(exe):
    # the reference's own formulation: one decode call per chunk row (batched_executor.cpp:454-466)
    w = make_prefill(2, 32, 8, 2, 128, 64, [200, 70], seed=7)
    got = run_gpu(exe, w)
    B, C, H, Hkv, D, P = (w[k] for k in ("B", "C", "H", "Hkv", "D", "P"))
    qf = w["q"].view(np.float16).astype(np.float32)
    bufs = [exe.allocateScratchBuffer(x.nbytes) for x in (w["k"], w["v"])]
    qb = exe.allocateScratchBuffer(B * H * D * 4)
    ob = exe.allocateScratchBuffer(B * H * D * 4)
    try:
        assert exe.uploadToBuffer(bufs[0], w["k"]) and exe.uploadToBuffer(bufs[1], w["v"])
        for i in range(C):
            assert exe.uploadToBuffer(qb, np.ascontiguousarray(qf[:, i]))
            pos = w["q_start"] + i
            assert exe.runPagedFlashAttention(qb, bufs[0], bufs[1], ob, w["flat"], w["off"], w["seq"],
                                              pos, B, H, Hkv, D, P, True), exe.lastError()
            row = np.empty((B, H, D), np.float32)
            assert exe.downloadFromBuffer(ob, row)
            assert np.max(np.abs(row - got[:, i])) < 2e-3, i
    finally:
        for b in bufs + [qb, ob]:
            exe.releaseScratchBuffer(b)


def test_prefill_encode_variant_and_rejections(exe):
    w = make_prefill(1, 32, 8, 2, 128, 64, [10], seed=8)
    a = run_gpu(exe, w, sync=True)
    b = run_gpu(exe, w, sync=False)
    assert np.array_equal(a, b)
    buf = exe.allocateScratchBuffer(1 << 20)
    try:
        args = (buf, buf, buf, buf, w["flat"], w["off"], w["seq"], w["q_start"], 1, 32, 8, 2)
        assert not exe.runPagedPrefillAttention(*args, 96, 64)     # head_dim
        assert not exe.runPagedPrefillAttention(*args, 128, 48)    # page size
        assert not exe.runPagedPrefillAttention(0, buf, buf, buf, *args[4:], 128, 64)
        assert not exe.runPagedPrefillAttention(buf, buf, buf, buf, w["flat"], w["off"], w["seq"],
                                                w["q_start"], 1, 32, 8, 3, 128, 64)
        assert not exe.runPagedPrefillAttention(*args, 128, 64, sync=False)  # no open pass
    finally:
        exe.releaseScratchBuffer(buf)


def test_prefill_baseline_config5_sampled(exe):
    """Benchmark configuration 5 at full size (B=8, 256-row chunk after 3840 cached tokens,
    32q/8kv, D=128); the oracle checks a sample of rows (first, diagonal-crossing, last)."""
    w = make_prefill(8, 256, 32, 8, 128, 64, [3840] * 8, seed=55)
    got = run_gpu(exe, w)
    assert np.all(np.isfinite(got))
    rows = [0, 1, 31, 32, 63, 64, 127, 200, 255]
    for r in (0, 5):
        sub = dict(w)
        sub.update(B=1, C=1)
        for i in rows:
            sub["q"] = np.ascontiguousarray(w["q"].reshape(8, 256, 32, 128)[r, i]).ravel()
            sub["flat"] = w["flat"][w["off"][r]:w["off"][r + 1]]
            sub["off"] = np.array([0, sub["flat"].size], np.uint32)
            sub["seq"] = w["seq"][r:r + 1]
            sub["q_start"] = np.array([3840 + i], np.uint32)
            want = oracle(sub)
            rep = po.per_head_report(got[r, i], want[0, 0], 128)
            assert rep["min_cosine"] >= MIN_COSINE and rep["max_abs"] <= MAX_ABS, (r, i, rep)


def test_prefill_baseline_config5_every_row_of_one_request(exe):
    """Configuration 5 at full size, all 256 chunk rows x 32 heads of one request against the
    oracle (the sampled test above covers two requests at nine rows each)."""
    w = make_prefill(8, 256, 32, 8, 128, 64, [3840] * 8, seed=55)
    got = run_gpu(exe, w)
    r = 3
    sub = dict(w)
    sub.update(B=1)
    sub["q"] = np.ascontiguousarray(w["q"].reshape(8, 256 * 32 * 128)[r])
    sub["flat"] = w["flat"][w["off"][r]:w["off"][r + 1]]
    sub["off"] = np.array([0, sub["flat"].size], np.uint32)
    sub["seq"], sub["q_start"] = w["seq"][r:r + 1], w["q_start"][r:r + 1]
    want = oracle(sub)
    rep = po.per_head_report(got[r], want[0], 128)
    print("[prefill] config 5, request 3, 256 rows:", rep, flush=True)
    assert rep["min_cosine"] >= MIN_COSINE and rep["max_abs"] <= MAX_ABS, rep


def test_prefill_32_rows_per_wave_kernel_for_small_gqa_ratios(exe):
    """GQA ratios up to 4 run the 64-rows-per-wave kernel by default; the 32-row kernel (the only
    one for ratio 8) must stay right for them too."""
    assert exe.setOption("prefill_rows64", 0)
    try:
        for H, Hkv, D in ((8, 2, 128), (8, 8, 64)):
            w = make_prefill(2, 40, H, Hkv, D, 64, [100, 0], seed=H + D + 1)
            check(exe, w, f"rows32 H{H} Hkv{Hkv} D{D}")
    finally:
        assert exe.setOption("prefill_rows64", 1)


def test_prefill_more_than_64_pages_and_one_tile_per_page(exe):
    """32-token pages (one K/V tile per page) and a sequence of more than 64 pages: the page ids
    are held 64 at a time; also a sequence shorter than the tiles kept in flight."""
    w = make_prefill(2, 64, 8, 2, 64, 32, [2500, 3], seed=21)
    check(exe, w, "80 pages of 32 tokens")
    w = make_prefill(1, 48, 4, 1, 128, 32, [2100], seed=22)
    check(exe, w, "68 pages, head_dim 128, one KV head")


@pytest.mark.parametrize("stages", [4, 8])
def test_prefill_other_stage_counts(exe, stages):
    """Six K/V tiles staged in LDS is the default; four and eight are selectable, and with eight
    the 64-rows-per-wave kernel lets its waves meet only after every second tile."""
    assert exe.setOption("prefill_stages", stages)
    try:
        for H, Hkv, D in ((8, 2, 128), (8, 8, 64), (8, 1, 128)):
            check(exe, make_prefill(2, 40, H, Hkv, D, 64, [100, 0], seed=H + D + stages), f"stages{stages} H{H}/{Hkv} D{D}")
        check(exe, make_prefill(2, 256, 8, 2, 128, 64, [1000, 517], seed=9 + stages), f"stages{stages} chunk 256")
        check(exe, make_prefill(2, 64, 8, 2, 64, 32, [2500, 3], seed=21 + stages), f"stages{stages} 80 pages of 32 tokens")
    finally:
        assert exe.setOption("prefill_stages", 0)
