"""Pins the CPU oracle (oracle/paged_oracle.c): against the reference's own code where it can
be compiled here (oracle/_ref), against the known answers and allocator sequences the
reference's tests hold, and against what the mathematics fixes.  No GPU needed."""
import os
import subprocess

import numpy as np
import pytest

from oracle import paged_oracle as po

HAVE_REF = po.ref_lib() is not None
needs_ref = pytest.mark.skipif(not HAVE_REF, reason="oracle/_ref not built (no reference checkout)")


# ---------------------------------------------------------------- fp16 conversions

def test_fp16_to_float_all_halves_match_ieee():
    h = np.arange(65536, dtype=np.uint16)
    got = po.fp16_to_float(h)
    want = h.view(np.float16).astype(np.float32)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))  # incl. subnormals, inf, nan payloads


def test_fp16_subnormals_known_values():
    # tests/test_runtime.cpp:63-70 checks subnormal decoding
    assert po.fp16_to_float([0x0001])[0] == np.float32(2.0 ** -24)
    assert po.fp16_to_float([0x03FF])[0] == np.float32(1023 * 2.0 ** -24)
    assert po.fp16_to_float([0x8001])[0] == np.float32(-(2.0 ** -24))
    assert po.fp16_to_float([0x3C00])[0] == 1.0


def test_float_to_fp16_rne_matches_numpy():
    rng = np.random.default_rng(0)
    x = np.concatenate([rng.standard_normal(1 << 18).astype(np.float32),
                        (rng.standard_normal(1 << 16) * 1e-6).astype(np.float32),
                        (rng.standard_normal(1 << 16) * 3e4).astype(np.float32),
                        np.array([0.0, -0.0, 65504.0, 65519.9, 65520.0, 1e9, -1e9, np.inf, -np.inf,
                                  2.0 ** -24, 2.0 ** -25, 2.0 ** -25 * 1.0001, 2.0 ** -26], np.float32)])
    with np.errstate(over="ignore"):
        want = x.astype(np.float16).view(np.uint16)
    assert np.array_equal(po.float_to_fp16_rne(x), want)


def test_float_to_fp16_ref_is_half_up_not_rne():
    # float_convert.hpp:57-76: adds 0x1000 and truncates -> ties go away from zero
    tie = np.float32(1.0 + 2.0 ** -11)        # exactly between 1.0 and 1.0009765625
    assert po.float_to_fp16_ref([tie])[0] == 0x3C01
    assert po.float_to_fp16_rne([tie])[0] == 0x3C00
    assert po.float_to_fp16_ref([np.float32(np.nan)])[0] & 0x7FFF == 0x7C00  # NaN -> Inf
    assert po.float_to_fp16_ref([np.float32(2.0 ** -26)])[0] == 0            # flush
    # every half survives fp16 -> fp32 -> fp16 (what makes passing cached rows back lossless)
    h = np.arange(65536, dtype=np.uint16)
    finite = (h & 0x7C00) != 0x7C00
    back = po.float_to_fp16_ref(po.fp16_to_float(h[finite]))
    assert np.array_equal(back, h[finite])


@needs_ref
def test_fp16_conversions_match_reference_build():
    h = np.arange(65536, dtype=np.uint16)
    assert np.array_equal(po.fp16_to_float(h).view(np.uint32), po.ref_fp16_to_float(h).view(np.uint32))
    rng = np.random.default_rng(1)
    x = np.concatenate([rng.standard_normal(1 << 19).astype(np.float32),
                        (rng.standard_normal(1 << 17) * 1e-5).astype(np.float32),
                        (rng.standard_normal(1 << 17) * 1e5).astype(np.float32),
                        po.fp16_to_float(h[(h & 0x7C00) != 0x7C00])])
    assert np.array_equal(po.float_to_fp16_ref(x), po.ref_float_to_fp16(x))


# ---------------------------------------------------------------- attention known answers

def _single(q, k_rows, v_rows, H, Hkv, D, P=4, causal=True, q_pos=None, fn=po.paged_attention_executor):
    """One request whose K/V rows ([S][Hkv][D] float) sit in ascending pages."""
    S = k_rows.shape[0]
    pages = max((S + P - 1) // P, 1)
    k = np.zeros((pages * P, Hkv, D), np.float16)
    v = np.zeros((pages * P, Hkv, D), np.float16)
    k[:S] = k_rows
    v[:S] = v_rows
    qp = [S - 1 if q_pos is None else q_pos]
    return fn(np.asarray(q, np.float32), k.view(np.uint16), v.view(np.uint16), np.arange(pages), [0, pages],
              [S], qp, 1, H, Hkv, D, P, causal)[0]


@pytest.mark.parametrize("fn", [po.paged_attention_executor, po.paged_attention_flashref])
def test_tiny_verify_identity_keys(fn):
    # compiler/main.cpp:4026-4031, 4264: Q=[1,0,0,0], K=V=I4 -> [0.354661, 0.215113 x3]
    eye = np.eye(4, dtype=np.float32).reshape(4, 1, 4)
    out = _single([[1, 0, 0, 0]], eye, eye, 1, 1, 4, fn=fn)
    e = np.exp(0.5)
    assert np.allclose(out[0], np.array([e, 1, 1, 1]) / (e + 3), atol=1e-6)
    assert np.allclose(out[0], [0.354661, 0.215113, 0.215113, 0.215113], atol=1e-6)


@pytest.mark.parametrize("fn", [po.paged_attention_executor, po.paged_attention_flashref])
def test_single_cached_row_returns_v(fn):
    # tests/test_runtime.cpp:1692-1705: q=[1,0], k=[.25,0], v=[.5,1] -> [.5, 1]
    out = _single([[1, 0]], np.array([[[0.25, 0]]], np.float32), np.array([[[0.5, 1.0]]], np.float32),
                  1, 1, 2, fn=fn)
    assert np.allclose(out[0], [0.5, 1.0], atol=1e-6)


@pytest.mark.parametrize("fn", [po.paged_attention_executor, po.paged_attention_flashref])
def test_masked_second_token_two_heads_one_kv_head(fn):
    # tests/test_runtime.cpp:3206-3263: 2 heads / 1 kv head, the second cached token masked
    # (mask [0, -1e9]) -> every head returns the first V row (10.0).  Here the mask is the
    # causal rule with q_position = 0.
    k = np.array([[[1.0, 0.0]], [[0.0, 1.0]]], np.float32)
    v = np.array([[[10.0, 10.0]], [[-5.0, 7.0]]], np.float32)
    out = _single([[1, 2], [3, -1]], k, v, 2, 1, 2, q_pos=0, fn=fn)
    assert np.allclose(out, 10.0, atol=1e-6)


@pytest.mark.parametrize("fn", [po.paged_attention_executor, po.paged_attention_flashref])
def test_closed_forms(fn):
    rng = np.random.default_rng(3)
    H, Hkv, D, S = 4, 2, 8, 13
    q = rng.standard_normal((H, D)).astype(np.float32)
    k = rng.standard_normal((S, Hkv, D)).astype(np.float16).astype(np.float32)
    v = rng.standard_normal((S, Hkv, D)).astype(np.float16).astype(np.float32)
    # all keys equal -> uniform weights -> mean of V
    keq = np.broadcast_to(k[:1], k.shape)
    out = _single(q, keq, v, H, Hkv, D, fn=fn)
    for h in range(H):
        assert np.allclose(out[h], v[:, h // 2].mean(0), atol=1e-5)
    # constant V -> that constant
    vc = np.broadcast_to(v[:1], v.shape)
    out = _single(q, k, vc, H, Hkv, D, fn=fn)
    for h in range(H):
        assert np.allclose(out[h], v[0, h // 2], atol=1e-5)
    # appending masked tokens changes nothing
    a = _single(q, k[:6], v[:6], H, Hkv, D, fn=fn)
    b = _single(q, k, v, H, Hkv, D, q_pos=5, fn=fn)
    assert np.allclose(a, b, atol=1e-7)
    # non causal sees everything regardless of q_position
    c = _single(q, k, v, H, Hkv, D, causal=False, q_pos=0, fn=fn)
    d = _single(q, k, v, H, Hkv, D, fn=fn)
    assert np.array_equal(c, d)


def _brute_f64(q, k_pages, v_pages, flat, off, seq, qpos, B, H, Hkv, D, P, causal):
    K = k_pages.view(np.float16).astype(np.float64).reshape(-1, P, Hkv, D)
    V = v_pages.view(np.float16).astype(np.float64).reshape(-1, P, Hkv, D)
    out = np.zeros((B, H, D))
    for r in range(B):
        lim = min(int(seq[r]), int(qpos[r]) + 1) if causal else int(seq[r])
        if lim == 0:
            continue
        pt = flat[off[r]:off[r + 1]]
        kk = K[pt].reshape(-1, Hkv, D)[:lim]
        vv = V[pt].reshape(-1, Hkv, D)[:lim]
        for h in range(H):
            s = kk[:, h * Hkv // H] @ q[r, h].astype(np.float64) / np.sqrt(D)
            w = np.exp(s - s.max())
            out[r, h] = (w / w.sum()) @ vv[:, h * Hkv // H]
    return out


@pytest.mark.parametrize("causal", [True, False])
def test_against_float64_brute_force(causal):
    from paged_cases import make_case
    c = make_case("bf", 5, 8, 2, 16, 8, [0, 1, 8, 23, 40], causal=causal,
                  q_positions=[0, 0, 3, 22, 17], seed=12)
    want = _brute_f64(c.q, c.k_pages, c.v_pages, c.page_tables_flat, c.page_table_offsets, c.seq_lens,
                      c.q_positions, 5, 8, 2, 16, 8, causal)
    for fn in (po.paged_attention_executor, po.paged_attention_flashref):
        got = fn(c.q, c.k_pages, c.v_pages, c.page_tables_flat, c.page_table_offsets, c.seq_lens,
                 c.q_positions, 5, 8, 2, 16, 8, causal)
        assert np.max(np.abs(got - want)) < 2e-6
        assert np.all(got[0] == 0)  # empty request -> zeros (metal_runtime.mm:2254-2257)


def test_page_permutation_leaves_output_bit_identical():
    from paged_cases import make_case
    a = make_case("pa", 2, 8, 2, 16, 8, [30, 9], capacity_pages=8, permute=False, seed=2)
    perm = np.random.default_rng(5).permutation(8).astype(np.uint32)
    kb = a.k_pages.reshape(8, -1)
    vb = a.v_pages.reshape(8, -1)
    k2 = np.empty_like(kb)
    v2 = np.empty_like(vb)
    k2[perm] = kb
    v2[perm] = vb
    args = (2, 8, 2, 16, 8, True)
    o1 = po.paged_attention_executor(a.q, a.k_pages, a.v_pages, a.page_tables_flat, a.page_table_offsets,
                                     a.seq_lens, a.q_positions, *args)
    o2 = po.paged_attention_executor(a.q, k2.ravel(), v2.ravel(), perm[a.page_tables_flat],
                                     a.page_table_offsets, a.seq_lens, a.q_positions, *args)
    assert np.array_equal(o1, o2)


def test_threads_do_not_change_results():
    from paged_cases import make_case
    c = make_case("thr", 4, 8, 2, 64, 64, [100, 64, 1, 130], seed=8)
    args = (c.q, c.k_pages, c.v_pages, c.page_tables_flat, c.page_table_offsets, c.seq_lens,
            c.q_positions, 4, 8, 2, 64, 64, True)
    assert np.array_equal(po.paged_attention_executor(*args, 1), po.paged_attention_executor(*args, 4))


def test_argument_errors_like_the_reference():
    from paged_cases import make_case
    c = make_case("err", 2, 8, 2, 16, 8, [10, 12], seed=1)
    ok = lambda **k: po.paged_attention_executor(
        c.q, c.k_pages, c.v_pages, k.get("flat", c.page_tables_flat), c.page_table_offsets, c.seq_lens,
        c.q_positions, k.get("B", 2), k.get("H", 8), k.get("Hkv", 2), k.get("D", 16), k.get("P", 8), True)
    assert ok() is not None
    # metal_runtime.mm:7742-7750
    assert ok(B=0) is None and ok(H=0) is None and ok(D=0) is None and ok(P=0) is None
    assert ok(Hkv=0) is None and ok(Hkv=3) is None and ok(D=512) is None
    assert ok(flat=c.page_tables_flat[:2]) is None


@needs_ref
@pytest.mark.parametrize("shape", [(32, 4, 64, 300), (8, 8, 32, 65), (32, 8, 128, 129), (4, 1, 16, 1)])
def test_executor_order_is_bit_exact_with_reference_run_attention_cpu(shape):
    """The real RunAttentionCPU (attention_cpu.cpp:272-478), compiled from the reference's own
    sources, on a gathered-contiguous copy of the same paged cache."""
    H, Hkv, D, S = shape
    P = 64
    rng = np.random.default_rng(S)
    pages = (S + P - 1) // P + 2
    K = rng.standard_normal(pages * P * Hkv * D).astype(np.float16).view(np.uint16)
    V = rng.standard_normal(pages * P * Hkv * D).astype(np.float16).view(np.uint16)
    pt = rng.permutation(pages)[:(S + P - 1) // P].astype(np.uint32)
    q = rng.standard_normal(H * D).astype(np.float32)
    mine = po.paged_attention_executor(q, K, V, pt, [0, pt.size], [S], [S - 1], 1, H, Hkv, D, P, True)[0]
    kc = np.zeros((Hkv, S, D), np.uint16)
    vc = np.zeros((Hkv, S, D), np.uint16)
    assert po.gather_kv_pages(K, pt, P, Hkv, D, S, kc, 2) and po.gather_kv_pages(V, pt, P, Hkv, D, S, vc, 2)
    ref = po.ref_run_attention_cpu(q, kc, vc, H, Hkv, D, S, S - 1, po.fp16_to_float(kc[:, S - 1, :]),
                                   po.fp16_to_float(vc[:, S - 1, :]))
    assert ref is not None
    assert np.array_equal(mine.view(np.uint32), ref.view(np.uint32))
    # the test-file ordering (tests/test_paged_flash.cpp:17-91) agrees to float rounding
    flash = po.paged_attention_flashref(q, K, V, pt, [0, pt.size], [S], [S - 1], 1, H, Hkv, D, P, True)[0]
    assert np.max(np.abs(flash - ref)) < 2e-6


def test_prefill_rows_equal_decode_rows_and_brute_force():
    rng = np.random.default_rng(21)
    B, C, H, Hkv, D, P = 2, 5, 4, 2, 16, 8
    ctx = np.array([9, 0])
    seq = (ctx + C).astype(np.uint32)
    pages = (seq + P - 1) // P
    flat = rng.permutation(int(pages.sum()) + 2)[:int(pages.sum())].astype(np.uint32)
    off = np.concatenate([[0], np.cumsum(pages)]).astype(np.uint32)
    n = (int(pages.sum()) + 2) * P * Hkv * D
    k = rng.standard_normal(n).astype(np.float16).view(np.uint16)
    v = rng.standard_normal(n).astype(np.float16).view(np.uint16)
    q16 = rng.standard_normal((B, C, H, D)).astype(np.float16)
    out = po.paged_attention_prefill(q16.view(np.uint16), k, v, flat, off, seq, ctx, B, C, H, Hkv, D, P)
    qf = q16.astype(np.float32)
    for i in range(C):
        row = po.paged_attention_executor(qf[:, i], k, v, flat, off, seq, ctx + i, B, H, Hkv, D, P, True)
        assert np.array_equal(out[:, i], row)
        want = _brute_f64(qf[:, i], k, v, flat, off, seq, ctx + i, B, H, Hkv, D, P, True)
        assert np.max(np.abs(out[:, i] - want)) < 2e-6


# ---------------------------------------------------------------- scatter / gather

def _pattern(pages, P, Hkv, D):
    p, s, h, d = np.meshgrid(np.arange(pages), np.arange(P), np.arange(Hkv), np.arange(D), indexing="ij")
    return (p * 1e5 + s * 1e3 + h * 10 + d).astype(np.float32)  # tests/test_paged_kv.cpp:219-241


def test_gather_closed_form_through_out_of_order_table():
    P, Hkv, D = 4, 2, 8
    pool = _pattern(12, P, Hkv, D)
    table = [7, 2, 11]  # tests/test_paged_kv.cpp:292
    out = np.zeros((Hkv, 10, D), np.float32)
    assert po.gather_kv_pages(pool, table, P, Hkv, D, 10, out, 4)
    for h in range(Hkv):
        for t in range(10):
            for d in range(D):
                assert out[h, t, d] == table[t // P] * 1e5 + (t % P) * 1e3 + h * 10 + d


def test_scatter_then_gather_is_identity_and_touches_nothing_else():
    # tests/test_paged_kv.cpp:404-474: start_slot 3, 11 tokens, pages {5, 1, ...}
    P, Hkv, D, tokens, start = 4, 2, 8, 11, 3
    rng = np.random.default_rng(4)
    for dtype, nbytes in ((np.float32, 4), (np.float16, 2)):
        pool = rng.standard_normal(10 * P * Hkv * D).astype(dtype)
        before = pool.copy()
        src = rng.standard_normal((Hkv, tokens, D)).astype(dtype)
        table = [5, 1, 8, 3]
        assert po.scatter_kv_paged(pool, table, P, Hkv, D, tokens, start, src, nbytes)
        full = np.zeros((Hkv, start + tokens, D), dtype)
        assert po.gather_kv_pages(pool, table, P, Hkv, D, start + tokens, full, nbytes)
        assert np.array_equal(full[:, start:], src)
        assert int((pool.view(np.uint8) != before.view(np.uint8)).any()) and \
            (pool != before).sum() <= tokens * Hkv * D
        # rows before start_slot of the first page are untouched
        assert np.array_equal(full[:, :start], before.reshape(10, P, Hkv, D)[5, :start].transpose(1, 0, 2))


def test_scatter_batched_index_formula_and_untouched_bytes():
    # metal_runtime.mm:420-422: dst = page*epp + slot*(Hkv*D) + kv*D + dim
    P, Hkv, D, B = 8, 3, 6, 4
    rng = np.random.default_rng(6)
    pool = rng.integers(0, 65536, 9 * P * Hkv * D, dtype=np.uint16)
    before = pool.copy()
    src = rng.integers(0, 65536, (B, Hkv, D), dtype=np.uint16)
    ids, slots = [3, 8, 0, 5], [7, 0, 2, 2]
    assert po.scatter_kv_paged_batched_f16(pool, ids, slots, P, Hkv, D, B, src)
    view = pool.reshape(9, P, Hkv, D)
    touched = np.zeros_like(view, bool)
    for r in range(B):
        assert np.array_equal(view[ids[r], slots[r]], src[r])
        touched[ids[r], slots[r]] = True
    assert np.array_equal(view[~touched], before.reshape(9, P, Hkv, D)[~touched])
    assert not po.scatter_kv_paged_batched_f16(pool, ids, slots, 0, Hkv, D, B, src)
    assert not po.scatter_kv_paged_batched_f16(pool, ids, slots, P, Hkv, D, 0, src)


def test_scatter_gather_reject_like_the_reference():
    pool = np.zeros(8 * 4 * 2 * 8, np.float32)
    buf = np.zeros((2, 16, 8), np.float32)
    # tests/test_paged_kv.cpp:541-595
    assert not po.gather_kv_pages(pool, [0], 4, 2, 8, 5, buf, 4)
    assert not po.gather_kv_pages(pool, [0], 4, 2, 8, 4, buf, 3)
    assert not po.gather_kv_pages(pool, [0], 4, 2, 8, 0, buf, 4)
    assert not po.scatter_kv_paged(pool, [0], 4, 2, 8, 4, 4, buf, 4)
    assert not po.scatter_kv_paged(pool, [0], 4, 2, 8, 5, 0, buf, 4)
    assert not po.scatter_kv_paged(pool, [0], 4, 2, 8, 4, 0, buf, 8)
    assert po.scatter_kv_paged(pool, [0], 4, 2, 8, 4, 0, buf, 4)


# ---------------------------------------------------------------- metrics

def test_metrics_definitions():
    a = np.array([1, 2, 3, 4], np.float32)
    b = np.array([1, 2, 3, 6], np.float32)
    m = po.metrics(a, b)
    assert m["max_abs"] == 2.0 and m["mean_abs"] == 0.5 and abs(m["rms"] - 1.0) < 1e-12
    assert abs(m["cosine"] - (1 + 4 + 9 + 24) / np.sqrt(30 * 50)) < 1e-12
    assert np.isnan(po.metrics(np.zeros(3, np.float32), a[:3])["cosine"])  # parity_harness.cpp:250-254
    assert po.cosine(np.zeros(3, np.float32), a[:3]) == 0.0                 # tests/test_paged_flash.cpp:100


# ---------------------------------------------------------------- allocator

def test_pool_fresh_ids_ascend_and_reuse_is_lifo():
    # tests/test_paged_kv.cpp:34-71
    pool = po.PagePool(4)
    assert [pool.allocate() for _ in range(4)] == [0, 1, 2, 3]
    assert pool.allocate() is None and pool.pages_in_use() == 4 and pool.pages_free() == 0
    pool.release(1)
    pool.release(3)
    assert pool.allocate() == 3 and pool.allocate() == 1


def test_pool_allocate_n_is_all_or_nothing():
    # tests/test_paged_kv.cpp:73-94
    pool = po.PagePool(5)
    assert pool.allocate_n(3) == [0, 1, 2]
    assert pool.allocate_n(3) is None and pool.pages_free() == 2
    assert pool.allocate_n(2) == [3, 4]


def test_request_state_slots_roll_over_pages():
    # tests/test_paged_kv.cpp:132-154: P=4 -> slots 0,1,2,3,0,... and a new page every 4 tokens
    pool = po.PagePool(3)
    st = po.RequestKVState(4)
    got = [st.extend_one_token(pool) for _ in range(9)]
    assert got == [(0, 0), (0, 1), (0, 2), (0, 3), (1, 0), (1, 1), (1, 2), (1, 3), (2, 0)]
    assert st.total_tokens() == 9 and st.page_table == [0, 1, 2] and st.tokens_in_last_page == 1
    for _ in range(3):
        assert st.extend_one_token(pool) is not None
    assert st.extend_one_token(pool) is None          # exhaustion, :156-169
    assert st.total_tokens() == 12
    assert st.locate(5) == (1, 1) and st.locate(11) == (2, 3) and st.locate(12) is None  # :171-189
    st.release_all(pool)
    assert pool.pages_in_use() == 0 and st.total_tokens() == 0   # :191-207


def test_requests_get_disjoint_pages():
    # tests/test_paged_kv.cpp:597-619
    pool = po.PagePool(16)
    reqs = [po.RequestKVState(4) for _ in range(3)]
    for t in range(10):
        for r in reqs:
            assert r.extend_one_token(pool) is not None
    tables = [set(r.page_table) for r in reqs]
    assert not (tables[0] & tables[1]) and not (tables[0] & tables[2]) and not (tables[1] & tables[2])


def replay_allocator_script(script):
    """Runs a PagePool / RequestKVState command script through the oracle and returns its
    replies in the text form of oracle/ref_alloc_driver.cpp."""
    pool, st, mine = None, None, []
    for line in script:
        cmd, *arg = line.split()
        a = int(arg[0]) if arg else 0
        if cmd == "pool":
            pool = po.PagePool(a)
            mine.append("ok")
        elif cmd == "req":
            st = po.RequestKVState(a, max_pages=64)
            mine.append("ok")
        elif cmd == "extend":
            r = st.extend_one_token(pool)
            mine.append("none" if r is None else f"{r[0]} {r[1]}")
        elif cmd == "reserve":
            ok = st.reserve(pool, a)
            mine.append(f"{int(ok)} {len(st.page_table)}")
        elif cmd == "locate":
            r = st.locate(a)
            mine.append("none" if r is None else f"{r[0]} {r[1]}")
        elif cmd == "total":
            mine.append(str(st.total_tokens()))
        elif cmd == "release_all":
            st.release_all(pool)
            mine.append("ok")
        elif cmd == "stats":
            mine.append(f"{pool.pages_in_use()} {pool.pages_free()}")
    return mine


@needs_ref
def test_allocator_transcript_matches_reference_build():
    """Replays a random script through the reference's PagePool/RequestKVState (compiled from
    compiler/runtime/paged_kv.cpp) and through the oracle, and compares every reply."""
    rng = np.random.default_rng(99)
    script = ["pool 24", "req 4"]
    for _ in range(300):
        r = rng.random()
        if r < 0.55:
            script.append("extend")
        elif r < 0.65:
            script.append(f"reserve {int(rng.integers(0, 40))}")
        elif r < 0.8:
            script.append(f"locate {int(rng.integers(0, 50))}")
        elif r < 0.9:
            script.append("total")
        elif r < 0.95:
            script.append("release_all")
        else:
            script.append("stats")
    ref_out = subprocess.run([po.REF_ALLOC_DRIVER], input="\n".join(script) + "\n", text=True,
                             capture_output=True, check=True).stdout.split("\n")
    mine = replay_allocator_script(script)
    assert mine == ref_out[:len(mine)]


# ------------------------------------------------- qkv split + RoPE + cast

ROPE_VEC = [1.7640524, 0.4001572, 0.9787380, 2.2408931, 1.8675580, -0.9772779, 0.95008844, -0.1513572]
ROPE_COS = [0.96366274, 0.3834415, 0.79172504, 0.5288949]
ROPE_SIN = [0.56804454, 0.92559665, 0.07103606, 0.0871293]
ROPE_EXPECTED = [1.4726444, 1.3876770, -1.6988745, 1.7651681, 1.5480144, -0.6410714, 0.5156846, 0.00272848]


def test_rope_known_answer_of_the_reference_test():
    """tests/test_runtime.cpp:799-818 (RotaryEmbeddingTest.CpuMatchesExpectedRotation), 1e-5."""
    qkv = np.array(ROPE_VEC * 3, np.float32)
    q, k, v, k16, v16 = po.qkv_split_rope_cast(qkv, ROPE_COS, ROPE_SIN, 1, 1, 1, 8, 24, 8, 8, 8, 8)
    assert np.max(np.abs(q[0] - np.array(ROPE_EXPECTED, np.float32))) <= 1e-5
    assert np.max(np.abs(k[0] - np.array(ROPE_EXPECTED, np.float32))) <= 1e-5
    assert np.array_equal(v[0], np.array(ROPE_VEC, np.float32))          # v is never rotated
    assert np.array_equal(k16[0], po.float_to_fp16_rne(k[0]))
    assert np.array_equal(v16[0], po.float_to_fp16_rne(v[0]))


def test_rope_split_closed_forms():
    rng = np.random.default_rng(5)
    B, H, Hkv, D, rot = 3, 4, 2, 16, 8
    q_rows, k_rows, v_rows = H * D, Hkv * D, Hkv * D
    qkv_rows = q_rows + k_rows + v_rows + 6           # padding after v is ignored
    qkv = rng.standard_normal((B, qkv_rows)).astype(np.float32)
    ang = rng.uniform(-3, 3, (B, rot // 2))
    cos, sin = np.cos(ang).astype(np.float32), np.sin(ang).astype(np.float32)
    q, k, v, k16, v16 = po.qkv_split_rope_cast(qkv, cos, sin, B, H, Hkv, D, qkv_rows, q_rows, k_rows,
                                               v_rows, rot)
    # split offsets (metal_runtime.mm:7962-7964) and untouched dims >= rotary_dim
    assert np.array_equal(v, qkv[:, q_rows + k_rows:q_rows + k_rows + v_rows])
    q_in = qkv[:, :q_rows].reshape(B, H, D)
    assert np.array_equal(q.reshape(B, H, D)[:, :, rot:], q_in[:, :, rot:])
    # rotation in float64 as the independent leg: pair norms are preserved, formula matches
    x0, x1 = q_in[:, :, 0:rot:2].astype(np.float64), q_in[:, :, 1:rot:2].astype(np.float64)
    c, s = cos[:, None, :].astype(np.float64), sin[:, None, :].astype(np.float64)
    want0, want1 = x0 * c - x1 * s, x0 * s + x1 * c
    got = q.reshape(B, H, D)
    assert np.max(np.abs(got[:, :, 0:rot:2] - want0)) < 1e-6
    assert np.max(np.abs(got[:, :, 1:rot:2] - want1)) < 1e-6
    # a transposed or sign-flipped rotation would fail this: rotating by -angle undoes it
    back = po.qkv_split_rope_cast(np.concatenate([q, k, v], axis=1), cos, -sin, B, H, Hkv, D,
                                  q_rows + k_rows + v_rows, q_rows, k_rows, v_rows, rot)
    assert np.max(np.abs(back[0] - qkv[:, :q_rows])) < 1e-6
    # rotary_dim 0: pure split + cast, tables may be absent
    q0, k0, v0, k160, _ = po.qkv_split_rope_cast(qkv, None, None, B, H, Hkv, D, qkv_rows, q_rows, k_rows,
                                                 v_rows, 0)
    assert np.array_equal(q0, qkv[:, :q_rows]) and np.array_equal(k0, qkv[:, q_rows:q_rows + k_rows])
    assert np.array_equal(k160, qkv[:, q_rows:q_rows + k_rows].astype(np.float16).view(np.uint16))
    # argument errors
    assert po.qkv_split_rope_cast(qkv, cos, sin, B, H, Hkv, D, q_rows, q_rows, k_rows, v_rows, rot) is None
    assert po.qkv_split_rope_cast(qkv, cos, sin, B, H, Hkv, D, qkv_rows, q_rows, k_rows, v_rows, D + 2) is None
    assert po.qkv_split_rope_cast(qkv, None, None, B, H, Hkv, D, qkv_rows, q_rows, k_rows, v_rows, rot) is None


def test_rotary_coefficients_closed_forms():
    cos, sin = po.rotary_coefficients(0, 64)
    assert np.all(cos == 1.0) and np.all(sin == 0.0)                   # position 0: identity
    cos, sin = po.rotary_coefficients(3, 8, 10000.0, 1.0)
    want = 3.0 * 10000.0 ** (-np.arange(4) * 2 / 8)
    assert np.max(np.abs(cos - np.cos(want))) < 1e-6 and np.max(np.abs(sin - np.sin(want))) < 1e-6
    # base <= 0 and scale == 0 fall back to 10000 and 1 (quantization.cpp:806-811)
    a, b = po.rotary_coefficients(7, 16, 0.0, 0.0), po.rotary_coefficients(7, 16, 10000.0, 1.0)
    assert np.array_equal(a[0], b[0]) and np.array_equal(a[1], b[1])
    assert po.rotary_coefficients(5, 1)[0].size == 0


@needs_ref
def test_rope_bit_exact_with_reference_build():
    """applyRotaryEmbedding / computeRotaryCoefficients compiled from
    compiler/runtime/quantization.cpp:772-823."""
    rng = np.random.default_rng(8)
    for D, rot, pos in [(64, 64, 1234), (128, 128, 8191), (64, 32, 17), (16, 8, 3)]:
        cos, sin = po.rotary_coefficients(pos, rot, 10000.0, 1.0)
        rc, rs = po.ref_rotary_coefficients(pos, rot, 10000.0, 1.0)
        assert np.array_equal(cos.view(np.uint32), rc.view(np.uint32))
        assert np.array_equal(sin.view(np.uint32), rs.view(np.uint32))
        H, Hkv = 4, 2
        qkv = rng.standard_normal((H + 2 * Hkv) * D).astype(np.float32)
        q, k, v, _, _ = po.qkv_split_rope_cast(qkv, cos, sin, 1, H, Hkv, D, qkv.size, H * D, Hkv * D,
                                               Hkv * D, rot)
        for h in range(H):
            want = po.ref_apply_rotary(qkv[h * D:(h + 1) * D], cos, sin, D, rot)
            assert np.array_equal(q[0, h * D:(h + 1) * D].view(np.uint32), want.view(np.uint32))
        for h in range(Hkv):
            want = po.ref_apply_rotary(qkv[(H + h) * D:(H + h + 1) * D], cos, sin, D, rot)
            assert np.array_equal(k[0, h * D:(h + 1) * D].view(np.uint32), want.view(np.uint32))


# ------------------------------------------------ walker layer operators

def test_rms_norm_closed_forms_and_reference_test_formula():
    rng = np.random.default_rng(3)
    B, L, eps = 4, 2048, 1e-5
    x = rng.uniform(-1, 1, (B, L)).astype(np.float32)
    w = rng.uniform(-1, 1, L).astype(np.float32)
    got = po.rms_norm_batched(x, w, eps, B, L)
    # tests/test_batched_elementwise.cpp:19-32 (double-precision sum), tolerance 1e-4 there
    want = x / np.sqrt((x.astype(np.float64) ** 2).mean(axis=1, keepdims=True) + eps) * w
    assert np.max(np.abs(got - want)) < 1e-5
    # constant rows: out = c / sqrt(c^2 + eps) * w
    c = np.full((2, 64), 3.0, np.float32)
    got = po.rms_norm_batched(c, np.ones(64, np.float32), eps, 2, 64)
    assert np.allclose(got, 3.0 / np.sqrt(9.0 + eps), rtol=1e-6)
    # scale invariance (up to eps) and the missing-weight rule (gamma = 1 past the end)
    a = po.rms_norm_batched(x * 4, w, 0.0, B, L)
    b = po.rms_norm_batched(x, w, 0.0, B, L)
    assert np.max(np.abs(a - b)) < 1e-5
    short = po.rms_norm_batched(x, w[:10], eps, B, L)
    full = po.rms_norm_batched(x, np.concatenate([w[:10], np.ones(L - 10, np.float32)]), eps, B, L)
    assert np.array_equal(short, full)
    assert po.rms_norm_batched(x, w, eps, 0, L) is None


def test_add_silu_gate_up_closed_forms():
    rng = np.random.default_rng(4)
    a, b = rng.standard_normal(1000).astype(np.float32), rng.standard_normal(1000).astype(np.float32)
    assert np.array_equal(po.add(a, b), a + b)
    g = np.array([0.0, 1.0, -1.0, 20.0, -20.0, 100.0, -100.0], np.float32)
    u = np.full(g.size, 2.0, np.float32)
    got = po.silu_mul(g, u)
    want = g.astype(np.float64) / (1 + np.exp(-g.astype(np.float64))) * 2
    assert np.allclose(got, want, rtol=1e-6, atol=1e-30)
    assert got[0] == 0.0 and got[5] == 200.0 and abs(got[6]) < 1e-30   # limits: 0, identity, 0
    B, inner, rows = 3, 8, 20
    gu = rng.standard_normal((B, rows)).astype(np.float32)
    gate, up, out = po.gate_up_split_silu_mul(gu, B, inner, rows)
    assert np.array_equal(gate, gu[:, :inner]) and np.array_equal(up, gu[:, inner:2 * inner])
    assert np.array_equal(out, po.silu_mul(gate, up))
    assert po.gate_up_split_silu_mul(gu, B, 11, rows) is None         # 2*inner > rows


def test_q4_0_known_block_and_dequant_formula():
    # one block by hand: d = 0.5, nibbles j -> weight j, j+16
    blk = np.zeros(18, np.uint8)
    blk[:2] = np.frombuffer(np.float16(0.5).tobytes(), np.uint8)
    lo = np.arange(16) % 16
    hi = (np.arange(16) * 3 + 1) % 16
    blk[2:] = (hi << 4 | lo).astype(np.uint8)
    w = np.concatenate([0.5 * (lo - 8), 0.5 * (hi - 8)]).astype(np.float32)
    x = np.linspace(-1, 1, 64).astype(np.float32)
    rows = np.tile(np.concatenate([blk, blk]), (4, 1))              # 4 rows x 64 cols
    got = po.matmul_q4_0_batched(rows, x[None, :], 1, 4, 64)
    want = float(np.dot(np.concatenate([w, w]).astype(np.float64), x.astype(np.float64)))
    assert np.allclose(got, want, rtol=1e-6)
    # constraints of the batched kernel (metal_runtime.mm:6942)
    assert po.matmul_q4_0_batched(rows, x[None, :32], 1, 4, 32) is None
    assert po.matmul_q4_0_batched(rows[:3], x[None, :], 1, 3, 64) is None


def test_q4_0_quantize_round_trip_error_bound():
    rng = np.random.default_rng(6)
    w = rng.standard_normal((8, 128)).astype(np.float32)
    q = po.quantize_q4_0(w)
    eye = np.eye(128, dtype=np.float32)
    deq = po.matmul_q4_0_batched(q, eye, 128, 8, 128).T            # row r of W = products with unit vectors
    d = np.abs(w).reshape(8, 4, 32).max(axis=2) / 8
    assert np.all(np.abs(deq - w).reshape(8, 4, 32) <= d[:, :, None] * 1.01 + 1e-6)


@needs_ref
def test_q4_0_bit_exact_with_reference_build():
    """quantizeRowQ4_0 / dotProductRowQ4_0 compiled from compiler/runtime/quantization.cpp."""
    R = po.ref_lib()
    rng = np.random.default_rng(12)
    for cols in (64, 96, 2048):
        w = (rng.standard_normal((4, cols)) * rng.uniform(0.01, 3)).astype(np.float32)
        q = po.quantize_q4_0(w)
        for r in range(4):
            buf = np.zeros(q.shape[1], np.uint8)
            n = R.ref_quantize_row_q4_0(w[r].ctypes.data_as(po._f32p), cols, buf.ctypes.data, buf.size)
            assert n == q.shape[1] and np.array_equal(buf, q[r])
        x = rng.standard_normal((3, cols)).astype(np.float32)
        got = po.matmul_q4_0_batched(q, x, 3, 4, cols)
        for b in range(3):
            for r in range(4):
                want = R.ref_dot_q4_0(q[r].ctypes.data, cols, x[b].ctypes.data_as(po._f32p))
                assert np.float32(want).view(np.uint32) == got[b, r].view(np.uint32)


def _q6k_block_by_hand(rng):
    """One Q6_K block written field by field, with the weights it stands for computed from the
    format's definition (quantization.cpp:142-147, 1469-1499): weight n of the block sits in
    half n / 128, quarter (n % 128) / 32, position l = n % 32; its low nibble is in ql[half*64 +
    (quarter & 1)*32 + l] (low nibble for quarters 0-1, high for 2-3), its two high bits in
    qh[half*32 + l] at bit 2*quarter, its scale is scales[half*8 + quarter*2 + l/16]."""
    q = rng.integers(0, 64, 256)
    sc = rng.integers(-100, 101, 16).astype(np.int8)
    d = np.float16(0.0123)
    blk = np.zeros(210, np.uint8)
    w = np.zeros(256, np.float64)
    for n in range(256):
        half, quarter, l = n // 128, (n % 128) // 32, n % 32
        qi = half * 64 + (quarter & 1) * 32 + l
        blk[qi] |= (q[n] & 0xF) << (4 if quarter >= 2 else 0)
        blk[128 + half * 32 + l] |= (q[n] >> 4) << (2 * quarter)
        w[n] = float(d) * float(sc[half * 8 + quarter * 2 + l // 16]) * (int(q[n]) - 32)
    blk[192:208] = sc.view(np.uint8)
    blk[208:210] = np.frombuffer(d.tobytes(), np.uint8)
    return blk, w


def test_q6_k_block_by_hand_and_constraints():
    rng = np.random.default_rng(66)
    blk, w = _q6k_block_by_hand(rng)
    deq = po.dequantize_q6_k(blk[None, :], 256)[0]
    assert np.allclose(deq, w, rtol=3e-7, atol=0)
    rows = np.tile(blk, (4, 1))
    x = rng.standard_normal((2, 256)).astype(np.float32)
    got = po.matmul_q6_k_batched(rows, x, 2, 4, 256)
    want = x.astype(np.float64) @ w
    assert np.allclose(got, want[:, None], rtol=1e-5, atol=1e-5)
    # constraints of the batched kernel (metal_runtime.mm:6985)
    assert po.matmul_q6_k_batched(rows[:3], x, 2, 3, 256) is None
    assert po.matmul_q6_k_batched(rows, x[:, :32], 2, 4, 32) is None


def test_q6_k_quantize_round_trip_error_bound():
    rng = np.random.default_rng(67)
    w = (rng.standard_normal((4, 512)) * rng.uniform(0.1, 4, (4, 1))).astype(np.float32)
    q = po.quantize_q6_k(w)
    deq = po.dequantize_q6_k(q, 512)
    # a group of 16 is quantised with step ~ max|group| / 32 (the scale code rounds it by up to
    # half a unit of max_scale / 127, the fp16 d by 2^-11): error <= 0.5 steps + the clamp at 31
    grp = np.abs(w).reshape(4, 32, 16).max(axis=2)
    blockmax = grp.reshape(4, 2, 16).max(axis=2).repeat(16, axis=1)
    step = grp / 32 + blockmax / 32 / 127
    assert np.all(np.abs(deq - w).reshape(4, 32, 16) <= 1.6 * step[:, :, None] + 1e-6)


@needs_ref
def test_q6_k_bit_exact_with_reference_build():
    """quantizeRowQ6_K / dequantizeRowQ6_K / dotProductRowQ6_K compiled from
    compiler/runtime/quantization.cpp."""
    R = po.ref_lib()
    rng = np.random.default_rng(68)
    for cols in (256, 320, 2048):     # 320: a partial last block
        w = (rng.standard_normal((4, cols)) * rng.uniform(0.01, 3)).astype(np.float32)
        q = po.quantize_q6_k(w)
        deq = po.dequantize_q6_k(q, cols)
        for r in range(4):
            buf = np.zeros(q.shape[1], np.uint8)
            n = R.ref_quantize_row_q6_k(w[r].ctypes.data_as(po._f32p), cols, buf.ctypes.data, buf.size)
            assert n == q.shape[1] and np.array_equal(buf, q[r])
            want = np.zeros(cols, np.float32)
            R.ref_dequantize_row_q6_k(q[r].ctypes.data, cols, want.ctypes.data_as(po._f32p))
            assert np.array_equal(want.view(np.uint32), deq[r].view(np.uint32))
        x = rng.standard_normal((3, cols)).astype(np.float32)
        got = po.matmul_q6_k_batched(q, x, 3, 4, cols)
        for b in range(3):
            for r in range(4):
                want = R.ref_dot_q6_k(q[r].ctypes.data, cols, x[b].ctypes.data_as(po._f32p))
                assert np.float32(want).view(np.uint32) == got[b, r].view(np.uint32)


def test_numpy_q4_0_encoder_is_bit_identical_to_the_oracle_quantiser():
    """The workload module's vectorised Q4_0 encoder against the oracle's restatement of
    quantizeRowQ4_0, including all-zero blocks and blocks whose extreme value is negative."""
    from mlcompiler_amd import workloads as wl
    rng = np.random.default_rng(5)
    w = (rng.standard_normal((37, 256)) * 0.05).astype(np.float32)
    w[3, 32:64] = 0.0
    w[5, :32] = -np.abs(w[5, :32])
    w[6, :32] = np.abs(w[6, :32])
    assert np.array_equal(wl.quantize_q4_0(w), po.quantize_q4_0(w))


def test_numpy_q6_k_encoder_decodes_within_half_a_step():
    """The workload module's Q6_K encoder is a plain round-to-nearest one (not the reference's
    scale search): what it writes must decode, through the oracle's dequantizeRowQ6_K, to within
    half a quantisation step of the input, and all-zero super-blocks must decode to zero."""
    from mlcompiler_amd import workloads as wl
    rng = np.random.default_rng(6)
    w = (rng.standard_normal((9, 1024)) * 0.03).astype(np.float32)
    w[2, 256:512] = 0.0
    enc = wl.quantize_q6_k(w)
    assert enc.shape == (9, po.q6_k_row_bytes(1024))
    back = po.dequantize_q6_k(enc, 1024)
    assert np.all(back[2, 256:512] == 0.0)
    step = np.abs(w).reshape(9, 64, 16).max(axis=2, keepdims=True) / 31.0
    err = np.abs(back - w).reshape(9, 64, 16)
    assert np.all(err <= 0.75 * step + 1e-7), float((err / (step + 1e-12)).max())
    # and it is about as good as the reference's quantiser on the same input
    ref = po.dequantize_q6_k(po.quantize_q6_k(w), 1024)
    assert np.abs(back - w).mean() <= 1.5 * np.abs(ref - w).mean()
