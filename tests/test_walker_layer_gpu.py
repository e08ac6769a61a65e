"""One whole decoder layer of the reference's batched decode step (the layer loop of
compiler/runtime/batched_walker.cpp:246-405) on the HIP path, every operator through the C ABI
in ONE open pass (no host round trip between them), against the same chain of CPU oracles:

  RMSNorm -> Q4_0 qkv matmul -> split + RoPE + fp16 cast + paged KV scatter -> paged decode
  attention -> Q4_0 out-projection -> residual add -> RMSNorm -> Q4_0 gate/up matmul ->
  gate/up split + SiLU*up -> Q4_0 down-projection -> residual add

TinyLlama-1.1B layer shape (hidden 2048, 32 q / 4 kv heads, head_dim 64, ffn 5632), random
Q4_0 weights, requests with different context lengths in a shared page pool."""
import numpy as np
import pytest

from oracle import paged_oracle as po

pytestmark = pytest.mark.gpu

from layer_case import D, FFN, H, HID, HKV, KV_ROWS, P, Q_ROWS, QKV_ROWS, make_layer_weights, oracle_chain, rotary_tables


@pytest.mark.timeout(300)
@pytest.mark.parametrize("kv_calls", ["one_call", "reference_calls"])
@pytest.mark.parametrize("fuse", [1, 0])
@pytest.mark.parametrize("batch", [6, 33])
def test_decoder_layer_matches_oracle_chain(exe, batch, fuse, kv_calls):
    """fuse = 1: the row-local operators between the matmuls run as fused launches (the default);
    fuse = 0: every operator is launched on its own.  Same expected values either way.
    kv_calls: the split + RoPE + cast + KV write as the one fused call, or as the walker's three
    calls (encodeQkvSplitRopeCast, then the batched scatters of its fp16 K and V rows,
    batched_walker.cpp:287-307)."""
    print(f"[layer] batch={batch} fuse_row_ops={fuse} {kv_calls}", flush=True)
    rng = np.random.default_rng(100 + batch)
    w = make_layer_weights(200 + batch)
    w_qkv, w_o, w_gu, w_down, g_attn, g_ffn = (w[n] for n in ("w_qkv", "w_o", "w_gu", "w_down", "g_attn", "g_ffn"))
    x = rng.standard_normal((batch, HID)).astype(np.float32)

    # paged KV state before the step: request r holds ctx[r] tokens; this step appends one
    ctx = rng.integers(0, 300, batch)
    pool = po.PagePool(int(((ctx + 1 + P - 1) // P).sum()) + 4)
    reqs = [po.RequestKVState(P, max_pages=64) for _ in range(batch)]
    for r, n in zip(reqs, ctx):
        for _ in range(int(n)):
            assert r.extend_one_token(pool) is not None
    cap = pool.capacity
    k_pool = rng.standard_normal(cap * P * KV_ROWS).astype(np.float16).view(np.uint16)
    v_pool = rng.standard_normal(cap * P * KV_ROWS).astype(np.float16).view(np.uint16)
    where = [r.extend_one_token(pool) for r in reqs]          # (page id, slot) of the new row
    page_ids = np.array([w[0] for w in where], np.uint32)
    slots = np.array([w[1] for w in where], np.uint32)
    seq = np.array([r.total_tokens() for r in reqs], np.uint32)
    qpos = seq - 1
    flat = np.concatenate([np.array(r.page_table, np.uint32) for r in reqs])
    off = np.concatenate([[0], np.cumsum([len(r.page_table) for r in reqs])]).astype(np.uint32)
    cos, sin = rotary_tables(qpos)

    # ---- oracle chain
    ref = oracle_chain(w, x, cos, sin, k_pool, v_pool, page_ids, slots, flat, off, seq, qpos)
    want, attn, k, want_k = ref["out"], ref["attn"], ref["k"], ref["k_pool"]

    # ---- the same on the device, one pass
    def dev(n_floats):
        return exe.allocateScratchBuffer(n_floats * 4)
    def up(a):
        a = np.ascontiguousarray(a)
        b = exe.allocateScratchBuffer(a.nbytes)
        assert exe.uploadToBuffer(b, a)
        return b
    d_x, d_cos, d_sin, d_k, d_v = up(x), up(cos), up(sin), up(k_pool), up(v_pool)
    d_n, d_qkv, d_q, d_attn, d_o, d_r1 = (dev(batch * n) for n in (HID, QKV_ROWS, Q_ROWS, HID, HID, HID))
    d_gu, d_gate, d_upb, d_mix, d_down, d_out = (dev(batch * n) for n in (2 * FFN, FFN, FFN, FFN, HID, HID))
    d_kf, d_vf = dev(batch * KV_ROWS), dev(batch * KV_ROWS)
    d_k16, d_v16 = exe.allocateScratchBuffer(batch * KV_ROWS * 2), exe.allocateScratchBuffer(batch * KV_ROWS * 2)
    bufs = [d_x, d_cos, d_sin, d_k, d_v, d_n, d_qkv, d_q, d_attn, d_o, d_r1, d_gu, d_gate, d_upb, d_mix,
            d_down, d_out, d_kf, d_vf, d_k16, d_v16]
    tag = f"layer{batch}"
    assert exe.setOption("fuse_row_ops", fuse)
    fused_before = exe.rowProgramLaunches()
    try:
        assert exe.beginForwardPassCB()
        ok = exe.encodeRmsNormBatched(d_x, g_attn, 1e-5, batch, HID, d_n)
        ok &= exe.encodeMatMulQ4_0Batched(tag + ".attn_qkv", w_qkv, d_n, batch, QKV_ROWS, HID, w_qkv.shape[1], 1, d_qkv)
        if kv_calls == "one_call":
            ok &= exe.encodeQkvSplitRopeScatter(d_qkv, d_q, d_k, d_v, d_cos, d_sin, page_ids, slots, P, batch, H,
                                                HKV, D, QKV_ROWS, Q_ROWS, KV_ROWS, KV_ROWS, D)
        else:
            ok &= exe.encodeQkvSplitRopeCast(d_qkv, d_q, d_kf, d_vf, d_k16, d_v16, d_cos, d_sin, batch, H, HKV, D,
                                             QKV_ROWS, Q_ROWS, KV_ROWS, KV_ROWS, D)
            ok &= exe.encodeScatterKVPagedBatched(d_k, page_ids, slots, P, HKV, D, batch, d_k16)
            ok &= exe.encodeScatterKVPagedBatched(d_v, page_ids, slots, P, HKV, D, batch, d_v16)
        ok &= exe.encodePagedFlashAttention(d_q, d_k, d_v, d_attn, flat, off, seq, qpos, batch, H, HKV, D, P, True)
        ok &= exe.encodeMatMulQ4_0Batched(tag + ".attn_output", w_o, d_attn, batch, HID, HID, w_o.shape[1], 1, d_o)
        ok &= exe.encodeAddBatched(d_x, d_o, d_r1, batch * HID)
        ok &= exe.encodeRmsNormBatched(d_r1, g_ffn, 1e-5, batch, HID, d_n)
        ok &= exe.encodeMatMulQ4_0Batched(tag + ".ffn_gate_up", w_gu, d_n, batch, 2 * FFN, HID, w_gu.shape[1], 1, d_gu)
        ok &= exe.encodeGateUpSplitSiluMul(d_gu, d_gate, d_upb, d_mix, batch, FFN, 2 * FFN)
        ok &= exe.encodeMatMulQ4_0Batched(tag + ".ffn_down", w_down, d_mix, batch, HID, FFN, w_down.shape[1], 1, d_down)
        ok &= exe.encodeAddBatched(d_r1, d_down, d_out, batch * HID)
        assert ok, exe.lastError()
        assert exe.flushForwardPassCB(), exe.lastError()
        got = np.empty((batch, HID), np.float32)
        got_attn = np.empty((batch, H, D), np.float32)
        got_k = np.empty_like(k_pool)
        assert exe.downloadFromBuffer(d_out, got) and exe.downloadFromBuffer(d_attn, got_attn)
        assert exe.downloadFromBuffer(d_k, got_k)
    finally:
        exe.setOption("fuse_row_ops", 1)
        for b in bufs:
            exe.releaseScratchBuffer(b)
    fused = exe.rowProgramLaunches() - fused_before
    print(f"  fused row-operator launches: {fused}", flush=True)
    assert (fused >= 2) if fuse else (fused == 0)

    # the KV rows written on the way: fp16 of values that went through two matmul implementations,
    # so equal up to one fp16 step on a few elements
    dk = np.abs(got_k.view(np.float16).astype(np.float32) - want_k.view(np.float16).astype(np.float32))
    assert np.count_nonzero(got_k != k_pool) <= batch * KV_ROWS
    assert np.max(dk) <= 2e-3 * max(1.0, float(np.max(np.abs(k)))), np.max(dk)
    rep = po.per_head_report(got_attn, attn, D)
    assert rep["min_cosine"] >= 0.9999 and rep["max_abs"] <= 2e-3, rep
    cosine = po.cosine(got.ravel(), want.ravel())
    rel = float(np.max(np.abs(got - want)) / np.max(np.abs(want)))
    print(f"  layer output: cosine {cosine:.8f}, max |diff| / max |want| = {rel:.2e}", flush=True)
    assert cosine >= 0.99999 and rel <= 1e-3
