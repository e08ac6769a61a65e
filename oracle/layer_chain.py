"""TEST INFRASTRUCTURE: the CPU oracles of one decoder layer of the reference's batched decode step
chained in the order of compiler/runtime/batched_walker.cpp:246-405 (RMSNorm, fused QKV matmul,
split + rotary + fp16 cast, K/V scatter, paged attention, output matmul, residual, RMSNorm,
gate/up matmul, SiLU*up, down matmul, residual).  Every link is a function of paged_oracle that is
pinned on its own; the chain adds only the order.  Used by the layer parity test and by the
benchmark's CPU baseline, never by the product."""
import numpy as np

from oracle import paged_oracle as po

# TinyLlama-1.1B layer shape
HID, H, HKV, D, FFN, P = 2048, 32, 4, 64, 5632, 64
Q_ROWS, KV_ROWS = H * D, HKV * D
QKV_ROWS = Q_ROWS + 2 * KV_ROWS


def rotary_tables(q_positions):
    cos = np.zeros((len(q_positions), D // 2), np.float32)
    sin = np.zeros((len(q_positions), D // 2), np.float32)
    for r, p in enumerate(q_positions):
        cos[r], sin[r] = po.rotary_coefficients(int(p), D)
    return cos, sin


def oracle_chain(w, x, cos, sin, k_pool, v_pool, page_ids, slots, flat, off, seq, qpos, n_threads=8):
    """Expected results of the layer for the requests given (x, cos, sin, page_ids, slots, off,
    seq, qpos all cover the same requests).  Returns a dict with the layer output, the attention
    output, the new K rows and the K/V pools after the write."""
    batch = x.shape[0]
    def mm(*a):
        return po.matmul_q4_0_batched(*a, n_threads=n_threads)
    n1 = po.rms_norm_batched(x, w["g_attn"], 1e-5, batch, HID)
    qkv = mm(w["w_qkv"], n1, batch, QKV_ROWS, HID)
    q, k, v, k16, v16 = po.qkv_split_rope_cast(qkv, cos, sin, batch, H, HKV, D, QKV_ROWS, Q_ROWS, KV_ROWS,
                                               KV_ROWS, D)
    want_k, want_v = k_pool.copy(), v_pool.copy()
    assert po.scatter_kv_paged_batched_f16(want_k, page_ids, slots, P, HKV, D, batch, k16)
    assert po.scatter_kv_paged_batched_f16(want_v, page_ids, slots, P, HKV, D, batch, v16)
    attn = po.paged_attention_executor(q, want_k, want_v, flat, off, seq, qpos, batch, H, HKV, D, P, True,
                                       n_threads)
    o = mm(w["w_o"], attn.reshape(batch, HID), batch, HID, HID)
    r1 = po.add(x, o)
    n2 = po.rms_norm_batched(r1, w["g_ffn"], 1e-5, batch, HID)
    gu = mm(w["w_gu"], n2, batch, 2 * FFN, HID)
    _, _, mix = po.gate_up_split_silu_mul(gu, batch, FFN, 2 * FFN)
    down = mm(w["w_down"], mix, batch, HID, FFN)
    return {"out": po.add(r1, down), "attn": attn, "k": k, "k_pool": want_k, "v_pool": want_v}
