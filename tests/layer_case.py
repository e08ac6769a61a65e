"""One TinyLlama-shape decoder layer of the reference's batched decode step
(compiler/runtime/batched_walker.cpp:246-405) as data: random Q4_0 weights, norm weights, an
input batch, and the chain of CPU oracles that gives the expected output.  Shared by the layer
parity test and the layer benchmark."""
import numpy as np

from oracle import paged_oracle as po

HID, H, HKV, D, FFN, P = 2048, 32, 4, 64, 5632, 64
Q_ROWS, KV_ROWS = H * D, HKV * D
QKV_ROWS = Q_ROWS + 2 * KV_ROWS


def q4_weights(rng, rows, cols, scale):
    return po.quantize_q4_0((rng.standard_normal((rows, cols)) * scale).astype(np.float32))


def make_layer_weights(seed):
    rng = np.random.default_rng(seed)
    return {
        "w_qkv": q4_weights(rng, QKV_ROWS, HID, 0.03),
        "w_o": q4_weights(rng, HID, HID, 0.03),
        "w_gu": q4_weights(rng, 2 * FFN, HID, 0.03),
        "w_down": q4_weights(rng, HID, FFN, 0.02),
        "g_attn": rng.uniform(0.5, 1.5, HID).astype(np.float32),
        "g_ffn": rng.uniform(0.5, 1.5, HID).astype(np.float32),
    }


def weight_bytes(w):
    return sum(w[k].nbytes for k in ("w_qkv", "w_o", "w_gu", "w_down"))


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
