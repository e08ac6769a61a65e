"""Writes a small synthetic Llama-topology GGUF (version 3) for the walker end-to-end test:
random weights, Q4_0 embeddings and projections, Q6_K output matrix, fp32 norm vectors -- the
tensor names, types and metadata keys of a llama.cpp export (what the reference's GGUFLoader,
compiler/frontends/gguf_loader.cpp, and its model-config reader, compiler/runtime/
kernel_scheduler.cpp:224-263, 354-394, look for).  The reference's own tests write their
synthetic files the same way (tests/test_runtime.cpp:110-169).

The quantisers are the oracle's (bit-identical to the reference's quantizeRowQ4_0 /
quantizeRowQ6_K): this script is test infrastructure.

  python tests/integration/make_tiny_llama_gguf.py OUT.gguf
"""
from __future__ import annotations

import os
import struct
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

# shape of the model: 8 query heads over 2 KV heads of 64 (GQA 4:1, so the decode attention runs on
# the tile-balanced kernel's matrix-pipe path), hidden 512, feed-forward 1024, 2 layers
# (the vocabulary is larger than the hidden size, as in every real model: the reference's embedding
# lookup takes a token_embd with fewer rows than columns for a transposed table, session.cpp:416-425)
SHAPE = dict(layers=2, hidden=512, heads=8, kv_heads=2, head_dim=64, ffn=1024, vocab=1024, context=512)
GGML_F32, GGML_Q4_0, GGML_Q6_K = 0, 2, 14
T_U32, T_F32, T_STR = 4, 6, 8
ALIGN = 32


def _s(text: str) -> bytes:
    b = text.encode()
    return struct.pack("<Q", len(b)) + b


def _kv(key: str, vtype: int, value) -> bytes:
    head = _s(key) + struct.pack("<I", vtype)
    if vtype == T_U32:
        return head + struct.pack("<I", value)
    if vtype == T_F32:
        return head + struct.pack("<f", value)
    return head + _s(value)


def build(seed: int = 20240607):
    from oracle import paged_oracle as po
    s = SHAPE
    rng = np.random.default_rng(seed)
    H, F, V = s["hidden"], s["ffn"], s["vocab"]
    q_rows, kv_rows = s["heads"] * s["head_dim"], s["kv_heads"] * s["head_dim"]

    def dense(rows, cols, scale):
        return (rng.standard_normal((rows, cols), dtype=np.float32) * scale).astype(np.float32)

    tensors = []   # (name, dims (ne0 = columns first), ggml type, bytes)

    def f32(name, arr):
        tensors.append((name, list(arr.shape[::-1]), GGML_F32, np.ascontiguousarray(arr, np.float32).tobytes()))

    def q4(name, rows, cols, scale):
        tensors.append((name, [cols, rows], GGML_Q4_0, po.quantize_q4_0(dense(rows, cols, scale)).tobytes()))

    q4("token_embd.weight", V, H, 1.0)
    for l in range(s["layers"]):
        p = f"blk.{l}."
        f32(p + "attn_norm.weight", 1.0 + 0.1 * rng.standard_normal(H, dtype=np.float32))
        q4(p + "attn_q.weight", q_rows, H, H ** -0.5)
        q4(p + "attn_k.weight", kv_rows, H, H ** -0.5)
        q4(p + "attn_v.weight", kv_rows, H, H ** -0.5)
        q4(p + "attn_output.weight", H, q_rows, q_rows ** -0.5)
        f32(p + "ffn_norm.weight", 1.0 + 0.1 * rng.standard_normal(H, dtype=np.float32))
        q4(p + "ffn_gate.weight", F, H, H ** -0.5)
        q4(p + "ffn_up.weight", F, H, H ** -0.5)
        q4(p + "ffn_down.weight", H, F, F ** -0.5)
    f32("output_norm.weight", 1.0 + 0.1 * rng.standard_normal(H, dtype=np.float32))
    tensors.append(("output.weight", [H, V], GGML_Q6_K, po.quantize_q6_k(dense(V, H, H ** -0.5)).tobytes()))

    kvs = [
        _kv("general.architecture", T_STR, "llama"),
        _kv("general.name", T_STR, "tiny synthetic llama for the walker test"),
        _kv("general.quantization_version", T_U32, 2),
        _kv("general.alignment", T_U32, ALIGN),
        _kv("llama.block_count", T_U32, s["layers"]),
        _kv("llama.embedding_length", T_U32, H),
        _kv("llama.feed_forward_length", T_U32, F),
        _kv("llama.attention.head_count", T_U32, s["heads"]),
        _kv("llama.attention.head_count_kv", T_U32, s["kv_heads"]),
        _kv("llama.context_length", T_U32, s["context"]),
        _kv("llama.rope.dimension_count", T_U32, s["head_dim"]),
        _kv("llama.rope.freq_base", T_F32, 10000.0),
        _kv("llama.attention.layer_norm_rms_epsilon", T_F32, 1e-5),
        _kv("general.vocab_size", T_U32, V),
    ]
    infos, data, off = b"", b"", 0
    for name, dims, ttype, raw in tensors:
        infos += _s(name) + struct.pack("<I", len(dims)) + b"".join(struct.pack("<Q", d) for d in dims)
        infos += struct.pack("<I", ttype) + struct.pack("<Q", off)
        pad = (-len(raw)) % ALIGN
        data += raw + b"\0" * pad
        off += len(raw) + pad
    head = struct.pack("<IIQQ", 0x46554747, 3, len(tensors), len(kvs)) + b"".join(kvs) + infos
    head += b"\0" * ((-len(head)) % ALIGN)
    return head + data


def main() -> int:
    out = sys.argv[1]
    blob = build()
    with open(out, "wb") as fh:
        fh.write(blob)
    import hashlib
    print(out, len(blob), "bytes, sha256", hashlib.sha256(blob).hexdigest())
    return 0


if __name__ == "__main__":
    sys.exit(main())
