"""Writes the golden fixtures of this directory from the reference's own code.

Needs oracle/_ref (the reference's attention_cpu.cpp / paged_kv.cpp / float_convert.hpp compiled
in place by `make -C oracle _ref`), i.e. a machine that has the reference checkout.  The fixtures
are plain data -- inputs and the outputs the reference code produced for them -- so the tests
that read them run anywhere:

  fp16_golden.npz        fp16ToFloat over all 65536 halves; floatToFp16 over a fixed set of
                         floats (ties, subnormals, overflow, NaN, random)
                         -- compiler/runtime/float_convert.hpp
  attention_golden.npz   RunAttentionCPU outputs (compiler/runtime/attention_cpu.cpp:272-478) for
                         small GQA decode cases, stored with their paged inputs
  allocator_golden.txt   a PagePool / RequestKVState script and the replies of
                         compiler/runtime/paged_kv.cpp, one "command => reply" per line
  quant_rope_golden.npz  quantizeRowQ4_0 / dotProductRowQ4_0, quantizeRowQ6_K / dequantizeRowQ6_K /
                         dotProductRowQ6_K (compiler/runtime/quantization.cpp:235-311, 1469-1663)
                         and computeRotaryCoefficients / applyRotaryEmbedding (:772-823) on seeded
                         rows, stored with their inputs

Run:  python tests/golden/make_golden.py
"""
import os
import subprocess
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

from oracle import paged_oracle as po  # noqa: E402

ATTENTION_CASES = [  # (H, Hkv, D, S, P, seed)
    (8, 2, 64, 130, 64, 1),
    (8, 8, 32, 65, 32, 2),
    (8, 2, 128, 70, 64, 3),
    (4, 1, 16, 1, 8, 4),
    (32, 4, 64, 200, 64, 5),
]


def float_inputs() -> np.ndarray:
    rng = np.random.default_rng(2024)
    halves = np.arange(0, 0x7C00, 37, dtype=np.uint16)            # finite halves ...
    lo = halves.view(np.float16).astype(np.float32)
    hi = (halves + 1).astype(np.uint16).view(np.float16).astype(np.float32)
    ties = (lo.astype(np.float64) + hi.astype(np.float64)) / 2     # ... and the exact midpoints
    special = np.array([0.0, -0.0, 65504.0, 65519.99, 65520.0, 65536.0, 1e9, -1e9, np.inf, -np.inf,
                        np.nan, 2.0 ** -24, 2.0 ** -25, 2.0 ** -26, 1.5 * 2.0 ** -25, 5.96e-8,
                        6.1e-5, 6.103515625e-05, 1e-10, -1e-10], np.float32)
    rnd = np.concatenate([rng.standard_normal(2000), rng.standard_normal(500) * 1e-6,
                          rng.standard_normal(500) * 3e4]).astype(np.float32)
    bits = rng.integers(0, 2 ** 32, 2000, dtype=np.uint64).astype(np.uint32).view(np.float32)
    x = np.concatenate([lo, ties.astype(np.float32), np.nextafter(ties.astype(np.float32), np.float32(0)),
                        -ties.astype(np.float32), special, rnd, bits])
    return np.ascontiguousarray(x, np.float32)


def main() -> int:
    if po.ref_lib() is None:
        print("oracle/_ref is not built: run `make -C oracle _ref` on a machine with the reference",
              file=sys.stderr)
        return 1
    # ---- fp16
    all_halves = np.arange(65536, dtype=np.uint32).astype(np.uint16)
    f = float_inputs()
    np.savez_compressed(os.path.join(HERE, "fp16_golden.npz"),
                        half_to_float_bits=po.ref_fp16_to_float(all_halves).view(np.uint32),
                        float_in_bits=f.view(np.uint32),
                        float_to_half=po.ref_float_to_fp16(f))
    # ---- attention
    out = {}
    for i, (H, Hkv, D, S, P, seed) in enumerate(ATTENTION_CASES):
        rng = np.random.default_rng(seed)
        n_tab = (S + P - 1) // P
        pages = n_tab + 2
        K = rng.standard_normal(pages * P * Hkv * D).astype(np.float16).view(np.uint16)
        V = rng.standard_normal(pages * P * Hkv * D).astype(np.float16).view(np.uint16)
        pt = rng.permutation(pages)[:n_tab].astype(np.uint32)
        q = rng.standard_normal(H * D).astype(np.float32)
        kc = np.zeros((Hkv, S, D), np.uint16)
        vc = np.zeros((Hkv, S, D), np.uint16)
        assert po.gather_kv_pages(K, pt, P, Hkv, D, S, kc, 2)
        assert po.gather_kv_pages(V, pt, P, Hkv, D, S, vc, 2)
        ref = po.ref_run_attention_cpu(q, kc, vc, H, Hkv, D, S, S - 1,
                                       po.fp16_to_float(kc[:, S - 1, :]),
                                       po.fp16_to_float(vc[:, S - 1, :]))
        assert ref is not None
        out[f"shape{i}"] = np.array([H, Hkv, D, S, P], np.int64)
        out[f"q{i}"], out[f"k{i}"], out[f"v{i}"], out[f"pt{i}"] = q, K, V, pt
        out[f"o_bits{i}"] = ref.view(np.uint32)
    np.savez_compressed(os.path.join(HERE, "attention_golden.npz"), **out)
    # ---- allocator
    rng = np.random.default_rng(99)
    script = ["pool 24", "req 4"]
    for _ in range(400):
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
    replies = subprocess.run([po.REF_ALLOC_DRIVER], input="\n".join(script) + "\n", text=True,
                             capture_output=True, check=True).stdout.split("\n")
    with open(os.path.join(HERE, "allocator_golden.txt"), "w") as fh:
        for cmd, rep in zip(script, replies):
            fh.write(f"{cmd} => {rep}\n")
    # ---- quantised rows and RoPE
    R = po.ref_lib()
    rng = np.random.default_rng(4242)
    out = {}
    for tag, cols in (("a", 64), ("b", 320), ("c", 2048)):       # 320: partial last Q6_K block
        w = (rng.standard_normal((4, cols)) * rng.uniform(0.01, 3)).astype(np.float32)
        x = rng.standard_normal((3, cols)).astype(np.float32)
        q4 = np.zeros((4, po.q4_0_row_bytes(cols)), np.uint8)
        q6 = np.zeros((4, po.q6_k_row_bytes(cols)), np.uint8)
        deq6 = np.zeros((4, cols), np.float32)
        dot4 = np.zeros((3, 4), np.float32)
        dot6 = np.zeros((3, 4), np.float32)
        for r in range(4):
            assert R.ref_quantize_row_q4_0(w[r].ctypes.data_as(po._f32p), cols, q4[r].ctypes.data, q4.shape[1]) == q4.shape[1]
            assert R.ref_quantize_row_q6_k(w[r].ctypes.data_as(po._f32p), cols, q6[r].ctypes.data, q6.shape[1]) == q6.shape[1]
            R.ref_dequantize_row_q6_k(q6[r].ctypes.data, cols, deq6[r].ctypes.data_as(po._f32p))
            for b in range(3):
                dot4[b, r] = R.ref_dot_q4_0(q4[r].ctypes.data, cols, x[b].ctypes.data_as(po._f32p))
                dot6[b, r] = R.ref_dot_q6_k(q6[r].ctypes.data, cols, x[b].ctypes.data_as(po._f32p))
        out.update({f"w_{tag}": w, f"x_{tag}": x, f"q4_{tag}": q4, f"q6_{tag}": q6,
                    f"deq6_bits_{tag}": deq6.view(np.uint32), f"dot4_bits_{tag}": dot4.view(np.uint32),
                    f"dot6_bits_{tag}": dot6.view(np.uint32)})
    rope = []
    for i, (pos, head_dim, rot, base, scale) in enumerate([(0, 64, 64, 10000.0, 1.0), (1, 64, 64, 10000.0, 1.0),
                                                           (1234, 128, 128, 500000.0, 1.0), (77, 64, 32, 10000.0, 0.5),
                                                           (4095, 20, 8, 10000.0, 1.0)]):
        cos, sin = po.ref_rotary_coefficients(pos, rot, base, scale)
        vec = rng.standard_normal(head_dim).astype(np.float32)
        out[f"rope_in_{i}"] = vec
        out[f"rope_cos_bits_{i}"], out[f"rope_sin_bits_{i}"] = cos.view(np.uint32), sin.view(np.uint32)
        out[f"rope_out_bits_{i}"] = po.ref_apply_rotary(vec, cos, sin, head_dim, rot).view(np.uint32)
        rope.append([pos, head_dim, rot, base, scale])
    out["rope_cases"] = np.array(rope, np.float64)
    np.savez_compressed(os.path.join(HERE, "quant_rope_golden.npz"), **out)
    print("wrote fp16_golden.npz, attention_golden.npz, allocator_golden.txt, quant_rope_golden.npz")
    return 0


if __name__ == "__main__":
    sys.exit(main())
