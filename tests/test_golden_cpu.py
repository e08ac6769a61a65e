"""The CPU oracle against the committed golden fixtures (tests/golden/, produced by the
reference's own code through tests/golden/make_golden.py).  Runs without the reference."""
import os

import numpy as np

from oracle import paged_oracle as po
from test_oracle_cpu import replay_allocator_script

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def test_fp16_to_float_all_halves_bit_exact():
    g = np.load(os.path.join(GOLDEN, "fp16_golden.npz"))
    halves = np.arange(65536, dtype=np.uint32).astype(np.uint16)
    got = po.fp16_to_float(halves).view(np.uint32)
    want = g["half_to_float_bits"]
    nan = (halves & 0x7FFF) > 0x7C00
    assert np.array_equal(got[~nan], want[~nan])
    assert np.all(np.isnan(got[nan].view(np.float32))) and np.all(np.isnan(want[nan].view(np.float32)))


def test_float_to_fp16_reference_rounding_bit_exact():
    g = np.load(os.path.join(GOLDEN, "fp16_golden.npz"))
    x = g["float_in_bits"].view(np.float32)
    assert np.array_equal(po.float_to_fp16_ref(x), g["float_to_half"])


def load_attention_cases():
    g = np.load(os.path.join(GOLDEN, "attention_golden.npz"))
    i = 0
    while f"shape{i}" in g:
        H, Hkv, D, S, P = (int(v) for v in g[f"shape{i}"])
        yield dict(H=H, Hkv=Hkv, D=D, S=S, P=P, q=g[f"q{i}"], k=g[f"k{i}"], v=g[f"v{i}"],
                   pt=g[f"pt{i}"], o=g[f"o_bits{i}"].view(np.float32).reshape(H, D))
        i += 1


def test_executor_path_bit_exact_with_golden_attention():
    n = 0
    for c in load_attention_cases():
        got = po.paged_attention_executor(c["q"], c["k"], c["v"], c["pt"], [0, c["pt"].size], [c["S"]],
                                          [c["S"] - 1], 1, c["H"], c["Hkv"], c["D"], c["P"], True)[0]
        assert np.array_equal(got.view(np.uint32), c["o"].view(np.uint32)), c["S"]
        flash = po.paged_attention_flashref(c["q"], c["k"], c["v"], c["pt"], [0, c["pt"].size], [c["S"]],
                                            [c["S"] - 1], 1, c["H"], c["Hkv"], c["D"], c["P"], True)[0]
        assert np.max(np.abs(flash - c["o"])) < 2e-6
        n += 1
    assert n >= 5


def test_allocator_replies_match_golden_transcript():
    script, want = [], []
    with open(os.path.join(GOLDEN, "allocator_golden.txt")) as fh:
        for line in fh:
            cmd, rep = line.rstrip("\n").split(" => ")
            script.append(cmd)
            want.append(rep)
    assert len(script) > 300
    assert replay_allocator_script(script) == want


def test_quantised_rows_bit_exact_with_golden():
    """Q4_0 / Q6_K quantise, dequantise and dot products as the reference's quantization.cpp
    produced them."""
    g = np.load(os.path.join(GOLDEN, "quant_rope_golden.npz"))
    for tag in "abc":
        w, x = g[f"w_{tag}"], g[f"x_{tag}"]
        cols = w.shape[1]
        assert np.array_equal(po.quantize_q4_0(w), g[f"q4_{tag}"])
        assert np.array_equal(po.quantize_q6_k(w), g[f"q6_{tag}"])
        assert np.array_equal(po.dequantize_q6_k(g[f"q6_{tag}"], cols).view(np.uint32), g[f"deq6_bits_{tag}"])
        got4 = po.matmul_q4_0_batched(g[f"q4_{tag}"], x, 3, 4, cols, n_threads=1)
        got6 = po.matmul_q6_k_batched(g[f"q6_{tag}"], x, 3, 4, cols, n_threads=1)
        assert np.array_equal(got4.view(np.uint32), g[f"dot4_bits_{tag}"])
        assert np.array_equal(got6.view(np.uint32), g[f"dot6_bits_{tag}"])


def test_rope_bit_exact_with_golden():
    """computeRotaryCoefficients and applyRotaryEmbedding outputs of the reference."""
    g = np.load(os.path.join(GOLDEN, "quant_rope_golden.npz"))
    for i, (pos, head_dim, rot, base, scale) in enumerate(g["rope_cases"]):
        pos, head_dim, rot = int(pos), int(head_dim), int(rot)
        cos, sin = po.rotary_coefficients(pos, rot, float(base), float(scale))
        assert np.array_equal(cos.view(np.uint32), g[f"rope_cos_bits_{i}"])
        assert np.array_equal(sin.view(np.uint32), g[f"rope_sin_bits_{i}"])
        # one request, one head: the fused-row layout of the operator is [q | k | v], q only here
        vec = g[f"rope_in_{i}"]
        qkv = np.concatenate([vec, np.zeros(2 * head_dim, np.float32)])[None, :]
        res = po.qkv_split_rope_cast(qkv, cos[None, :], sin[None, :], 1, 1, 1, head_dim, 3 * head_dim,
                                     head_dim, head_dim, head_dim, rot)
        assert res is not None
        assert np.array_equal(res[0][0].view(np.uint32), g[f"rope_out_bits_{i}"])
