"""The HIP decode path against the committed golden outputs of the reference's own
RunAttentionCPU (tests/golden/attention_golden.npz) -- no oracle in between.  Tolerance as
for every attention parity test: per-head cosine >= 0.9999, max-abs <= 2e-3."""
import numpy as np
import pytest

from paged_cases import DecodeCase, DeviceCase, assert_parity
from test_golden_cpu import load_attention_cases

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("c", list(load_attention_cases()), ids=lambda c: f"H{c['H']}kv{c['Hkv']}D{c['D']}S{c['S']}")
@pytest.mark.parametrize("kernel", ["balanced", "generic"])
def test_decode_matches_golden_reference_outputs(exe, c, kernel):
    generic = 1 if kernel == "generic" else 0
    P, S = c["P"], c["S"]
    pool_pages = c["k"].size // (P * c["Hkv"] * c["D"])
    case = DecodeCase(name="golden", batch=1, num_heads=c["H"], kv_heads=c["Hkv"], head_dim=c["D"],
                      page_size=P, capacity_pages=pool_pages,
                      seq_lens=np.array([S], np.uint32), q_positions=np.array([S - 1], np.uint32),
                      page_tables_flat=c["pt"].astype(np.uint32),
                      page_table_offsets=np.array([0, c["pt"].size], np.uint32), apply_causal=True,
                      q=c["q"].reshape(1, c["H"], c["D"]), k_pages=c["k"], v_pages=c["v"])
    print(f"[golden] H={c['H']}/{c['Hkv']} D={c['D']} S={S} P={P} kernel={kernel}", flush=True)
    assert exe.setOption("decode_force_generic", generic)
    dev = DeviceCase(exe, case)
    try:
        got = dev.run(sync=True)
    finally:
        dev.free()
        exe.setOption("decode_force_generic", 0)
    assert_parity(got.reshape(1, c["H"], c["D"]), c["o"].reshape(1, c["H"], c["D"]), c["D"], "golden")


def _golden_quant():
    import os
    from test_golden_cpu import GOLDEN
    return np.load(os.path.join(GOLDEN, "quant_rope_golden.npz"))


@pytest.mark.parametrize("tag", ["a", "b", "c"])
def test_quantised_matmuls_match_golden_reference_dots(exe, tag):
    """Q4_0 and Q6_K matmuls on the weights the reference quantised, against the dot products the
    reference computed (dotProductRowQ4_0 / dotProductRowQ6_K): within 2e-5 of sum |w x| (the
    reference's own fp32 loop is that far from the exact value, see the matmul tests)."""
    g = _golden_quant()
    x = g[f"x_{tag}"]
    cols = x.shape[1]
    w = g[f"w_{tag}"].astype(np.float64)
    scale = np.abs(x.astype(np.float64)) @ np.abs(w).T + 1e-30
    d_in, d_out = exe.allocateScratchBuffer(x.nbytes), exe.allocateScratchBuffer(3 * 4 * 4)
    try:
        assert exe.uploadToBuffer(d_in, x)
        got = np.empty((3, 4), np.float32)
        q4 = np.ascontiguousarray(g[f"q4_{tag}"])
        assert exe.encodeMatMulQ4_0Batched(f"golden.q4.{tag}", q4, d_in, 3, 4, cols, q4.shape[1], 1, d_out, sync=True)
        assert exe.downloadFromBuffer(d_out, got)
        assert np.max(np.abs(got - g[f"dot4_bits_{tag}"].view(np.float32)) / scale) < 2e-5
        q6 = np.ascontiguousarray(g[f"q6_{tag}"])
        assert exe.encodeMatMulQ6KBatched(f"golden.q6.{tag}", q6, d_in, 3, 4, cols, q6.shape[1], d_out, sync=True)
        assert exe.downloadFromBuffer(d_out, got)
        assert np.max(np.abs(got - g[f"dot6_bits_{tag}"].view(np.float32)) / scale) < 2e-5
    finally:
        exe.releaseScratchBuffer(d_in)
        exe.releaseScratchBuffer(d_out)


def test_rope_matches_golden_reference_rotations_bit_exact(exe):
    """encodeQkvSplitRopeCast on the vectors the reference rotated (applyRotaryEmbedding)."""
    g = _golden_quant()
    for i, (pos, head_dim, rot, base, scale) in enumerate(g["rope_cases"]):
        head_dim, rot = int(head_dim), int(rot)
        cos = g[f"rope_cos_bits_{i}"].view(np.float32)
        sin = g[f"rope_sin_bits_{i}"].view(np.float32)
        qkv = np.concatenate([g[f"rope_in_{i}"], np.zeros(2 * head_dim, np.float32)])
        bufs = [exe.allocateScratchBuffer(n) for n in (qkv.nbytes, head_dim * 4, head_dim * 4, head_dim * 4,
                                                       head_dim * 2, head_dim * 2, max(cos.nbytes, 16), max(sin.nbytes, 16))]
        try:
            assert exe.uploadToBuffer(bufs[0], qkv)
            if cos.size:
                assert exe.uploadToBuffer(bufs[6], cos) and exe.uploadToBuffer(bufs[7], sin)
            assert exe.encodeQkvSplitRopeCast(bufs[0], bufs[1], bufs[2], bufs[3], bufs[4], bufs[5], bufs[6], bufs[7],
                                              1, 1, 1, head_dim, 3 * head_dim, head_dim, head_dim, head_dim, rot,
                                              sync=True), exe.lastError()
            got = np.empty(head_dim, np.float32)
            assert exe.downloadFromBuffer(bufs[1], got)
        finally:
            for b in bufs:
                exe.releaseScratchBuffer(b)
        assert np.array_equal(got.view(np.uint32), g[f"rope_out_bits_{i}"]), i
