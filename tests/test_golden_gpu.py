"""The HIP decode path against the committed golden outputs of the reference's own
RunAttentionCPU (tests/golden/attention_golden.npz) -- no oracle in between.  Tolerance as
for every attention parity test: per-head cosine >= 0.9999, max-abs <= 2e-3."""
import numpy as np
import pytest

from paged_cases import DecodeCase, DeviceCase, assert_parity
from test_golden_cpu import load_attention_cases

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("c", list(load_attention_cases()), ids=lambda c: f"H{c['H']}kv{c['Hkv']}D{c['D']}S{c['S']}")
@pytest.mark.parametrize("generic", [0, 1], ids=["fast", "generic"])
def test_decode_matches_golden_reference_outputs(exe, c, generic):
    P, S = c["P"], c["S"]
    pool_pages = c["k"].size // (P * c["Hkv"] * c["D"])
    case = DecodeCase(name="golden", batch=1, num_heads=c["H"], kv_heads=c["Hkv"], head_dim=c["D"],
                      page_size=P, capacity_pages=pool_pages,
                      seq_lens=np.array([S], np.uint32), q_positions=np.array([S - 1], np.uint32),
                      page_tables_flat=c["pt"].astype(np.uint32),
                      page_table_offsets=np.array([0, c["pt"].size], np.uint32), apply_causal=True,
                      q=c["q"].reshape(1, c["H"], c["D"]), k_pages=c["k"], v_pages=c["v"])
    print(f"[golden] H={c['H']}/{c['Hkv']} D={c['D']} S={S} P={P} generic={generic}", flush=True)
    assert exe.setOption("decode_force_generic", generic)
    dev = DeviceCase(exe, case)
    try:
        got = dev.run(sync=True)
    finally:
        dev.free()
        exe.setOption("decode_force_generic", 0)
    assert_parity(got.reshape(1, c["H"], c["D"]), c["o"].reshape(1, c["H"], c["D"]), c["D"], "golden")
