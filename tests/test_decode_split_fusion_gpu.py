"""The decode attention and the matmul after it: a decode call of an open pass that is followed by
the Q4_0 matmul that reads its output (the out-projection, compiler/runtime/batched_walker.cpp:
333-345) also writes that output as the matmul's split-fp16 activations, one power-of-two scale per
(request, block of 32 columns), and the split kernel is not launched.  The attention's output must
agree with the call launched on its own to the last bit or two and with the oracle like it; the
matmul's agrees with the oracle's matmul of the GPU's own attention output like any other Q4_0
matmul."""
import numpy as np
import pytest

from oracle import paged_oracle as po
from paged_cases import DeviceCase, assert_parity, make_case, oracle_decode

pytestmark = pytest.mark.gpu


def _run(exe, case, w, rows_out, form, fuse, options=()):
    """form: 'proj' (attention, then the matmul that reads its output), 'alone' (attention, then the
    pass ends), 'other' (attention, then a matmul that reads another buffer), 'twice' (two attention
    calls into the same buffer, then the matmul), 'download' (attention, then its output is read back
    while the pass is still open, then the matmul)."""
    B, cols = case.batch, case.num_heads * case.head_dim
    dev = DeviceCase(exe, case)
    other = np.random.default_rng(3).standard_normal((B, cols)).astype(np.float32)
    d_other = exe.allocateScratchBuffer(other.nbytes)
    d_out = exe.allocateScratchBuffer(B * rows_out * 4)
    assert exe.uploadToBuffer(d_other, other)
    assert exe.setOption("fuse_row_ops", fuse)
    for name, value in options:
        assert exe.setOption(name, value)
    before = exe.fusedDecodeSplitLaunches()
    args = (dev.q_buf, dev.k_buf, dev.v_buf, dev.o_buf, case.page_tables_flat, case.page_table_offsets, case.seq_lens,
            case.q_positions, B, case.num_heads, case.kv_heads, case.head_dim, case.page_size, case.apply_causal)
    try:
        assert exe.beginForwardPassCB()
        assert exe.encodePagedFlashAttention(*args), exe.lastError()
        if form == "twice":
            assert exe.encodePagedFlashAttention(*args), exe.lastError()
        if form == "download":
            early = np.empty(case.q.shape, np.float32)
            assert exe.downloadFromBuffer(dev.o_buf, early)      # no flush in between
            assert not np.isnan(early).any()
        if form != "alone":
            assert exe.encodeMatMulQ4_0Batched(f"{case.name}.proj", w, d_other if form == "other" else dev.o_buf, B, rows_out,
                                               cols, po.q4_0_row_bytes(cols), 1, d_out), exe.lastError()
        assert exe.flushForwardPassCB(), exe.lastError()
        o = np.empty(case.q.shape, np.float32)
        out = np.empty((B, rows_out), np.float32)
        assert exe.downloadFromBuffer(dev.o_buf, o) and exe.downloadFromBuffer(d_out, out)
        kernel = exe.lastDecodeKernel()
    finally:
        exe.setOption("fuse_row_ops", 1)
        for name, _ in options:
            exe.setOption(name, {"decode_mfma": 1}.get(name, 0))
        dev.free()
        exe.releaseScratchBuffer(d_other)
        exe.releaseScratchBuffer(d_out)
    return o, out, other, exe.fusedDecodeSplitLaunches() - before, kernel


def _lens(rng, B, kind):
    if kind == "ragged":
        lens = rng.integers(1, 700, B)
        lens[rng.random(B) < 0.2] = 0          # requests without visible tokens: rows of zeros
        lens[0] = 0
        return lens
    return rng.integers(900, 1400, B)


SHAPES = {
    "tinyllama": dict(B=32, H=32, Hkv=4, D=64, P=64, rows_out=2048, kind="long"),
    "ragged_two_batch_tiles": dict(B=37, H=16, Hkv=4, D=64, P=64, rows_out=192, kind="ragged"),
    "head_dim_128": dict(B=9, H=16, Hkv=2, D=128, P=32, rows_out=128, kind="ragged"),
    "gqa_16": dict(B=5, H=32, Hkv=2, D=64, P=64, rows_out=64, kind="ragged"),
    "one_wave_groups": dict(B=6, H=4, Hkv=4, D=64, P=64, rows_out=64, kind="ragged"),
    "two_wave_groups_128": dict(B=33, H=4, Hkv=2, D=128, P=32, rows_out=64, kind="ragged"),
}


@pytest.mark.parametrize("form", ["proj", "alone", "other", "twice", "download"])
@pytest.mark.parametrize("shape", list(SHAPES), ids=list(SHAPES))
def test_attention_writes_the_next_matmuls_activations(exe, shape, form):
    kw = SHAPES[shape]
    rng = np.random.default_rng(len(shape) * 131 + len(form))
    B, H, D = kw["B"], kw["H"], kw["D"]
    case = make_case(f"split.{shape}.{form}", B, H, kw["Hkv"], D, kw["P"], _lens(rng, B, kw["kind"]), seed=7)
    w = po.quantize_q4_0((rng.standard_normal((kw["rows_out"], H * D)) * 0.05).astype(np.float32))
    print(f"[case] {shape} {form} B={B} H={H}/{kw['Hkv']} D={D} rows_out={kw['rows_out']}", flush=True)
    o_plain, out_plain, other, n_plain, _ = _run(exe, case, w, kw["rows_out"], form, fuse=0)
    o_fused, out_fused, _, n_fused, kernel = _run(exe, case, w, kw["rows_out"], form, fuse=1)
    assert kernel.startswith("stream<")
    assert n_plain == 0 and n_fused == (1 if form in ("proj", "twice") else 0)
    # (two builds of the kernel: the compiler may contract a multiply and an add in one and not in
    # the other, so the last bit can differ)
    err = float(np.abs(o_plain - o_fused).max() / max(float(np.abs(o_plain).max()), 1e-30))
    print(f"[case] attention output, fused against plain: {err:.2e} of the largest value", flush=True)
    assert err <= 5e-7
    assert_parity(o_fused, oracle_decode(case), D, case.name)
    if form != "alone":
        src = other if form == "other" else o_fused.reshape(B, H * D)
        want = po.matmul_q4_0_batched(w, src, B, kw["rows_out"], H * D)
        scale = np.maximum(np.abs(want).max(axis=1, keepdims=True), 1e-30)
        for got in (out_plain, out_fused):
            assert (np.abs(got - want) <= 2e-5 * scale).all()
        if form == "other":
            assert np.array_equal(out_plain, out_fused)


def test_vector_pipe_attention_splits_as_well(exe):
    rng = np.random.default_rng(5)
    case = make_case("split.vector", 12, 32, 4, 64, 64, _lens(rng, 12, "ragged"), seed=9)
    w = po.quantize_q4_0((rng.standard_normal((256, 2048)) * 0.05).astype(np.float32))
    o, out, _, n, kernel = _run(exe, case, w, 256, "proj", fuse=1, options=(("decode_mfma", 0),))
    assert n == 1 and "mfma" not in kernel
    assert_parity(o, oracle_decode(case), 64, case.name)
    want = po.matmul_q4_0_batched(w, o.reshape(12, 2048), 12, 256, 2048)
    scale = np.maximum(np.abs(want).max(axis=1, keepdims=True), 1e-30)
    assert (np.abs(out - want) <= 2e-5 * scale).all()


def test_outputs_of_very_different_size_per_block(exe):
    """V rows whose magnitude differs by 2^20 between KV heads and by 2^6 inside a head: the
    per-block scales of one request differ widely, and every block keeps its own accuracy."""
    rng = np.random.default_rng(17)
    B, H, Hkv, D, P = 8, 16, 4, 64, 64
    case = make_case("split.spread", B, H, Hkv, D, P, rng.integers(100, 400, B), seed=3)
    v = case.v_pages.view(np.float16).reshape(-1, Hkv, D).astype(np.float32)
    v *= np.exp2(np.array([-10.0, 0.0, 5.0, 10.0], np.float32))[None, :, None]
    v[:, :, 32:] *= 1.0 / 64.0
    case.v_pages[:] = v.astype(np.float16).view(np.uint16).reshape(case.v_pages.shape)
    # one output row per block of 32 columns, reading only that block: its result is measured
    # against that block's own size
    nblk = H * D // 32
    wf = np.zeros((64, H * D), np.float32)
    for r in range(64):
        blk = r % nblk
        wf[r, blk * 32:(blk + 1) * 32] = rng.standard_normal(32)
    w = po.quantize_q4_0(wf)
    o, out, _, n, _ = _run(exe, case, w, 64, "proj", fuse=1)
    assert n == 1
    want = po.matmul_q4_0_batched(w, o.reshape(B, H * D), B, 64, H * D)
    blk_max = np.abs(o.reshape(B, nblk, 32)).max(axis=2)                       # [B][nblk]
    # 32 terms with |w| < 4 and a split good to 2^-22 of the block's largest value: 6e-6 expected
    assert (np.abs(out - want) <= 1e-4 * blk_max[:, np.arange(64) % nblk] + 1e-30).all()
