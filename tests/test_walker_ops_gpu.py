"""The small per-layer operators of the batched decode step (RMSNorm, add, SiLU*up, gate/up
split) against the CPU oracle through the C ABI.  add and the split copies are bit-exact; the
others agree with the CPU formulas to a few units in the last place (tolerances below: the GPU
sums squares in a tree, and its expf / division differ from glibc's by at most a few ulp)."""
import numpy as np
import pytest

from oracle import paged_oracle as po

pytestmark = pytest.mark.gpu


def _up(exe, arr):
    arr = np.ascontiguousarray(arr)
    buf = exe.allocateScratchBuffer(max(arr.nbytes, 16))
    assert buf and exe.uploadToBuffer(buf, arr)
    return buf


def _down(exe, buf, shape, dtype=np.float32):
    out = np.empty(shape, dtype)
    assert exe.downloadFromBuffer(buf, out)
    return out


@pytest.mark.parametrize("batch,length", [(4, 2048), (64, 2048), (32, 4096), (3, 100), (1, 7)])
@pytest.mark.parametrize("sync", [True, False])
def test_rms_norm_batched(exe, batch, length, sync):
    print(f"[rmsnorm] batch={batch} length={length} sync={sync}", flush=True)
    rng = np.random.default_rng(batch * 31 + length)
    x = (rng.uniform(-1, 1, (batch, length)) * rng.uniform(0.1, 30, (batch, 1))).astype(np.float32)
    w = rng.uniform(-1, 1, length).astype(np.float32)
    want = po.rms_norm_batched(x, w, 1e-5, batch, length)
    d_in, d_out = _up(exe, x), exe.allocateScratchBuffer(x.nbytes)
    try:
        if not sync:
            assert exe.beginForwardPassCB()
        assert exe.encodeRmsNormBatched(d_in, w, 1e-5, batch, length, d_out, sync=sync), exe.lastError()
        if not sync:
            assert exe.flushForwardPassCB()
        got = _down(exe, d_out, x.shape)
    finally:
        exe.releaseScratchBuffer(d_in)
        exe.releaseScratchBuffer(d_out)
    # the reference's own gate between its kernel and a CPU formula is 1e-4 absolute
    # (tests/test_batched_elementwise.cpp:77); here: 4 ulp-ish relative
    assert np.max(np.abs(got - want) / (np.abs(want) + 1e-6)) < 5e-6


def test_rms_norm_short_weight_counts_as_one(exe):
    x = np.linspace(-2, 2, 2 * 64, dtype=np.float32).reshape(2, 64)
    w = np.full(10, 0.5, np.float32)
    want = po.rms_norm_batched(x, w, 1e-5, 2, 64)
    d_in, d_out = _up(exe, x), exe.allocateScratchBuffer(x.nbytes)
    try:
        assert exe.encodeRmsNormBatched(d_in, w, 1e-5, 2, 64, d_out, sync=True)
        got = _down(exe, d_out, x.shape)
    finally:
        exe.releaseScratchBuffer(d_in)
        exe.releaseScratchBuffer(d_out)
    assert np.allclose(got, want, rtol=5e-6, atol=1e-7)


@pytest.mark.parametrize("n", [1, 255, 64 * 2048, 64 * 5632])
def test_add_batched_bit_exact(exe, n):
    rng = np.random.default_rng(n)
    a, b = rng.standard_normal(n).astype(np.float32), rng.standard_normal(n).astype(np.float32)
    d_a, d_b, d_o = _up(exe, a), _up(exe, b), exe.allocateScratchBuffer(n * 4)
    try:
        assert exe.encodeAddBatched(d_a, d_b, d_o, n, sync=True), exe.lastError()
        got = _down(exe, d_o, (n,))
    finally:
        for x in (d_a, d_b, d_o):
            exe.releaseScratchBuffer(x)
    assert np.array_equal(got.view(np.uint32), po.add(a, b).view(np.uint32))


@pytest.mark.parametrize("batch,inner,pad", [(1, 5632, 0), (64, 5632, 0), (5, 100, 7)])
def test_gate_up_split_silu_mul(exe, batch, inner, pad):
    print(f"[gate_up] batch={batch} inner={inner} pad={pad}", flush=True)
    rng = np.random.default_rng(batch + inner)
    rows = 2 * inner + pad
    gu = (rng.standard_normal((batch, rows)) * 3).astype(np.float32)
    gu[0, :6] = [0.0, 30.0, -30.0, 88.0, -88.0, -104.0]          # saturation of exp(-g)
    gate, up, out = po.gate_up_split_silu_mul(gu, batch, inner, rows)
    d_gu = _up(exe, gu)
    bufs = [exe.allocateScratchBuffer(batch * inner * 4) for _ in range(4)]
    try:
        assert exe.beginForwardPassCB()
        assert exe.encodeGateUpSplitSiluMul(d_gu, bufs[0], bufs[1], bufs[2], batch, inner, rows), exe.lastError()
        assert exe.encodeSiluMulBatched(bufs[0], bufs[1], bufs[3], batch * inner), exe.lastError()
        assert exe.flushForwardPassCB()
        g_gate, g_up, g_out, g_out2 = (_down(exe, b, (batch, inner)) for b in bufs)
    finally:
        for b in (d_gu, *bufs):
            exe.releaseScratchBuffer(b)
    assert np.array_equal(g_gate, gate) and np.array_equal(g_up, up)          # copies: bit-exact
    assert np.array_equal(g_out.view(np.uint32), g_out2.view(np.uint32))      # fused == unfused
    assert np.all(np.isfinite(g_out))
    assert np.max(np.abs(g_out - out) / (np.abs(out) + 1e-30)) < 2e-6


def test_walker_ops_argument_errors(exe):
    buf = exe.allocateScratchBuffer(1024)
    try:
        assert not exe.hasForwardPassCB()
        assert not exe.encodeAddBatched(buf, buf, buf, 16) and "open forward pass" in exe.lastError()
        assert not exe.encodeAddBatched(buf, None, buf, 16, sync=True)
        assert not exe.encodeAddBatched(buf, buf, buf, 0, sync=True)
        assert not exe.encodeAddBatched(buf, buf, buf, 1024, sync=True)        # 4 KiB > 1 KiB buffer
        assert not exe.encodeRmsNormBatched(buf, np.ones(4, np.float32), 1e-5, 0, 4, buf, sync=True)
        assert not exe.encodeGateUpSplitSiluMul(buf, buf, buf, buf, 2, 8, 12, sync=True)  # 2*inner > rows
    finally:
        exe.releaseScratchBuffer(buf)


# ---- operators encoded back to back in one pass run as one fused launch: same results ---------

def _chain_case(rng, batch, hid, ffn):
    x = rng.standard_normal((batch, hid)).astype(np.float32)
    y = rng.standard_normal((batch, hid)).astype(np.float32)
    w = rng.uniform(0.5, 1.5, hid).astype(np.float32)
    gu = rng.standard_normal((batch, 2 * ffn)).astype(np.float32)
    return x, y, w, gu


@pytest.mark.parametrize("batch,hid,ffn", [(5, 2048, 5632), (33, 256, 64), (64, 4096, 1024), (2, 16384, 8)])
@pytest.mark.parametrize("fuse", [1, 0])
def test_add_then_rms_norm_in_one_pass(exe, batch, hid, ffn, fuse):
    """add -> RMSNorm (the residual add of one layer and the norm of the next), then a second,
    unrelated add: with fusion on, the first two are one launch; all three outputs are written."""
    print(f"[chain add+rms] batch={batch} hid={hid} fuse={fuse}", flush=True)
    rng = np.random.default_rng(batch + hid)
    x, y, w, _ = _chain_case(rng, batch, hid, ffn)
    r1 = po.add(x, y)
    want_n = po.rms_norm_batched(r1, w, 1e-5, batch, hid)
    bufs = [_up(exe, x), _up(exe, y)] + [exe.allocateScratchBuffer(x.nbytes) for _ in range(3)]
    d_x, d_y, d_r1, d_n, d_z = bufs
    assert exe.setOption("fuse_row_ops", fuse)
    before = exe.rowProgramLaunches()
    try:
        assert exe.beginForwardPassCB()
        assert exe.encodeAddBatched(d_x, d_y, d_r1, batch * hid)
        assert exe.encodeRmsNormBatched(d_r1, w, 1e-5, batch, hid, d_n)
        assert exe.encodeAddBatched(d_n, d_x, d_z, batch * hid)      # reads the chain's result
        assert exe.flushForwardPassCB(), exe.lastError()
        got_r1, got_n, got_z = (_down(exe, b, x.shape) for b in (d_r1, d_n, d_z))
    finally:
        exe.setOption("fuse_row_ops", 1)
        for b in bufs:
            exe.releaseScratchBuffer(b)
    assert np.array_equal(got_r1, r1)
    assert np.max(np.abs(got_n - want_n) / (np.abs(want_n) + 1e-6)) < 5e-6
    assert np.array_equal(got_z, got_n + x)
    launches = exe.rowProgramLaunches() - before
    assert launches == (1 if fuse else 0), launches


@pytest.mark.parametrize("fuse", [1, 0])
def test_in_place_add_and_download_without_flush(exe, fuse):
    """out == a (the residual stream updated in place), and the result read back while the pass
    is still open: the download has to see the pending operators' results."""
    rng = np.random.default_rng(3)
    a = rng.standard_normal((7, 512)).astype(np.float32)
    b = rng.standard_normal((7, 512)).astype(np.float32)
    d_a, d_b = _up(exe, a), _up(exe, b)
    assert exe.setOption("fuse_row_ops", fuse)
    try:
        assert exe.beginForwardPassCB()
        assert exe.encodeAddBatched(d_a, d_b, d_a, a.size)
        got = _down(exe, d_a, a.shape)            # no flush before
        assert exe.encodeAddBatched(d_a, d_b, d_a, a.size)
        assert exe.flushForwardPassCB()
        got2 = _down(exe, d_a, a.shape)
    finally:
        exe.setOption("fuse_row_ops", 1)
        exe.releaseScratchBuffer(d_a)
        exe.releaseScratchBuffer(d_b)
    assert np.array_equal(got, a + b)
    assert np.array_equal(got2, (a + b) + b)


@pytest.mark.parametrize("batch,hid,ffn,rows", [(6, 2048, 5632, 2048), (33, 256, 64, 192), (64, 1024, 512, 64)])
@pytest.mark.parametrize("fuse", [1, 0])
def test_gate_up_then_matmul_then_add_in_one_pass(exe, batch, hid, ffn, rows, fuse):
    """gate/up split + SiLU -> Q4_0 down-projection -> residual add: the fp16 split of the
    matmul's input joins the SiLU launch and (when the matmul splits K) the sum of its slices
    joins the add.  Every buffer the three operators are specified to write is checked."""
    print(f"[chain silu+matmul+add] batch={batch} ffn={ffn} rows={rows} fuse={fuse}", flush=True)
    rng = np.random.default_rng(batch * 7 + ffn)
    _, _, _, gu = _chain_case(rng, batch, hid, ffn)
    resid = rng.standard_normal((batch, rows)).astype(np.float32)
    wq = po.quantize_q4_0((rng.standard_normal((rows, ffn)) * 0.05).astype(np.float32))
    want_gate, want_up, want_mix = po.gate_up_split_silu_mul(gu, batch, ffn, 2 * ffn)
    want_down = po.matmul_q4_0_batched(wq, want_mix, batch, rows, ffn)
    want_out = po.add(resid, want_down)
    d_gu, d_res = _up(exe, gu), _up(exe, resid)
    d_gate, d_upb, d_mix = (exe.allocateScratchBuffer(batch * ffn * 4) for _ in range(3))
    d_down, d_out = (exe.allocateScratchBuffer(batch * rows * 4) for _ in range(2))
    bufs = [d_gu, d_res, d_gate, d_upb, d_mix, d_down, d_out]
    assert exe.setOption("fuse_row_ops", fuse)
    try:
        for ks in (0, 2):   # automatic, and a forced K split (the sum of the slices joins the add)
            assert exe.setOption("q4_ksplit", ks)
            assert exe.beginForwardPassCB()
            assert exe.encodeGateUpSplitSiluMul(d_gu, d_gate, d_upb, d_mix, batch, ffn, 2 * ffn)
            assert exe.encodeMatMulQ4_0Batched(f"chain.down.{rows}x{ffn}", wq, d_mix, batch, rows, ffn,
                                               wq.shape[1], 1, d_down), exe.lastError()
            assert exe.encodeAddBatched(d_res, d_down, d_out, batch * rows)
            assert exe.flushForwardPassCB(), exe.lastError()
            got_gate, got_up, got_mix = (_down(exe, b, (batch, ffn)) for b in (d_gate, d_upb, d_mix))
            got_down, got_out = (_down(exe, b, (batch, rows)) for b in (d_down, d_out))
            assert np.array_equal(got_gate, want_gate) and np.array_equal(got_up, want_up)
            assert np.max(np.abs(got_mix - want_mix) / (np.abs(want_mix) + 1e-6)) < 5e-6
            scale = float(np.max(np.abs(want_down)))
            assert np.max(np.abs(got_down - want_down)) < 2e-5 * scale
            assert np.array_equal(got_out, resid + got_down)
            assert np.max(np.abs(got_out - want_out)) < 2e-5 * max(scale, 1.0)
    finally:
        exe.setOption("fuse_row_ops", 1)
        exe.setOption("q4_ksplit", 0)
        for b in bufs:
            exe.releaseScratchBuffer(b)


def test_long_rows_between_two_matmuls(exe):
    """A matmul whose output rows are longer than the fused row kernel handles (20480 > 16384),
    split over K so that the sum of its slices is pending, feeding another matmul directly: the
    sum and the split of the second matmul's input then run as separate kernels."""
    rng = np.random.default_rng(21)
    batch, k1, mid, rows2 = 3, 1024, 20480, 64
    w1 = po.quantize_q4_0((rng.standard_normal((mid, k1)) * 0.05).astype(np.float32))
    w2 = po.quantize_q4_0((rng.standard_normal((rows2, mid)) * 0.02).astype(np.float32))
    x = rng.standard_normal((batch, k1)).astype(np.float32)
    want_mid = po.matmul_q4_0_batched(w1, x, batch, mid, k1)
    want = po.matmul_q4_0_batched(w2, want_mid, batch, rows2, mid)
    d_x, d_mid, d_out = _up(exe, x), exe.allocateScratchBuffer(batch * mid * 4), exe.allocateScratchBuffer(batch * rows2 * 4)
    try:
        assert exe.setOption("q4_ksplit", 2)
        assert exe.beginForwardPassCB()
        assert exe.encodeMatMulQ4_0Batched("long.a", w1, d_x, batch, mid, k1, w1.shape[1], 1, d_mid), exe.lastError()
        assert exe.encodeMatMulQ4_0Batched("long.b", w2, d_mid, batch, rows2, mid, w2.shape[1], 1, d_out), exe.lastError()
        assert exe.flushForwardPassCB(), exe.lastError()
        got_mid, got = _down(exe, d_mid, (batch, mid)), _down(exe, d_out, (batch, rows2))
    finally:
        exe.setOption("q4_ksplit", 0)
        for b in (d_x, d_mid, d_out):
            exe.releaseScratchBuffer(b)
    assert np.max(np.abs(got_mid - want_mid)) < 2e-5 * float(np.max(np.abs(want_mid)))
    assert np.max(np.abs(got - want)) < 1e-4 * float(np.max(np.abs(want)))
