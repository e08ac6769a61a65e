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
