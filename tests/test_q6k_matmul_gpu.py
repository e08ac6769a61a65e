"""Batched Q6_K matmul (the lm_head of the batched decode step) against the CPU oracle
(dotProductRowQ6_K order, bit-exact with the reference build) and against a float64 product of
the dequantised weights, through the C ABI.

Tolerances, per output element, relative to A = sum_c |w_c * x_c|: the fp32 sequential oracle is
itself within about cols * 2^-24 * A of the exact value; the matrix-core path multiplies exact
integers with activations split into fp16 pairs (relative error 2^-22 per product), scales each
group of 16 in fp32 and accumulates in fp32, so it must be within 4e-6 * A of the exact value
and within 2e-5 * A of the oracle.  The scalar kernel is held to the same bounds."""
import numpy as np
import pytest

from oracle import paged_oracle as po

pytestmark = pytest.mark.gpu


def run(exe, name, q, x, batch, rows, cols, stride, sync=True):
    d_in = exe.allocateScratchBuffer(x.nbytes)
    d_out = exe.allocateScratchBuffer(batch * rows * 4)
    assert exe.uploadToBuffer(d_in, x)
    assert exe.uploadToBuffer(d_out, np.full(batch * rows, np.nan, np.float32))
    try:
        if not sync:
            assert exe.beginForwardPassCB()
        assert exe.encodeMatMulQ6KBatched(name, q, d_in, batch, rows, cols, stride, d_out, sync=sync), exe.lastError()
        if not sync:
            assert exe.flushForwardPassCB()
        out = np.empty((batch, rows), np.float32)
        assert exe.downloadFromBuffer(d_out, out)
    finally:
        exe.releaseScratchBuffer(d_in)
        exe.releaseScratchBuffer(d_out)
    return out


def check(got, q, x, batch, rows, cols, stride):
    assert np.all(np.isfinite(got))
    w = po.dequantize_q6_k(np.ascontiguousarray(q[:, :po.q6_k_row_bytes(cols)]), cols).astype(np.float64)
    exact = x.astype(np.float64) @ w.T
    scale = np.abs(x.astype(np.float64)) @ np.abs(w).T + 1e-30
    oracle = po.matmul_q6_k_batched(q, x, batch, rows, cols, stride)
    assert oracle is not None
    err_exact = np.max(np.abs(got - exact) / scale)
    err_oracle = np.max(np.abs(got - oracle) / scale)
    print(f"  max |got-exact|/A = {err_exact:.2e}, |got-oracle|/A = {err_oracle:.2e}, "
          f"|oracle-exact|/A = {np.max(np.abs(oracle - exact) / scale):.2e}", flush=True)
    assert err_exact < 4e-6 and err_oracle < 2e-5


def make(rows, cols, batch, seed, pad=0, x_scale=1.0):
    rng = np.random.default_rng(seed)
    w = (rng.standard_normal((rows, cols)) * 0.05 * rng.uniform(0.2, 3.0, (rows, 1))).astype(np.float32)
    q = po.quantize_q6_k(w)
    if pad:
        q = np.concatenate([q, rng.integers(0, 256, (rows, pad), dtype=np.uint8)], axis=1)
    x = (rng.standard_normal((batch, cols)) * x_scale).astype(np.float32)
    return np.ascontiguousarray(q), x, q.shape[1]


MFMA_SHAPES = [  # rows, cols, batch: a slice of the TinyLlama lm_head (32000 x 2048), odd sizes
    (4096, 2048, 32), (2048, 2048, 64), (32, 256, 1), (96, 512, 33), (16384, 256, 5), (64, 4096, 100),
]


@pytest.mark.parametrize("rows,cols,batch", MFMA_SHAPES)
def test_q6k_matmul_mfma_path(exe, rows, cols, batch):
    print(f"[q6k mfma] rows={rows} cols={cols} batch={batch}", flush=True)
    q, x, stride = make(rows, cols, batch, rows + cols + batch)
    got = run(exe, f"q6k.{rows}x{cols}", q, x, batch, rows, cols, stride)
    check(got, q, x, batch, rows, cols, stride)


@pytest.mark.parametrize("x_scale", [1e-20, 1e-3, 1e4, 1e18])
def test_q6k_matmul_activation_ranges(exe, x_scale):
    """the per-request power-of-two scale keeps the fp16 split exact-ish over the fp32 range"""
    rows, cols, batch = 64, 512, 9
    q, x, stride = make(rows, cols, batch, 5, x_scale=x_scale)
    x[3] *= 1e-3  # requests with very different magnitudes in one batch
    x[4] = 0.0
    got = run(exe, "q6k.ranges", q, x, batch, rows, cols, stride)
    check(got, q, x, batch, rows, cols, stride)
    assert np.all(got[4] == 0.0)


@pytest.mark.parametrize("rows,cols,batch,pad", [(68, 320, 3, 0), (4, 64, 1, 0), (100, 700, 5, 0),
                                                 (64, 2048, 4, 6), (256, 256, 9, 2)])
def test_q6k_matmul_scalar_path(exe, rows, cols, batch, pad):
    """shapes the matrix-core kernel does not take (rows % 32, a partial last block), and row
    strides with padding; (64, 2048, pad 6) and (256, 256, pad 2) take the matrix-core path with
    a padded stride"""
    print(f"[q6k scalar] rows={rows} cols={cols} batch={batch} pad={pad}", flush=True)
    q, x, stride = make(rows, cols, batch, rows * 3 + cols, pad=pad)
    got = run(exe, f"q6k.s.{rows}x{cols}.{pad}", q, x, batch, rows, cols, stride)
    check(got, q, x, batch, rows, cols, stride)
    assert exe.setOption("q4_force_generic", 1)
    try:
        got = run(exe, f"q6k.s.{rows}x{cols}.{pad}", q, x, batch, rows, cols, stride)
    finally:
        exe.setOption("q4_force_generic", 0)
    check(got, q, x, batch, rows, cols, stride)


def test_q6k_matmul_encode_in_pass_and_weight_cache(exe):
    rows, cols, batch = 128, 512, 6
    q, x, stride = make(rows, cols, batch, 77)
    a = run(exe, "q6k.cache", q, x, batch, rows, cols, stride, sync=True)
    b = run(exe, "q6k.cache", q, x, batch, rows, cols, stride, sync=False)   # cached weights, encode form
    assert np.array_equal(a, b)
    # the same name with other contents of another size replaces the cached matrix
    q2, x2, stride2 = make(64, 256, 2, 78)
    got = run(exe, "q6k.cache", q2, x2, 2, 64, 256, stride2)
    check(got, q2, x2, 2, 64, 256, stride2)


def test_q6k_matmul_argument_checks(exe):
    q, x, stride = make(64, 256, 2, 3)
    d_in, d_out = exe.allocateScratchBuffer(x.nbytes), exe.allocateScratchBuffer(2 * 64 * 4)
    try:
        assert not exe.encodeMatMulQ6KBatched("q6k.bad", q, d_in, 2, 64, 256, stride, d_out)          # no open pass
        assert not exe.encodeMatMulQ6KBatched("q6k.bad", q, d_in, 2, 62, 256, stride, d_out, sync=True)   # rows % 4
        assert not exe.encodeMatMulQ6KBatched("q6k.bad", q, d_in, 2, 64, 32, stride, d_out, sync=True)    # cols < 64
        assert not exe.encodeMatMulQ6KBatched("q6k.bad", q, d_in, 2, 64, 256, 100, d_out, sync=True)      # stride too small
        assert not exe.encodeMatMulQ6KBatched("q6k.bad", q[:32], d_in, 2, 64, 256, stride, d_out, sync=True)  # bytes short
        assert not exe.encodeMatMulQ6KBatched("q6k.bad", q, 0, 2, 64, 256, stride, d_out, sync=True)      # null input
    finally:
        exe.releaseScratchBuffer(d_in)
        exe.releaseScratchBuffer(d_out)


def test_final_norm_then_lm_head_in_one_pass(exe):
    """RMSNorm -> Q6_K matmul, the end of the batched step (batched_walker.cpp:415-431): the fp16
    split of the matmul's input joins the norm's launch."""
    rows, cols, batch = 1024, 2048, 17
    rng = np.random.default_rng(9)
    q, x, stride = make(rows, cols, batch, 91)
    g = rng.uniform(0.5, 1.5, cols).astype(np.float32)
    want_n = po.rms_norm_batched(x, g, 1e-5, batch, cols)
    d_x, d_n, d_o = (exe.allocateScratchBuffer(n) for n in (x.nbytes, x.nbytes, batch * rows * 4))
    before = exe.rowProgramLaunches()
    try:
        assert exe.uploadToBuffer(d_x, x)
        assert exe.beginForwardPassCB()
        assert exe.encodeRmsNormBatched(d_x, g, 1e-5, batch, cols, d_n)
        assert exe.encodeMatMulQ6KBatched("q6k.head", q, d_n, batch, rows, cols, stride, d_o), exe.lastError()
        assert exe.flushForwardPassCB()
        got_n, got = np.empty_like(x), np.empty((batch, rows), np.float32)
        assert exe.downloadFromBuffer(d_n, got_n) and exe.downloadFromBuffer(d_o, got)
    finally:
        for b in (d_x, d_n, d_o):
            exe.releaseScratchBuffer(b)
    assert exe.rowProgramLaunches() - before == 1
    assert np.max(np.abs(got_n - want_n) / (np.abs(want_n) + 1e-6)) < 5e-6
    check(got, q, got_n, batch, rows, cols, stride)
