"""Batched Q4_0 matmul (the walker's projection / FFN matmuls) against the CPU oracle
(dotProductRowQ4_0 order, bit-exact with the reference build) and against a float64 product of
the dequantised weights, through the C ABI.

Tolerances, per output element, relative to A = sum_c |w_c * x_c| (the scale of the rounding
errors of any summation): the fp32 sequential oracle itself is within about cols * 2^-24 * A of the
exact value; the MFMA path multiplies the exact integers q - 8 with activations split into fp16
pairs (relative error 2^-22 per product), accumulates in fp32 and applies the block scale in
fp32, so it must be within 4e-6 * A of the exact value and within 2e-5 * A of the oracle.  The scalar fallback kernel is held to the same bounds."""
import numpy as np
import pytest

from oracle import paged_oracle as po

pytestmark = pytest.mark.gpu


def dequant(q: np.ndarray, cols: int) -> np.ndarray:
    rows = q.shape[0]
    nb = (cols + 31) // 32
    blk = q[:, :nb * 18].reshape(rows, nb, 18)
    d = blk[:, :, :2].copy().view(np.float16).astype(np.float64)[:, :, 0]
    lo = (blk[:, :, 2:] & 0x0F).astype(np.float64) - 8
    hi = (blk[:, :, 2:] >> 4).astype(np.float64) - 8
    w = np.concatenate([lo, hi], axis=2) * d[:, :, None]
    return w.reshape(rows, nb * 32)[:, :cols]


def run(exe, name, q, x, batch, rows, cols, stride, sync=True):
    d_in = exe.allocateScratchBuffer(x.nbytes)
    d_out = exe.allocateScratchBuffer(batch * rows * 4)
    assert exe.uploadToBuffer(d_in, x)
    assert exe.uploadToBuffer(d_out, np.full(batch * rows, np.nan, np.float32))
    try:
        if not sync:
            assert exe.beginForwardPassCB()
        assert exe.encodeMatMulQ4_0Batched(name, q, d_in, batch, rows, cols, stride, 1, d_out, sync=sync), exe.lastError()
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
    w = dequant(q, cols)
    exact = x.astype(np.float64) @ w.T
    scale = np.abs(x.astype(np.float64)) @ np.abs(w).T + 1e-30
    oracle = po.matmul_q4_0_batched(q, x, batch, rows, cols, stride)
    assert oracle is not None
    err_exact = np.max(np.abs(got - exact) / scale)
    err_oracle = np.max(np.abs(got - oracle) / scale)
    print(f"  max |got-exact|/A = {err_exact:.2e}, |got-oracle|/A = {err_oracle:.2e}, "
          f"|oracle-exact|/A = {np.max(np.abs(oracle - exact) / scale):.2e}", flush=True)
    assert err_exact < 4e-6 and err_oracle < 2e-5


def make(rows, cols, batch, seed, pad=0, x_scale=1.0):
    rng = np.random.default_rng(seed)
    w = (rng.standard_normal((rows, cols)) * 0.05).astype(np.float32)
    q = po.quantize_q4_0(w)
    if pad:
        q = np.concatenate([q, rng.integers(0, 256, (rows, pad), dtype=np.uint8)], axis=1)
    x = (rng.standard_normal((batch, cols)) * x_scale).astype(np.float32)
    return np.ascontiguousarray(q), x, q.shape[1]


MFMA_SHAPES = [  # rows, cols, batch: TinyLlama qkv / out-proj / gate_up / down, odd batches, Llama-3-8B
    (2560, 2048, 32), (2048, 2048, 64), (11264, 2048, 64), (2048, 5632, 64),
    (64, 64, 1), (128, 96, 33), (256, 2048, 7), (192, 160, 100),
    (6144, 4096, 5), (4096, 14336, 3), (28672, 4096, 2),    # Llama-3-8B qkv / down / gate_up
    # one batch tile of more than 16 requests on a small grid: two workgroups per row tile, half of the
    # requests each (with K split over workgroups as well; the odd batches leave one half ragged)
    (512, 4096, 20), (1024, 512, 17), (3200, 256, 31), (4096, 2048, 32),
]


@pytest.mark.parametrize("rows,cols,batch", MFMA_SHAPES)
def test_q4_matmul_mfma_path(exe, rows, cols, batch):
    print(f"[q4 mfma] rows={rows} cols={cols} batch={batch}", flush=True)
    q, x, stride = make(rows, cols, batch, rows + cols + batch)
    got = run(exe, f"w_{rows}_{cols}", q, x, batch, rows, cols, stride)
    check(got, q, x, batch, rows, cols, stride)


@pytest.mark.parametrize("rows,cols,batch", [(2560, 2048, 32), (11264, 2048, 64), (128, 96, 33), (4096, 14336, 3)])
def test_q4_matmul_weights_as_fp16_pairs(exe, rows, cols, batch):
    # q4_int_operand = 0: the earlier arithmetic (d * (q - 8) as an exact fp16 pair, three MFMAs per
    # k step) stays selectable and is held to the same bounds
    q, x, stride = make(rows, cols, batch, rows + cols + batch + 1)
    assert exe.setOption("q4_int_operand", 0)
    try:
        got = run(exe, f"p_{rows}_{cols}", q, x, batch, rows, cols, stride)
    finally:
        assert exe.setOption("q4_int_operand", 1)
    check(got, q, x, batch, rows, cols, stride)


@pytest.mark.parametrize("ksplit", [1, 2, 8, 64])
def test_q4_matmul_k_split_is_deterministic_and_correct(exe, ksplit):
    rows, cols, batch = 512, 2048, 40
    q, x, stride = make(rows, cols, batch, 99)
    assert exe.setOption("q4_ksplit", ksplit)
    try:
        a = run(exe, "w_ksplit", q, x, batch, rows, cols, stride)
        b = run(exe, "w_ksplit", q, x, batch, rows, cols, stride, sync=False)
    finally:
        exe.setOption("q4_ksplit", 0)
    assert np.array_equal(a.view(np.uint32), b.view(np.uint32))     # fixed summation order
    check(a, q, x, batch, rows, cols, stride)


@pytest.mark.parametrize("rows,cols,batch,pad", [(68, 96, 3, 0), (4, 64, 1, 0), (100, 200, 5, 0),
                                                 (64, 2048, 4, 6), (256, 128, 9, 1)])
def test_q4_matmul_scalar_path(exe, rows, cols, batch, pad):
    # shapes the MFMA path does not take (rows % 64, cols % 32, odd strides) and forced fallback
    print(f"[q4 scalar] rows={rows} cols={cols} batch={batch} pad={pad}", flush=True)
    q, x, stride = make(rows, cols, batch, rows * 3 + cols + pad, pad=pad)
    assert exe.setOption("q4_force_generic", 1)
    try:
        got = run(exe, f"s_{rows}_{cols}_{pad}", q, x, batch, rows, cols, stride)
    finally:
        exe.setOption("q4_force_generic", 0)
    check(got, q, x, batch, rows, cols, stride)
    if rows % 64 == 0 and cols % 32 == 0:   # the same call without the switch takes the MFMA path
        check(run(exe, f"s_{rows}_{cols}_{pad}", q, x, batch, rows, cols, stride), q, x, batch, rows, cols, stride)


@pytest.mark.parametrize("x_scale", [1e-6, 1.0, 3e4, 1e12])
def test_q4_matmul_activation_range(exe, x_scale):
    # the per-request power-of-two scaling keeps the fp16 split exact-ish over the fp32 range;
    # one request is all zeros, one has a single huge outlier
    rows, cols, batch = 128, 256, 6
    q, x, stride = make(rows, cols, batch, 5, x_scale=x_scale)
    x[2] = 0.0
    x[3, 17] = 1e4 * x_scale
    got = run(exe, "w_range", q, x, batch, rows, cols, stride)
    assert np.all(got[2] == 0.0)
    check(got, q, x, batch, rows, cols, stride)


def test_q4_matmul_weight_cache_and_errors(exe):
    rows, cols, batch = 64, 64, 2
    q, x, stride = make(rows, cols, batch, 1)
    q2, _, _ = make(rows, cols, batch, 2)
    a = run(exe, "w_cache", q, x, batch, rows, cols, stride)
    # like getOrCacheWeight, the name decides: a second call with the same name and size reuses
    # the device copy, whatever the host bytes now hold
    b = run(exe, "w_cache", q2, x, batch, rows, cols, stride)
    assert np.array_equal(a, b)
    c = run(exe, "w_cache_other", q2, x, batch, rows, cols, stride)
    assert not np.array_equal(a, c)
    buf = exe.allocateScratchBuffer(4096)
    try:
        assert not exe.hasForwardPassCB()
        assert not exe.encodeMatMulQ4_0Batched("e", q, buf, batch, rows, cols, stride, 1, buf)
        assert "open forward pass" in exe.lastError()
        assert not exe.encodeMatMulQ4_0Batched("e", q, buf, batch, rows, 32, 18, 1, buf, sync=True)   # cols < 64
        assert not exe.encodeMatMulQ4_0Batched("e", q, buf, batch, 6, cols, stride, 1, buf, sync=True)  # rows % 4
        assert not exe.encodeMatMulQ4_0Batched("e", q[:10], buf, batch, rows, cols, stride, 1, buf, sync=True)
        assert not exe.encodeMatMulQ4_0Batched("e", q, None, batch, rows, cols, stride, 1, buf, sync=True)
    finally:
        exe.releaseScratchBuffer(buf)
