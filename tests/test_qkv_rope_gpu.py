"""The step before the KV write -- fused qkv split + RoPE + fp32->fp16 cast, and its form fused
with the paged scatter -- against the CPU oracle through the C ABI.  Every output is compared
BIT-EXACTLY: the kernel rounds each product and sum on its own like the CPU rotation
(compiler/runtime/quantization.cpp:772-793) and casts with round-to-nearest-even like MSL
half() (compiler/runtime/metal_runtime.mm:457-464)."""
import numpy as np
import pytest

from oracle import paged_oracle as po

pytestmark = pytest.mark.gpu

SHAPES = [  # B, H, Hkv, D, rotary_dim, extra qkv padding
    (1, 32, 4, 64, 64, 0),      # TinyLlama row, batch 1
    (32, 32, 4, 64, 64, 0),
    (64, 32, 8, 128, 128, 0),   # Llama-3-8B row
    (5, 8, 2, 64, 32, 10),      # partial rotary, padded qkv rows
    (3, 4, 4, 16, 0, 0),        # no rotation
    (7, 6, 2, 20, 8, 2),
]


def _up(exe, arr):
    arr = np.ascontiguousarray(arr)
    buf = exe.allocateScratchBuffer(max(arr.nbytes, 16))
    assert buf and exe.uploadToBuffer(buf, arr)
    return buf


def _down(exe, buf, shape, dtype):
    out = np.empty(shape, dtype)
    assert exe.downloadFromBuffer(buf, out)
    return out


def _inputs(B, H, Hkv, D, rot, pad, seed):
    rng = np.random.default_rng(seed)
    q_rows, k_rows, v_rows = H * D, Hkv * D, Hkv * D
    qkv_rows = q_rows + k_rows + v_rows + pad
    qkv = rng.standard_normal((B, qkv_rows)).astype(np.float32)
    # values that sit on fp16 rounding ties, subnormals and overflow in the v segment
    ties = np.array([1.00048828125, 1.00146484375, 2049.0, 2051.0, 65519.9, 65520.0, 7e4, 3e-8, 5.97e-8,
                     -1.00048828125, 6.1e-5, 0.0, -0.0], np.float32)
    qkv[0, q_rows + k_rows:q_rows + k_rows + min(ties.size, v_rows)] = ties[:v_rows]
    pos = rng.integers(0, 8192, B)
    cos = np.ones((B, max(rot // 2, 1)), np.float32)
    sin = np.zeros((B, max(rot // 2, 1)), np.float32)
    for r in range(B):
        if rot:
            cos[r], sin[r] = po.rotary_coefficients(int(pos[r]), rot)
    return qkv, cos, sin, (qkv_rows, q_rows, k_rows, v_rows)


@pytest.mark.parametrize("B,H,Hkv,D,rot,pad", SHAPES)
@pytest.mark.parametrize("sync", [True, False])
def test_split_rope_cast_bit_exact(exe, B, H, Hkv, D, rot, pad, sync):
    print(f"[rope] B={B} H={H}/{Hkv} D={D} rot={rot} pad={pad} sync={sync}", flush=True)
    qkv, cos, sin, (qkv_rows, q_rows, k_rows, v_rows) = _inputs(B, H, Hkv, D, rot, pad, B * 7 + D)
    want = po.qkv_split_rope_cast(qkv, cos if rot else None, sin if rot else None, B, H, Hkv, D,
                                  qkv_rows, q_rows, k_rows, v_rows, rot)
    assert want is not None
    d_qkv, d_cos, d_sin = _up(exe, qkv), _up(exe, cos), _up(exe, sin)
    outs = [exe.allocateScratchBuffer(n) for n in (B * q_rows * 4, B * k_rows * 4, B * v_rows * 4,
                                                   B * k_rows * 2, B * v_rows * 2)]
    try:
        if not sync:
            assert exe.beginForwardPassCB()
        assert exe.encodeQkvSplitRopeCast(d_qkv, *outs, d_cos, d_sin, B, H, Hkv, D, qkv_rows, q_rows,
                                          k_rows, v_rows, rot, sync=sync), exe.lastError()
        if not sync:
            assert exe.flushForwardPassCB()
        got = [_down(exe, outs[0], (B, q_rows), np.float32), _down(exe, outs[1], (B, k_rows), np.float32),
               _down(exe, outs[2], (B, v_rows), np.float32), _down(exe, outs[3], (B, k_rows), np.uint16),
               _down(exe, outs[4], (B, v_rows), np.uint16)]
    finally:
        for b in (d_qkv, d_cos, d_sin, *outs):
            exe.releaseScratchBuffer(b)
    for name, g, w in zip(("q", "k", "v"), got[:3], want[:3]):
        assert np.array_equal(g.view(np.uint32), w.view(np.uint32)), name
    assert np.array_equal(got[3], want[3]), "k_f16"
    assert np.array_equal(got[4], want[4]), "v_f16"


@pytest.mark.parametrize("B,H,Hkv,D,rot,pad", SHAPES[:4])
def test_fused_scatter_equals_cast_then_two_scatters(exe, B, H, Hkv, D, rot, pad):
    print(f"[rope+scatter] B={B} H={H}/{Hkv} D={D} rot={rot}", flush=True)
    P = 64
    qkv, cos, sin, (qkv_rows, q_rows, k_rows, v_rows) = _inputs(B, H, Hkv, D, rot, pad, B * 11 + D)
    rng = np.random.default_rng(B)
    cap = 2 * B + 3
    k_pool = rng.integers(0, 65536, cap * P * Hkv * D, dtype=np.uint16)
    v_pool = rng.integers(0, 65536, cap * P * Hkv * D, dtype=np.uint16)
    page_ids = rng.permutation(cap)[:B].astype(np.uint32)
    slots = rng.integers(0, P, B).astype(np.uint32)
    q, k, v, k16, v16 = po.qkv_split_rope_cast(qkv, cos, sin, B, H, Hkv, D, qkv_rows, q_rows, k_rows,
                                               v_rows, rot)
    want_k, want_v = k_pool.copy(), v_pool.copy()
    assert po.scatter_kv_paged_batched_f16(want_k, page_ids, slots, P, Hkv, D, B, k16)
    assert po.scatter_kv_paged_batched_f16(want_v, page_ids, slots, P, Hkv, D, B, v16)
    d_qkv, d_cos, d_sin = _up(exe, qkv), _up(exe, cos), _up(exe, sin)
    d_k, d_v = _up(exe, k_pool), _up(exe, v_pool)
    d_q = exe.allocateScratchBuffer(B * q_rows * 4)
    d_kf = exe.allocateScratchBuffer(B * k_rows * 4)
    try:
        assert exe.beginForwardPassCB()
        # k fp32 copy requested, v fp32 copy left out
        assert exe.encodeQkvSplitRopeScatter(d_qkv, d_q, d_k, d_v, d_cos, d_sin, page_ids, slots, P, B,
                                             H, Hkv, D, qkv_rows, q_rows, k_rows, v_rows, rot,
                                             k_f32_buf=d_kf), exe.lastError()
        assert exe.flushForwardPassCB()
        got_q = _down(exe, d_q, (B, q_rows), np.float32)
        got_kf = _down(exe, d_kf, (B, k_rows), np.float32)
        got_k, got_v = _down(exe, d_k, k_pool.shape, np.uint16), _down(exe, d_v, v_pool.shape, np.uint16)
    finally:
        for b in (d_qkv, d_cos, d_sin, d_k, d_v, d_q, d_kf):
            exe.releaseScratchBuffer(b)
    assert np.array_equal(got_q.view(np.uint32), q.view(np.uint32))
    assert np.array_equal(got_kf.view(np.uint32), k.view(np.uint32))
    assert np.array_equal(got_k, want_k) and np.array_equal(got_v, want_v)
    assert int((got_k != k_pool).sum()) <= B * k_rows      # nothing else in the pool moved


def test_rope_known_answer_of_the_reference_test(exe):
    """tests/test_runtime.cpp:799-818 through the HIP kernel."""
    from test_oracle_cpu import ROPE_COS, ROPE_EXPECTED, ROPE_SIN, ROPE_VEC
    qkv = np.array(ROPE_VEC * 3, np.float32)
    d_qkv, d_cos, d_sin = _up(exe, qkv), _up(exe, np.array(ROPE_COS, np.float32)), _up(exe, np.array(ROPE_SIN, np.float32))
    outs = [exe.allocateScratchBuffer(64) for _ in range(5)]
    try:
        assert exe.encodeQkvSplitRopeCast(d_qkv, *outs, d_cos, d_sin, 1, 1, 1, 8, 24, 8, 8, 8, 8, sync=True)
        q = _down(exe, outs[0], (8,), np.float32)
    finally:
        for b in (d_qkv, d_cos, d_sin, *outs):
            exe.releaseScratchBuffer(b)
    assert np.max(np.abs(q - np.array(ROPE_EXPECTED, np.float32))) <= 1e-5


def test_rope_argument_errors(exe):
    buf = exe.allocateScratchBuffer(4096)
    try:
        ok = lambda **kw: exe.encodeQkvSplitRopeCast(  # noqa: E731
            kw.get("qkv", buf), buf, buf, buf, buf, buf, kw.get("cos", buf), buf, 1, 2, 1, 8,
            kw.get("qkv_rows", 32), 16, 8, 8, kw.get("rot", 8), sync=kw.get("sync", True))
        assert not exe.hasForwardPassCB()
        assert not ok(sync=False) and "open forward pass" in exe.lastError()
        assert not ok(qkv=None)
        assert not ok(qkv_rows=30)          # q + k + v do not fit
        assert not ok(rot=10)               # rotary_dim > head_dim
        assert not ok(cos=None)             # rotation without tables
        assert not ok(rot=3)                # odd
    finally:
        exe.releaseScratchBuffer(buf)
