"""The gate/up projection and the two steps after it: a Q4_0 matmul of an open pass that is followed
by the gate/up split + SiLU * up of its output (compiler/runtime/batched_walker.cpp:366-384) does
that work in its epilogue, and when the call after that is the Q4_0 matmul that reads the products
(the down-projection, :386-396) the epilogue also writes that matmul's split-fp16 activations, with
one power-of-two scale per (request, block of 32 columns) instead of one per request.  Every
buffer the calls are specified to write must come out bit-identical to the calls launched one by
one, except the last matmul's output, whose activations are split with other (finer) scales: it
must agree with the oracle's matmul of the GPU's own products like any other Q4_0 matmul."""
import zlib

import numpy as np
import pytest

from oracle import paged_oracle as po

pytestmark = pytest.mark.gpu


def _pool(exe, host: np.ndarray) -> int:
    buf = exe.allocateScratchBuffer(host.nbytes)
    assert buf and exe.uploadToBuffer(buf, host)
    return buf


def _read(exe, buf, like: np.ndarray) -> np.ndarray:
    out = np.empty_like(like)
    assert exe.downloadFromBuffer(buf, out)
    return out


class Case:
    def __init__(self, B, hid, ffn, rows_out, seed=0, spread=False):
        self.B, self.hid, self.ffn, self.rows_out = B, hid, ffn, rows_out
        rng = np.random.default_rng(seed)
        self.w_gu = po.quantize_q4_0((rng.standard_normal((2 * ffn, hid)) * 0.05).astype(np.float32))
        self.w_down = po.quantize_q4_0((rng.standard_normal((rows_out, ffn)) * 0.05).astype(np.float32))
        self.x = rng.standard_normal((B, hid)).astype(np.float32)
        if spread:  # requests and columns of very different magnitude: the per-block scales differ widely
            self.x *= np.exp2(rng.integers(-12, 12, (B, 1))).astype(np.float32)
            self.x[:, ::7] *= 64.0
        self.other = rng.standard_normal((B, ffn)).astype(np.float32)
        self.name = f"silu.{B}.{hid}.{ffn}.{rows_out}.{seed}"


def _run(exe, c: Case, form: str, fuse: int):
    """form: 'down' (split + SiLU, then the matmul that reads the products), 'alone' (split + SiLU,
    then the pass ends), 'other' (split + SiLU, then a matmul that reads another buffer)."""
    B = c.B
    like = {"gate_up": np.empty((B, 2 * c.ffn), np.float32), "gate": np.empty((B, c.ffn), np.float32),
            "up": np.empty((B, c.ffn), np.float32), "prod": np.empty((B, c.ffn), np.float32),
            "down": np.empty((B, c.rows_out), np.float32)}
    d = {n: _pool(exe, np.zeros(a.shape, a.dtype)) for n, a in like.items()}
    d_x, d_other = _pool(exe, c.x), _pool(exe, c.other)
    assert exe.setOption("fuse_row_ops", fuse)
    before = exe.fusedMatmulSiluLaunches(), exe.fusedMatmulSiluSplitLaunches()
    try:
        assert exe.beginForwardPassCB()
        assert exe.encodeMatMulQ4_0Batched(c.name + ".gu", c.w_gu, d_x, B, 2 * c.ffn, c.hid, po.q4_0_row_bytes(c.hid), 1,
                                           d["gate_up"]), exe.lastError()
        assert exe.encodeGateUpSplitSiluMul(d["gate_up"], d["gate"], d["up"], d["prod"], B, c.ffn, 2 * c.ffn), exe.lastError()
        if form != "alone":
            assert exe.encodeMatMulQ4_0Batched(c.name + ".down", c.w_down, d["prod"] if form == "down" else d_other, B,
                                               c.rows_out, c.ffn, po.q4_0_row_bytes(c.ffn), 1, d["down"]), exe.lastError()
        assert exe.flushForwardPassCB(), exe.lastError()
        got = {n: _read(exe, d[n], like[n]) for n in like}
    finally:
        exe.setOption("fuse_row_ops", 1)
        for b in list(d.values()) + [d_x, d_other]:
            exe.releaseScratchBuffer(b)
    return got, (exe.fusedMatmulSiluLaunches() - before[0], exe.fusedMatmulSiluSplitLaunches() - before[1])


# fused where the gate/up rows make more than 256 tiles of 32 (two row tiles per workgroup)
SHAPES = {
    "tinyllama": dict(B=32, hid=2048, ffn=5632, rows_out=2048, fused=True),
    "two_batch_tiles": dict(B=40, hid=256, ffn=4128, rows_out=192, fused=True),
    "ragged_batch": dict(B=5, hid=128, ffn=4160, rows_out=64, fused=True, spread=True),
    "down_not_split_over_k": dict(B=20, hid=64, ffn=4128, rows_out=8192 + 64, fused=True, spread=True),
    # (two batch tiles and two row tiles per workgroup: no kernel for block-wise scales, the split stays a launch)
    "down_two_tiles_each_way": dict(B=33, hid=64, ffn=4128, rows_out=8192 + 64, fused=True, split=False, spread=True),
    "few_rows": dict(B=9, hid=256, ffn=512, rows_out=256, fused=False),
}


@pytest.mark.parametrize("form", ["down", "alone", "other"])
@pytest.mark.parametrize("shape", list(SHAPES), ids=list(SHAPES))
def test_matmul_with_silu_epilogue_matches_separate_launches(exe, shape, form):
    kw = dict(SHAPES[shape])
    expect_fused = kw.pop("fused")
    expect_split = kw.pop("split", True)
    c = Case(seed=zlib.crc32(f"{shape}.{form}".encode()) % 1000, **kw)
    print(f"[case] {shape} {form} B={c.B} hid={c.hid} ffn={c.ffn} rows_out={c.rows_out}", flush=True)
    plain, n_plain = _run(exe, c, form, fuse=0)
    fused, n_fused = _run(exe, c, form, fuse=1)
    assert n_plain == (0, 0)
    assert n_fused == ((1, 1 if form == "down" and expect_split else 0) if expect_fused else (0, 0))
    for n in ("gate_up", "gate", "up", "prod"):
        assert np.array_equal(plain[n].view(np.uint8), fused[n].view(np.uint8)), n
    # against the oracle: the projection, the split + SiLU of the GPU's own projection (expf and the
    # division are the device's: a few ulps), the matmul of the GPU's own products
    want_gu = po.matmul_q4_0_batched(c.w_gu, c.x, c.B, 2 * c.ffn, c.hid)
    assert np.abs(fused["gate_up"] - want_gu).max() <= 2e-5 * np.abs(want_gu).max()
    wg, wu, wp = po.gate_up_split_silu_mul(fused["gate_up"], c.B, c.ffn, 2 * c.ffn)
    assert np.array_equal(fused["gate"], wg) and np.array_equal(fused["up"], wu)
    assert np.max(np.abs(fused["prod"] - wp) / (np.abs(wp) + 1e-30)) < 5e-6
    if form != "alone":
        src = fused["prod"] if form == "down" else c.other
        want_down = po.matmul_q4_0_batched(c.w_down, src, c.B, c.rows_out, c.ffn)
        for got in (plain["down"], fused["down"]):
            # per request: a request's error is measured against that request's largest output
            scale = np.abs(want_down).max(axis=1, keepdims=True)
            assert (np.abs(got - want_down) <= 2e-5 * scale).all()
        if form == "other":
            assert np.array_equal(plain["down"], fused["down"])


def test_silu_epilogue_inside_a_row_chain_of_layers(exe):
    """Two rounds of projection -> split + SiLU -> down-projection in one pass, the second reading the
    first's output: the fragments and scales of the first round are not overwritten before their
    reader ran, and the second round's are its own."""
    c = Case(B=32, hid=2048, ffn=5632, rows_out=2048, seed=11)
    B = c.B
    outs = {}
    for fuse in (0, 1):
        d_x = _pool(exe, c.x)
        d_gu, d_g, d_u, d_p = (exe.allocateScratchBuffer(B * n * 4) for n in (2 * c.ffn, c.ffn, c.ffn, c.ffn))
        d_h1, d_h2 = (exe.allocateScratchBuffer(B * c.rows_out * 4) for _ in range(2))
        assert exe.setOption("fuse_row_ops", fuse)
        before = exe.fusedMatmulSiluSplitLaunches()
        try:
            assert exe.beginForwardPassCB()
            for src, dst in ((d_x, d_h1), (d_h1, d_h2)):
                assert exe.encodeMatMulQ4_0Batched(c.name + ".gu", c.w_gu, src, B, 2 * c.ffn, c.hid,
                                                   po.q4_0_row_bytes(c.hid), 1, d_gu), exe.lastError()
                assert exe.encodeGateUpSplitSiluMul(d_gu, d_g, d_u, d_p, B, c.ffn, 2 * c.ffn), exe.lastError()
                assert exe.encodeMatMulQ4_0Batched(c.name + ".down", c.w_down, d_p, B, c.rows_out, c.ffn,
                                                   po.q4_0_row_bytes(c.ffn), 1, dst), exe.lastError()
            assert exe.flushForwardPassCB(), exe.lastError()
            outs[fuse] = [_read(exe, b, np.empty((B, c.rows_out), np.float32)) for b in (d_h1, d_h2)]
            assert exe.fusedMatmulSiluSplitLaunches() - before == (2 if fuse else 0)
        finally:
            exe.setOption("fuse_row_ops", 1)
            for b in (d_x, d_gu, d_g, d_u, d_p, d_h1, d_h2):
                exe.releaseScratchBuffer(b)
    for a, b in zip(outs[0], outs[1]):
        scale = np.abs(a).max(axis=1, keepdims=True)
        assert (np.abs(a - b) <= 4e-5 * scale).all()
