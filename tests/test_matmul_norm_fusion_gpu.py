"""The out-projection and the three steps after it: a Q4_0 matmul of an open pass that is followed
by the residual add of its output, the RMSNorm of the sum and the Q4_0 matmul that reads the norm
(compiler/runtime/batched_walker.cpp:333-365) runs as two launches.  The first matmul's epilogue
adds the residual, leaves every request's sums of squares and writes (sum * gamma) as the second
matmul's split-fp16 input, one scale per (request, block of 32 columns); the second matmul
multiplies its result with the norm's per-request factor and writes the norm's own output.  The
first matmul's output and the sum must be bit-identical to the calls launched one by one; the
norm and what follows differ in the order of their roundings and are checked against the oracle."""
import zlib

import numpy as np
import pytest

from oracle import paged_oracle as po

pytestmark = pytest.mark.gpu

EPS = 1e-5


def _pool(exe, host: np.ndarray) -> int:
    buf = exe.allocateScratchBuffer(host.nbytes)
    assert buf and exe.uploadToBuffer(buf, host)
    return buf


def _read(exe, buf, like: np.ndarray) -> np.ndarray:
    out = np.empty_like(like)
    assert exe.downloadFromBuffer(buf, out)
    return out


class Case:
    def __init__(self, B, k_in, hid, rows2, ffn_form=False, n_gamma=None, spread=False, seed=0):
        """proj = W1[hid x k_in] x; h = resid + proj; xn = rmsnorm(h) * gamma; y = W2[rows2 x hid] xn
        (ffn_form: rows2 = 2 * ffn, followed by the gate/up split + SiLU and a down-projection to hid)."""
        self.B, self.k_in, self.hid, self.rows2, self.ffn_form = B, k_in, hid, rows2, ffn_form
        rng = np.random.default_rng(seed)
        self.w1 = po.quantize_q4_0((rng.standard_normal((hid, k_in)) * 0.05).astype(np.float32))
        self.w2 = po.quantize_q4_0((rng.standard_normal((rows2, hid)) * 0.05).astype(np.float32))
        self.w3 = po.quantize_q4_0((rng.standard_normal((hid, rows2 // 2)) * 0.05).astype(np.float32)) if ffn_form else None
        self.x = rng.standard_normal((B, k_in)).astype(np.float32)
        self.resid = rng.standard_normal((B, hid)).astype(np.float32)
        if spread:   # requests and column ranges of very different size
            self.x *= np.exp2(rng.integers(-8, 8, (B, 1))).astype(np.float32)
            self.resid *= np.exp2(rng.integers(-8, 8, (B, 1))).astype(np.float32)
            self.resid[:, : hid // 4] *= 1e-3
        self.gamma = (1.0 + 0.3 * rng.standard_normal(hid if n_gamma is None else n_gamma)).astype(np.float32)
        self.name = f"norm.{B}.{k_in}.{hid}.{rows2}.{seed}"


def _run(exe, c: Case, form: str, fuse: int, resid_first=True):
    """form: 'full' (matmul, add, norm, matmul [, gate/up split + SiLU, down-projection]), 'no_reader'
    (matmul, add, norm), 'add_only' (matmul, add), 'other_reader' (the last matmul reads another
    buffer), 'in_place' (the sum is written over the residual)."""
    B = c.B
    like = {"proj": np.empty((B, c.hid), np.float32), "h": np.empty((B, c.hid), np.float32),
            "xn": np.empty((B, c.hid), np.float32), "y": np.empty((B, c.rows2), np.float32)}
    if c.ffn_form:
        like.update(gate=np.empty((B, c.rows2 // 2), np.float32), up=np.empty((B, c.rows2 // 2), np.float32),
                    prod=np.empty((B, c.rows2 // 2), np.float32), down=np.empty((B, c.hid), np.float32))
    d = {n: _pool(exe, np.zeros(a.shape, a.dtype)) for n, a in like.items()}
    other = np.random.default_rng(9).standard_normal((B, c.hid)).astype(np.float32)
    d_x, d_res, d_other = _pool(exe, c.x), _pool(exe, c.resid), _pool(exe, other)
    d_h = d_res if form == "in_place" else d["h"]
    assert exe.setOption("fuse_row_ops", fuse)
    before = exe.fusedMatmulNormLaunches()
    try:
        assert exe.beginForwardPassCB()
        assert exe.encodeMatMulQ4_0Batched(c.name + ".1", c.w1, d_x, B, c.hid, c.k_in, po.q4_0_row_bytes(c.k_in), 1,
                                           d["proj"]), exe.lastError()
        a, b = (d_res, d["proj"]) if resid_first else (d["proj"], d_res)
        assert exe.encodeAddBatched(a, b, d_h, B * c.hid), exe.lastError()
        if form != "add_only":
            assert exe.encodeRmsNormBatched(d_h, c.gamma, EPS, B, c.hid, d["xn"]), exe.lastError()
        if form in ("full", "other_reader", "in_place"):
            assert exe.encodeMatMulQ4_0Batched(c.name + ".2", c.w2, d_other if form == "other_reader" else d["xn"], B, c.rows2,
                                               c.hid, po.q4_0_row_bytes(c.hid), 1, d["y"]), exe.lastError()
            if c.ffn_form:
                ffn = c.rows2 // 2
                assert exe.encodeGateUpSplitSiluMul(d["y"], d["gate"], d["up"], d["prod"], B, ffn, c.rows2), exe.lastError()
                assert exe.encodeMatMulQ4_0Batched(c.name + ".3", c.w3, d["prod"], B, c.hid, ffn, po.q4_0_row_bytes(ffn), 1,
                                                   d["down"]), exe.lastError()
        assert exe.flushForwardPassCB(), exe.lastError()
        got = {n: _read(exe, d[n], like[n]) for n in like}
        if form == "in_place":
            got["h"] = _read(exe, d_res, like["h"])
    finally:
        exe.setOption("fuse_row_ops", 1)
        for buf in list(d.values()) + [d_x, d_res, d_other]:
            exe.releaseScratchBuffer(buf)
    return got, other, exe.fusedMatmulNormLaunches() - before


SHAPES = {
    "tinyllama": dict(B=32, k_in=2048, hid=2048, rows2=11264, ffn_form=True),
    "two_batch_tiles": dict(B=40, k_in=256, hid=512, rows2=1024),
    "ragged_batch_spread": dict(B=5, k_in=128, hid=1024, rows2=2048, spread=True),
    "short_gamma": dict(B=9, k_in=64, hid=256, rows2=512, n_gamma=100),
    "reader_split_over_k": dict(B=3, k_in=64, hid=4096, rows2=1024, spread=True),
    "too_few_workgroups_to_write_the_norm": dict(B=30, k_in=64, hid=4096, rows2=64),   # falls back
}


def _rel(a, b):
    return float(np.abs(a - b).max() / max(float(np.abs(b).max()), 1e-30))


@pytest.mark.parametrize("form", ["full", "no_reader", "add_only", "other_reader", "in_place"])
@pytest.mark.parametrize("shape", list(SHAPES), ids=list(SHAPES))
def test_matmul_add_norm_matmul_in_two_launches(exe, shape, form):
    c = Case(seed=zlib.crc32(f"{shape}.{form}".encode()) % 1000, **SHAPES[shape])
    print(f"[case] {shape} {form} B={c.B} k_in={c.k_in} hid={c.hid} rows2={c.rows2}", flush=True)
    plain, other, n_plain = _run(exe, c, form, fuse=0)
    fused, _, n_fused = _run(exe, c, form, fuse=1, resid_first=(len(shape) % 2 == 0))
    expect = 1 if form in ("full", "in_place") and shape != "too_few_workgroups_to_write_the_norm" else 0
    assert n_plain == 0 and n_fused == expect
    assert np.array_equal(plain["proj"].view(np.uint32), fused["proj"].view(np.uint32))
    assert np.array_equal(plain["h"].view(np.uint32), fused["h"].view(np.uint32))
    want_proj = po.matmul_q4_0_batched(c.w1, c.x, c.B, c.hid, c.k_in)
    assert (np.abs(fused["proj"] - want_proj) <= 2e-5 * np.abs(want_proj).max(axis=1, keepdims=True)).all()
    assert np.array_equal(fused["h"], po.add(c.resid, fused["proj"]))
    if form == "add_only":
        return
    want_xn = po.rms_norm_batched(fused["h"], c.gamma, EPS, c.B, c.hid)
    for got in (plain, fused):
        assert (np.abs(got["xn"] - want_xn) <= 2e-6 * np.abs(want_xn).max(axis=1, keepdims=True)).all()
    if form == "no_reader":
        return
    src = other if form == "other_reader" else fused["xn"]
    want_y = po.matmul_q4_0_batched(c.w2, src, c.B, c.rows2, c.hid)
    scale = np.abs(want_y).max(axis=1, keepdims=True)
    for got in (plain, fused):
        assert (np.abs(got["y"] - want_y) <= 2e-5 * scale).all()
    if c.ffn_form:
        ffn = c.rows2 // 2
        wg, wu, wp = po.gate_up_split_silu_mul(fused["y"], c.B, ffn, c.rows2)
        assert np.array_equal(fused["gate"], wg) and np.array_equal(fused["up"], wu)
        assert np.max(np.abs(fused["prod"] - wp) / (np.abs(wp) + 1e-30)) < 5e-6
        want_down = po.matmul_q4_0_batched(c.w3, fused["prod"], c.B, c.hid, ffn)
        assert (np.abs(fused["down"] - want_down) <= 2e-5 * np.abs(want_down).max(axis=1, keepdims=True)).all()
