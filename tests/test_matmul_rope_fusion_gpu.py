"""The qkv projection and the step after it in one launch: a Q4_0 matmul of an open pass that is
followed by the split + RoPE + cast of its output (encodeQkvSplitRopeCast with the batched
scatters of compiler/runtime/batched_walker.cpp:287-307, or the fused split + RoPE + scatter
call) does that work in its epilogue.  Every buffer the calls are specified to write must come
out bit-identical to the calls launched one by one, and the rotation must be the oracle's
applied to the matmul's own output."""
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
    def __init__(self, B, H, Hkv, D, hid, rotary=None, P=16, seed=0):
        self.B, self.H, self.Hkv, self.D, self.hid, self.P = B, H, Hkv, D, hid, P
        self.rotary = D if rotary is None else rotary
        self.q_rows, self.kv_rows = H * D, Hkv * D
        self.rows = self.q_rows + 2 * self.kv_rows
        rng = np.random.default_rng(seed)
        self.w = po.quantize_q4_0((rng.standard_normal((self.rows, hid)) * 0.05).astype(np.float32))
        self.x = rng.standard_normal((B, hid)).astype(np.float32)
        pos = rng.integers(0, 3000, B)
        self.cos = np.zeros((B, max(self.rotary // 2, 1)), np.float32)
        self.sin = np.zeros((B, max(self.rotary // 2, 1)), np.float32)
        for r in range(B):
            if self.rotary:
                self.cos[r], self.sin[r] = po.rotary_coefficients(int(pos[r]), self.rotary)
        cap = 2 * B
        self.k_pool, self.v_pool = (rng.integers(0, 65536, cap * P * self.kv_rows, dtype=np.uint16) for _ in range(2))
        self.ids = rng.permutation(cap)[:B].astype(np.uint32)
        self.slots = rng.integers(0, P, B).astype(np.uint32)
        self.name = f"fusion.{B}.{H}.{Hkv}.{D}.{hid}.{seed}"


def _run(exe, c: Case, form: str, fuse: int):
    """form: 'scatter' (fused call), 'cast2' (cast + K and V scatters), 'cast1' (cast + K scatter),
    'cast0' (cast alone).  Returns every buffer the calls write and the counter's increase."""
    B = c.B
    like = {"qkv": np.empty((B, c.rows), np.float32), "q": np.empty((B, c.q_rows), np.float32),
            "k": np.empty((B, c.kv_rows), np.float32), "v": np.empty((B, c.kv_rows), np.float32),
            "k16": np.empty((B, c.kv_rows), np.uint16), "v16": np.empty((B, c.kv_rows), np.uint16),
            "kp": c.k_pool, "vp": c.v_pool}
    d = {n: _pool(exe, a if n in ("kp", "vp") else np.zeros(a.shape, a.dtype)) for n, a in like.items()}
    d_x, d_cos, d_sin = (_pool(exe, a) for a in (c.x, c.cos, c.sin))
    assert exe.setOption("fuse_row_ops", fuse)
    before = exe.fusedMatmulRopeLaunches()
    try:
        assert exe.beginForwardPassCB()
        assert exe.encodeMatMulQ4_0Batched(c.name, c.w, d_x, B, c.rows, c.hid, po.q4_0_row_bytes(c.hid), 1,
                                           d["qkv"]), exe.lastError()
        if form == "scatter":
            assert exe.encodeQkvSplitRopeScatter(d["qkv"], d["q"], d["kp"], d["vp"], d_cos, d_sin, c.ids, c.slots,
                                                 c.P, B, c.H, c.Hkv, c.D, c.rows, c.q_rows, c.kv_rows, c.kv_rows,
                                                 c.rotary, k_f32_buf=d["k"], v_f32_buf=d["v"]), exe.lastError()
        else:
            assert exe.encodeQkvSplitRopeCast(d["qkv"], d["q"], d["k"], d["v"], d["k16"], d["v16"], d_cos, d_sin,
                                              B, c.H, c.Hkv, c.D, c.rows, c.q_rows, c.kv_rows, c.kv_rows,
                                              c.rotary), exe.lastError()
            if form in ("cast1", "cast2"):
                assert exe.encodeScatterKVPagedBatched(d["kp"], c.ids, c.slots, c.P, c.Hkv, c.D, B, d["k16"])
            if form == "cast2":
                assert exe.encodeScatterKVPagedBatched(d["vp"], c.ids, c.slots, c.P, c.Hkv, c.D, B, d["v16"])
        assert exe.flushForwardPassCB(), exe.lastError()
        got = {n: _read(exe, d[n], like[n]) for n in like}
    finally:
        exe.setOption("fuse_row_ops", 1)
        for b in list(d.values()) + [d_x, d_cos, d_sin]:
            exe.releaseScratchBuffer(b)
    return got, exe.fusedMatmulRopeLaunches() - before


SHAPES = {
    "small": dict(B=9, H=8, Hkv=2, D=64, hid=256),
    "tinyllama": dict(B=32, H=32, Hkv=4, D=64, hid=2048),
    "two_batch_tiles": dict(B=40, H=4, Hkv=4, D=128, hid=512),
    "partial_rotary": dict(B=5, H=8, Hkv=4, D=64, hid=256, rotary=32),
    "no_rotary": dict(B=3, H=4, Hkv=2, D=64, hid=128, rotary=0),
    "two_row_tiles": dict(B=7, H=64, Hkv=8, D=128, hid=256),
}


@pytest.mark.parametrize("form", ["scatter", "cast2", "cast1", "cast0"])
@pytest.mark.parametrize("shape", list(SHAPES), ids=list(SHAPES))
def test_matmul_with_rope_epilogue_matches_separate_launches(exe, shape, form):
    c = Case(seed=zlib.crc32(f"{shape}.{form}".encode()) % 1000, **SHAPES[shape])
    print(f"[case] {shape} {form} B={c.B} rows={c.rows} hid={c.hid}", flush=True)
    plain, n_plain = _run(exe, c, form, fuse=0)
    fused, n_fused = _run(exe, c, form, fuse=1)
    assert n_plain == 0 and n_fused == 1
    written = {"scatter": ("qkv", "q", "k", "v", "kp", "vp"), "cast2": ("qkv", "q", "k", "v", "k16", "v16", "kp", "vp"),
               "cast1": ("qkv", "q", "k", "v", "k16", "v16", "kp", "vp"),
               "cast0": ("qkv", "q", "k", "v", "k16", "v16", "kp", "vp")}[form]
    for n in written:
        assert np.array_equal(plain[n].view(np.uint8), fused[n].view(np.uint8)), n
    # the matmul against the oracle's, and the rotation: the oracle's applied to the GPU's own qkv
    want_qkv = po.matmul_q4_0_batched(c.w, c.x, c.B, c.rows, c.hid)
    scale = np.abs(want_qkv).max()
    assert np.abs(fused["qkv"] - want_qkv).max() <= 2e-5 * scale
    wq, wk, wv, wk16, wv16 = po.qkv_split_rope_cast(fused["qkv"], c.cos, c.sin, c.B, c.H, c.Hkv, c.D, c.rows,
                                                    c.q_rows, c.kv_rows, c.kv_rows, c.rotary)
    want_k, want_v = c.k_pool.copy(), c.v_pool.copy()
    if form != "cast0":
        assert po.scatter_kv_paged_batched_f16(want_k, c.ids, c.slots, c.P, c.Hkv, c.D, c.B, wk16)
    if form in ("scatter", "cast2"):
        assert po.scatter_kv_paged_batched_f16(want_v, c.ids, c.slots, c.P, c.Hkv, c.D, c.B, wv16)
    wants = {"q": wq, "k": wk, "v": wv, "kp": want_k, "vp": want_v}
    if form != "scatter":
        wants.update(k16=wk16, v16=wv16)
    for n, want in wants.items():
        assert np.array_equal(fused[n].view(np.uint8), np.ascontiguousarray(want).view(np.uint8)), n


def test_matmul_followed_by_something_else_is_launched_as_it_is(exe):
    """The held-back matmul goes out unchanged when the next call is not the split of its output:
    a download, a split of another buffer, a second matmul."""
    c = Case(seed=5, **SHAPES["small"])
    B = c.B
    want_qkv = po.matmul_q4_0_batched(c.w, c.x, B, c.rows, c.hid)
    other = np.random.default_rng(6).standard_normal((B, c.rows)).astype(np.float32)
    d_x, d_cos, d_sin, d_other = (_pool(exe, a) for a in (c.x, c.cos, c.sin, other))
    d_qkv = exe.allocateScratchBuffer(B * c.rows * 4)
    d_qkv2 = exe.allocateScratchBuffer(B * c.rows * 4)
    d_q = exe.allocateScratchBuffer(B * c.q_rows * 4)
    d_kp, d_vp = _pool(exe, c.k_pool), _pool(exe, c.v_pool)
    bufs = [d_x, d_cos, d_sin, d_other, d_qkv, d_qkv2, d_q, d_kp, d_vp]
    before = exe.fusedMatmulRopeLaunches()
    stride = po.q4_0_row_bytes(c.hid)
    try:
        assert exe.beginForwardPassCB()
        assert exe.encodeMatMulQ4_0Batched(c.name, c.w, d_x, B, c.rows, c.hid, stride, 1, d_qkv)
        got = np.empty((B, c.rows), np.float32)
        assert exe.downloadFromBuffer(d_qkv, got)          # no flush in between
        assert np.abs(got - want_qkv).max() <= 2e-5 * np.abs(want_qkv).max()
        assert exe.encodeMatMulQ4_0Batched(c.name, c.w, d_x, B, c.rows, c.hid, stride, 1, d_qkv)
        assert exe.encodeQkvSplitRopeScatter(d_other, d_q, d_kp, d_vp, d_cos, d_sin, c.ids, c.slots, c.P, B, c.H,
                                             c.Hkv, c.D, c.rows, c.q_rows, c.kv_rows, c.kv_rows, c.rotary)
        assert exe.encodeMatMulQ4_0Batched(c.name, c.w, d_x, B, c.rows, c.hid, stride, 1, d_qkv)
        assert exe.encodeMatMulQ4_0Batched(c.name, c.w, d_x, B, c.rows, c.hid, stride, 1, d_qkv2)
        assert exe.flushForwardPassCB(), exe.lastError()
        q = _read(exe, d_q, np.empty((B, c.q_rows), np.float32))
        a, b = (_read(exe, x, got) for x in (d_qkv, d_qkv2))
    finally:
        for x in bufs:
            exe.releaseScratchBuffer(x)
    assert exe.fusedMatmulRopeLaunches() == before
    wq = po.qkv_split_rope_cast(other, c.cos, c.sin, B, c.H, c.Hkv, c.D, c.rows, c.q_rows, c.kv_rows, c.kv_rows,
                                c.rotary)[0]
    assert np.array_equal(q, wq)
    assert np.array_equal(a, got) and np.array_equal(b, got)
