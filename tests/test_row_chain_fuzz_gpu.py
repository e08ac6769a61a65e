"""Random sequences of the row-local operators (add, RMSNorm, gate/up SiLU, Q4_0 matmul), of the
paged decode attention (whose launch may be held back for the matmul behind it) and of
the KV write (split + RoPE + cast, with the batched scatters or fused with them) with
shared and in-place buffers, encoded in one pass twice: with the fused chains (the default) and
with every operator launched on its own.  Deferring and fusing must never change what a
sequence computes: every buffer is compared at the end (and after a read-back in the middle of
the pass).  add is exact; RMSNorm sums in another order in the fused kernel, so buffers are
compared to 1e-4 of their largest value."""
import numpy as np
import pytest

from oracle import paged_oracle as po

pytestmark = pytest.mark.gpu

B, L = 5, 256
# a [B][2L] buffer read as a fused qkv row: 4 query heads and 2 KV heads of 64
H, HKV, D, P, CAP = 4, 2, 64, 8, 12
KV_ROWS = HKV * D
# the attention op: an [B][L] buffer as q of 4 heads over one KV head, pools of its own with 64-token pages
A_HKV, A_P = 1, 64


def _program(rng, n_ops):
    """ops over buffers: 'n' = [B][L] (indices 0..5), 'w' = [B][2L] (indices 0..1)"""
    ops = []
    for _ in range(n_ops):
        kind = rng.choice(["add", "add", "rms", "rms", "mm_n", "mm_n", "mm_w", "mm_w", "silu", "peek", "rope", "ropec",
                           "attn", "attn", "layer_like", "layer_like"])
        if kind == "layer_like":
            # the order of a decoder layer's middle, buffers drawn at random (they may alias where the
            # operators allow it): attention -> matmul -> + residual -> norm -> matmul, any prefix of it cut off
            q, o, proj, res, h, xn = (int(v) for v in rng.permutation(6))
            if rng.random() < 0.3:
                h = res                                          # the sum written over the residual
            seq = [("attn", q, o), ("mm_n", o, proj), ("add", proj, res, h) if rng.random() < 0.5 else ("add", res, proj, h),
                   ("rms", h, xn, int(rng.integers(0, 2))), ("mm_w", xn, int(rng.integers(0, 2)))]
            first = int(rng.integers(0, 2))                      # with or without the attention in front
            ops.extend(seq[first:int(rng.integers(first + 2, len(seq) + 1))])
            continue
        if kind == "add":
            a, b, c = (int(v) for v in rng.integers(0, 6, 3))
            ops.append(("add", a, b, c))                       # c may alias a or b
        elif kind == "rms":
            a, c = (int(v) for v in rng.integers(0, 6, 2))
            ops.append(("rms", a, c, int(rng.integers(0, 2))))  # c may alias a; one of two weight vectors
        elif kind == "mm_n":
            a = int(rng.integers(0, 6))
            c = int(rng.choice([i for i in range(6) if i != a]))
            ops.append(("mm_n", a, c))
        elif kind == "mm_w":
            ops.append(("mm_w", int(rng.integers(0, 6)), int(rng.integers(0, 2))))
        elif kind == "attn":
            a = int(rng.integers(0, 6))
            ops.append(("attn", a, int(rng.choice([i for i in range(6) if i != a]))))
        elif kind == "silu":
            g, u, m = (int(v) for v in rng.choice(6, 3, replace=False))
            ops.append(("silu", int(rng.integers(0, 2)), g, u, m))
        elif kind in ("rope", "ropec"):
            # q goes to an [B][L] buffer; "ropec": cast form, then the scatters of its K (and V) rows
            ops.append((kind, int(rng.integers(0, 2)), int(rng.integers(0, 6)), int(rng.integers(0, 3))))
        else:
            ops.append(("peek", int(rng.integers(0, 6))))
    return ops


def _run(exe, ops, init_n, init_w, weights, gammas, fuse, ksplit, kv):
    # options are set before the pass: setting one launches what is pending
    assert exe.setOption("fuse_row_ops", fuse)
    assert exe.setOption("q4_ksplit", ksplit)
    n = [exe.allocateScratchBuffer(B * L * 4) for _ in range(6)]
    w = [exe.allocateScratchBuffer(B * 2 * L * 4) for _ in range(2)]
    peeks = []
    kvb = {k: exe.allocateScratchBuffer(a.nbytes) for k, a in kv["init"].items()}
    try:
        for buf, a in zip(n + w, init_n + init_w):
            assert exe.uploadToBuffer(buf, a)
        for k, a in kv["init"].items():
            assert exe.uploadToBuffer(kvb[k], a)
        assert exe.beginForwardPassCB()
        for op in ops:
            if op[0] == "add":
                assert exe.encodeAddBatched(n[op[1]], n[op[2]], n[op[3]], B * L)
            elif op[0] == "rms":
                assert exe.encodeRmsNormBatched(n[op[1]], gammas[op[3]], 1e-5, B, L, n[op[2]])
            elif op[0] == "mm_n":
                assert exe.encodeMatMulQ4_0Batched("fuzz.n", weights["n"], n[op[1]], B, L, L, weights["n"].shape[1], 1,
                                                   n[op[2]]), exe.lastError()
            elif op[0] == "mm_w":
                assert exe.encodeMatMulQ4_0Batched("fuzz.w", weights["w"], n[op[1]], B, 2 * L, L, weights["w"].shape[1], 1,
                                                   w[op[2]]), exe.lastError()
            elif op[0] == "silu":
                assert exe.encodeGateUpSplitSiluMul(w[op[1]], n[op[2]], n[op[3]], n[op[4]], B, L, 2 * L)
            elif op[0] == "attn":
                at = kv["attn"]
                assert exe.encodePagedFlashAttention(n[op[1]], kvb["a_k"], kvb["a_v"], n[op[2]], at["flat"], at["off"],
                                                     at["lens"], at["pos"], B, H, A_HKV, D, A_P, True), exe.lastError()
            elif op[0] == "rope":
                assert exe.encodeQkvSplitRopeScatter(w[op[1]], n[op[2]], kvb["kp"], kvb["vp"], kvb["cos"], kvb["sin"],
                                                     kv["ids"], kv["slots"], P, B, H, HKV, D, 2 * L, L, KV_ROWS,
                                                     KV_ROWS, D), exe.lastError()
            elif op[0] == "ropec":
                assert exe.encodeQkvSplitRopeCast(w[op[1]], n[op[2]], kvb["k"], kvb["v"], kvb["k16"], kvb["v16"],
                                                  kvb["cos"], kvb["sin"], B, H, HKV, D, 2 * L, L, KV_ROWS, KV_ROWS,
                                                  D), exe.lastError()
                if op[3] >= 1:
                    assert exe.encodeScatterKVPagedBatched(kvb["kp"], kv["ids"], kv["slots"], P, HKV, D, B, kvb["k16"])
                if op[3] >= 2:
                    assert exe.encodeScatterKVPagedBatched(kvb["vp"], kv["ids"], kv["slots"], P, HKV, D, B, kvb["v16"])
            else:
                out = np.empty((B, L), np.float32)
                assert exe.downloadFromBuffer(n[op[1]], out)      # in the middle of the pass
                peeks.append(out)
        assert exe.flushForwardPassCB(), exe.lastError()
        final = []
        for buf, shape in zip(n + w, [(B, L)] * 6 + [(B, 2 * L)] * 2):
            out = np.empty(shape, np.float32)
            assert exe.downloadFromBuffer(buf, out)
            final.append(out)
        for k in ("k", "v", "k16", "v16", "kp", "vp"):
            out = np.empty_like(kv["init"][k])
            assert exe.downloadFromBuffer(kvb[k], out)
            final.append(out.astype(np.float32) if out.dtype == np.float32 else out.view(np.float16).astype(np.float32))
    finally:
        exe.setOption("fuse_row_ops", 1)
        exe.setOption("q4_ksplit", 0)
        for buf in n + w + list(kvb.values()):
            exe.releaseScratchBuffer(buf)
    return final, peeks


@pytest.mark.parametrize("seed", range(40))
def test_fused_and_unfused_sequences_agree(exe, seed):
    rng = np.random.default_rng(1000 + seed)
    ops = _program(rng, 14)
    print(f"[fuzz {seed}] " + " ".join(o[0] + ":" + ",".join(str(v) for v in o[1:]) for o in ops), flush=True)
    init_n = [rng.standard_normal((B, L)).astype(np.float32) for _ in range(6)]
    init_w = [rng.standard_normal((B, 2 * L)).astype(np.float32) for _ in range(2)]
    weights = {"n": po.quantize_q4_0((rng.standard_normal((L, L)) * 0.06).astype(np.float32)),
               "w": po.quantize_q4_0((rng.standard_normal((2 * L, L)) * 0.06).astype(np.float32))}
    gammas = [rng.uniform(0.5, 1.5, L).astype(np.float32) for _ in range(2)]
    ksplit = int(rng.choice([0, 2]))     # 2: the matmuls leave K slices for the next chain to sum
    cos, sin = np.zeros((B, D // 2), np.float32), np.zeros((B, D // 2), np.float32)
    for r in range(B):
        cos[r], sin[r] = po.rotary_coefficients(int(rng.integers(0, 2000)), D)
    kv = {"ids": rng.permutation(CAP)[:B].astype(np.uint32), "slots": rng.integers(0, P, B).astype(np.uint32),
          "init": {"cos": cos, "sin": sin, "k": np.zeros((B, KV_ROWS), np.float32), "v": np.zeros((B, KV_ROWS), np.float32),
                   "k16": np.zeros((B, KV_ROWS), np.uint16), "v16": np.zeros((B, KV_ROWS), np.uint16),
                   "kp": np.zeros(CAP * P * KV_ROWS, np.uint16), "vp": np.zeros(CAP * P * KV_ROWS, np.uint16)}}
    a_lens = rng.integers(0, 200, B).astype(np.uint32)          # (a request without tokens now and then: a row of zeros)
    a_pages = (a_lens.astype(np.int64) + A_P - 1) // A_P
    a_off = np.zeros(B + 1, np.uint32)
    a_off[1:] = np.cumsum(a_pages)
    n_pages = max(int(a_pages.sum()), 1)
    kv["attn"] = {"lens": a_lens, "pos": np.where(a_lens > 0, a_lens - 1, 0).astype(np.uint32), "off": a_off,
                  "flat": rng.permutation(n_pages)[:int(a_pages.sum())].astype(np.uint32)}
    for name in ("a_k", "a_v"):
        kv["init"][name] = rng.standard_normal(n_pages * A_P * A_HKV * D).astype(np.float16).view(np.uint16)
    before = exe.rowProgramLaunches()
    before_mm = exe.fusedMatmulRopeLaunches()
    before_more = exe.fusedDecodeSplitLaunches(), exe.fusedMatmulNormLaunches()
    fused, fused_peeks = _run(exe, ops, init_n, init_w, weights, gammas, 1, ksplit, kv)
    n_fused = exe.rowProgramLaunches() - before
    print(f"[fuzz {seed}] fused chains {n_fused}, matmuls with the RoPE epilogue "
          f"{exe.fusedMatmulRopeLaunches() - before_mm}, attention launches that split their output "
          f"{exe.fusedDecodeSplitLaunches() - before_more[0]}, matmuls that took over add + norm "
          f"{exe.fusedMatmulNormLaunches() - before_more[1]}", flush=True)
    plain, plain_peeks = _run(exe, ops, init_n, init_w, weights, gammas, 0, ksplit, kv)
    assert exe.rowProgramLaunches() - before == n_fused       # none with fusion off
    n_final = len(fused)
    for i, (a, b) in enumerate(list(zip(fused, plain)) + list(zip(fused_peeks, plain_peeks))):
        assert np.all(np.isfinite(a)) and np.all(np.isfinite(b))
        scale = max(float(np.max(np.abs(b))), 1e-30)
        # the last four final buffers hold fp16 rows: a last-bit difference of an fp32 value can
        # move its cast by one fp16 step (2^-11 of the value)
        tol = 1e-3 if n_final - 4 <= i < n_final else 1e-4
        assert float(np.max(np.abs(a - b))) <= tol * scale, (i, float(np.max(np.abs(a - b))), scale)
