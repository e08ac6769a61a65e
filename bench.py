#!/usr/bin/env python3
"""Benchmark of the paged decode attention hot path on one MI355X.

A step is one decode-attention layer call over one batch (the reference's
per-layer encodePagedFlashAttention, compiler/runtime/batched_walker.cpp:326)
on synthetic data already resident in HBM.  The default workload is the
batch-32 TinyLlama-shape configuration; consecutive steps walk over 22
independent per-layer K/V pools so the working set (~0.8 GB touched) does not
sit in the 256 MB Infinity Cache.

Prints ONE JSON line: the KV-read GB/s of the whole job, the roofline of the
decode kernel measured with HIP events on the kernel's stream (with a plain
streaming read of the same bytes beside it), and the CPU baseline timed on
this host's cores in the same run.  The default run adds config.per_config:
configurations 1, 3 (with its KV write), 4 and 5 (chunked prefill), each with
its own time, rate, roofline fraction and bounded CPU baseline.
--workload cfg1|cfg3|cfg4|cfg5 print one of those as a line of its own,
--workload refbench the reference's own micro-benchmark grid, --workload
layer|step a whole decoder layer / decode step.
"""
from __future__ import annotations

import argparse
import json
import os
import statistics
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0  # MI355X HBM3E, published
MFMA_F16_PEAK_TFLOPS = 2500.0  # MI355X dense fp16 MFMA, published
N_CU = 256  # MI355X compute units (8 XCDs of 32)


def bench_copy(args) -> int:
    """Plain copy kernel of known size: calibrates FETCH_SIZE / WRITE_SIZE and gives the
    practical streaming ceiling at the decode workload's size."""
    import ctypes as C

    from mlcompiler_amd import HipExecutor
    from mlcompiler_amd.build import BENCH_LIB_PATH
    exe = HipExecutor.Instance()
    exe.requireAvailable()
    bl = C.CDLL(BENCH_LIB_PATH)
    nbytes = args.copy_mib << 20
    pairs = [(exe.allocateScratchBuffer(nbytes), exe.allocateScratchBuffer(nbytes)) for _ in range(8)]
    for s_, d_ in pairs:
        exe.zeroBuffer(s_, nbytes)
    ms = C.c_float()
    total_ms = 0.0
    for rep in range(2):   # first pass warms up
        total_ms = 0.0
        for s_, d_ in pairs:  # rotate buffers so the data does not sit in the Infinity Cache
            assert bl.mlc_bench_copy_loop(C.c_void_p(s_), C.c_void_p(d_), C.c_size_t(nbytes),
                                          C.c_size_t(max(args.steps // 8, 1)), C.byref(ms))
            total_ms += ms.value
    n = max(args.steps // 8, 1) * 8
    us = total_ms / n * 1e3
    print(json.dumps({"metric": "plain copy kernel", "bytes_read_per_launch": nbytes,
                      "bytes_written_per_launch": nbytes, "us_per_launch": round(us, 3),
                      "read_plus_write_GBs": round(2 * nbytes / us / 1e3, 1), "launches": n}))
    return 0


def prefill_traffic():
    """HBM bytes per launch of the prefill kernel at configuration 5 (profiles/traffic.json)."""
    try:
        with open(os.path.join(ROOT, "profiles", "traffic.json")) as fh:
            return json.load(fh).get("prefill", {}).get("cfg5", {}).get("hbm_bytes_per_launch")
    except (OSError, ValueError):
        return None


def bench_prefill(args) -> dict:
    """Chunked prefill (benchmark configuration 5): B=8, 256-row fp16 query chunk after 3840
    cached tokens, 32q/8kv heads, head_dim 128.  Reports TFLOP/s on the exact causal FLOPs."""
    import ctypes as C

    from mlcompiler_amd import HipExecutor
    from mlcompiler_amd.build import BENCH_LIB_PATH
    from mlcompiler_amd.workloads import make_prefill
    exe = HipExecutor.Instance()
    exe.requireAvailable()
    if args.prefill_stages and not exe.setOption("prefill_stages", args.prefill_stages):
        raise SystemExit("bench.py: --prefill-stages must be 2, 4, 6 or 8")
    B, Cc, H, Hkv, D, P, ctx = 8, 256, 32, 8, 128, 64, 3840
    w = make_prefill(B, Cc, H, Hkv, D, P, [ctx] * B, seed=55)
    bufs = [exe.allocateScratchBuffer(w[n].nbytes) for n in ("q", "k", "v")]
    for b, n in zip(bufs, ("q", "k", "v")):
        assert exe.uploadToBuffer(b, w[n])
    ob = exe.allocateScratchBuffer(B * Cc * H * D * 4)
    bl = C.CDLL(BENCH_LIB_PATH)
    u32p = C.POINTER(C.c_uint32)
    meta = [np.ascontiguousarray(w[k], np.uint32) for k in ("flat", "off", "seq", "q_start")]

    def loop(steps):
        ms, wall_s = C.c_float(), C.c_double()
        ok = bl.mlc_bench_prefill_loop(
            C.c_void_p(bufs[0]), C.c_void_p(bufs[1]), C.c_void_p(bufs[2]), C.c_void_p(ob),
            meta[0].ctypes.data_as(u32p), C.c_size_t(meta[0].size), meta[1].ctypes.data_as(u32p),
            meta[2].ctypes.data_as(u32p), meta[3].ctypes.data_as(u32p), C.c_size_t(B), C.c_size_t(Cc),
            C.c_size_t(H), C.c_size_t(Hkv), C.c_size_t(D), C.c_size_t(P), C.c_size_t(steps),
            C.byref(ms), C.byref(wall_s))
        if not ok:
            raise RuntimeError("prefill loop failed: " + exe.lastError())
        return ms.value, wall_s.value

    steps = min(args.steps, 200) if args.workload == "cfg5" else 100
    loop(max(1, min(args.warmup, 10)))
    ev_ms, wall = loop(steps)
    flops = 4 * D * H * B * sum(ctx + i + 1 for i in range(Cc))  # exact causal count
    tflops = flops / (wall / steps) / 1e12
    ach = flops / (ev_ms / steps * 1e-3) / 1e12
    kv_bytes = B * (ctx + Cc) * 4 * Hkv * D
    result = {
        "metric": "chunked-prefill paged attention TFLOP/s (exact causal FLOPs), config 5",
        "value": round(tflops, 2), "unit": "TFLOP/s", "n_gpus": 1, "steps": steps,
        "warmup": min(args.warmup, 10), "ms_per_step": round(wall / steps * 1e3, 5),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f16 (fp16 q/K/V, MFMA with fp32 accumulate, fp32 output)", "data": "synthetic",
        "config": {"workload": f"cfg5_chunked_prefill: batch {B}, {Cc}-row chunk after {ctx} cached "
                               f"tokens, {H}q/{Hkv}kv heads, head_dim {D}, {P}-token pages",
                   "flop_per_step": flops, "kv_bytes_per_step": kv_bytes},
        "roofline": {"bound": "mfma", "achieved": round(ach, 2), "peak": MFMA_F16_PEAK_TFLOPS,
                     "unit": "TFLOP/s", "frac": round(ach / MFMA_F16_PEAK_TFLOPS, 4),
                     "traffic": prefill_traffic() if not args.prefill_stages else None,
                     "us_per_launch": round(ev_ms / steps * 1e3, 2)},
    }
    if not args.no_cpu:
        from oracle import paged_oracle as po
        sub = dict(w)
        sub.update(B=1)
        for k_ in ("q",):
            sub[k_] = w["q"].reshape(B, -1)[0]
        sub["flat"] = w["flat"][w["off"][0]:w["off"][1]]
        sub["off"] = np.array([0, sub["flat"].size], np.uint32)
        sub["seq"], sub["q_start"] = w["seq"][:1], w["q_start"][:1]
        rows = 8   # bounded sample: the first 8 chunk rows of request 0, all heads, one thread
        sub["C"] = rows
        sub["q"] = np.ascontiguousarray(w["q"].reshape(B, Cc, H * D)[0, :rows]).ravel()
        t0 = time.perf_counter()
        want = po.paged_attention_prefill(sub["q"], sub["k"], sub["v"], sub["flat"], sub["off"], sub["seq"],
                                          sub["q_start"], 1, rows, H, Hkv, D, P, 1)
        dt = time.perf_counter() - t0
        f_s = 4 * D * H * sum(ctx + i + 1 for i in range(rows))
        got = np.empty((B, Cc, H, D), np.float32)
        exe.downloadFromBuffer(ob, got)
        rep = po.per_head_report(got[0, :rows], want[0], D)
        result["cpu_baseline"] = {"value": round(f_s / dt / 1e12, 6), "unit": "TFLOP/s", "cores": 1,
                                  "kind": "port",
                                  "sample": f"{rows} of {Cc} chunk rows of request 0 (all heads), {dt:.2f} s"}
        result["parity_vs_cpu_baseline"] = {"min_cosine": round(rep["min_cosine"], 7),
                                            "max_abs": float(f"{rep['max_abs']:.3e}")}
    return result


def bench_layer(args, workload=None, steps=None) -> dict:
    """One whole decoder layer per step (TinyLlama-1.1B shape, Q4_0 weights) around the paged
    decode attention of configuration 2: the eleven operators of the reference's layer loop
    (compiler/runtime/batched_walker.cpp:246-405) enqueued through the C ABI with no host wait
    between them.  Reports the algorithmic bytes (Q4_0 weights + KV read) per second."""
    import ctypes as C

    from mlcompiler_amd import HipExecutor
    from mlcompiler_amd import workloads as lc
    from mlcompiler_amd.build import BENCH_LIB_PATH
    workload = workload or args.workload
    steps = steps or args.steps
    exe = HipExecutor.Instance()
    exe.requireAvailable()
    if args.q4_ksplit:
        exe.setOption("q4_ksplit", args.q4_ksplit)
    if args.no_fuse:
        exe.setOption("fuse_row_ops", 0)
    case, n_layers = build_workload("cfg2")
    c = case
    B = c.batch
    w = lc.make_layer_weights(7)
    rng = np.random.default_rng(8)
    x = rng.standard_normal((B, lc.HID)).astype(np.float32)
    qpos = c.q_positions.astype(np.uint32)
    cos, sin = lc.rotary_tables(qpos)
    # the step's new K/V row of request r goes to the slot of its newest position
    page_ids = np.array([c.page_tables_flat[c.page_table_offsets[r] + qpos[r] // c.page_size]
                         for r in range(B)], np.uint32)
    slots = (qpos % c.page_size).astype(np.uint32)

    keep, held = [], []

    def up(a):
        a = np.ascontiguousarray(a)
        b = exe.allocateScratchBuffer(a.nbytes)
        assert b and exe.uploadToBuffer(b, a), "out of device memory"
        keep.append(a)
        held.append(b)
        return b

    def dev(n_floats):
        b = exe.allocateScratchBuffer(n_floats * 4)
        assert b
        held.append(b)
        return b

    def release():
        while held:
            exe.releaseScratchBuffer(held.pop())

    k_bufs = [up(c.k_pages) for _ in range(n_layers)]
    v_bufs = [up(c.v_pages) for _ in range(n_layers)]
    u32p, f32p = C.POINTER(C.c_uint32), C.POINTER(C.c_float)

    class Layer(C.Structure):
        _fields_ = ([(n, C.c_void_p) for n in
                     ("x", "norm", "qkv", "q", "attn", "o", "resid", "gate_up", "gate", "up", "mix",
                      "down", "out", "out2", "cos", "sin")]
                    + [("attn_norm_w", f32p), ("ffn_norm_w", f32p)]
                    + [(n, t) for wn in ("w_qkv", "w_o", "w_gate_up", "w_down")
                       for n, t in ((wn, C.c_void_p), (wn + "_bytes", C.c_size_t))]
                    + [(n, C.c_size_t) for n in ("hidden", "ffn_inner", "num_heads", "kv_heads",
                                                 "head_dim", "page_size_tokens", "batch")]
                    + [("page_ids", u32p), ("slots", u32p), ("page_tables_flat", u32p),
                       ("n_flat", C.c_size_t), ("page_table_offsets", u32p), ("seq_lens", u32p),
                       ("q_positions", u32p), ("head_norm_w", f32p), ("head_w", C.c_void_p),
                       ("head_bytes", C.c_size_t), ("head_rows", C.c_size_t), ("logits", C.c_void_p),
                       ("enqueue_s", C.POINTER(C.c_double))])

    meta = {n: np.ascontiguousarray(a, np.uint32) for n, a in
            (("page_ids", page_ids), ("slots", slots), ("page_tables_flat", c.page_tables_flat),
             ("page_table_offsets", c.page_table_offsets), ("seq_lens", c.seq_lens),
             ("q_positions", qpos))}
    L = Layer()
    L.x, L.cos, L.sin = up(x), up(cos), up(sin)
    for n, cols in (("norm", lc.HID), ("qkv", lc.QKV_ROWS), ("q", lc.Q_ROWS), ("attn", lc.HID),
                    ("o", lc.HID), ("resid", lc.HID), ("gate_up", 2 * lc.FFN), ("gate", lc.FFN),
                    ("up", lc.FFN), ("mix", lc.FFN), ("down", lc.HID), ("out", lc.HID)):
        setattr(L, n, dev(B * cols))
    L.attn_norm_w = w["g_attn"].ctypes.data_as(f32p)
    L.ffn_norm_w = w["g_ffn"].ctypes.data_as(f32p)
    for field, key in (("w_qkv", "w_qkv"), ("w_o", "w_o"), ("w_gate_up", "w_gu"), ("w_down", "w_down")):
        setattr(L, field, w[key].ctypes.data)
        setattr(L, field + "_bytes", w[key].nbytes)
    L.hidden, L.ffn_inner, L.num_heads, L.kv_heads = lc.HID, lc.FFN, lc.H, lc.HKV
    L.head_dim, L.page_size_tokens, L.batch = lc.D, c.page_size, B
    for n, a in meta.items():
        setattr(L, n, a.ctypes.data_as(u32p))
    L.n_flat = meta["page_tables_flat"].size
    enqueue_s = C.c_double()
    L.enqueue_s = C.pointer(enqueue_s)

    whole_step = workload == "step"
    VOCAB = lc.VOCAB
    if whole_step:   # final RMSNorm + Q6_K lm_head after every 22nd layer: one decode step of the model
        head_norm, w_head = lc.make_head_weights(rng)
        keep.extend([head_norm, w_head])
        L.head_norm_w = head_norm.ctypes.data_as(f32p)
        L.head_w, L.head_bytes, L.head_rows = w_head.ctypes.data, w_head.nbytes, VOCAB
        L.logits = dev(B * VOCAB)

    bl = C.CDLL(BENCH_LIB_PATH)
    kp = (C.c_void_p * n_layers)(*k_bufs)
    vp = (C.c_void_p * n_layers)(*v_bufs)

    def loop(steps):
        ms, wall_s = C.c_float(), C.c_double()
        if not bl.mlc_bench_layer_loop(C.byref(L), kp, vp, C.c_size_t(n_layers), C.c_size_t(steps),
                                       C.byref(ms), C.byref(wall_s)):
            raise RuntimeError("layer loop failed: " + exe.lastError())
        return ms.value, wall_s.value

    loop(max(args.warmup, n_layers))     # also uploads and repacks the weights (first use of a name)
    # timed: every step reads the step before's output, like the layers of a model (the
    # residual add of one layer and the RMSNorm of the next are neighbours in the pass)
    L.out2 = dev(B * lc.HID)
    if whole_step:
        try:
            return finish_step(args, steps, exe, L, loop, lc, c, w, x, cos, sin, page_ids, slots, qpos,
                               n_layers, VOCAB, head_norm, w_head)
        finally:
            release()
    enqueue_s.value = 0.0
    ev_ms, wall = loop(steps)
    host_encode_us = enqueue_s.value / steps * 1e6
    graph_us = graph_nodes = None
    if args.graph:   # the same n_layers launches captured once into a HIP graph and replayed
        g_ms, g_nodes = C.c_float(), C.c_size_t()
        replays = max(1, steps // n_layers)
        loop(n_layers)                   # the same pass launched call by call: the replays must reproduce it
        eager_out = np.empty((B, lc.HID), np.float32)
        exe.downloadFromBuffer(L.out2, eager_out)
        rc = bl.mlc_bench_layer_loop_graph(C.byref(L), kp, vp, C.c_size_t(n_layers), C.c_size_t(replays),
                                           C.byref(g_ms), C.byref(g_nodes))
        if rc == 0:
            raise RuntimeError("graph replay of the layer loop failed: " + exe.lastError())
        graph_nodes = g_nodes.value
        replay_out = np.empty((B, lc.HID), np.float32)
        exe.downloadFromBuffer(L.out2, replay_out)
        if not np.array_equal(eager_out, replay_out):
            raise RuntimeError("graph replays of the layer loop differ from the eager pass")
        graph_us = round(g_ms.value / (replays * n_layers) * 1e3, 2)
    L.out2 = None
    loop(1)                              # one step from the known input, for the parity check
    out = np.empty((B, lc.HID), np.float32)
    exe.downloadFromBuffer(L.out, out)

    w_bytes = lc.weight_bytes(w)
    alg_bytes = w_bytes + c.kv_bytes
    us = wall / steps * 1e6
    ev_us = ev_ms / steps * 1e3
    value = alg_bytes / (wall / steps) / 1e9
    ach = alg_bytes / (ev_us * 1e-6) / 1e9
    result = {
        "metric": "decoder layer (Q4_0 weights + KV read) GB/s & us/layer, TinyLlama shape B=32",
        "value": round(value, 2), "unit": "GB/s", "n_gpus": 1, "steps": steps,
        "warmup": max(args.warmup, n_layers), "ms_per_step": round(us / 1e3, 6),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32 (Q4_0 weights, fp16 K/V storage; matmuls on split-fp16 MFMA with fp32 accumulate)",
        "data": "synthetic",
        "config": {
            "workload": f"decoder layer, TinyLlama-1.1B shape (hidden {lc.HID}, {lc.H}q/{lc.HKV}kv heads, "
                        f"head_dim {lc.D}, ffn {lc.FFN}), batch {B}, contexts of {c.name} "
                        f"(sum {int(c.seq_lens.sum())}), 11 operators per step, each step's output is the next "
                        f"step's input, {n_layers} K/V pools and {n_layers} device copies of the weights rotated",
            "weight_bytes_per_step": w_bytes, "kv_bytes_per_step": c.kv_bytes,
            "us_per_layer": round(us, 2),
            "host_encode_us_per_layer": round(host_encode_us, 2),
            "tokens_per_s_at_22_layers": round(B / (22 * us * 1e-6), 1),
            **({"us_per_layer_graph_replay": graph_us, "graph_nodes": graph_nodes} if args.graph else {}),
        },
        "roofline": {"bound": "hbm", "achieved": round(ach, 2), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(ach / HBM_PEAK_GBS, 4), "traffic": None,
                     "us_per_launch": round(ev_us, 2),
                     "note": "whole layer (all its kernels) between HIP events / steps; per-kernel "
                             "durations are in the rocprofv3 summary of this workload"},
    }
    if not args.no_cpu:
        from oracle import paged_oracle as po
        from oracle.layer_chain import oracle_chain
        nb = 8   # bounded sample: the first 8 requests of the batch, one thread
        off = c.page_table_offsets
        flat = c.page_tables_flat[:off[nb]]
        t0 = time.perf_counter()
        ref = oracle_chain(w, x[:nb], cos[:nb], sin[:nb], c.k_pages, c.v_pages, page_ids[:nb],
                              slots[:nb], flat, off[:nb + 1], c.seq_lens[:nb], qpos[:nb], n_threads=1)
        dt = time.perf_counter() - t0
        # the CPU reads the weights once per request: bytes that count are per request
        b_s = (w_bytes + int(c.seq_lens[:nb].sum()) * 4 * lc.HKV * lc.D / nb) * nb
        result["cpu_baseline"] = {"value": round(b_s / dt / 1e9, 4), "unit": "GB/s", "cores": 1,
                                  "kind": "port",
                                  "sample": f"{nb} of {B} requests through the same 11 operators, "
                                            f"{dt:.2f} s ({dt / nb * 1e3:.1f} ms per token-layer)",
                                  "us_per_layer_at_full_batch": round(dt / nb * B * 1e6, 1)}
        got = out[:nb]
        rel = float(np.max(np.abs(got - ref["out"])) / np.max(np.abs(ref["out"])))
        result["parity_vs_cpu_baseline"] = {"cosine": round(po.cosine(got.ravel(), ref["out"].ravel()), 8),
                                            "max_abs_over_max": float(f"{rel:.3e}"),
                                            "requests_checked": nb}
    release()
    return result


def finish_step(args, steps, exe, L, loop, lc, c, w, x, cos, sin, page_ids, slots, qpos, n_layers, VOCAB,
                head_norm, w_head) -> dict:
    """--workload step: times whole decode steps of a TinyLlama-1.1B-shape model (22 decoder
    layers, final RMSNorm, Q6_K lm_head) and checks the logits of one step against the CPU chain."""
    B = c.batch
    steps = max(1, min(steps, 200))
    loop(n_layers)                                  # first use of the lm_head: upload and repack
    ev_ms, wall = loop(steps * n_layers)
    loop(n_layers)                                  # one step from the known input, for the parity check
    # (with out2 set, layer 0 of a loop reads x and every later layer the one before: a whole step)
    logits = np.empty((B, VOCAB), np.float32)
    exe.downloadFromBuffer(L.logits, logits)
    w_bytes = lc.weight_bytes(w) * n_layers + w_head.nbytes
    alg_bytes = w_bytes + c.kv_bytes * n_layers
    s_per_step = wall / steps
    ev_s = ev_ms / steps * 1e-3
    result = {
        "metric": "decode step tokens/s (22 decoder layers + final norm + lm_head), TinyLlama-1.1B shape B=32",
        "value": round(B / s_per_step, 1), "unit": "tokens/s", "n_gpus": 1, "steps": steps,
        "warmup": 2, "ms_per_step": round(s_per_step * 1e3, 5), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None,
        "dtype": "f32 (Q4_0 / Q6_K weights, fp16 K/V storage; matmuls on split-fp16 MFMA with fp32 accumulate)",
        "data": "synthetic",
        "config": {
            "workload": f"decode step: {n_layers} decoder layers (hidden {lc.HID}, {lc.H}q/{lc.HKV}kv heads, "
                        f"head_dim {lc.D}, ffn {lc.FFN}, Q4_0) + RMSNorm + lm_head ({VOCAB} x {lc.HID}, Q6_K), "
                        f"batch {B}, contexts of {c.name} (sum {int(c.seq_lens.sum())}), random weights "
                        f"(one host copy, {n_layers} device copies), one open pass per step loop",
            "weight_bytes_per_step": w_bytes, "kv_bytes_per_step": c.kv_bytes * n_layers,
            "us_per_layer": round((s_per_step * 1e6) / n_layers, 2),
        },
        "roofline": {"bound": "hbm", "achieved": round(alg_bytes / ev_s / 1e9, 2), "peak": HBM_PEAK_GBS,
                     "unit": "GB/s", "frac": round(alg_bytes / ev_s / 1e9 / HBM_PEAK_GBS, 4), "traffic": None,
                     "us_per_launch": round(ev_s * 1e6, 2),
                     "note": "a whole step (200 kernels) between HIP events / steps; algorithmic bytes = all "
                             "weights once + the K/V of all layers"},
    }
    if not args.no_cpu:
        from oracle import paged_oracle as po
        from oracle.layer_chain import oracle_chain
        nb = 16 if args.workload == "step" else 4   # bounded sample: the first requests of the batch through all
        off = c.page_table_offsets                    # 22 layers and the head, 8 threads
        flat = c.page_tables_flat[:off[nb]]
        n_thr = min(os.cpu_count() or 1, 8)
        t0 = time.perf_counter()
        h = x[:nb]
        for _ in range(n_layers):
            h = oracle_chain(w, h, cos[:nb], sin[:nb], c.k_pages, c.v_pages, page_ids[:nb], slots[:nb],
                                flat, off[:nb + 1], c.seq_lens[:nb], qpos[:nb], n_threads=n_thr)["out"]
        hn = po.rms_norm_batched(h, head_norm, 1e-5, nb, lc.HID)
        want = po.matmul_q6_k_batched(w_head, hn, nb, VOCAB, lc.HID, n_threads=n_thr)
        dt = time.perf_counter() - t0
        result["cpu_baseline"] = {"value": round(nb / dt, 3), "unit": "tokens/s", "cores": n_thr, "kind": "port",
                                  "sample": f"{nb} of {B} requests through the same step, {dt:.2f} s"}
        got = logits[:nb]
        result["parity_vs_cpu_baseline"] = {
            "cosine": round(po.cosine(got.ravel(), want.ravel()), 8),
            "max_abs_over_max": float(f"{float(np.max(np.abs(got - want)) / np.max(np.abs(want))):.3e}"),
            "argmax_agree": int(np.sum(np.argmax(got, axis=1) == np.argmax(want, axis=1))),
            "requests_checked": nb}
    return result


def build_workload(name: str, batch=None):
    """The benchmark configuration `name`; batch: another batch size of the same shape and length
    distribution (cfg2 - cfg4; an experiment, not a benchmark configuration)."""
    from mlcompiler_amd.workloads import baseline_config
    idx = {"cfg1": 1, "cfg2": 2, "cfg3": 3, "cfg4": 4}[name]
    case = baseline_config(idx, batch=batch) if batch and idx > 1 else baseline_config(idx)
    layers = {"cfg1": 22, "cfg2": 22, "cfg3": 8, "cfg4": 1}[name]
    return case, layers


def cpu_baseline(case, budget_s: float):
    """Times the CPU path on a bounded sample of the same workload.  Uses the
    reference's own RunAttentionCPU build when it travelled with the tree
    (oracle/_ref), else the oracle port; one thread, like the reference."""
    from oracle import paged_oracle as po
    c = case
    kind = "reference" if po.ref_lib() is not None else "port"
    bytes_per_tok = 4 * c.kv_heads * c.head_dim
    done_bytes, spent, outs = 0, 0.0, {}
    order = list(range(c.batch))
    for r in order:
        S = int(c.seq_lens[r])
        if S == 0:
            continue
        pt = c.page_tables_flat[c.page_table_offsets[r]:c.page_table_offsets[r + 1]]
        if kind == "reference":
            kc = np.zeros((c.kv_heads, S, c.head_dim), np.uint16)
            vc = np.zeros((c.kv_heads, S, c.head_dim), np.uint16)
            po.gather_kv_pages(c.k_pages, pt, c.page_size, c.kv_heads, c.head_dim, S, kc, 2)
            po.gather_kv_pages(c.v_pages, pt, c.page_size, c.kv_heads, c.head_dim, S, vc, 2)
            kn = po.fp16_to_float(kc[:, S - 1, :])
            vn = po.fp16_to_float(vc[:, S - 1, :])
            t0 = time.perf_counter()
            o = po.ref_run_attention_cpu(c.q[r], kc, vc, c.num_heads, c.kv_heads, c.head_dim, S,
                                         S - 1, kn, vn)
            spent += time.perf_counter() - t0
        else:
            t0 = time.perf_counter()
            o = po.paged_attention_executor(c.q[r:r + 1], c.k_pages, c.v_pages, pt, [0, pt.size],
                                            [S], [S - 1], 1, c.num_heads, c.kv_heads, c.head_dim,
                                            c.page_size, True, 1)[0]
            spent += time.perf_counter() - t0
        outs[r] = o
        done_bytes += S * bytes_per_tok
        if spent > budget_s:
            break
    sample = f"{len(outs)} of {c.batch} requests of the same batch, {done_bytes} KV bytes, {spent:.2f} s"
    # all host cores, OpenMP over (request, head): reported beside the 1-thread figure
    # (the oracle's OpenMP loop is given at most 16 threads: the share of the host a one-GPU
    # box has; the host's own count is reported beside it)
    n = min(os.cpu_count() or 1, 16)
    t0 = time.perf_counter()
    po.paged_attention_executor(c.q, c.k_pages, c.v_pages, c.page_tables_flat,
                                c.page_table_offsets, c.seq_lens, c.q_positions, c.batch,
                                c.num_heads, c.kv_heads, c.head_dim, c.page_size, c.apply_causal, n)
    t_all = time.perf_counter() - t0
    return {
        "value": round(done_bytes / spent / 1e9, 4) if spent > 0 else None,
        "unit": "GB/s",
        "cores": 1,
        "kind": kind,
        "sample": sample,
        "all_cores": {"value": round(case.kv_bytes / t_all / 1e9, 4), "cores": n, "kind": "port",
                      "host_cores": os.cpu_count()},
    }, outs


def load_traffic(workload: str, kernel: str, work_items: int):
    """HBM bytes per launch of the decode kernel as profiled with rocprofv3 (FETCH_SIZE and
    WRITE_SIZE, scaled by the copy-kernel calibration), from profiles/traffic.json.  The figure
    belongs to one kernel variant and one split of the work: None when this run's differ."""
    try:
        with open(os.path.join(ROOT, "profiles", "traffic.json")) as fh:
            table = json.load(fh)
    except (OSError, ValueError):
        return None
    e = table.get("decode", {}).get(workload)
    if not e or e.get("kernel") != kernel or e.get("work_items") != work_items:
        return None
    return e.get("hbm_bytes_per_launch")


def probe_timeline(n_wg: int) -> dict:
    """Per-workgroup time stamps of the last tile-balanced decode launch, from a library built with
    -DMLC_STREAM_PROBE (MLC_HIPCC_EXTRA; add -DMLC_STREAM_PROBE_TILES for three stamps per tile).
    Thread 0 of every workgroup writes the 100 MHz counter at fixed points; the figures are us
    after the first workgroup's entry, min / median / p90 / max over the workgroups."""
    import ctypes as C

    from mlcompiler_amd._lib import load
    lib = load()
    if not hasattr(lib, "mlc_hip_debug_probe"):
        raise SystemExit("--probe needs a library built with MLC_HIPCC_EXTRA=-DMLC_STREAM_PROBE")
    buf = np.zeros((n_wg, 32), np.uint64)
    lib.mlc_hip_debug_probe.argtypes = [C.c_void_p, C.c_size_t]
    if not lib.mlc_hip_debug_probe(buf.ctypes.data, n_wg):
        raise RuntimeError("mlc_hip_debug_probe failed")
    t = buf.astype(np.int64)
    if os.environ.get("MLC_PROBE_RAW"):   # the raw stamps, for offline analysis
        np.save(os.environ["MLC_PROBE_RAW"], t)
    us = lambda x: (x - t[:, 0].min()) / 100.0

    def st(x):
        x = np.sort(np.asarray(x, np.float64))
        if x.size == 0:
            return None
        return {"min": round(float(x[0]), 2), "median": round(float(x[x.size // 2]), 2),
                "p90": round(float(x[x.size * 9 // 10]), 2), "max": round(float(x[-1]), 2)}
    names = ["entry", "per_request_figures_known", "page_ids_fetched", "first_tile_landed", "last_tile_consumed", "exit"]
    out = {"workgroups": n_wg, "tiles_per_workgroup": sorted(set(int(v) for v in t[:, 6]))}
    for i, nm in enumerate(names):
        out[nm] = st(us(t[:, i]))
    xcc = (t[:, 7] >> 32) & 0xF
    out["workgroups_not_on_xcd_blockidx_mod_8"] = int((xcc != (np.arange(n_wg) % 8)).sum())
    out["xcd_of_first_16_workgroups"] = [int(v) for v in xcc[:16]]
    lastc, ex = us(t[:, 4]), us(t[:, 5])
    pub = (t[:, 26] >= t[:, 0]) & (t[:, 26] <= t[:, 5])
    mer = (t[:, 28] >= t[:, 0]) & (t[:, 28] <= t[:, 5])
    out["published"] = int(pub.sum())
    out["partial_stores_issued_after_last_tile"] = st((us(t[:, 26]) - lastc)[pub])
    out["merged_by_wave_0"] = int(mer.sum())
    out["merge_begins_after_last_tile"] = st((us(t[:, 28]) - lastc)[mer])
    out["exit_after_merge_begins"] = st((ex - us(t[:, 28]))[mer])
    out["exit_after_last_tile_mergers"] = st((ex - lastc)[mer])
    out["exit_after_last_tile_others"] = st((ex - lastc)[~mer])
    if t[:, 8].max() > 0:  # stamps per tile: wait and work on each of the first six tiles
        n = t[:, 6]
        per_tile = []
        for k in range(6):
            m = n > k
            if not m.any():
                break
            wb, ab, ac = us(t[m, 8 + 3 * k]), us(t[m, 9 + 3 * k]), us(t[m, 10 + 3 * k])
            per_tile.append({"tile": k, "workgroups": int(m.sum()), "wait": st(ab - wb), "work": st(ac - ab), "done": st(ac)})
        out["per_tile"] = per_tile
    return out


def run_decode(args, name: str, steps: int, warmup: int, cpu_budget: float, full: bool) -> dict:
    """Times one decode configuration through the C ABI and frees its buffers again.
    full: also the one-launch-at-a-time distribution, the changing-tables loop, the fp32-weight
    variant and the streaming-read ceiling (the headline configuration's extras)."""
    import ctypes as C

    from mlcompiler_amd import HipExecutor
    from mlcompiler_amd.build import BENCH_LIB_PATH
    exe = HipExecutor.Instance()
    case, n_layers = build_workload(name, getattr(args, "batch", 0) if name == args.workload else None)
    c = case
    pool_bytes = c.k_pages.nbytes
    q_buf = exe.allocateScratchBuffer(c.q.nbytes)
    o_buf = exe.allocateScratchBuffer(c.q.nbytes)
    assert exe.uploadToBuffer(q_buf, c.q)
    k_bufs, v_bufs = [], []
    for _ in range(n_layers):
        kb = exe.allocateScratchBuffer(pool_bytes)
        vb = exe.allocateScratchBuffer(pool_bytes)
        assert kb and vb, "out of device memory"
        assert exe.uploadToBuffer(kb, c.k_pages) and exe.uploadToBuffer(vb, c.v_pages)
        k_bufs.append(kb)
        v_bufs.append(vb)

    bl = C.CDLL(BENCH_LIB_PATH)   # native loop around the C ABI (no Python between launches)
    u32p = C.POINTER(C.c_uint32)
    meta = [np.ascontiguousarray(x, np.uint32) for x in
            (c.page_tables_flat, c.page_table_offsets, c.seq_lens, c.q_positions)]
    kp = (C.c_void_p * n_layers)(*k_bufs)
    vp = (C.c_void_p * n_layers)(*v_bufs)

    def native_loop(n: int):
        ms, wall_s = C.c_float(), C.c_double()
        ok = bl.mlc_bench_decode_loop(
            C.c_void_p(q_buf), kp, vp, C.c_size_t(n_layers), C.c_void_p(o_buf),
            meta[0].ctypes.data_as(u32p), C.c_size_t(meta[0].size), meta[1].ctypes.data_as(u32p),
            meta[2].ctypes.data_as(u32p), meta[3].ctypes.data_as(u32p), C.c_size_t(c.batch),
            C.c_size_t(c.num_heads), C.c_size_t(c.kv_heads), C.c_size_t(c.head_dim),
            C.c_size_t(c.page_size), C.c_int(int(c.apply_causal)), C.c_size_t(n),
            C.byref(ms), C.byref(wall_s))
        if not ok:
            raise RuntimeError("decode loop failed: " + exe.lastError())
        return ms.value, wall_s.value

    def step(layer: int, flat=None, pos=None, causal=None) -> None:
        ok = exe.encodePagedFlashAttention(q_buf, k_bufs[layer], v_bufs[layer], o_buf,
                                           c.page_tables_flat if flat is None else flat,
                                           c.page_table_offsets, c.seq_lens,
                                           c.q_positions if pos is None else pos, c.batch, c.num_heads,
                                           c.kv_heads, c.head_dim, c.page_size,
                                           c.apply_causal if causal is None else causal)
        if not ok:
            raise RuntimeError("encodePagedFlashAttention failed: " + exe.lastError())

    # set-up: one untimed pass over every pool (the first launch that touches a pool pays for its
    # address translations), then the --warmup steps
    native_loop(n_layers)
    if warmup:
        native_loop(warmup)

    # ---- timed region: exactly `steps` steps, device idle on both sides (the loop starts on an
    # idle stream and returns after the stream has drained); HIP events bracket the same region
    # on the kernels' stream.
    ev_ms, wall = native_loop(steps)
    r = {"case": c, "n_layers": n_layers, "steps": steps, "ev_us": ev_ms / steps * 1e3, "wall_us": wall / steps * 1e6,
         "launches": exe.lastDecodeLaunches(), "items": exe.lastDecodeWorkItems(), "kernel": exe.lastDecodeKernel()}
    if args.probe:
        r["probe_timeline"] = probe_timeline(r["items"])

    if full:
        # ---- one launch at a time, HIP events around each (the reference's harness reports its
        # timings this way: warm-up, >= 200 iterations, median and p10 / p90,
        # tools/paged_flash_bench.cpp:55-76)
        singles = []
        exe.beginForwardPassCB()
        for i in range(203):
            exe.timerStart()
            step(i % n_layers)
            t = exe.timerStopMs()
            if i >= 3:
                singles.append(t * 1e3)
        exe.flushForwardPassCB()
        singles.sort()
        r["single_us"] = {"median": round(singles[len(singles) // 2], 2), "p10": round(singles[len(singles) // 10], 2),
                          "p90": round(singles[len(singles) * 9 // 10], 2), "n": len(singles)}

        # ---- boundary-inclusive figures: what a caller sees whose tables change with every call.
        # (a) the per-request arrays change (one query position alternates); (b) the page table's
        # content changes too (two page ids of one request trade places: same bytes read), so
        # the device copy of the table is refreshed by every call.
        # (their own step count and a warm-up pass each: at the driver's --steps 20 a one-off upload or
        # the first launches of a mode would dominate the figure)
        n_b = 500
        for key, swap_pages in (("tables_change_us", False), ("page_table_changes_us", True)):
            pos = c.q_positions.copy()
            flat2 = c.page_tables_flat.copy()
            big = int(np.argmax(c.seq_lens))
            o0 = int(c.page_table_offsets[big])
            if int(c.page_table_offsets[big + 1]) - o0 >= 2:
                flat2[o0], flat2[o0 + 1] = flat2[o0 + 1], flat2[o0]
            pos_alt = [pos.copy(), pos.copy()]
            pos_alt[1][0] = pos[0] - 1

            def changing(i):
                step(i % n_layers, flat=(flat2 if (swap_pages and i % 2) else None), pos=pos_alt[i % 2], causal=False)

            exe.beginForwardPassCB()
            for i in range(2 * n_layers):
                changing(i)
            assert exe.flushForwardPassCB()
            exe.beginForwardPassCB()
            exe.timerStart()
            tb = time.perf_counter()
            for i in range(n_b):
                changing(i)
            ev = exe.timerStopMs()
            assert exe.flushForwardPassCB()
            r[key] = {"wall": round((time.perf_counter() - tb) / n_b * 1e6, 3), "events": round(ev / n_b * 1e3, 3),
                      "steps": n_b}

        # ---- softmax weights rounded to fp16 for P.V (option decode_pv_fp16 = 1; the default keeps them
        # fp32-grade and meets the reference's 1e-5 stress gate)
        n_x = max(steps, 500)
        assert exe.setOption("decode_pv_fp16", 1)
        native_loop(2 * n_layers)
        ev16, _ = native_loop(n_x)
        assert exe.setOption("decode_pv_fp16", 0)
        r["pv_fp16_us"] = ev16 / n_x * 1e3

        # ---- products on the vector pipe (decode_mfma = 0), fp16 softmax weights as in the default
        if any(kv.startswith("decode_mfma=") for kv in args.opt):
            r["vector_pipe_us"] = float("nan")  # the caller chose the mode: nothing to compare
        else:
            assert exe.setOption("decode_mfma", 0)
            native_loop(2 * n_layers)
            evv, _ = native_loop(n_x)
            assert exe.setOption("decode_mfma", 1)
            r["vector_pipe_us"] = evv / n_x * 1e3

        # ---- a plain streaming read of the same number of bytes from the same pools
        each = min(c.kv_bytes // 2 // 16 * 16, pool_bytes)
        r["stream_read"] = stream_read_sweep(bl, kp, vp, n_layers, each, N_CU)

    # ---- the layer as the batched step runs it (batched_walker.cpp:304-331): write the step's
    # new K row and V row (they land on the newest position: the bytes read stay the same), then
    # attend.  Three encode calls per layer; the attention launch carries the two scatters.
    rng = np.random.default_rng(5)
    row = c.kv_heads * c.head_dim
    new_k = rng.standard_normal((c.batch, row)).astype(np.float16)
    new_v = rng.standard_normal((c.batch, row)).astype(np.float16)
    nk_buf, nv_buf = exe.allocateScratchBuffer(new_k.nbytes), exe.allocateScratchBuffer(new_v.nbytes)
    assert exe.uploadToBuffer(nk_buf, new_k) and exe.uploadToBuffer(nv_buf, new_v)
    last = np.maximum(c.seq_lens.astype(np.int64) - 1, 0)
    ids = np.array([c.page_tables_flat[c.page_table_offsets[i] + last[i] // c.page_size] if c.seq_lens[i] else 0
                    for i in range(c.batch)], np.uint32)
    slots = (last % c.page_size).astype(np.uint32)
    n_w = 500
    ms_w, wall_w = C.c_float(), C.c_double()

    def step_loop(n: int):
        return bl.mlc_bench_decode_step_loop(
            C.c_void_p(q_buf), kp, vp, C.c_size_t(n_layers), C.c_void_p(o_buf), C.c_void_p(nk_buf), C.c_void_p(nv_buf),
            ids.ctypes.data_as(u32p), slots.ctypes.data_as(u32p),
            meta[0].ctypes.data_as(u32p), C.c_size_t(meta[0].size), meta[1].ctypes.data_as(u32p),
            meta[2].ctypes.data_as(u32p), meta[3].ctypes.data_as(u32p), C.c_size_t(c.batch),
            C.c_size_t(c.num_heads), C.c_size_t(c.kv_heads), C.c_size_t(c.head_dim), C.c_size_t(c.page_size),
            C.c_size_t(n), C.byref(ms_w), C.byref(wall_w))

    ok = step_loop(2 * n_layers) and step_loop(n_w)
    if not ok:
        raise RuntimeError("decode step loop failed: " + exe.lastError())
    r["kv_write_us"] = ms_w.value / n_w * 1e3
    r["kv_write_steps"] = n_w
    # the pools now hold the new rows at the newest positions: the parity check below uses them
    for attr, new in (("k_pages", new_k), ("v_pages", new_v)):
        p2 = getattr(c, attr).copy().view(np.uint16).reshape(-1, c.page_size, row)
        for i in range(c.batch):
            if c.seq_lens[i]:
                p2[ids[i], slots[i]] = new[i].view(np.uint16)
        setattr(c, attr, p2.reshape(-1))

    out = np.empty(c.q.shape, np.float32)
    exe.beginForwardPassCB()
    step(0)
    exe.flushForwardPassCB()
    exe.downloadFromBuffer(o_buf, out)
    for b in [q_buf, o_buf, nk_buf, nv_buf] + k_bufs + v_bufs:
        exe.releaseScratchBuffer(b)

    if not args.no_cpu:
        cpu, outs = cpu_baseline(case, cpu_budget)
        from oracle import paged_oracle as po
        worst_cos, worst_abs = 1.0, 0.0
        for i, o in outs.items():
            rep = po.per_head_report(out[i], o, c.head_dim)
            worst_cos = min(worst_cos, rep["min_cosine"])
            worst_abs = max(worst_abs, rep["max_abs"])
        r["cpu"] = cpu
        r["parity"] = {"min_cosine": round(worst_cos, 7), "max_abs": float(f"{worst_abs:.3e}"),
                       "requests_checked": len(outs)}
    return r


def stream_read_sweep(bl, kp, vp, n_layers: int, each: int, n_cu: int, launches: int = 300) -> dict:
    """The practical ceiling of the memory system for a launch that reads `each` bytes of a K pool and
    of a V pool and does nothing else: the streaming-read kernels of csrc/bench_loop.cpp (loads into
    registers with 1..8 independent 16-byte loads per tensor in flight per lane, and global -> LDS
    loads shaped like the decode kernel's tile loads, each with ordinary and with non-temporal
    loads) swept over 1, 2, 4 and 8 workgroups per CU,
    each timed like the decode loop (same pools, rotated, HIP events around `launches` launches).
    Reports the best average, the best block of a repeat run of that combination, and the untuned
    grid-stride kernel."""
    import ctypes as C
    ms = C.c_float()

    def tuned(kind, unroll, grid, n):
        ok = bl.mlc_bench_read_tuned_loop(kp, vp, C.c_size_t(n_layers), C.c_size_t(each), C.c_size_t(n),
                                          C.c_int(kind), C.c_int(unroll), C.c_uint(grid), C.byref(ms))
        return ms.value / n * 1e3 if ok else None

    bl.mlc_bench_read_loop(kp, vp, C.c_size_t(n_layers), C.c_size_t(each), C.c_size_t(n_layers), C.byref(ms))
    assert bl.mlc_bench_read_loop(kp, vp, C.c_size_t(n_layers), C.c_size_t(each), C.c_size_t(launches), C.byref(ms))
    plain_us = ms.value / launches * 1e3
    rows = []
    names = {0: "registers", 1: "global->LDS", 2: "registers, non-temporal", 3: "global->LDS, non-temporal"}
    for kind, unrolls in ((0, (1, 2, 4, 8)), (1, (1, 2, 4)), (2, (1, 2, 4, 8)), (3, (1, 2, 4))):
        for u in unrolls:
            for per_cu in (1, 2, 4, 8):
                if kind % 2 == 1 and per_cu * 2 * 2 * u * 4096 > 160 * 1024:
                    continue   # the LDS stages of that many workgroups do not fit a CU
                grid = n_cu * per_cu
                if tuned(kind, u, grid, n_layers) is None:
                    continue
                rows.append({"kind": names[kind], "loads_in_flight_per_lane": 2 * u * (1 if kind % 2 == 0 else 2),
                             "wgs_per_cu": per_cu, "us": round(tuned(kind, u, grid, launches), 3),
                             "_k": kind, "_u": u, "_g": grid})
    best = min(rows, key=lambda x: x["us"])
    blocks = [tuned(best["_k"], best["_u"], best["_g"], 100) for _ in range(10)]
    for x in rows:
        for k in ("_k", "_u", "_g"):
            x.pop(k, None)
    return {"bytes": 2 * each, "us_per_launch": best["us"], "best": best, "best_block_of_100_us": round(min(blocks), 3),
            "untuned_grid_stride_us": round(plain_us, 3), "sweep": rows}


def workload_text(c, n_layers) -> str:
    return (f"{c.name}: batched paged decode attention, batch {c.batch}, "
            f"{c.num_heads}q/{c.kv_heads}kv heads, head_dim {c.head_dim}, "
            f"contexts {int(c.seq_lens.min())}..{int(c.seq_lens.max())} "
            f"(sum {int(c.seq_lens.sum())}), {c.page_size}-token fp16 pages permuted in a "
            f"{c.capacity_pages}-page pool, {n_layers} layer pools rotated")


def per_config_entry(name: str, r: dict) -> dict:
    """One decode configuration as an entry of config.per_config: every figure can be recomputed
    from kv_bytes_per_step and the microseconds beside it."""
    c = r["case"]
    with_write = name == "cfg3"   # the step of configuration 3 is scatter K, scatter V, attention
    us = r["kv_write_us"] if with_write else r["ev_us"]
    e = {"workload": workload_text(c, r["n_layers"]),
         "step": "scatter K row, scatter V row, attention (one launch: the attention kernel carries the write)"
                 if with_write else "attention",
         "steps": r["kv_write_steps"] if with_write else r["steps"],
         "kv_bytes_per_step": c.kv_bytes, "us_per_step": round(us, 3),
         "GBs": round(c.kv_bytes / us / 1e3, 1), "frac_of_hbm_peak": round(c.kv_bytes / us / 1e3 / HBM_PEAK_GBS, 4),
         "us_attention_only": round(r["ev_us"], 3), "kernel": r["kernel"], "work_items": r["items"],
         "traffic": load_traffic(name, r["kernel"], r["items"])}
    if "cpu" in r:
        e["cpu_baseline"] = r["cpu"]
        e["parity_vs_cpu_baseline"] = r["parity"]
    return e


def bench_refbench(args) -> dict:
    """The reference's own micro-benchmark grid (tools/paged_flash_bench.cpp:29-34, 206-226):
    32 query heads, 4 KV heads, head_dim 64, one 64-token page per request, batch 1, 2, 4, 8;
    3 warm-up calls, then 200 synchronous runPagedFlashAttention calls timed one by one on the
    host clock (as the reference's harness does, :55-76), median / p10 / p90 in microseconds; beside
    it the same calls timed with a HIP event pair on the stream."""
    from mlcompiler_amd import HipExecutor
    from mlcompiler_amd.workloads import DeviceCase, make_case
    exe = HipExecutor.Instance()
    exe.requireAvailable()
    rows = []
    for b in (1, 2, 4, 8):
        case = make_case(f"refbench_b{b}", b, 32, 4, 64, 64, [64] * b, capacity_pages=b, permute=False, seed=42,
                         dist="uniform")
        d = DeviceCase(exe, case)
        host, dev = [], []
        a = (d.q_buf, d.k_buf, d.v_buf, d.o_buf, case.page_tables_flat, case.page_table_offsets, case.seq_lens,
             case.q_positions, case.batch, case.num_heads, case.kv_heads, case.head_dim, case.page_size,
             case.apply_causal)
        for i in range(203):
            t0 = time.perf_counter()
            assert exe.runPagedFlashAttention(*a), exe.lastError()
            t = (time.perf_counter() - t0) * 1e6
            if i >= 3:
                host.append(t)
        exe.beginForwardPassCB()
        for i in range(203):
            exe.timerStart()
            assert exe.encodePagedFlashAttention(*a), exe.lastError()
            t = exe.timerStopMs() * 1e3
            if i >= 3:
                dev.append(t)
        exe.flushForwardPassCB()
        d.free()
        host.sort()
        dev.sort()
        pick = lambda v: {"median": round(v[len(v) // 2], 2), "p10": round(v[len(v) // 10], 2),
                          "p90": round(v[len(v) * 9 // 10], 2)}
        rows.append({"batch": b, "host_sync_call_us": pick(host), "stream_event_us": pick(dev), "n": len(host)})
    return ({"metric": "paged flash attention micro-benchmark of the reference (median us per call)",
                      "value": rows[-1]["host_sync_call_us"]["median"], "unit": "us", "n_gpus": 1, "steps": 200,
                      "warmup": 3, "higher_is_better": False, "scaling": "weak", "vs_baseline": None,
                      "dtype": "f32 (fp16 K/V storage, fp32 q, accumulate and output)", "data": "synthetic",
                      "config": {"workload": "tools/paged_flash_bench.cpp grid: 32q/4kv heads, head_dim 64, one "
                                             "64-token page per request, batch 1/2/4/8, uniform(-0.5, 0.5) inputs",
                                 "rows": rows}})


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=2000)
    ap.add_argument("--warmup", type=int, default=100)
    ap.add_argument("--workload", default="cfg2",
                    choices=["cfg1", "cfg2", "cfg3", "cfg4", "cfg5", "layer", "step", "copy", "refbench"])
    ap.add_argument("--per-config", type=int, default=-1,
                    help="1: add config.per_config (configurations 1, 3, 4 and 5, each with its own bounded CPU "
                         "baseline) to the line; default: only for the default workload")
    ap.add_argument("--batch", type=int, default=0,
                    help="cfg2 - cfg4: another batch size of the same shape (an experiment; the line then is not "
                         "the benchmark configuration's)")
    ap.add_argument("--copy-mib", type=int, default=32, help="size of the calibration copy")
    ap.add_argument("--cpu-budget", type=float, default=15.0, help="seconds of CPU baseline work")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--wgs-per-cu", type=int, default=0, help="tile-balanced kernel: workgroups per CU (0 = automatic)")
    ap.add_argument("--stages", type=int, default=0, help="tile-balanced kernel: LDS stages (0 = automatic)")
    ap.add_argument("--read-sweep", action="store_true",
                    help="decode: print every row of the streaming-read sweep, not only the best")
    ap.add_argument("--probe", action="store_true",
                    help="decode: print the per-workgroup timeline of the last launch as config.probe_timeline "
                         "(needs a library built with MLC_HIPCC_EXTRA=-DMLC_STREAM_PROBE; its times mean nothing)")
    ap.add_argument("--opt", action="append", default=[], metavar="NAME=VALUE",
                    help="library tunable (mlc_hip_set_option), may be repeated")
    ap.add_argument("--prefill-stages", type=int, default=0, help="cfg5: LDS pipeline depth (0 = automatic)")
    ap.add_argument("--q4-ksplit", type=int, default=0, help="layer: K slices of the Q4_0 matmuls (0 = automatic)")
    ap.add_argument("--graph", action="store_true",
                    help="layer workload: also replay the layers from a captured HIP graph")
    ap.add_argument("--no-fuse", action="store_true", help="layer: launch every operator on its own")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on ONE GPU only (no collectives, no sharding); "
              "use --gpus 1", file=sys.stderr)
        return 2

    if args.opt:
        from mlcompiler_amd import HipExecutor
        for kv in args.opt:
            name, value = kv.split("=")
            assert HipExecutor.Instance().setOption(name, int(value)), f"unknown option {kv}"

    if args.workload == "cfg5":
        print(json.dumps(bench_prefill(args)))
        return 0
    if args.workload == "copy":
        return bench_copy(args)
    if args.workload == "refbench":
        print(json.dumps(bench_refbench(args)))
        return 0
    if args.workload in ("layer", "step"):
        print(json.dumps(bench_layer(args)))
        return 0

    from mlcompiler_amd import HipExecutor
    exe = HipExecutor.Instance()
    exe.requireAvailable()
    if args.wgs_per_cu:
        assert exe.setOption("decode_wgs_per_cu", args.wgs_per_cu)
    if args.stages:
        assert exe.setOption("decode_stages", args.stages)
    per_config = args.per_config == 1 or (args.per_config < 0 and args.workload == "cfg2" and not args.no_cpu)
    r = run_decode(args, args.workload, args.steps, args.warmup, args.cpu_budget, full=True)
    c = r["case"]
    kv_bytes = c.kv_bytes
    # `value` and `ms_per_step` come from the HIP-event time of the timed region (device time of
    # exactly --steps steps, gaps between launches included).  The host clock around the same
    # region adds the one-off latency of the first launch and of the final synchronisation
    # (about 40 us): at --steps 20 that is a tenth of the region, so it is reported beside it
    # (wall_us_per_step) instead of being folded into the rate.
    ev_us = r["ev_us"]
    value = kv_bytes / ev_us / 1e3
    sr = r["stream_read"]
    result = {
        "metric": "decode attn KV-read GB/s (% of HBM peak) & us/layer, TinyLlama shape B=32",
        "value": round(value, 2),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ev_us / 1e3, 6),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32 (fp16 K/V storage, fp32 q, accumulate and output; fp32-grade products, no operand rounded: on "
                 "the f16 MFMA q and the softmax weights enter as sums of two fp16 numbers; option decode_pv_fp16 = 1 "
                 "rounds the weights to fp16, us_per_layer_pv_fp16 is its time; option decode_mfma = 0: every product "
                 "on the vector pipe, us_per_layer_vector_pipe is its time)",
        "data": "synthetic",
        "config": {
            "workload": workload_text(c, r["n_layers"]),
            "kv_bytes_per_step": kv_bytes,
            "us_per_layer": round(ev_us, 3),
            "wall_us_per_step": round(r["wall_us"], 3),
            "setup_steps_before_warmup": r["n_layers"],
            "pct_of_hbm_peak": round(100.0 * value / HBM_PEAK_GBS, 2),
            "kernels_per_step": r["launches"],
            "kernel": r["kernel"],
            "work_items": r["items"],
            "us_per_layer_pv_fp16": round(r["pv_fp16_us"], 3),
            "us_per_layer_vector_pipe": None if r["vector_pipe_us"] != r["vector_pipe_us"] else round(r["vector_pipe_us"], 3),
            "us_per_layer_tables_change": r["tables_change_us"],
            "us_per_layer_page_table_changes": r["page_table_changes_us"],
            "single_launch_us": r["single_us"],
            "us_per_layer_with_kv_write": round(r["kv_write_us"], 3),
            "host_cores": os.cpu_count(),
            **({"probe_timeline": r["probe_timeline"]} if "probe_timeline" in r else {}),
        },
        "roofline": {
            "bound": "hbm",
            "achieved": round(value, 2),
            "peak": HBM_PEAK_GBS,
            "unit": "GB/s",
            "frac": round(value / HBM_PEAK_GBS, 4),
            "traffic": load_traffic(args.workload, r["kernel"], r["items"]),
            "traffic_source": "profiles/traffic.json (rocprofv3 FETCH_SIZE / WRITE_SIZE of this kernel variant and "
                              "work split; null when this run's differ from the profiled ones)",
            "us_per_launch": round(ev_us, 3),
            "stream_read_ceiling": {"bytes": sr["bytes"], "us_per_launch": round(sr["us_per_launch"], 3),
                                    "GBs": round(sr["bytes"] / sr["us_per_launch"] / 1e3, 1),
                                    "frac": round(sr["bytes"] / sr["us_per_launch"] / 1e3 / HBM_PEAK_GBS, 4),
                                    "best": sr["best"], "best_block_of_100_us": sr["best_block_of_100_us"],
                                    "untuned_grid_stride_us": sr["untuned_grid_stride_us"],
                                    **({"sweep": sr["sweep"]} if args.read_sweep else {}),
                                    "note": "kernels that only read the same number of bytes contiguously from the "
                                            "same pools, same run, same timing: best of a sweep over loads in "
                                            "flight per lane (registers or global->LDS) and workgroups per CU"},
            "note": "HIP events around the timed region on the library stream / steps: one step = one "
                    "decode kernel (split requests are merged inside it by the last workgroup to arrive)",
        },
    }
    if "cpu" in r:
        result["cpu_baseline"] = r["cpu"]
        result["parity_vs_cpu_baseline"] = r["parity"]
    if per_config:
        pc = {}
        # (their own step counts, stated in each entry and independent of --steps: a 20-step region
        # of a 7 us kernel would mostly measure its first launches)
        for name, st, wu in (("cfg1", 2000, 20), ("cfg3", 500, 20), ("cfg4", 300, 50)):
            sub = run_decode(args, name, st, wu, 4.0, full=False)
            pc[name] = per_config_entry(name, sub)
        p5 = bench_prefill(args)
        pc["cfg5"] = {"workload": p5["config"]["workload"], "steps": p5["steps"],
                      "flop_per_step": p5["config"]["flop_per_step"],
                      "us_per_step": p5["roofline"]["us_per_launch"], "TFLOPs": p5["roofline"]["achieved"],
                      "frac_of_mfma_f16_peak": p5["roofline"]["frac"], "traffic": p5["roofline"]["traffic"],
                      **{k: p5[k] for k in ("cpu_baseline", "parity_vs_cpu_baseline") if k in p5}}
        # the reference's own micro-benchmark grid, one decoder layer and one whole decode step
        rb = bench_refbench(args)
        pc["refbench"] = {"workload": rb["config"]["workload"], "calls_per_batch": 200, "rows": rb["config"]["rows"]}
        for name, st in (("layer", 2000), ("step", 100)):
            sub = bench_layer(args, name, st)
            pc[name] = {"workload": sub["config"]["workload"], "steps": sub["steps"], "metric": sub["metric"],
                        "value": sub["value"], "unit": sub["unit"], "us_per_step": round(sub["ms_per_step"] * 1e3, 2),
                        **{k: sub["config"][k] for k in ("weight_bytes_per_step", "kv_bytes_per_step", "us_per_layer",
                                                        "host_encode_us_per_layer", "tokens_per_s_at_22_layers")
                           if k in sub["config"]},
                        "frac_of_hbm_peak": sub["roofline"]["frac"],
                        **{k: sub[k] for k in ("cpu_baseline", "parity_vs_cpu_baseline") if k in sub}}
        result["config"]["per_config"] = pc
    print(json.dumps(result))
    return 0


if __name__ == "__main__":
    sys.exit(main())
