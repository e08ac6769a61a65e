"""The reference's unchanged BatchedWalker::step on top of libmlc_hip.so, end to end, as the
reference tests it (tests/test_batched_walker_h1.cpp:62-180): per request and step, the logits of
the batched walker against those of the reference's single-stream CPU runner on the same model,
cosine >= 0.999 (the reference's bar), and the same arg-max.

The model is the synthetic Llama-topology GGUF of tests/integration/make_tiny_llama_gguf.py
(2 layers, hidden 512, 8 query / 2 KV heads of 64, Q4_0 projections, Q6_K output matrix); the
expected logits are a committed fixture written by tests/golden/make_walker_golden.py from the
reference's own DecodeRunner.  The program under test is oracle/_ref/integration/walker_end_to_end,
built from the reference's batched_walker.cpp / batched_executor.cpp where they lie plus this
repository's binding (tests/integration/Makefile); it is run as a child process."""
import hashlib
import os
import subprocess
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, os.path.join(ROOT, "tests", "integration"))
sys.path.insert(0, os.path.join(ROOT, "tests", "golden"))

pytestmark = pytest.mark.gpu

PROGRAM = os.path.join(ROOT, "oracle", "_ref", "integration", "walker_end_to_end")


@pytest.fixture(scope="module")
def model(tmp_path_factory):
    import make_tiny_llama_gguf as gen
    golden = np.load(os.path.join(ROOT, "tests", "golden", "walker_tiny_llama.npz"))
    blob = gen.build()
    if hashlib.sha256(blob).hexdigest() != str(golden["gguf_sha256"]):
        pytest.fail("the generated model differs from the one the fixture was computed on "
                    "(another numpy random stream?): run tests/golden/make_walker_golden.py")
    path = tmp_path_factory.mktemp("walker") / "tiny.gguf"
    path.write_bytes(blob)
    return str(path), golden["logits"], golden["long_logits"]


@pytest.mark.parametrize("requests", [1, 2, 4])
def test_walker_logits_match_the_single_stream_cpu_runner(model, requests, tmp_path):
    from make_walker_golden import STEPS, read_logits
    path, want, _ = model
    if not os.path.exists(PROGRAM):
        pytest.fail(f"{PROGRAM} is not built (make -C tests/integration, needs the reference checkout)")
    out = str(tmp_path / "logits.bin")
    print(f"[walker] {requests} request(s) x {STEPS} steps", flush=True)
    proc = subprocess.run([PROGRAM, "walker", path, out, str(requests), str(STEPS)], stdout=subprocess.PIPE,
                          stderr=subprocess.STDOUT, text=True, timeout=110)
    assert proc.returncode == 0, proc.stdout
    got = read_logits(out)
    assert got.shape == (requests, STEPS, want.shape[2])
    worst = 1.0
    for r in range(requests):
        for i in range(STEPS):
            a, b = got[r, i].astype(np.float64), want[r, i].astype(np.float64)
            cos = float(a @ b / np.sqrt((a @ a) * (b @ b)))
            worst = min(worst, cos)
            assert cos >= 0.999, (r, i, cos)
            assert int(np.argmax(a)) == int(np.argmax(b)), (r, i)
    print(f"[walker] worst cosine {worst:.7f}", flush=True)


def test_walker_across_a_page_boundary(model, tmp_path):
    """72 steps per request: the reference's PagePool hands every request a second 64-token page on
    the way, the KV writes and the paged attention go on across it; the last steps' logits against the
    single-stream CPU runner's."""
    from make_walker_golden import LONG_KEPT, LONG_REQUESTS, LONG_STEPS, read_logits
    path, _, want = model
    if not os.path.exists(PROGRAM):
        pytest.fail(f"{PROGRAM} is not built (make -C tests/integration, needs the reference checkout)")
    out = str(tmp_path / "logits_long.bin")
    print(f"[walker] {LONG_REQUESTS} requests x {LONG_STEPS} steps", flush=True)
    proc = subprocess.run([PROGRAM, "walker", path, out, str(LONG_REQUESTS), str(LONG_STEPS)], stdout=subprocess.PIPE,
                          stderr=subprocess.STDOUT, text=True, timeout=110)
    assert proc.returncode == 0, proc.stdout
    got = read_logits(out)[:, LONG_STEPS - LONG_KEPT:]
    assert got.shape == want.shape
    worst = 1.0
    for r in range(LONG_REQUESTS):
        for i in range(LONG_KEPT):
            a, b = got[r, i].astype(np.float64), want[r, i].astype(np.float64)
            cos = float(a @ b / np.sqrt((a @ a) * (b @ b)))
            worst = min(worst, cos)
            assert cos >= 0.999, (r, i, cos)
            assert int(np.argmax(a)) == int(np.argmax(b)), (r, i)
    print(f"[walker] worst cosine {worst:.7f}", flush=True)
