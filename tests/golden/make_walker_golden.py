"""Writes tests/golden/walker_tiny_llama.npz: the logits of the reference's own single-stream CPU
runner (DecodeRunner, compiler/runtime/decode_runner.cpp) on the synthetic model that
tests/integration/make_tiny_llama_gguf.py writes, for 4 requests x 8 steps and (the last steps of) 2 requests x 72 steps -- what the reference's
walker test compares BatchedWalker::step against (tests/test_batched_walker_h1.cpp:62-180).

Runs in the build container only (needs the reference checkout): it executes
oracle/_ref/integration/walker_end_to_end in `reference` mode, a program built from the
reference's sources where they lie (tests/integration/Makefile).  No GPU is involved: without a
gfx950 device the reference's operators take their CPU paths.

  make -C tests/integration && python tests/golden/make_walker_golden.py
"""
from __future__ import annotations

import hashlib
import os
import subprocess
import sys
import tempfile

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, os.path.join(ROOT, "tests", "integration"))

REQUESTS, STEPS = 4, 8
# a second run long enough for every request to open a second 64-token page: 2 requests x 72 steps,
# of which the last LONG_KEPT steps' logits are kept
LONG_REQUESTS, LONG_STEPS, LONG_KEPT = 2, 72, 8


def read_logits(path: str) -> np.ndarray:
    raw = np.fromfile(path, np.uint32, 3)
    n_req, n_steps, vocab = (int(v) for v in raw)
    return np.fromfile(path, np.float32, offset=12).reshape(n_req, n_steps, vocab)


def main() -> int:
    import make_tiny_llama_gguf as gen
    blob = gen.build()
    exe = os.path.join(ROOT, "oracle", "_ref", "integration", "walker_end_to_end")
    with tempfile.TemporaryDirectory() as tmp:
        model, out = os.path.join(tmp, "tiny.gguf"), os.path.join(tmp, "logits.bin")
        with open(model, "wb") as fh:
            fh.write(blob)
        subprocess.check_call([exe, "reference", model, out, str(REQUESTS), str(STEPS)])
        logits = read_logits(out)
        subprocess.check_call([exe, "reference", model, out, str(LONG_REQUESTS), str(LONG_STEPS)])
        long_logits = read_logits(out)[:, LONG_STEPS - LONG_KEPT:]
    np.savez_compressed(os.path.join(HERE, "walker_tiny_llama.npz"), logits=logits, long_logits=long_logits,
                        gguf_sha256=np.array(hashlib.sha256(blob).hexdigest()))
    print("wrote walker_tiny_llama.npz", logits.shape, long_logits.shape, "model sha256",
          hashlib.sha256(blob).hexdigest())
    return 0


if __name__ == "__main__":
    sys.exit(main())
