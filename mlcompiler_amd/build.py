"""Builds the in-tree native libraries of the package with hipcc for gfx950.

  libmlc_hip.so       HIP kernels + the C ABI declared in include/mlc_hip.h
  libhip_executor.so  the C++ HipExecutor class (mirror of the reference's
                      MetalExecutor paged-path methods) on top of that ABI
  libmlc_bench.so     native benchmark loops that call the ABI, plus a plain copy kernel
                      used to calibrate the HBM traffic counters
"""
from __future__ import annotations

import hashlib
import os
import shutil
import subprocess

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(PKG_DIR, "csrc")
LIB_PATH = os.path.join(CSRC, "libmlc_hip.so")
EXECUTOR_LIB_PATH = os.path.join(CSRC, "libhip_executor.so")
BENCH_LIB_PATH = os.path.join(CSRC, "libmlc_bench.so")
STAMP_PATH = os.path.join(CSRC, "libmlc_hip.stamp")   # hash of the sources the libraries were built from

# Packed FP32 instructions (v_pk_*_f32) are switched off on purpose: some of their forms have
# produced wrong results on the target machines.  hipcc's host pass prints a harmless
# "not a recognized feature" warning for the flag.
HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-fno-honor-nans",
    "-Wno-inline-asm",  # the global->LDS load in paged_prefill_kernels.h names m0 as clobbered
]


# extra compiler flags for experiments (for example -DMLC_STREAM_PROBE: time stamps per workgroup)
HIPCC_FLAGS += os.environ.get("MLC_HIPCC_EXTRA", "").split()


def source_hash() -> str:
    """Hash over every source the native libraries are built from (and the flags)."""
    h = hashlib.sha256(" ".join(HIPCC_FLAGS).encode())
    files = [os.path.join(CSRC, n) for n in sorted(os.listdir(CSRC))
             if n.endswith((".h", ".hpp", ".hip", ".cpp"))]
    files.append(os.path.join(os.path.dirname(PKG_DIR), "include", "mlc_hip.h"))
    for f in files:
        h.update(os.path.basename(f).encode())
        with open(f, "rb") as fh:
            h.update(fh.read())
    return h.hexdigest()


def built_from_current_sources() -> bool:
    """True when the libraries exist and were built from the sources as they are now."""
    if not all(os.path.exists(p) for p in (LIB_PATH, EXECUTOR_LIB_PATH, BENCH_LIB_PATH, STAMP_PATH)):
        return False
    with open(STAMP_PATH) as fh:
        return fh.read().strip() == source_hash()


def hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found; the HIP extension cannot be built")
    return exe


def _run(cmd: list[str]) -> None:
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if proc.returncode != 0:
        raise RuntimeError("build failed: " + " ".join(cmd) + "\n" + proc.stdout)


def build_all(verbose: bool = False) -> None:
    """Compiles the decode-kernel variants and the runtime in parallel, then links them."""
    from concurrent.futures import ThreadPoolExecutor

    cc = hipcc()
    if os.path.exists(STAMP_PATH):
        os.remove(STAMP_PATH)   # no stamp while the libraries are being replaced
    obj_dir = os.path.join(CSRC, "build")
    os.makedirs(obj_dir, exist_ok=True)
    jobs = []
    for d in (64, 128):
        for h in (1, 2, 4, 8):
            obj = os.path.join(obj_dir, f"decode_d{d}_h{h}.o")
            jobs.append(([cc, *HIPCC_FLAGS, f"-DMLC_D={d}", f"-DMLC_HPW={h}", "-c",
                          os.path.join(CSRC, "paged_decode_inst.hip"), "-o", obj], obj))
    rt_obj = os.path.join(obj_dir, "mlc_hip.o")
    jobs.append(([cc, *HIPCC_FLAGS, "-c", os.path.join(CSRC, "mlc_hip.hip"), "-o", rt_obj], rt_obj))
    with ThreadPoolExecutor(max_workers=min(8, os.cpu_count() or 1)) as pool:
        list(pool.map(lambda j: _run(j[0]), jobs))
    _run([cc, "--offload-arch=gfx950", "-shared", "-fPIC", *[j[1] for j in jobs], "-o", LIB_PATH])
    _run(["g++", "-O2", "-std=c++17", "-fPIC", "-shared", os.path.join(CSRC, "hip_executor.cpp"),
          "-o", EXECUTOR_LIB_PATH, "-L" + CSRC, "-lmlc_hip", "-Wl,-rpath,$ORIGIN"])
    _run([cc, *HIPCC_FLAGS, "-shared", "-x", "hip", os.path.join(CSRC, "bench_loop.cpp"),
          "-o", BENCH_LIB_PATH, "-L" + CSRC, "-lmlc_hip", "-Wl,-rpath,$ORIGIN"])
    with open(STAMP_PATH, "w") as fh:
        fh.write(source_hash() + "\n")
    if verbose:
        print("built", LIB_PATH, EXECUTOR_LIB_PATH, BENCH_LIB_PATH)


if __name__ == "__main__":
    build_all(verbose=True)
