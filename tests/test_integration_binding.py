"""The reference-side binding (tests/integration/metal_runtime_hip.cpp) compiled against the
reference's own metal_runtime.hpp and linked with the reference's paged_kv.cpp on top of
libmlc_hip.so.  The objects and the program are built by __graft_entry__.build() (make -C
tests/integration) where the reference checkout exists and travel with the tree; they are never
part of history."""
import os
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
OUT = os.path.join(ROOT, "oracle", "_ref", "integration")
PROGRAM = os.path.join(OUT, "paged_kv_roundtrip")


def _symbols(path, undefined):
    out = subprocess.run(["nm", "-C", "-u" if undefined else "--defined-only", path], capture_output=True,
                         text=True, check=True).stdout
    syms = set()
    for line in out.splitlines():
        parts = line.split(None, 1 if undefined else 2)
        name = parts[-1].strip()
        if "mlc::runtime::MetalExecutor::" in name:
            syms.add(name)
    return syms


def _need_objects():
    if not os.path.exists(os.path.join(OUT, "metal_runtime_hip.o")):
        pytest.skip("integration objects not built (no reference checkout at build time)")
    if shutil.which("nm") is None:
        pytest.skip("binutils nm not available")


def test_binding_defines_every_executor_symbol_the_paged_path_callers_use():
    """paged_kv.cpp and batched_walker.cpp of the reference, compiled as they are, must find every
    MetalExecutor method they call in the binding: no undefined MetalExecutor symbol is left."""
    _need_objects()
    defined = _symbols(os.path.join(OUT, "metal_runtime_hip.o"), undefined=False)
    assert len(defined) >= 25
    for obj in ("paged_kv.o", "batched_walker.o"):
        wanted = _symbols(os.path.join(OUT, obj), undefined=True)
        assert wanted, obj + " calls no executor method?"
        missing = sorted(wanted - defined)
        assert not missing, f"{obj}: not defined by the binding: {missing}"


def test_program_links_against_the_abi_library_only():
    """The program made of the binding, the reference's paged_kv.cpp and the driver links with
    libmlc_hip.so and nothing else of this repository (no oracle, no Python)."""
    _need_objects()
    assert os.path.exists(PROGRAM)
    out = subprocess.run(["nm", "-C", "-u", PROGRAM], capture_output=True, text=True, check=True).stdout
    mlc = sorted({l.split()[-1] for l in out.splitlines() if "mlc_hip_" in l})
    assert "mlc_hip_paged_attn_decode" in mlc and "mlc_hip_scatter_kv_paged" in mlc
    assert "oracle" not in out


@pytest.mark.gpu
def test_reference_paged_kv_storage_runs_on_the_hip_library(exe):
    """PagedKVStorage::initialize, the scatter(start_slot=3, 11 tokens) / gather round trips of
    tests/test_paged_kv.cpp:404-560 and a decode step, through MetalExecutor::Instance()."""
    assert os.path.exists(PROGRAM), "build it with __graft_entry__.build() where the reference checkout exists"
    proc = subprocess.run([PROGRAM], capture_output=True, text=True, timeout=120)
    print(proc.stdout, proc.stderr, flush=True)
    assert proc.returncode == 0, proc.stdout + proc.stderr
    for name in ("storage_is_zero_filled", "scatter_gather_round_trip_f32", "scatter_gather_round_trip_f16",
                 "decode_step_on_storage"):
        assert name + " ok" in proc.stdout
