"""Host-side checks that need no GPU: the native library loads, exports every symbol that
include/mlc_hip.h declares, and fails loudly (never falls back) without a device."""
import ctypes as C
import os
import re

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_symbols():
    text = open(os.path.join(ROOT, "include", "mlc_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(mlc_hip_\w+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    from mlcompiler_amd._lib import SIGNATURES, load
    lib = load()
    declared = _declared_symbols()
    assert len(declared) >= 20
    for name in declared:
        assert hasattr(lib, name), f"{name} declared in include/mlc_hip.h but not exported"
    assert sorted(SIGNATURES) == declared, "ctypes binding and header disagree"


def test_cpp_executor_and_bench_libraries_load():
    from mlcompiler_amd.build import BENCH_LIB_PATH, EXECUTOR_LIB_PATH
    for path in (EXECUTOR_LIB_PATH, BENCH_LIB_PATH):
        assert os.path.exists(path), path
        C.CDLL(path)
    lib = C.CDLL(BENCH_LIB_PATH)
    for name in ("mlc_bench_decode_loop", "mlc_bench_decode_step_loop", "mlc_bench_prefill_loop"):
        assert hasattr(lib, name)


def test_no_silent_fallback_without_a_gpu():
    import torch  # noqa: F401  (only to ask whether a device exists)
    from mlcompiler_amd import HipExecutor, NativeLibraryError
    exe = HipExecutor.Instance()
    if exe.isAvailable():
        pytest.skip("a gfx950 device is present")
    with pytest.raises(NativeLibraryError):
        exe.requireAvailable()
    assert exe.allocateScratchBuffer(64) == 0
    dummy = np.zeros(4, np.uint32)
    assert not exe.runPagedFlashAttention(1, 1, 1, 1, dummy[:1], dummy[:2], dummy[:1], dummy[:1],
                                          1, 8, 2, 64, 64, True)
    assert not exe.scatterKVPagedBatched(1, [0], [0], 64, 2, 64, 1, 1)
    assert "unavailable" in exe.lastError().lower() or "no hip device" in exe.lastError().lower()
    assert not exe.beginForwardPassCB()


def test_product_package_never_imports_the_oracle():
    pkg = os.path.join(ROOT, "mlcompiler_amd")
    for dirpath, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".cpp", ".hip", ".h", ".hpp")):
                text = open(os.path.join(dirpath, f)).read()
                assert "oracle" not in text.lower() or f == "__init__.py" and "oracle" not in text, \
                    f"{f} mentions the oracle"


def test_reference_scenarios_are_well_formed():
    from paged_cases import baseline_config, reference_scenarios
    sc = reference_scenarios()
    assert [s.name for s in sc][:2] == ["SingleRequestSmall", "TwoRequestsDisjointPages"]
    for s in sc:
        assert s.page_table_offsets[-1] == s.page_tables_flat.size <= s.capacity_pages
    c2 = baseline_config(2)
    assert c2.batch == 32 and c2.num_heads == 32 and c2.kv_heads == 4 and c2.head_dim == 64
    assert 128 <= c2.seq_lens.min() and c2.seq_lens.max() <= 2048
    assert c2.kv_bytes == int(c2.seq_lens.sum()) * 1024
    assert len(set(c2.page_tables_flat.tolist())) == c2.page_tables_flat.size  # disjoint pages
