"""Determinism soak of the tile-balanced decode kernel: thousands of launches back to back (no wait
between them inside a batch of 50), at the benchmark's batch-32 and batch-64 configurations and
with the grid size varied, every output compared bit for bit with the first launch of its grid.
A split pair is summed in workgroup order from tagged partials, so the result must not depend on
which workgroup finishes when; a launch that read a partial of the launch before, or summed in
another order, shows up as a mismatch.  Stops at the first one."""
import numpy as np
import pytest

from paged_cases import DeviceCase, baseline_config

pytestmark = pytest.mark.gpu


def _soak(exe, case, grids, launches_per_grid, batch_of=50):
    dev = DeviceCase(exe, case)
    c = case
    nbytes = c.q.nbytes
    outs = [exe.allocateScratchBuffer(nbytes) for _ in range(batch_of)]
    got = np.empty_like(c.q)
    try:
        for grid in grids:
            assert exe.setOption("decode_grid_wgs", grid)
            first = None
            done = 0
            while done < launches_per_grid:
                n = min(batch_of, launches_per_grid - done)
                assert exe.beginForwardPassCB()
                for i in range(n):
                    assert exe.encodePagedFlashAttention(dev.q_buf, dev.k_buf, dev.v_buf, outs[i], c.page_tables_flat,
                                                         c.page_table_offsets, c.seq_lens, c.q_positions, c.batch,
                                                         c.num_heads, c.kv_heads, c.head_dim, c.page_size,
                                                         c.apply_causal), exe.lastError()
                assert exe.flushForwardPassCB(), exe.lastError()
                for i in range(n):
                    assert exe.downloadFromBuffer(outs[i], got)
                    if first is None:
                        first = got.copy()
                        assert np.isfinite(first).all()
                    elif not np.array_equal(got, first):
                        pytest.fail(f"{case.name}: launch {done + i} on a grid of {grid or 'default'} workgroups "
                                    f"differs from the first one (max abs {np.abs(got - first).max():.3e})")
                done += n
            print(f"[soak] {case.name} grid {grid or 'default'}: {launches_per_grid} launches bit-identical", flush=True)
    finally:
        exe.setOption("decode_grid_wgs", 0)
        for o in outs:
            exe.releaseScratchBuffer(o)
        dev.free()


def test_2000_launches_batch32_are_bit_identical(exe):
    _soak(exe, baseline_config(2), grids=(0, 384, 768, 1000), launches_per_grid=500)


def test_500_launches_batch64_are_bit_identical(exe):
    _soak(exe, baseline_config(3), grids=(0, 640), launches_per_grid=250)
