"""The synthetic workloads of the paged attention path (built by mlcompiler_amd.workloads) plus
the two helpers that compare a result with the CPU oracle."""
from __future__ import annotations

import numpy as np

from mlcompiler_amd.workloads import (DecodeCase, DeviceCase, baseline_config, make_case,  # noqa: F401
                                      reference_scenarios)


def oracle_decode(case: DecodeCase, n_threads=8):
    from oracle import paged_oracle as po
    c = case
    return po.paged_attention_executor(c.q, c.k_pages, c.v_pages, c.page_tables_flat,
                                       c.page_table_offsets, c.seq_lens, c.q_positions, c.batch,
                                       c.num_heads, c.kv_heads, c.head_dim, c.page_size,
                                       c.apply_causal, n_threads)


# acceptance bar of the benchmark definition: per (request, head)
MIN_COSINE = 0.9999
MAX_ABS = 2e-3


def assert_parity(got, want, head_dim, what=""):
    from oracle import paged_oracle as po
    assert np.all(np.isfinite(got)), f"{what}: non-finite output"
    rep = po.per_head_report(got, want, head_dim)
    assert rep["min_cosine"] >= MIN_COSINE, f"{what}: {rep}"
    assert rep["max_abs"] <= MAX_ABS, f"{what}: {rep}"
    return rep
