"""One TinyLlama-shape decoder layer of the reference's batched decode step
(compiler/runtime/batched_walker.cpp:246-405): inputs from mlcompiler_amd.workloads, expected
output from the chain of CPU oracles."""
from mlcompiler_amd.workloads import (D, FFN, H, HID, HKV, KV_ROWS, P, Q_ROWS, QKV_ROWS,  # noqa: F401
                                      make_layer_weights, weight_bytes)
from oracle.layer_chain import oracle_chain, rotary_tables  # noqa: F401
