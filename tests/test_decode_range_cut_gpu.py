"""The tile-balanced decode kernel cuts the batch's KV tiles into one range per workgroup of equal
cost (a tile one unit, the end of a (request, KV head) pair `decode_pair_cost` units).  Which
workgroups share a pair, where their partials go and who writes a pair's output all follow from
that cut, so it is fuzzed here: random batches (empty requests, one-tile requests, long ones),
GQA ratios, head dims, pair costs and grid sizes, each under two different cuts against the CPU
oracle."""
import numpy as np
import pytest

from paged_cases import DeviceCase, assert_parity, make_case, oracle_decode

pytestmark = pytest.mark.gpu


def _run(exe, case, pair_cost, grid):
    assert exe.setOption("decode_pair_cost", pair_cost)
    assert exe.setOption("decode_grid_wgs", grid)
    dev = DeviceCase(exe, case)
    try:
        return dev.run(sync=True)
    finally:
        dev.free()
        exe.setOption("decode_pair_cost", -1)
        exe.setOption("decode_grid_wgs", 0)


@pytest.mark.parametrize("seed", range(64))
def test_random_batches_under_random_cuts(exe, seed):
    rng = np.random.default_rng(1000 + seed)
    head_dim = int(rng.choice([64, 128]))
    kv_heads = int(rng.choice([1, 2, 4, 8]))
    ratio = int(rng.choice([1, 2, 4, 8, 16]))
    batch = int(rng.choice([1, 2, 5, 17, 40, 64, 65, 90]))
    kind = rng.integers(0, 3)
    if kind == 0:      # many short requests, some empty: ranges that hold many pairs
        lens = rng.integers(0, 3 * 64, batch)
        lens[rng.random(batch) < 0.25] = 0
    elif kind == 1:    # a few long ones among short ones: pairs cut many times
        lens = rng.integers(1, 200, batch)
        lens[rng.integers(0, batch, max(1, batch // 8))] = rng.integers(1500, 5000)
    else:              # lengths around tile and page boundaries
        lens = rng.choice([1, 31, 32, 33, 63, 64, 65, 127, 128, 129, 640], batch)
    if not lens.any():
        lens[0] = 70
    case = make_case(f"cut{seed}", batch, kv_heads * ratio, kv_heads, head_dim, 64, lens, seed=seed)
    pair_cost = int(rng.integers(0, 8))
    grid = int(rng.choice([0, 1, 3, 17, 100, 512, 1000]))
    print(f"[cut] seed={seed} B={batch} H={kv_heads * ratio}/{kv_heads} D={head_dim} lens(sum)={int(lens.sum())} "
          f"pair_cost={pair_cost} grid={grid}", flush=True)
    got = _run(exe, case, pair_cost, grid)
    want = oracle_decode(case)
    assert want is not None
    assert_parity(got, want, head_dim, case.name)
    # another cut of the same call (other partials, merged in another order)
    other = _run(exe, case, (pair_cost + 3) % 8, 0 if grid else 37)
    assert_parity(other, want, head_dim, case.name + " (second cut)")
