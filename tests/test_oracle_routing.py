"""Pins the routing-metadata oracle: the reference's worked example plus invariants."""

import json
import os

import numpy as np
import pytest

from oracle import moe_oracle as O

GOLDEN = os.path.join(os.path.dirname(__file__), "golden", "routing_scatter_example.json")


def test_reference_worked_example():
    with open(GOLDEN) as f:
        g = json.load(f)
    meta = O.routing_metadata(np.asarray(g["top_k_index"], dtype=np.int32), g["E"], block_m=g["BLOCK_M_TOKEN"])
    assert meta.expert_start.tolist() == g["expert_start"]
    assert meta.counts.tolist() == g["counts"]
    assert meta.s_scatter_idx.tolist() == g["s_scatter_idx"]
    assert meta.s_reverse_scatter_idx.tolist() == g["s_reverse_scatter_idx"]
    assert meta.x_gather_idx.tolist() == g["x_gather_idx"]
    assert meta.tile_row_start.tolist() == g["tile_row_start"]
    assert meta.tile_expert.tolist() == g["tile_expert"]


@pytest.mark.parametrize("T,E,K,seed", [(1, 3, 1, 0), (7, 3, 2, 1), (33, 8, 3, 2), (257, 64, 2, 3), (1000, 8, 2, 4)])
def test_invariants(T, E, K, seed):
    rng = np.random.Generator(np.random.Philox(seed))
    idx = rng.integers(0, E, size=(T, K)).astype(np.int32)
    if E > 2:
        idx[idx == 1] = 0                     # leave an empty expert
    m = O.routing_metadata(idx, E)
    TK = T * K
    flat = idx.reshape(-1)
    assert m.expert_start[0] == 0 and m.expert_start[-1] == TK
    assert np.array_equal(np.diff(m.expert_start), m.counts)
    assert np.array_equal(m.s_reverse_scatter_idx[m.s_scatter_idx], np.arange(TK))
    assert np.array_equal(m.x_gather_idx, m.s_scatter_idx // K)
    sorted_e = flat[m.s_scatter_idx]
    assert np.all(np.diff(sorted_e) >= 0)
    for e in range(E):
        seg = m.s_scatter_idx[m.expert_start[e]:m.expert_start[e + 1]]
        assert np.all(np.diff(seg) > 0)       # ascending entry inside an expert
        assert np.all(flat[seg] == e)
    assert len(m.tile_row_start) == sum(-(-int(c) // 64) for c in m.counts)
