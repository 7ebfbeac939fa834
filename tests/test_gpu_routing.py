"""HIP routing metadata against the oracle and the reference's worked example: bit-exact."""

import json
import os

import numpy as np
import pytest
import torch

from oracle import moe_oracle as O
from tests.helpers import hip_backend

pytestmark = pytest.mark.gpu

GOLDEN = os.path.join(os.path.dirname(__file__), "golden", "routing_scatter_example.json")


def _run(idx, E, block_m=64):
    from minitrain_amd.kernels.hip.fused_moe import compute_routing_metadata

    out = compute_routing_metadata(torch.from_numpy(idx).cuda(), E, block_m)
    torch.cuda.synchronize()
    names = ("counts", "expert_start", "x_gather", "s_scatter", "s_reverse", "tile_row_start", "tile_expert",
             "tile_count")
    return {n: t.cpu().numpy() for n, t in zip(names, out)}


def _compare(idx, E, block_m=64):
    got = _run(idx, E, block_m)
    want = O.routing_metadata(idx, E, block_m)
    assert np.array_equal(got["counts"], want.counts)
    assert np.array_equal(got["expert_start"], want.expert_start)
    kept = int(want.expert_start[-1])               # rows exist for the kept routes only (dropped ones carry -1)
    assert np.array_equal(got["s_scatter"][:kept], want.s_scatter_idx[:kept]) and len(want.s_scatter_idx) == kept
    assert np.array_equal(got["s_reverse"], want.s_reverse_scatter_idx)
    assert np.array_equal(got["x_gather"][:kept], want.x_gather_idx[:kept])
    n = int(got["tile_count"][0])
    assert n == len(want.tile_row_start)
    assert np.array_equal(got["tile_row_start"][:n], want.tile_row_start)
    assert np.array_equal(got["tile_expert"][:n], want.tile_expert)


def test_reference_worked_example():
    with open(GOLDEN) as f:
        g = json.load(f)
    got = _run(np.asarray(g["top_k_index"], dtype=np.int32), g["E"], g["BLOCK_M_TOKEN"])
    assert got["expert_start"].tolist() == g["expert_start"]
    assert got["counts"].tolist() == g["counts"]
    assert got["s_scatter"].tolist() == g["s_scatter_idx"]
    assert got["s_reverse"].tolist() == g["s_reverse_scatter_idx"]
    assert got["x_gather"].tolist() == g["x_gather_idx"]
    n = int(got["tile_count"][0])
    assert got["tile_row_start"][:n].tolist() == g["tile_row_start"]
    assert got["tile_expert"][:n].tolist() == g["tile_expert"]


@pytest.mark.parametrize("T,E,K", [(1, 3, 1), (7, 3, 2), (33, 8, 3), (257, 64, 2), (1000, 8, 2), (4097, 8, 2),
                                   (24576, 8, 2), (98304, 8, 2), (5000, 1024, 4), (3000, 300, 8)])
def test_against_oracle(T, E, K):
    print(f"routing T={T} E={E} K={K}", flush=True)
    rng = np.random.Generator(np.random.Philox(T + E + K))
    idx = rng.integers(0, E, size=(T, K)).astype(np.int32)
    _compare(idx, E)


@pytest.mark.parametrize("T,E,K,dropped", [(700, 1025, 2, False), (5000, 3000, 4, True), (300, 65534, 2, False),
                                           (4097, 2048, 8, True)])
def test_more_experts_than_one_window(T, E, K, dropped):
    """Beyond 1024 experts the three kernels run once per window of 1024 expert ids; row offsets and the
    tile list carry over from window to window.  Up to the reference's limit of 65534 experts."""
    print(f"routing windows T={T} E={E} K={K} dropped={dropped}", flush=True)
    rng = np.random.Generator(np.random.Philox(T + E + K))
    idx = rng.integers(0, E, size=(T, K)).astype(np.int32)
    idx[:: max(T // 7, 1), 0] = E - 1                      # the last expert of the last window is used
    if dropped:
        idx[rng.random((T, K)) < 0.15] = -1
    _compare(idx, E)


def test_edge_patterns():
    rng = np.random.Generator(np.random.Philox(8))
    # only experts 0 and 1 of 8 used, the same expert several times within a token (K=3)
    T = 33
    idx = np.stack([(np.arange(T) + s) % 2 for s in range(3)], axis=1).astype(np.int32)
    _compare(idx, 8)
    # every route to the last expert
    _compare(np.full((513, 2), 7, dtype=np.int32), 8)
    # Zipf-like imbalance
    p = np.arange(1, 9) ** -1.2
    p /= p.sum()
    idx = rng.choice(8, size=(24576, 2), p=p).astype(np.int32)
    _compare(idx, 8)
    _compare(idx, 8, block_m=256)


@pytest.mark.parametrize("T,K,E", [(1, 1, 3), (257, 2, 8), (24576, 2, 8), (5000, 3, 64)])
def test_expert_counts_only_mode_matches_bincount(T, K, E):
    """mts_moe_route without the permutation arrays: the router module's count of routes."""
    ops = hip_backend()
    rng = np.random.Generator(np.random.Philox(T + K + E))
    idx = torch.from_numpy(rng.integers(0, E, size=(T, K), dtype=np.int32))
    got = ops.expert_counts(idx.cuda(), E)
    assert got.dtype == torch.int32 and got.shape == (E,)
    assert torch.equal(got.cpu().long(), torch.bincount(idx.flatten().long(), minlength=E))
