"""Pins the capacity-mask oracle and checks the host-side selection of the router module
against it.  The rule (minitrain/model/moe_router.py:43-61): inside an expert routes are
ranked by descending weight, equal weights by ascending flat entry; rank < capacity stays."""

import numpy as np
import pytest
import torch

from oracle import moe_oracle as O


def _brute(idx, w, E, capacity):
    flat_e = idx.reshape(-1).tolist()
    flat_w = w.reshape(-1).tolist()
    keep = [False] * len(flat_e)
    for e in range(E):
        entries = [n for n, x in enumerate(flat_e) if x == e]
        entries.sort(key=lambda n: (-flat_w[n], n))
        for n in entries[:max(capacity, 0)]:
            keep[n] = True
    return np.asarray(keep).reshape(idx.shape)


def _case(seed, T, K, E, levels=None):
    rng = np.random.Generator(np.random.Philox(seed))
    idx = rng.integers(0, E, size=(T, K)).astype(np.int32)
    w = rng.random(size=(T, K)).astype(np.float32)
    if levels:                                   # few distinct weights: many ties
        w = (np.floor(w * levels) / levels).astype(np.float32)
    return idx, w


@pytest.mark.parametrize("T,K,E,capacity,levels", [
    (1, 1, 3, 1, None), (7, 2, 3, 2, None), (33, 3, 8, 4, 4), (64, 2, 4, 16, 2), (200, 2, 8, 30, None),
    (200, 2, 8, 1000, None), (50, 4, 5, 7, 3), (40, 1, 2, 5, 1),
])
def test_matches_per_expert_sort(T, K, E, capacity, levels):
    idx, w = _case(T * 31 + K, T, K, E, levels)
    got = O.capacity_mask(torch.from_numpy(idx), torch.from_numpy(w), E, capacity).numpy()
    assert np.array_equal(got, _brute(idx, w, E, capacity))


@pytest.mark.parametrize("levels", [None, 5])
def test_invariants(levels):
    T, K, E, capacity = 3000, 2, 8, 500
    idx, w = _case(5, T, K, E, levels)
    keep = O.capacity_mask(torch.from_numpy(idx), torch.from_numpy(w), E, capacity).numpy()
    flat_e, flat_w, flat_k = idx.reshape(-1), w.reshape(-1), keep.reshape(-1)
    for e in range(E):
        mine = np.flatnonzero(flat_e == e)
        kept, dropped = mine[flat_k[mine]], mine[~flat_k[mine]]
        assert kept.size == min(mine.size, capacity)
        if dropped.size:
            assert flat_w[kept].min() >= flat_w[dropped].max()
            edge = flat_w[kept].min()
            tied_kept, tied_dropped = kept[flat_w[kept] == edge], dropped[flat_w[dropped] == edge]
            if tied_dropped.size:
                assert tied_kept.max() < tied_dropped.min()


def test_all_ties_keep_the_first_tokens():
    # K = 1 with normalised weights: every weight is exactly 1
    T, E, capacity = 100, 3, 10
    idx = (np.arange(T) % E).astype(np.int32).reshape(T, 1)
    keep = O.capacity_mask(torch.from_numpy(idx), torch.ones(T, 1), E, capacity).numpy().reshape(-1)
    for e in range(E):
        mine = np.flatnonzero(idx.reshape(-1) == e)
        assert keep[mine[:capacity]].all() and not keep[mine[capacity:]].any()


def test_expert_capacity_formula():
    assert O.expert_capacity(24576, 2, 8, 1.0, 4) == 6144
    assert O.expert_capacity(24576, 2, 8, 1.25, 4) == 7680
    assert O.expert_capacity(10, 2, 8, 1.0, 4) == 4          # the floor wins
    assert O.expert_capacity(7, 2, 3, 1.0, 1) == 5           # ceil(14/3)


def test_apply_capacity_renormalises_per_token():
    w = torch.tensor([[0.75, 0.25], [0.5, 0.5], [0.9, 0.1]])
    keep = torch.tensor([[True, False], [True, True], [False, False]])
    out = O.apply_capacity(w, keep, normalize=True)
    assert torch.allclose(out, torch.tensor([[1.0, 0.0], [0.5, 0.5], [0.0, 0.0]]))
    out = O.apply_capacity(w, keep, normalize=False)
    assert torch.equal(out, torch.tensor([[0.75, 0.0], [0.5, 0.5], [0.0, 0.0]]))


@pytest.mark.parametrize("T,K,E,capacity,levels", [(257, 2, 8, 40, None), (500, 3, 16, 50, 4), (64, 1, 4, 9, 1)])
def test_module_selection_matches_oracle(T, K, E, capacity, levels):
    from minitrain_amd.model.moe_router import capacity_selection

    idx, w = _case(T + K + E, T, K, E, levels)
    idx_t, w_t = torch.from_numpy(idx), torch.from_numpy(w)
    keep, kept_index, accepted = capacity_selection(idx_t, w_t, E, capacity)
    want = O.capacity_mask(idx_t, w_t, E, capacity)
    assert torch.equal(keep, want)
    assert torch.equal(kept_index, torch.where(want, idx_t, torch.full_like(idx_t, -1)))
    assert accepted.tolist() == np.minimum(np.bincount(idx.reshape(-1), minlength=E), capacity).tolist()


def test_dropped_routes_equal_zero_weights_in_the_expert_loop():
    x, _, w1, w2, g = O.make_inputs(3, 40, 16, 4, 24)
    idx, w = _case(9, 40, 2, 4)
    idx_t, w_t = torch.from_numpy(idx), torch.from_numpy(w)
    keep = O.capacity_mask(idx_t, w_t, 4, 12)
    assert not keep.all()
    masked_w = O.apply_capacity(w_t, keep, normalize=True)

    def run(index):
        leaves = [t.clone().requires_grad_(True) for t in (x, w1, w2, masked_w)]
        out = O.fused_moe(leaves[0], leaves[1], leaves[2], index, leaves[3])
        (out * g).sum().backward()
        return out.detach(), [l.grad for l in leaves]

    out_zero, grads_zero = run(idx_t)
    out_drop, grads_drop = run(torch.where(keep, idx_t, torch.full_like(idx_t, -1)))
    assert torch.allclose(out_zero, out_drop, atol=1e-6)
    for a, b in zip(grads_zero[:3], grads_drop[:3]):
        assert torch.allclose(a, b, atol=1e-6)
    # the gradient of a dropped route's weight is defined at zero weight and vanishes once the
    # route has left the dispatch; the router sees neither, both pass through the mask
    assert torch.allclose(grads_zero[3] * keep, grads_drop[3], atol=1e-6)
    assert torch.equal(grads_drop[3][~keep], torch.zeros_like(grads_drop[3][~keep]))


def test_routing_metadata_skips_dropped_routes():
    idx, _ = _case(4, 300, 2, 8)
    idx[::7, 0] = -1
    idx[5::11, 1] = -1
    m = O.routing_metadata(idx, 8)
    flat = idx.reshape(-1)
    kept = np.flatnonzero(flat >= 0)
    assert m.expert_start[-1] == kept.size == m.s_scatter_idx.size
    assert np.array_equal(m.counts, np.bincount(flat[kept], minlength=8))
    assert np.all(m.s_reverse_scatter_idx[flat < 0] == -1)
    assert np.array_equal(m.s_reverse_scatter_idx[m.s_scatter_idx], np.arange(kept.size))
    assert np.all(np.diff(flat[m.s_scatter_idx]) >= 0)


def test_router_metric_record_from_fused_statistics_matches_the_torch_path():
    """Host logic of the router module: the monitoring record taken as views of a backend's
    load statistics carries the same keys and values as the one computed with torch ops
    (keys and formulas of minitrain/model/moe_router.py:113-135)."""
    import math
    import sys
    from pathlib import Path
    from types import SimpleNamespace

    sys.path.insert(0, str(Path(__file__).resolve().parents[1] / "mini-train-sys_amd"))
    from minitrain_amd.model.moe_router import load_metrics, load_metrics_from_stats

    E, routes = 8, 4096
    counts = torch.tensor([900, 0, 300, 512, 512, 1000, 72, 800])
    assert int(counts.sum()) == routes
    frac = counts.double() / routes
    entropy = torch.tensor(1.234)
    stats = torch.cat([frac, torch.tensor([counts.max(), counts.min(), frac.std(unbiased=False) * E, frac.max() * E,
                                           (counts == 0).sum(), 0.0, 1.234 / math.log(E)], dtype=torch.float64)]).float()
    route = SimpleNamespace(entropy=entropy, probability_per_expert=torch.full((E,), 1.0 / E), load_stats=stats)
    fused = load_metrics_from_stats(route, E)
    plain = load_metrics(route, counts.float(), routes, torch.zeros(()), E)
    assert set(fused) == set(plain)
    for key in plain:
        torch.testing.assert_close(fused[key].float(), plain[key].float(), rtol=1e-6, atol=1e-7, msg=key)
        assert fused[key].shape == plain[key].shape, key
