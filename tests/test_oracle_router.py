"""Pins the router part of the CPU oracle against library routines, closed forms,
finite differences and constructed ties (no GPU)."""

import numpy as np
import pytest
import scipy.special as sp
import torch

from oracle import moe_oracle as O


def _logits(T, E, seed, scale=2.0):
    rng = np.random.Generator(np.random.Philox(seed))
    return torch.from_numpy((rng.standard_normal((T, E)) * scale).astype(np.float32))


@pytest.mark.parametrize("T,E,K", [(1, 3, 1), (7, 3, 2), (33, 8, 2), (257, 64, 2), (256, 4, 3)])
@pytest.mark.parametrize("normalize", [True, False])
def test_forward_matches_library_closed_forms(T, E, K, normalize):
    logits = _logits(T, E, 17)
    out = O.router_postprocess(logits, K, normalize=normalize)
    l64 = logits.double().numpy()
    L = sp.logsumexp(l64, axis=1)
    p = sp.softmax(l64, axis=1)
    # untied rows: any correct sort agrees
    ref_idx = np.argsort(-l64, axis=1, kind="stable")[:, :K]
    assert np.array_equal(out.expert_indices.numpy(), ref_idx)
    assert out.expert_indices.dtype == torch.int32
    sel = np.take_along_axis(p, ref_idx, axis=1)
    if normalize:
        # normalised weights are a softmax over the selected logits only
        sel = sp.softmax(np.take_along_axis(l64, ref_idx, axis=1), axis=1)
    np.testing.assert_allclose(out.expert_weights.numpy(), sel, rtol=2e-5, atol=2e-6)
    np.testing.assert_allclose(out.probability_per_expert.numpy(), p.mean(0), rtol=2e-5, atol=1e-7)
    np.testing.assert_allclose(float(out.z_loss), (L ** 2).mean(), rtol=2e-5)
    H = -(p * np.log(np.maximum(p, 1e-9))).sum(1).mean()
    np.testing.assert_allclose(float(out.entropy), H, rtol=2e-5)
    if normalize:
        np.testing.assert_allclose(out.expert_weights.sum(1).numpy(), 1.0, rtol=1e-6)
    # rank order: column 0 carries the largest weight
    assert bool((out.expert_weights[:, :-1] >= out.expert_weights[:, 1:]).all())


def test_tie_rule_lowest_index_wins():
    # all equal: the first K experts, in order
    out = O.router_postprocess(torch.zeros(2, 8), 2, normalize=True)
    assert out.expert_indices.tolist() == [[0, 1], [0, 1]]
    # tie for rank 1/2
    l = torch.tensor([[0.0, 5.0, 1.0, 5.0], [3.0, 1.0, 3.0, 3.0], [9.0, 2.0, 2.0, 2.0]])
    assert O.router_postprocess(l, 2, normalize=False).expert_indices.tolist() == [[1, 3], [0, 2], [0, 1]]
    assert O.router_postprocess(l, 3, normalize=False).expert_indices.tolist() == [[1, 3, 2], [0, 2, 3], [0, 1, 2]]
    # iterative arg-max written out, against the sort-based selection
    rng = np.random.Generator(np.random.Philox(5))
    l = torch.from_numpy(rng.integers(0, 3, size=(500, 8)).astype(np.float32))
    got = O.select_topk_lowest_index(l, 3).numpy()
    for t in range(l.shape[0]):
        row = l[t].clone().numpy()
        for j in range(3):
            e = int(np.argmax(row))            # numpy arg-max returns the first maximum
            assert got[t, j] == e
            row[e] = -np.inf


def test_validation_errors():
    with pytest.raises(ValueError):
        O.router_postprocess(torch.zeros(4), 1, normalize=True)
    with pytest.raises(ValueError):
        O.router_postprocess(torch.zeros(0, 4), 1, normalize=True)
    with pytest.raises(ValueError):
        O.router_postprocess(torch.zeros(3, 4), 5, normalize=True)
    with pytest.raises(ValueError):
        O.router_postprocess(torch.zeros(3, 4), 0, normalize=True)
    with pytest.raises(ValueError):
        O.router_postprocess(torch.zeros(3, 4, dtype=torch.bfloat16), 1, normalize=True)


def _objective(logits, K, normalize, g_w, g_p, g_z):
    out = O.router_postprocess(logits, K, normalize=normalize)
    return (out.expert_weights * g_w).sum() + (out.probability_per_expert * g_p).sum() + g_z * out.z_loss


@pytest.mark.parametrize("T,E,K", [(7, 3, 2), (33, 8, 2), (5, 8, 3), (9, 4, 1)])
@pytest.mark.parametrize("normalize", [True, False])
def test_backward_closed_form_vs_autograd_and_finite_differences(T, E, K, normalize):
    rng = np.random.Generator(np.random.Philox(3))
    logits = torch.from_numpy(rng.standard_normal((T, E))).double()
    g_w = torch.from_numpy(rng.standard_normal((T, K))).double()
    g_p = torch.from_numpy(rng.standard_normal(E)).double()
    g_z = 0.13
    l = logits.clone().requires_grad_(True)
    _objective(l, K, normalize, g_w, g_p, g_z).backward()
    out = O.router_postprocess(logits, K, normalize=normalize)
    closed = O.router_backward_closed(logits, out.expert_indices, out.expert_weights, g_w, g_p, g_z,
                                      normalize=normalize)
    np.testing.assert_allclose(closed, l.grad.numpy(), rtol=1e-9, atol=1e-12)
    # central differences (selection is locally constant on untied rows)
    eps = 1e-6
    fd = np.zeros((T, E))
    for t in range(T):
        for e in range(E):
            lp = logits.clone(); lp[t, e] += eps
            lm = logits.clone(); lm[t, e] -= eps
            fd[t, e] = float(_objective(lp, K, normalize, g_w, g_p, g_z)
                             - _objective(lm, K, normalize, g_w, g_p, g_z)) / (2 * eps)
    np.testing.assert_allclose(closed, fd, rtol=1e-5, atol=1e-7)
