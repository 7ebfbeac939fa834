"""Pins the fused-MoE part of the CPU oracle: brute force, closed-form gradients,
finite differences (no GPU)."""

import numpy as np
import pytest
import torch

from oracle import moe_oracle as O


def _case(T, E, K, H, I, seed, *, empty_expert=True, zero_weight=True, duplicate=False):
    rng = np.random.Generator(np.random.Philox(seed))
    x = torch.from_numpy(rng.standard_normal((T, H)))
    w1 = torch.from_numpy(rng.standard_normal((E, 2 * I, H)) * 0.3)
    w2 = torch.from_numpy(rng.standard_normal((E, H, I)) * 0.3)
    idx = np.stack([rng.permutation(E)[:K] for _ in range(T)]).astype(np.int32)
    if duplicate:
        idx[::2, -1] = idx[::2, 0]            # same expert twice within a token
    if empty_expert and E > 2:
        idx[idx == E - 1] = 0 if duplicate else idx[idx == E - 1]
        if not duplicate:
            # remap the last expert onto a free one per row where possible
            for t in range(T):
                for k in range(K):
                    if idx[t, k] == E - 1:
                        free = [e for e in range(E - 1) if e not in idx[t]]
                        idx[t, k] = free[0] if free else 0
    s = torch.from_numpy(rng.random((T, K)))
    if zero_weight:
        s[::2, -1] = 0.0
    g = torch.from_numpy(rng.standard_normal((T, H)))
    return x, w1, w2, torch.from_numpy(idx), s, g


@pytest.mark.parametrize("T,E,K,H,I,dup", [(7, 3, 2, 4, 5, False), (5, 4, 3, 6, 3, True), (1, 2, 1, 3, 2, False)])
def test_forward_vs_bruteforce(T, E, K, H, I, dup):
    x, w1, w2, idx, s, _ = _case(T, E, K, H, I, 11, duplicate=dup)
    got = O.fused_moe(x, w1, w2, idx, s)
    want = O.fused_moe_bruteforce(x, w1, w2, idx, s)
    np.testing.assert_allclose(got.numpy(), want, rtol=1e-12, atol=1e-13)


@pytest.mark.parametrize("T,E,K,H,I,dup", [(7, 3, 2, 4, 5, False), (6, 4, 3, 5, 3, True)])
def test_backward_closed_form_vs_autograd_and_finite_differences(T, E, K, H, I, dup):
    x, w1, w2, idx, s, g = _case(T, E, K, H, I, 12, duplicate=dup)
    leaves = [t.clone().requires_grad_(True) for t in (x, w1, w2, s)]
    out = O.fused_moe(leaves[0], leaves[1], leaves[2], idx, leaves[3])
    (out * g).sum().backward()
    dx, dw1, dw2, dS = O.fused_moe_backward_closed(x, w1, w2, idx, s, g)
    for got, want in zip((dx, dw1, dw2, dS), (l.grad.numpy() for l in leaves)):
        np.testing.assert_allclose(got, want, rtol=1e-10, atol=1e-12)
    # zero-weight routes still receive a gradient
    assert np.abs(dS[::2, -1]).min() > 0
    # experts without routes get exactly zero weight gradients
    used = set(idx.flatten().tolist())
    for e in range(E):
        if e not in used:
            assert not dw1[e].any() and not dw2[e].any()

    def f(xx, a, b, ss):
        return float((O.fused_moe(xx, a, b, idx, ss) * g).sum())

    eps = 1e-6
    rng = np.random.Generator(np.random.Philox(1))
    for which, (tensor, grad) in enumerate(zip((x, w1, w2, s), (dx, dw1, dw2, dS))):
        flat = tensor.flatten()
        for pos in rng.choice(flat.numel(), size=min(25, flat.numel()), replace=False):
            args_p = [x.clone(), w1.clone(), w2.clone(), s.clone()]
            args_m = [x.clone(), w1.clone(), w2.clone(), s.clone()]
            args_p[which].view(-1)[pos] += eps
            args_m[which].view(-1)[pos] -= eps
            fd = (f(*args_p) - f(*args_m)) / (2 * eps)
            np.testing.assert_allclose(grad.reshape(-1)[pos], fd, rtol=2e-5, atol=1e-7)


def test_input_dtype_path_matches_wide_path_in_fp32():
    x, w_r, w1, w2, g = O.make_inputs(0, 256, 64, 4, 128)
    hidden, r = O.moe_feed_forward(x, w_r, w1, w2, 2)
    wide, _ = O.moe_feed_forward(x, w_r, w1, w2, 2, compute_dtype=torch.float64)
    st = O.error_stats(hidden, wide)
    assert st["max_rel_scaled"] < 1e-5, st
    # caller arithmetic: aux = E * sum_e f_e * pbar_e with f from the assignment counts
    counts = np.bincount(r.expert_indices.flatten().numpy(), minlength=4)
    aux = 4 * float((torch.from_numpy(counts / counts.sum()).float() * r.route.probability_per_expert).sum())
    np.testing.assert_allclose(float(r.auxiliary_loss), aux, rtol=1e-6)
    assert r.expert_indices.dtype == torch.int32 and r.expert_weights.dtype == x.dtype


def test_make_inputs_is_deterministic_and_scaled():
    a = O.make_inputs(1, 64, 16, 4, 8)
    b = O.make_inputs(1, 64, 16, 4, 8)
    for u, v in zip(a, b):
        assert torch.equal(u, v)
    assert abs(float(a[0].std()) - 1.0) < 0.1 and abs(float(a[2].std()) - 0.02) < 0.004


def test_tie_injection_straddles_the_boundary():
    logits = torch.zeros(300, 8).normal_(generator=torch.Generator().manual_seed(0))
    tied = O.inject_ties(logits, 0.05, 3)
    changed = (tied != logits).any(dim=1)
    assert 10 <= int(changed.sum()) <= 20
    srt = torch.sort(tied[changed], dim=1, descending=True).values
    assert bool(((srt[:, 0] == srt[:, 1]) | (srt[:, 1] == srt[:, 2])).all())
