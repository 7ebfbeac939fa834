"""HIP router post-process against the CPU oracle (through the C ABI)."""

import numpy as np
import pytest
import torch

from oracle import moe_oracle as O
from tests.helpers import hip_backend

pytestmark = pytest.mark.gpu

FWD_TOL = 2e-5   # weights / mean probability / z-loss / entropy
BWD_TOL = 5e-5   # dlogits


def _logits(T, E, seed, scale=1.5):
    rng = np.random.Generator(np.random.Philox(seed))
    return torch.from_numpy((rng.standard_normal((T, E)) * scale).astype(np.float32))


def _check(logits, K, normalize, *, tied=False):
    ops = hip_backend()
    ref = O.router_postprocess(logits, K, normalize=normalize)
    lg = logits.cuda().requires_grad_(True)
    got = ops.router_postprocess(lg, K, normalize=normalize)
    assert got.expert_indices.dtype == torch.int32 and got.expert_weights.dtype == torch.float32
    assert torch.equal(got.expert_indices.cpu(), ref.expert_indices), "routing indices must be bit-exact"
    torch.testing.assert_close(got.expert_weights.cpu(), ref.expert_weights, rtol=FWD_TOL, atol=FWD_TOL)
    torch.testing.assert_close(got.probability_per_expert.cpu(), ref.probability_per_expert, rtol=FWD_TOL, atol=FWD_TOL)
    torch.testing.assert_close(got.z_loss.cpu(), ref.z_loss, rtol=FWD_TOL, atol=FWD_TOL)
    torch.testing.assert_close(got.entropy.cpu(), ref.entropy, rtol=FWD_TOL, atol=FWD_TOL)
    assert not got.expert_indices.requires_grad and not got.entropy.requires_grad
    # the bookkeeping of the router module, computed in the same pass: routes per expert (exact)
    # and the load-balancing term E * sum_e f_e * pbar_e
    T_, E_ = logits.shape
    ref_counts = torch.bincount(ref.expert_indices.flatten().long(), minlength=E_)
    assert got.expert_counts.dtype == torch.int32 and torch.equal(got.expert_counts.cpu().long(), ref_counts)
    ref_lb = E_ * torch.sum(ref_counts.double() / (T_ * K) * ref.probability_per_expert.double())
    torch.testing.assert_close(got.load_balance_loss.cpu().double(), ref_lb, rtol=FWD_TOL, atol=FWD_TOL)
    # the module's load metrics (minitrain/model/moe_router.py:113-135) from the same pass, against numpy in fp64
    frac = ref_counts.double().numpy() / (T_ * K)
    want = np.concatenate([frac, [ref_counts.max().item(), ref_counts.min().item(), frac.std() * E_, frac.max() * E_,
                                  float((ref_counts == 0).sum()), 0.0,
                                  float(ref.entropy) / (np.log(E_) if E_ > 1 else 1.0)]])
    stats = got.load_stats.cpu().double().numpy()
    assert got.load_stats.dtype == torch.float32 and stats.shape == (E_ + 7,) and not got.load_stats.requires_grad
    np.testing.assert_allclose(stats, want, rtol=2e-5, atol=2e-6)
    assert stats[E_] == want[E_] and stats[E_ + 1] == want[E_ + 1] and stats[E_ + 4] == want[E_ + 4]   # counts are exact
    # backward through the combined objective of the reference's parity probe
    T, E = logits.shape
    rng = np.random.Generator(np.random.Philox(99))
    g_w = torch.from_numpy(rng.standard_normal((T, K)).astype(np.float32))
    g_p = torch.from_numpy(rng.standard_normal(E).astype(np.float32))
    obj = ((got.expert_weights * g_w.cuda()).sum() + (got.probability_per_expert * g_p.cuda()).sum()
           + 0.13 * got.z_loss + 0.37 * got.load_balance_loss)
    obj.backward()
    # the load-balancing term reaches the logits through the mean probability only
    g_p_eff = g_p + (0.37 * E * ref_counts.double() / (T * K)).float()
    closed = O.router_backward_closed(logits, ref.expert_indices, ref.expert_weights.double(), g_w, g_p_eff, 0.13,
                                      normalize=normalize)
    np.testing.assert_allclose(lg.grad.cpu().numpy(), closed, rtol=BWD_TOL, atol=BWD_TOL)


@pytest.mark.parametrize("T", [1, 7, 33, 256, 257])
@pytest.mark.parametrize("E,K", [(3, 1), (3, 2), (4, 2), (8, 2), (8, 3), (64, 2), (64, 3)])
@pytest.mark.parametrize("normalize", [True, False])
def test_router_matrix(T, E, K, normalize):
    print(f"router T={T} E={E} K={K} normalize={normalize}", flush=True)
    _check(_logits(T, E, 17 + T + E), K, normalize)


@pytest.mark.parametrize("E,K", [(16, 2), (40, 4), (129, 8), (300, 2), (512, 2), (1000, 8), (1024, 2)])
def test_router_wide(E, K):
    print(f"router wide E={E} K={K}", flush=True)
    _check(_logits(97, E, E), K, True)
    _check(_logits(97, E, E + 1), K, False)


def test_router_ties_lowest_index_wins():
    print("router ties", flush=True)
    ops = hip_backend()
    l = torch.zeros(5, 8)
    got = ops.router_postprocess(l.cuda(), 2, normalize=True)
    assert got.expert_indices.cpu().tolist() == [[0, 1]] * 5
    rng = np.random.Generator(np.random.Philox(5))
    for E, K in [(8, 2), (8, 3), (4, 2), (64, 2), (200, 3)]:
        l = torch.from_numpy(rng.integers(0, 3, size=(4099, E)).astype(np.float32))
        got = ops.router_postprocess(l.cuda(), K, normalize=False)
        want = O.router_postprocess(l, K, normalize=False)
        assert torch.equal(got.expert_indices.cpu(), want.expert_indices)
        torch.testing.assert_close(got.expert_weights.cpu(), want.expert_weights, rtol=FWD_TOL, atol=FWD_TOL)


def test_router_config2_and_config4_shapes():
    print("router 24576x8 incl. Zipf bias and injected ties", flush=True)
    x, w_r, _, _, _ = O.make_inputs(3, 24576, 768, 8, 8)
    logits = torch.nn.functional.linear(x.bfloat16().float(), w_r) + O.zipf_log_bias(8)
    logits = O.inject_ties(logits, 0.01, 3)
    _check(logits, 2, True)
    ref = O.router_postprocess(logits, 2, normalize=True)
    share = np.bincount(ref.expert_indices.flatten().numpy(), minlength=8) / ref.expert_indices.numel()
    assert share.max() > 0.25          # the load really is imbalanced


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("normalize", [True, False])
def test_router_weights_in_the_activation_dtype(dtype, normalize):
    """``weights_dtype`` adds the copy of the weights the router module makes for the MoE block
    (minitrain/model/moe_router.py:139-140): bit-identical to ``expert_weights.to(dtype)``, and a
    gradient that arrives at it gives the logits gradient the cast's own backward would give."""
    print(f"router weights cast {dtype} normalize={normalize}", flush=True)
    ops = hip_backend()
    assert ops.casts_router_weights
    T, E, K = 1000, 8, 2
    logits = _logits(T, E, 17)
    g = torch.from_numpy(np.random.Generator(np.random.Philox(5)).standard_normal((T, K)).astype(np.float32)).cuda()
    a = logits.cuda().requires_grad_(True)
    got = ops.router_postprocess(a, K, normalize=normalize, weights_dtype=dtype)
    assert got.expert_weights_cast.dtype == dtype and got.expert_weights.dtype == torch.float32
    assert torch.equal(got.expert_weights_cast, got.expert_weights.to(dtype))
    ((got.expert_weights_cast.float() * g).sum() + 0.5 * got.expert_weights.sum()).backward()
    b = logits.cuda().requires_grad_(True)
    plain = ops.router_postprocess(b, K, normalize=normalize)
    assert plain.expert_weights_cast is None
    ((plain.expert_weights.to(dtype).float() * g).sum() + 0.5 * plain.expert_weights.sum()).backward()
    # the same numbers enter the same kernel, once as a 16-bit tensor and once widened by torch
    assert torch.equal(a.grad, b.grad)
    with pytest.raises(ValueError):
        ops.router_postprocess(a, K, normalize=normalize, weights_dtype=torch.float64)


def test_router_errors_and_determinism():
    ops = hip_backend()
    with pytest.raises(ValueError):
        ops.router_postprocess(torch.zeros(4, device="cuda"), 1, normalize=True)
    with pytest.raises(ValueError):
        ops.router_postprocess(torch.zeros(0, 4, device="cuda"), 1, normalize=True)
    with pytest.raises(ValueError):
        ops.router_postprocess(torch.zeros(3, 4, device="cuda"), 5, normalize=True)
    with pytest.raises(ValueError):
        ops.router_postprocess(torch.zeros(3, 4, device="cuda", dtype=torch.bfloat16), 1, normalize=True)
    with pytest.raises(RuntimeError):
        ops.router_postprocess(torch.zeros(3, 4), 1, normalize=True)          # CPU tensor: no fallback
    with pytest.raises(RuntimeError):
        ops.router_postprocess(torch.zeros(3, 16, device="cuda"), 9, normalize=True)
    l = _logits(5000, 8, 1).cuda()
    a = ops.router_postprocess(l, 2, normalize=True)
    b = ops.router_postprocess(l, 2, normalize=True)
    for u, v in zip((a.expert_weights, a.probability_per_expert, a.z_loss, a.entropy),
                    (b.expert_weights, b.probability_per_expert, b.z_loss, b.entropy)):
        assert torch.equal(u, v), "statistics must be bit-stable from run to run"
    # non-contiguous logits are accepted
    wide = _logits(64, 16, 2).cuda()
    got = ops.router_postprocess(wide[:, ::2], 2, normalize=True)
    want = O.router_postprocess(wide[:, ::2].cpu().contiguous(), 2, normalize=True)
    assert torch.equal(got.expert_indices.cpu(), want.expert_indices)
