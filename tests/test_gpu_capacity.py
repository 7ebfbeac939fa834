"""Capacity-limited dispatch on the GPU: the accepted-route mask (bit-exact against the
oracle), routing metadata and fused MoE with dropped routes, and the router module."""

import numpy as np
import pytest
import torch

from oracle import moe_oracle as O
from tests.helpers import BF16_TOL, assert_close_scaled, hip_backend, hip_moe_grads, oracle_moe_grads, routed_case

pytestmark = pytest.mark.gpu


def _mask_case(seed, T, K, E, levels=None, zipf=False):
    rng = np.random.Generator(np.random.Philox(seed))
    if zipf:
        p = np.arange(1, E + 1) ** -1.2
        idx = rng.choice(E, size=(T, K), p=p / p.sum()).astype(np.int32)
    else:
        idx = rng.integers(0, E, size=(T, K)).astype(np.int32)
    w = rng.random(size=(T, K)).astype(np.float32)
    if levels:
        w = (np.floor(w * levels) / levels).astype(np.float32)
    return torch.from_numpy(idx), torch.from_numpy(w)


def _check_mask(idx, w, E, capacity):
    ops = hip_backend()
    keep, kept_index, accepted = ops.capacity_mask(idx.cuda(), w.cuda(), E, capacity)
    torch.cuda.synchronize()
    want = O.capacity_mask(idx, w, E, capacity)
    assert keep.dtype == torch.bool and kept_index.dtype == torch.int32 and accepted.dtype == torch.int32
    assert torch.equal(keep.cpu(), want)
    assert torch.equal(kept_index.cpu(), torch.where(want, idx, torch.full_like(idx, -1)))
    counts = torch.bincount(idx.flatten().long(), minlength=E)
    assert torch.equal(accepted.cpu().long(), counts.clamp(max=max(capacity, 0)))


@pytest.mark.parametrize("T,K,E,capacity,levels,zipf", [
    (1, 1, 3, 1, None, False), (7, 2, 3, 2, None, False), (257, 3, 8, 40, 4, False), (1000, 2, 8, 250, None, False),
    (1000, 2, 8, 5000, None, False), (5000, 1, 4, 900, 1, False), (24576, 2, 8, 6144, None, False),
    (24576, 2, 8, 6144, None, True), (24576, 2, 8, 6144, 7, True), (98304, 2, 8, 24576, None, True),
    (5000, 4, 300, 50, 3, False), (3000, 8, 1024, 4, None, False), (4097, 2, 8, 1, 2, False),
])
def test_mask_matches_oracle(T, K, E, capacity, levels, zipf):
    print(f"capacity mask T={T} K={K} E={E} C={capacity} levels={levels} zipf={zipf}", flush=True)
    idx, w = _mask_case(T + K + E + capacity, T, K, E, levels, zipf)
    _check_mask(idx, w, E, capacity)


def test_mask_on_router_output_with_exact_ties():
    """Weights as the router makes them: K=1 normalised gives 1.0 everywhere, so the whole
    decision rests on the entry order; K=2 on tied logits gives pairs of equal weights."""
    print("capacity mask router ties", flush=True)
    case = routed_case(3, 4096, 64, 8, 64, 1)
    _check_mask(case["idx"], case["route"].expert_weights, 8, 300)
    case = routed_case(4, 4096, 64, 8, 64, 2, tie_fraction=0.2)
    _check_mask(case["idx"], case["route"].expert_weights, 8, 700)


def _routing(idx, E):
    from minitrain_amd.kernels.hip.fused_moe import compute_routing_metadata

    out = compute_routing_metadata(idx.cuda(), E, 64)
    torch.cuda.synchronize()
    names = ("counts", "expert_start", "x_gather", "s_scatter", "s_reverse", "tile_row_start", "tile_expert",
             "tile_count")
    return {n: t.cpu().numpy() for n, t in zip(names, out)}


@pytest.mark.parametrize("T,K,E", [(7, 2, 3), (1000, 2, 8), (24576, 2, 8), (5000, 3, 64)])
def test_routing_metadata_with_dropped_routes(T, K, E):
    print(f"routing with drops T={T} K={K} E={E}", flush=True)
    idx, w = _mask_case(T, T, K, E, zipf=E == 8)
    keep = O.capacity_mask(idx, w, E, max(1, T * K // E // 2))
    dropped = torch.where(keep, idx, torch.full_like(idx, -1))
    got = _routing(dropped, E)
    want = O.routing_metadata(dropped.numpy(), E, 64)
    kept = int(want.expert_start[-1])
    assert kept < T * K
    assert np.array_equal(got["counts"], want.counts)
    assert np.array_equal(got["expert_start"], want.expert_start)
    assert np.array_equal(got["s_reverse"], want.s_reverse_scatter_idx)
    assert np.array_equal(got["s_scatter"][:kept], want.s_scatter_idx)
    assert np.array_equal(got["x_gather"][:kept], want.x_gather_idx)
    n = int(got["tile_count"][0])
    assert n == len(want.tile_row_start)
    assert np.array_equal(got["tile_row_start"][:n], want.tile_row_start)
    assert np.array_equal(got["tile_expert"][:n], want.tile_expert)


def _moe_with_drops(case, capacity, *, tol):
    """The compacted dispatch must give what the reference's convention for a dropped route,
    a zero weight on a route that is still dispatched, gives: outputs, dx, dW1, dW2, and the
    weight gradient on the routes that stayed (zero on the ones that left)."""
    E = case["w1"].shape[0]
    keep = O.capacity_mask(case["idx"], case["route"].expert_weights, E, capacity)
    assert not keep.all()
    w = O.apply_capacity(case["route"].expert_weights, keep, normalize=True).to(case["x"].dtype)
    dropped = torch.where(keep, case["idx"], torch.full_like(case["idx"], -1))
    out, grads = hip_moe_grads(case["x"], case["w1"], case["w2"], dropped, w, case["g"])
    ref_out, ref_grads = oracle_moe_grads(case["x"], case["w1"], case["w2"], case["idx"], w, case["g"])
    assert_close_scaled(out, ref_out, tol, "out")
    for name, got, want in zip(("dx", "dW1", "dW2"), grads, ref_grads):
        assert_close_scaled(got, want, tol, name)
    assert_close_scaled(grads[3], ref_grads[3] * keep, tol, "dS")
    assert not grads[3].cpu()[~keep].any()
    # and the same numbers as the uncompacted HIP path with those zero weights
    out_zero, grads_zero = hip_moe_grads(case["x"], case["w1"], case["w2"], case["idx"], w, case["g"])
    assert_close_scaled(out, out_zero, tol, "out vs zero-weight dispatch")
    return keep


@pytest.mark.parametrize("T,H,E,I,K,capacity", [(256, 64, 4, 128, 2, 100), (700, 72, 3, 40, 2, 300),
                                                (129, 32, 4, 24, 3, 20), (64, 64, 4, 64, 1, 5)])
def test_fused_moe_with_dropped_routes_small(T, H, E, I, K, capacity):
    print(f"moe with drops T={T} H={H} E={E} I={I} K={K} C={capacity}", flush=True)
    _moe_with_drops(routed_case(40 + T, T, H, E, I, K), capacity, tol=BF16_TOL)


def test_fused_moe_with_dropped_routes_fp32():
    print("moe with drops fp32", flush=True)
    _moe_with_drops(routed_case(0, 256, 64, 4, 128, 2, dtype=torch.float32), 100, tol=1e-5)


def test_fused_moe_with_dropped_routes_layer_size_zipf():
    print("moe with drops 24576 zipf", flush=True)
    case = routed_case(3, 24576, 768, 8, 1024, 2, bias=O.zipf_log_bias(8))
    capacity = O.expert_capacity(24576, 2, 8, 1.0, 4)
    E = 8
    keep = O.capacity_mask(case["idx"], case["route"].expert_weights, E, capacity)
    w = O.apply_capacity(case["route"].expert_weights, keep, normalize=True).to(torch.bfloat16)
    dropped = torch.where(keep, case["idx"], torch.full_like(case["idx"], -1))
    out, grads = hip_moe_grads(case["x"], case["w1"], case["w2"], dropped, w, case["g"])
    ref_out, ref_grads = oracle_moe_grads(case["x"], case["w1"], case["w2"], case["idx"], w, case["g"], device="cuda")
    assert_close_scaled(out, ref_out, BF16_TOL, "out")
    for name, got, want in zip(("dx", "dW1", "dW2"), grads, ref_grads):
        assert_close_scaled(got, want, BF16_TOL, name)
    assert_close_scaled(grads[3], ref_grads[3] * keep.cuda(), BF16_TOL, "dS")


def test_every_route_dropped_gives_zeros():
    print("moe all dropped", flush=True)
    case = routed_case(8, 100, 64, 4, 64, 2)
    idx = torch.full_like(case["idx"], -1)
    out, grads = hip_moe_grads(case["x"], case["w1"], case["w2"], idx, case["w"], case["g"])
    assert not out.any()
    for g in grads:
        assert not g.any()


def test_router_module_with_capacity_matches_oracle():
    """TopKRouter + MoEFeedForward under a capacity factor, GPU `hip` against the oracle."""
    print("module with capacity", flush=True)
    from minitrain_amd.model.blocks import MoEFeedForward
    from minitrain_amd.model.config import ModelConfig

    T, H, E, I, K = 512, 64, 4, 128, 2
    cfg = ModelConfig(n_layers=2, n_heads=1, hidden_size=H, intermediate_size=I, num_experts=E, experts_per_token=K,
                      expert_capacity_factor=0.75, expert_min_capacity=4)
    x, w_r, w1, w2, g = O.make_inputs(6, T, H, E, I)
    block = MoEFeedForward(cfg)
    with torch.no_grad():
        block.router.weight.copy_(w_r)
        block.gate_up_proj.copy_(w1)
        block.down_proj.copy_(w2)
    block = block.cuda()
    xg = x.cuda().requires_grad_(True)
    out = block(xg, hip_backend())
    loss = (out.hidden_states * g.cuda()).sum() + 0.01 * out.router_aux_loss + 0.001 * out.router_z_loss
    loss.backward()
    torch.cuda.synchronize()

    leaves = [t.clone().requires_grad_(True) for t in (x, w_r, w1, w2)]
    r = O.topk_router(leaves[0], leaves[1], K, normalize=True)
    capacity = O.expert_capacity(T, K, E, 0.75, 4)
    keep = O.capacity_mask(r.expert_indices, r.route.expert_weights, E, capacity)
    w = O.apply_capacity(r.route.expert_weights, keep, normalize=True)
    ref = O.fused_moe(leaves[0], leaves[2], leaves[3], r.expert_indices, w.to(x.dtype))
    ref_loss = (ref * g).sum() + 0.01 * r.auxiliary_loss + 0.001 * r.z_loss
    ref_loss.backward()

    assert float(out.router_metrics["moe/dropped_route_fraction"]) == pytest.approx(1.0 - keep.float().mean().item())
    assert out.router_metrics["moe/max_expert_load"].item() <= capacity
    assert_close_scaled(out.hidden_states.detach(), ref.detach(), 1e-5, "hidden")
    assert_close_scaled(xg.grad, leaves[0].grad, 1e-4, "dx")
    assert_close_scaled(block.router.weight.grad, leaves[1].grad, 1e-4, "dW_r")
    assert_close_scaled(block.gate_up_proj.grad, leaves[2].grad, 1e-4, "dW1")
    assert_close_scaled(block.down_proj.grad, leaves[3].grad, 1e-4, "dW2")
