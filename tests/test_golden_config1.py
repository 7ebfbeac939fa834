"""The 256-token fp32 debug configuration: oracle against the committed vectors (CPU), and
the HIP fp32 path against both (GPU).  fp32 gate: max|a-b| / max|b| <= 1e-5 per tensor."""

import os

import numpy as np
import pytest
import torch

from oracle import moe_oracle as O
from tests.golden.make_config1_golden import CONFIG1, evaluate

FP32_TOL = 1e-5
GOLDEN = np.load(os.path.join(os.path.dirname(__file__), "golden", "config1_fp32.npz"))


def _close(a, b, what, tol=FP32_TOL):
    st = O.error_stats(torch.as_tensor(np.asarray(a)), torch.as_tensor(np.asarray(b)))
    assert st["max_rel_scaled"] <= tol, (what, st)


def test_oracle_reproduces_the_committed_vectors():
    now = evaluate()
    assert np.array_equal(now["expert_indices"], GOLDEN["expert_indices"])
    assert np.array_equal(now["x_head"], GOLDEN["x_head"])
    for key in ("expert_weights", "probability_per_expert", "z_loss", "auxiliary_loss", "hidden", "dx", "d_router",
                "d_gate_up", "d_down"):
        _close(now[key], GOLDEN[key], key, 1e-6)


def test_fp32_torch_semantics_path_within_1e5_of_the_float64_evaluation():
    """The input-dtype expert loop (what the reference's PyTorch backend runs on the CPU) in fp32."""
    c = CONFIG1
    x, w_r, w1, w2, g = O.make_inputs(c["seed"], c["T"], c["H"], c["E"], c["I"])
    leaves = [t.clone().requires_grad_(True) for t in (x, w_r, w1, w2)]
    hidden, r = O.moe_feed_forward(*leaves, c["K"])
    ((hidden * g).sum() + 0.01 * r.auxiliary_loss + 0.001 * r.z_loss).backward()
    _close(hidden.detach(), GOLDEN["hidden"], "hidden")
    for leaf, key in zip(leaves, ("dx", "d_router", "d_gate_up", "d_down")):
        _close(leaf.grad, GOLDEN[key], key)


@pytest.mark.gpu
def test_hip_fp32_layer_matches_the_vectors():
    from minitrain_amd.model.blocks import MoEFeedForward
    from minitrain_amd.model.config import ModelConfig
    from minitrain_amd.model.ops import get_ops_backend

    c = CONFIG1
    print("config1 fp32 on the GPU", flush=True)
    x, w_r, w1, w2, g = O.make_inputs(c["seed"], c["T"], c["H"], c["E"], c["I"])
    cfg = ModelConfig(hidden_size=c["H"], n_heads=1, intermediate_size=c["I"], num_experts=c["E"], experts_per_token=c["K"])
    block = MoEFeedForward(cfg).cuda()
    with torch.no_grad():
        block.router.weight.copy_(w_r)
        block.gate_up_proj.copy_(w1)
        block.down_proj.copy_(w2)
    xg = x.cuda().requires_grad_(True)
    out = block(xg.view(2, 128, c["H"]), get_ops_backend("hip"))
    loss = (out.hidden_states.view(c["T"], c["H"]) * g.cuda()).sum() + 0.01 * out.router_aux_loss + 0.001 * out.router_z_loss
    loss.backward()
    torch.cuda.synchronize()
    assert out.hidden_states.dtype == torch.float32
    _close(out.hidden_states.view(c["T"], c["H"]).detach().cpu(), GOLDEN["hidden"], "hidden")
    _close(out.router_aux_loss.detach().cpu(), GOLDEN["auxiliary_loss"], "aux")
    _close(out.router_z_loss.detach().cpu(), GOLDEN["z_loss"], "z")
    _close(xg.grad.cpu(), GOLDEN["dx"], "dx")
    _close(block.router.weight.grad.cpu(), GOLDEN["d_router"], "dRouter")
    _close(block.gate_up_proj.grad.cpu(), GOLDEN["d_gate_up"], "dW1")
    _close(block.down_proj.grad.cpu(), GOLDEN["d_down"], "dW2")


@pytest.mark.gpu
@pytest.mark.parametrize("T,H,E,I,K", [(33, 36, 8, 24, 3), (257, 64, 4, 128, 2), (700, 72, 3, 40, 2), (1, 8, 2, 4, 1)])
def test_hip_fp32_operator_small_shapes(T, H, E, I, K):
    from tests.helpers import hip_moe_grads, oracle_moe_grads, routed_case

    print(f"fp32 moe T={T} H={H} E={E} I={I} K={K}", flush=True)
    case = routed_case(50 + T, T, H, E, I, K, dtype=torch.float32)
    out, grads = hip_moe_grads(case["x"], case["w1"], case["w2"], case["idx"], case["w"], case["g"])
    ref_out, ref_grads = oracle_moe_grads(case["x"], case["w1"], case["w2"], case["idx"], case["w"], case["g"],
                                          compute_dtype=torch.float64)
    assert out.dtype == torch.float32
    _close(out.cpu(), ref_out, "out")
    for name, a, b in zip(("dx", "dW1", "dW2", "dS"), grads, ref_grads):
        assert a.dtype == torch.float32
        _close(a.cpu(), b, name)
