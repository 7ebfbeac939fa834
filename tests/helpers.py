"""Shared pieces of the GPU parity tests."""

import numpy as np
import torch

from oracle import moe_oracle as O

# bf16 parity gate: max|a-b| / max|b| per tensor against an fp32-accumulated reference
BF16_TOL = 2e-2


def hip_backend():
    from minitrain_amd.model.ops import get_ops_backend

    return get_ops_backend("hip")


def routed_case(seed, T, H, E, I, K, *, dtype=torch.bfloat16, bias=None, tie_fraction=0.0, normalize=True):
    """x, W_r, W1, W2, G plus the routing the oracle derives from the fp32 logits."""
    x, w_r, w1, w2, g = O.make_inputs(seed, T, H, E, I)
    x, w1, w2, g = (t.to(dtype) for t in (x, w1, w2, g))
    logits = torch.nn.functional.linear(x.float(), w_r)
    if bias is not None:
        logits = logits + bias
    if tie_fraction:
        logits = O.inject_ties(logits, tie_fraction, seed)
    route = O.router_postprocess(logits, K, normalize=normalize)
    return dict(x=x, w_r=w_r, w1=w1, w2=w2, g=g, logits=logits, idx=route.expert_indices,
                w=route.expert_weights.to(dtype), route=route)


def oracle_moe_grads(x, w1, w2, idx, w, g, *, device="cpu", compute_dtype=torch.float32):
    """fp32-accumulated forward and gradients of the oracle on ``device``."""
    leaves = [t.detach().to(device).to(compute_dtype).requires_grad_(True) for t in (x, w1, w2, w)]
    out = O.fused_moe(leaves[0], leaves[1], leaves[2], idx.to(device), leaves[3])
    (out * g.to(device).to(compute_dtype)).sum().backward()
    return out.detach(), [l.grad for l in leaves]


def hip_moe_grads(x, w1, w2, idx, w, g):
    ops = hip_backend()
    leaves = [t.detach().cuda().requires_grad_(True) for t in (x, w1, w2, w)]
    out = ops.fused_moe(leaves[0], leaves[1], leaves[2], idx.cuda(), leaves[3])
    out.backward(g.cuda().to(out.dtype))
    torch.cuda.synchronize()
    return out.detach(), [l.grad for l in leaves]


def assert_close_scaled(actual, expected, tol, what):
    st = O.error_stats(actual, expected)
    assert st["max_rel_scaled"] <= tol, f"{what}: {st}"
    return st


def np_i32(t):
    return t.detach().cpu().numpy().astype(np.int32)
