"""Operator boundary between the model code and the kernel backends.

The interface is the reference's (minitrain/model/ops.py:7-112): a result record for the router
post-process, a structural protocol with eight operators, and a factory that builds a backend
from its name.  Only the names, arguments and return types are shared with it; this package
ships one backend, ``hip``.
"""

from dataclasses import dataclass
from typing import Protocol

import torch

Tensor = torch.Tensor


@dataclass
class RouterPostprocessOutput:
    """What ``router_postprocess`` hands back, whichever backend computed it."""

    expert_weights: Tensor           # [T, K] fp32, weight of each selected expert
    expert_indices: Tensor           # [T, K] expert ids, rank 0 first
    probability_per_expert: Tensor   # [E] mean softmax probability over the tokens
    z_loss: Tensor                   # [] mean squared log-partition
    entropy: Tensor                  # [] mean routing entropy, detached
    # Not in the reference's record (minitrain/model/ops.py:7-15); a backend that has them from the
    # same pass fills them in, None leaves the computation to the caller: routes per expert (int32
    # [E], no gradient), E * sum_e (routes_e / routes) * probability_per_expert_e, which carries a
    # gradient through the mean probability, and the load statistics below.
    expert_counts: Tensor | None = None
    load_balance_loss: Tensor | None = None
    # fp32 [E + 7], no gradient: what the router module's load metrics need when no route is dropped --
    # the fraction of the routes per expert, then the largest and the smallest route count, the
    # population standard deviation of the fractions x E, the largest fraction x E, the number of
    # experts without a route, 0 (the dropped-route fraction) and entropy / log E
    load_stats: Tensor | None = None
    # [T, K] in the dtype asked for with ``weights_dtype``: expert_weights rounded to it, differentiable
    # (what the router module hands to fused_moe); None when not asked for or not offered
    expert_weights_cast: Tensor | None = None


class OpsBackend(Protocol):
    """The eight operators a backend provides; the model only ever sees this protocol."""

    name: str

    # dense operators: stay on stock PyTorch-ROCm in the ``hip`` backend
    def rmsnorm(self, x: Tensor, weight: Tensor, eps: float) -> Tensor: ...

    def rope(self, q: Tensor, k: Tensor, cos: Tensor, sin: Tensor) -> tuple[Tensor, Tensor]: ...

    def swiglu(self, gate: Tensor, up: Tensor) -> Tensor: ...

    def attention(self, q: Tensor, k: Tensor, v: Tensor, *, is_causal: bool, dropout_p: float) -> Tensor: ...

    def cross_entropy(self, logits: Tensor, targets: Tensor) -> Tensor: ...

    def fused_linear_cross_entropy(self, x: Tensor, weight: Tensor, targets: Tensor) -> Tensor: ...

    # the two MoE operators
    def router_postprocess(self, logits: Tensor, top_k: int, *, normalize: bool) -> RouterPostprocessOutput:
        """fp32 logits ``[T, E]`` -> top-k weights and indices plus the routing statistics; differentiable
        through the weights, the mean probability and the z-loss."""
        ...

    def fused_moe(
        self, x: Tensor, gate_up_proj: Tensor, down_proj: Tensor, top_k_index: Tensor, top_k_weights: Tensor
    ) -> Tensor:
        """``out[t] = sum_k w[t,k] * W2[e] (silu(g) * u)`` with ``[g; u] = W1[e] x[t]``, ``e = index[t,k]``."""
        ...


def get_ops_backend(name: str) -> OpsBackend:
    """Backend instance for ``name``; unknown names raise ``ValueError`` as in the reference."""
    if name != "hip":
        raise ValueError(f"Unknown ops backend: {name}")
    from minitrain_amd.kernels.hip import HipOpsBackend

    return HipOpsBackend()
