"""Operator boundary between the MoE block and kernel backends.

Mirror of the reference's ``minitrain/model/ops.py:7-112``: the same record type,
the same protocol (eight methods) and the same factory function, plus the
``hip`` branch a maintainer would add there.
"""

from dataclasses import dataclass
from typing import Protocol

import torch


@dataclass
class RouterPostprocessOutput:
    """Backend-neutral result of processing fp32 router logits."""

    expert_weights: torch.Tensor
    expert_indices: torch.Tensor
    probability_per_expert: torch.Tensor
    z_loss: torch.Tensor
    entropy: torch.Tensor
    # Beyond the reference's record (minitrain/model/ops.py:7-15), filled by backends that
    # compute them in the same pass: routes per expert (int32 [E], no gradient) and the
    # load-balancing term E * sum_e (routes_e / routes) * probability_per_expert_e, which is
    # differentiable through the mean probability.  None means the caller computes them.
    expert_counts: torch.Tensor | None = None
    load_balance_loss: torch.Tensor | None = None


class OpsBackend(Protocol):
    name: str

    def rmsnorm(self, x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor: ...

    def rope(self, q, k, cos, sin) -> tuple[torch.Tensor, torch.Tensor]: ...

    def swiglu(self, gate: torch.Tensor, up: torch.Tensor) -> torch.Tensor: ...

    def attention(self, q, k, v, *, is_causal: bool, dropout_p: float) -> torch.Tensor: ...

    def cross_entropy(self, logits: torch.Tensor, targets: torch.Tensor) -> torch.Tensor: ...

    def fused_linear_cross_entropy(self, x, weight, targets) -> torch.Tensor: ...

    def router_postprocess(
        self, logits: torch.Tensor, top_k: int, *, normalize: bool
    ) -> RouterPostprocessOutput:
        """Process fp32 router logits and return differentiable routing statistics."""
        ...

    def fused_moe(
        self,
        x: torch.Tensor,
        gate_up_proj: torch.Tensor,
        down_proj: torch.Tensor,
        top_k_index: torch.Tensor,
        top_k_weights: torch.Tensor,
    ) -> torch.Tensor:
        """Apply routed SwiGLU experts and aggregate the selected outputs."""
        ...


def get_ops_backend(name: str) -> OpsBackend:
    """Construct an operator backend by name (only ``hip`` lives in this package)."""

    if name == "hip":
        from minitrain_amd.kernels.hip import HipOpsBackend

        return HipOpsBackend()
    raise ValueError(f"Unknown ops backend: {name}")
