"""Top-k router module: the caller of ``ops.router_postprocess``.

Same arithmetic and record as the reference's ``TopKRouter``
(minitrain/model/moe_router.py:12-144): fp32 router GEMM with autocast off, the
post-process operator, assignment counts, the load-balancing loss
``E * sum_e f_e * pbar_e`` and the load metrics; indices are returned as int32 and
weights in the activation dtype.
"""

import math
from dataclasses import dataclass

import torch
import torch.nn.functional as F
from torch import nn

from minitrain_amd.model.config import ModelConfig
from minitrain_amd.model.ops import OpsBackend


@dataclass
class RouterOutput:
    expert_indices: torch.Tensor
    expert_weights: torch.Tensor
    auxiliary_loss: torch.Tensor
    z_loss: torch.Tensor
    metrics: dict[str, torch.Tensor]


class TopKRouter(nn.Module):
    def __init__(self, cfg: ModelConfig) -> None:
        super().__init__()
        self.cfg = cfg
        self.weight = nn.Parameter(torch.empty(cfg.num_experts, cfg.hidden_size))
        nn.init.normal_(self.weight, mean=0.0, std=0.02)

    def forward(self, hidden_states: torch.Tensor, ops: OpsBackend) -> RouterOutput:
        cfg = self.cfg
        jitter = self.training and cfg.router_jitter_noise
        # a backend may offer the projection straight from the activation dtype (same fp32
        # arithmetic, no fp32 copy of the activations); jitter noise needs the fp32 copy
        fused_logits = None if jitter else getattr(ops, "router_logits", None)
        logits = None
        if fused_logits is not None and hidden_states.ndim == 2:
            with torch.autocast(device_type=hidden_states.device.type, enabled=False):
                logits = fused_logits(hidden_states, self.weight)
        if logits is None:
            router_input = hidden_states.float()
            if jitter:
                noise = torch.empty_like(router_input).uniform_(
                    1.0 - cfg.router_jitter_noise, 1.0 + cfg.router_jitter_noise
                )
                router_input = router_input * noise

        with torch.autocast(device_type=hidden_states.device.type, enabled=False):
            if logits is None:
                logits = F.linear(router_input, self.weight.float())
            route = ops.router_postprocess(logits, cfg.experts_per_token, normalize=cfg.router_normalize_topk)
            expert_weights = route.expert_weights
            expert_indices = route.expert_indices

            route_counts = getattr(route, "expert_counts", None)
            auxiliary_loss = getattr(route, "load_balance_loss", None)
            if route_counts is None:
                count_routes = getattr(ops, "expert_counts", None)
                if count_routes is not None and expert_indices.is_cuda and expert_indices.dtype == torch.int32:
                    route_counts = count_routes(expert_indices, cfg.num_experts)
                else:
                    route_counts = torch.bincount(expert_indices.flatten().long(), minlength=cfg.num_experts)
            if auxiliary_loss is None:
                tokens_per_expert = route_counts.float() / expert_indices.numel()
                # the assignment fraction carries no gradient; it enters through the mean probability
                auxiliary_loss = cfg.num_experts * torch.sum(tokens_per_expert * route.probability_per_expert)

            accepted = route_counts.float()
            load_fraction = accepted / max(expert_indices.numel(), 1)
            uniform = 1.0 / cfg.num_experts
            metrics = {
                "moe/router_entropy": route.entropy,
                "moe/router_entropy_normalized": (
                    route.entropy / (math.log(cfg.num_experts) if cfg.num_experts > 1 else 1.0)
                ).detach(),
                "moe/dropped_route_fraction": expert_weights.new_zeros(()).detach(),
                "moe/max_expert_load": accepted.max().detach(),
                "moe/min_expert_load": accepted.min().detach(),
                "moe/expert_load_cv": (load_fraction.std(unbiased=False) / uniform).detach(),
                "moe/max_to_mean_load": (load_fraction.max() / uniform).detach(),
                "moe/dead_expert_count": (accepted == 0).sum().detach(),
                "moe/expert_load_fraction": load_fraction.detach(),
                "moe/expert_probability": route.probability_per_expert.detach(),
            }

        return RouterOutput(
            expert_indices=expert_indices.to(torch.int32),
            expert_weights=expert_weights.to(hidden_states.dtype),
            auxiliary_loss=auxiliary_loss,
            z_loss=route.z_loss,
            metrics=metrics,
        )
