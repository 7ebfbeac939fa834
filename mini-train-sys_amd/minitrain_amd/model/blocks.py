"""MoE feed-forward block: parameter owner and caller of ``ops.fused_moe``.

Same parameter layout, initialisation and call sequence as the reference's
``MoEFeedForward`` (minitrain/model/blocks.py:71-102): ``gate_up_proj [E,2I,H]``
with rows ``0..I-1`` = gate and ``I..2I-1`` = up, ``down_proj [E,H,I]``.
"""

import math
from dataclasses import dataclass, field

import torch
from torch import nn

from minitrain_amd.model.config import ModelConfig
from minitrain_amd.model.moe_router import TopKRouter, load_metrics_from_stats
from minitrain_amd.model.ops import OpsBackend, RouterPostprocessOutput


@dataclass
class FeedForwardOutput:
    hidden_states: torch.Tensor
    router_aux_loss: torch.Tensor | None = None
    router_z_loss: torch.Tensor | None = None
    router_metrics: dict[str, torch.Tensor] = field(default_factory=dict)


class MoEFeedForward(nn.Module):
    """Owner of the expert parameters; calls the router and ``ops.fused_moe`` on flattened tokens."""

    def __init__(self, cfg: ModelConfig) -> None:
        super().__init__()
        E, H, I = cfg.num_experts, cfg.hidden_size, cfg.intermediate_size
        self.cfg = cfg
        self.router = TopKRouter(cfg)
        # rows 0..I-1 of an expert's gate_up_proj are the gate, rows I..2I-1 the up projection
        self.gate_up_proj = nn.Parameter(torch.empty(E, 2 * I, H))
        self.down_proj = nn.Parameter(torch.empty(E, H, I))
        self.dropout = nn.Dropout(cfg.dropout)
        with torch.no_grad():
            self.gate_up_proj.normal_(0.0, 0.02)
            self.down_proj.normal_(0.0, 0.02 / math.sqrt(2 * cfg.n_layers))   # residual-branch scaling

    def _whole_layer(self, tokens: torch.Tensor, ops: OpsBackend):
        """The layer as one node of a backend that offers it (dropless routing without jitter noise):
        same outputs as the router module followed by ``ops.fused_moe``, or None."""
        cfg = self.cfg
        layer = getattr(ops, "moe_layer", None)
        if layer is None or cfg.expert_capacity_factor is not None or (self.training and cfg.router_jitter_noise):
            return None
        result = layer(tokens, self.router.weight, self.gate_up_proj, self.down_proj, cfg.experts_per_token,
                       normalize=cfg.router_normalize_topk)
        if result is None:
            return None
        mixed, aux_loss, z_loss, prob_mean, entropy, counts, load_stats, indices, weights = result
        route = RouterPostprocessOutput(expert_weights=weights, expert_indices=indices, probability_per_expert=prob_mean,
                                        z_loss=z_loss, entropy=entropy, expert_counts=counts, load_balance_loss=aux_loss,
                                        load_stats=load_stats)
        return mixed, aux_loss, z_loss, load_metrics_from_stats(route, cfg.num_experts)

    def forward(self, x: torch.Tensor, ops: OpsBackend) -> FeedForwardOutput:
        tokens = x.reshape(-1, x.shape[-1])
        whole = self._whole_layer(tokens, ops)
        if whole is not None:
            mixed, aux_loss, z_loss, metrics = whole
            return FeedForwardOutput(hidden_states=self.dropout(mixed.view(x.shape)), router_aux_loss=aux_loss,
                                     router_z_loss=z_loss, router_metrics=metrics)
        route = self.router(tokens, ops)
        # under a capacity limit the router may hand over a dispatch in which dropped routes carry -1
        dispatch = route.expert_indices if route.dispatch_indices is None else route.dispatch_indices
        mixed = ops.fused_moe(tokens, self.gate_up_proj, self.down_proj, dispatch, route.expert_weights)
        return FeedForwardOutput(
            hidden_states=self.dropout(mixed.view(x.shape)),
            router_aux_loss=route.auxiliary_loss,
            router_z_loss=route.z_loss,
            router_metrics=route.metrics,
        )
