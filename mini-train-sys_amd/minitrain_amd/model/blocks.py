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
from minitrain_amd.model.moe_router import TopKRouter
from minitrain_amd.model.ops import OpsBackend


@dataclass
class FeedForwardOutput:
    hidden_states: torch.Tensor
    router_aux_loss: torch.Tensor | None = None
    router_z_loss: torch.Tensor | None = None
    router_metrics: dict[str, torch.Tensor] = field(default_factory=dict)


class MoEFeedForward(nn.Module):
    def __init__(self, cfg: ModelConfig) -> None:
        super().__init__()
        self.cfg = cfg
        self.router = TopKRouter(cfg)
        self.gate_up_proj = nn.Parameter(torch.empty(cfg.num_experts, 2 * cfg.intermediate_size, cfg.hidden_size))
        self.down_proj = nn.Parameter(torch.empty(cfg.num_experts, cfg.hidden_size, cfg.intermediate_size))
        self.dropout = nn.Dropout(cfg.dropout)
        nn.init.normal_(self.gate_up_proj, mean=0.0, std=0.02)
        nn.init.normal_(self.down_proj, mean=0.0, std=0.02 / math.sqrt(2 * cfg.n_layers))

    def forward(self, x: torch.Tensor, ops: OpsBackend) -> FeedForwardOutput:
        shape = x.shape
        flat_x = x.reshape(-1, shape[-1])
        route = self.router(flat_x, ops)
        # under a capacity limit the router may hand over a dispatch in which dropped routes carry -1
        dispatch = route.expert_indices if route.dispatch_indices is None else route.dispatch_indices
        hidden = ops.fused_moe(flat_x, self.gate_up_proj, self.down_proj, dispatch, route.expert_weights).view(shape)
        return FeedForwardOutput(
            hidden_states=self.dropout(hidden),
            router_aux_loss=route.auxiliary_loss,
            router_z_loss=route.z_loss,
            router_metrics=route.metrics,
        )
