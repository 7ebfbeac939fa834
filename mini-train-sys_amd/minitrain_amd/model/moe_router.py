"""Top-k router module: the caller of ``ops.router_postprocess``.

Same arithmetic and record as the reference's ``TopKRouter``
(minitrain/model/moe_router.py:12-144): fp32 router GEMM with autocast off, the
post-process operator, assignment counts, the load-balancing loss
``E * sum_e f_e * pbar_e`` and the load metrics; indices are returned as int32 and
weights in the activation dtype.

With ``cfg.expert_capacity_factor`` set, the capacity limit the reference keeps switched
off (moe_router.py:29-61 and the commented block at :92-110) is applied: an expert accepts
its ``capacity`` most confident routes, the weights of dropped routes become zero, the
remaining weights of a token are renormalised, and ``dispatch_indices`` tells a backend
that compacts its dispatch (``ops.drops_routes``) which routes to leave out.
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
    # what fused_moe is called with when it differs from expert_indices: -1 marks a dropped route
    dispatch_indices: torch.Tensor | None = None


def _order_key(weights: torch.Tensor) -> torch.Tensor:
    """int64 key that grows with the fp32 weight (-0 and +0 alike)."""
    w = torch.where(weights == 0, torch.zeros_like(weights), weights).float().contiguous()
    bits = w.view(torch.int32).long() & 0xFFFFFFFF
    return torch.where(bits >= 2**31, 0xFFFFFFFF - bits, bits + 2**31)


def capacity_selection(expert_indices: torch.Tensor, expert_weights: torch.Tensor, num_experts: int, capacity: int):
    """``(keep, kept_index, accepted)``: per expert the ``capacity`` routes with the largest
    weight, equal weights in ascending flat-entry order (the rule of the reference's
    ``_capacity_mask``, minitrain/model/moe_router.py:43-61), from one stable sort of a
    composite (expert, descending weight) key."""
    flat_experts = expert_indices.flatten().long()
    composite = flat_experts * 2**32 + (0xFFFFFFFF - _order_key(expert_weights.detach().flatten()))
    order = torch.sort(composite, stable=True).indices
    counts = torch.bincount(flat_experts, minlength=num_experts)
    first_row = counts.cumsum(0) - counts
    rank = torch.arange(order.numel(), device=order.device) - first_row[flat_experts[order]]
    keep = torch.empty_like(flat_experts, dtype=torch.bool)
    keep[order] = rank < capacity
    keep = keep.view_as(expert_indices)
    kept_index = torch.where(keep, expert_indices, torch.full_like(expert_indices, -1))
    return keep, kept_index, counts.clamp(max=capacity)


def load_metrics_from_stats(route, num_experts: int):
    """The same record from a backend's ``load_stats`` (dropless routing): views of one tensor, no launches."""
    stats, E = route.load_stats, num_experts
    record = {
        "moe/router_entropy": route.entropy,
        "moe/router_entropy_normalized": stats[E + 6],
        "moe/dropped_route_fraction": stats[E + 5],
        "moe/max_expert_load": stats[E],
        "moe/min_expert_load": stats[E + 1],
        "moe/expert_load_cv": stats[E + 2],
        "moe/max_to_mean_load": stats[E + 3],
        "moe/dead_expert_count": stats[E + 4],
        "moe/expert_load_fraction": stats[:E],
        "moe/expert_probability": route.probability_per_expert,
    }
    return {k: (v if k == "moe/router_entropy" else v.detach()) for k, v in record.items()}


def load_metrics(route, accepted: torch.Tensor, routes: int, dropped_fraction: torch.Tensor, num_experts: int):
    """The router's monitoring record, keys as in the reference (minitrain/model/moe_router.py:113-135);
    ``accepted`` = routes each expert takes, as floats."""
    share = accepted / max(routes, 1)
    scale = float(num_experts)                      # 1 / (uniform share)
    log_e = math.log(num_experts) if num_experts > 1 else 1.0
    record = {
        "moe/router_entropy": route.entropy,
        "moe/router_entropy_normalized": route.entropy / log_e,
        "moe/dropped_route_fraction": dropped_fraction,
        "moe/max_expert_load": accepted.max(),
        "moe/min_expert_load": accepted.min(),
        "moe/expert_load_cv": share.std(unbiased=False) * scale,
        "moe/max_to_mean_load": share.max() * scale,
        "moe/dead_expert_count": (accepted == 0).sum(),
        "moe/expert_load_fraction": share,           # per expert: stacked by layer for heat maps
        "moe/expert_probability": route.probability_per_expert,
    }
    return {k: (v if k == "moe/router_entropy" else v.detach()) for k, v in record.items()}


class TopKRouter(nn.Module):
    def __init__(self, cfg: ModelConfig) -> None:
        super().__init__()
        self.cfg = cfg
        self.weight = nn.Parameter(torch.empty(cfg.num_experts, cfg.hidden_size))
        with torch.no_grad():
            self.weight.normal_(0.0, 0.02)

    def _logits(self, hidden_states: torch.Tensor, ops: OpsBackend) -> torch.Tensor:
        """fp32 router projection with autocast off (minitrain/model/moe_router.py:64-76)."""
        cfg = self.cfg
        jitter = self.training and cfg.router_jitter_noise
        device_type = hidden_states.device.type
        # a backend may offer the projection straight from the activation dtype (same fp32
        # arithmetic, no fp32 copy of the activations); jitter noise needs the fp32 copy
        fused = None if jitter else getattr(ops, "router_logits", None)
        if fused is not None and hidden_states.ndim == 2:
            with torch.autocast(device_type=device_type, enabled=False):
                logits = fused(hidden_states, self.weight)
            if logits is not None:
                return logits
        wide = hidden_states.float()
        if jitter:
            low, high = 1.0 - cfg.router_jitter_noise, 1.0 + cfg.router_jitter_noise
            wide = wide * torch.empty_like(wide).uniform_(low, high)
        with torch.autocast(device_type=device_type, enabled=False):
            return F.linear(wide, self.weight.float())

    def _limit_capacity(self, ops: OpsBackend, expert_indices: torch.Tensor, expert_weights: torch.Tensor):
        """Masked and renormalised weights, dispatch indices (or None), accepted counts, dropped fraction."""
        cfg = self.cfg
        tokens, top_k = expert_indices.shape
        capacity = max(cfg.expert_min_capacity, math.ceil(cfg.expert_capacity_factor * tokens * top_k / cfg.num_experts))
        select = getattr(ops, "capacity_mask", None)
        selection = select(expert_indices, expert_weights, cfg.num_experts, capacity) if select is not None else None
        if selection is None:
            selection = capacity_selection(expert_indices, expert_weights, cfg.num_experts, capacity)
        keep, kept_index, accepted_counts = selection
        weights = expert_weights * keep
        if cfg.router_normalize_topk:
            total = weights.sum(dim=-1, keepdim=True)
            smallest = torch.finfo(weights.dtype).eps
            weights = torch.where(total > 0, weights / total.clamp_min(smallest), weights)   # a token may lose every route
        dispatch = kept_index.to(torch.int32) if getattr(ops, "drops_routes", False) else None
        return weights, dispatch, accepted_counts.float(), 1.0 - keep.float().mean()

    def forward(self, hidden_states: torch.Tensor, ops: OpsBackend) -> RouterOutput:
        cfg = self.cfg
        logits = self._logits(hidden_states, ops)
        with torch.autocast(device_type=hidden_states.device.type, enabled=False):
            # a backend may write the copy of the weights in the activation dtype in the same pass
            want_cast = (
                getattr(ops, "casts_router_weights", False)
                and cfg.expert_capacity_factor is None
                and hidden_states.dtype in (torch.bfloat16, torch.float16)
            )
            extra = {"weights_dtype": hidden_states.dtype} if want_cast else {}
            route = ops.router_postprocess(logits, cfg.experts_per_token, normalize=cfg.router_normalize_topk, **extra)
            expert_weights, expert_indices = route.expert_weights, route.expert_indices

            route_counts = getattr(route, "expert_counts", None)
            auxiliary_loss = getattr(route, "load_balance_loss", None)
            if route_counts is None:
                count_routes = getattr(ops, "expert_counts", None)
                if count_routes is not None and expert_indices.is_cuda and expert_indices.dtype == torch.int32:
                    route_counts = count_routes(expert_indices, cfg.num_experts)
                else:
                    route_counts = torch.bincount(expert_indices.flatten().long(), minlength=cfg.num_experts)
            if auxiliary_loss is None:
                # E * sum_e f_e * pbar_e; the route fractions f carry no gradient, the mean probability does
                route_fraction = route_counts.float() / expert_indices.numel()
                auxiliary_loss = cfg.num_experts * torch.sum(route_fraction * route.probability_per_expert)

            dispatch_indices = None
            if cfg.expert_capacity_factor is not None:
                expert_weights, dispatch_indices, accepted, dropped_fraction = self._limit_capacity(
                    ops, expert_indices, expert_weights
                )
                metrics = load_metrics(route, accepted, expert_indices.numel(), dropped_fraction, cfg.num_experts)
            elif getattr(route, "load_stats", None) is not None:
                metrics = load_metrics_from_stats(route, cfg.num_experts)
            else:
                metrics = load_metrics(
                    route, route_counts.float(), expert_indices.numel(), expert_weights.new_zeros(()), cfg.num_experts
                )

        cast = getattr(route, "expert_weights_cast", None) if want_cast else None
        return RouterOutput(
            expert_indices=expert_indices.to(torch.int32),
            expert_weights=cast if cast is not None else expert_weights.to(hidden_states.dtype),
            auxiliary_loss=auxiliary_loss,
            z_loss=route.z_loss,
            metrics=metrics,
            dispatch_indices=dispatch_indices,
        )
