"""`hip` operator backend: MoE operators on hand-written gfx950 kernels.

Counterpart of the reference's ``TritonOpsBackend``
(minitrain/kernels/triton/__init__.py:36-113) for the two MoE methods.  Unlike
that class there is no fallback: an unsupported tensor contract raises.
"""

from minitrain_amd.kernels.dense_ops import DenseTorchOps
from minitrain_amd.kernels.hip.capacity import capacity_mask, is_capacity_mask_supported
from minitrain_amd.kernels.hip.fused_moe import expert_counts, fused_moe, is_fused_moe_supported
from minitrain_amd.kernels.hip.moe_layer import moe_layer, moe_layer_violation
from minitrain_amd.kernels.hip.switches import SWITCHES
from minitrain_amd.kernels.hip.router import (
    is_router_logits_supported,
    is_router_postprocess_supported,
    router_logits,
    router_postprocess,
)


class HipOpsBackend(DenseTorchOps):
    name = "hip"
    # fused_moe gives a route whose expert index is negative no row in the expert GEMMs
    drops_routes = True

    # router_postprocess takes ``weights_dtype`` and then also returns the weights rounded to it
    # (a comparison switch leaves the cast to the caller, see switches.py)
    casts_router_weights = SWITCHES.router_cast

    def router_postprocess(self, logits, top_k, *, normalize, weights_dtype=None):
        return router_postprocess(logits, top_k, normalize=normalize, weights_dtype=weights_dtype)

    def fused_moe(self, x, gate_up_proj, down_proj, top_k_index, top_k_weights):
        return fused_moe(x, gate_up_proj, down_proj, top_k_index, top_k_weights)

    def expert_counts(self, expert_indices, num_experts):
        """Extension: routes per expert (int32 ``[E]``) without a host synchronisation."""
        return expert_counts(expert_indices, num_experts)

    def capacity_mask(self, expert_indices, expert_weights, num_experts, capacity):
        """Extension: ``(keep, kept_index, accepted)`` of a capacity-limited dispatch, or None when
        the contract is not supported (the caller then uses its own sort-based selection)."""
        if not is_capacity_mask_supported(expert_indices, expert_weights, num_experts):
            return None
        return capacity_mask(expert_indices, expert_weights, num_experts, capacity)

    # a comparison switch keeps the layer on the three separate operators (switches.py); an instance may also set
    # this attribute to False, e.g. to have forward hooks on the router module fire (the one-node path does not
    # call that module)
    offers_moe_layer = SWITCHES.layer_node

    def moe_layer(self, x, router_weight, gate_up_proj, down_proj, top_k, *, normalize):
        """Extension: router projection, post-process, routing metadata and the experts as one autograd
        node (see ``kernels/hip/moe_layer.py``).  Returns None when the contract is not supported; the
        caller then composes the layer from ``router_postprocess`` and ``fused_moe``."""
        if not self.offers_moe_layer or moe_layer_violation(x, router_weight, gate_up_proj, down_proj, top_k) is not None:
            return None
        return moe_layer(x, router_weight, gate_up_proj, down_proj, top_k, normalize=normalize)

    def router_logits(self, hidden_states, weight):
        """Extension beyond the reference's operator interface: the router projection in fp32
        straight from the activation dtype.  Returns None when the contract is not supported,
        and the caller then runs its own ``F.linear``."""
        if not is_router_logits_supported(hidden_states, weight):
            return None
        return router_logits(hidden_states, weight)


__all__ = [
    "HipOpsBackend",
    "capacity_mask",
    "expert_counts",
    "fused_moe",
    "is_capacity_mask_supported",
    "is_fused_moe_supported",
    "is_router_logits_supported",
    "is_router_postprocess_supported",
    "moe_layer",
    "router_logits",
    "router_postprocess",
]
