"""Capacity-limited dispatch: which routes an expert accepts.

The selection rule is that of the reference's ``TopKRouter._capacity_mask``
(minitrain/model/moe_router.py:29-61): per expert the ``capacity`` routes with the
largest router weight, equal weights in ascending flat-entry order.  The reference keeps
the helper for experiments and routes droplessly, "until capacity-aware compaction is
implemented in the routing metadata and forward/backward kernels"
(moe_router.py:92-97); here the dropped routes leave the dispatch: ``kept_index`` carries
-1 for them, the routing metadata gives them no row, and the expert GEMMs of
``fused_moe`` run on the accepted routes only.
"""

import math

import torch

from minitrain_amd import _lib


def expert_capacity(tokens: int, top_k: int, num_experts: int, factor: float, min_capacity: int) -> int:
    """Rows an expert accepts (minitrain/model/moe_router.py:38-42)."""
    return max(int(min_capacity), math.ceil(factor * tokens * top_k / num_experts))


def is_capacity_mask_supported(expert_indices: torch.Tensor, expert_weights: torch.Tensor, num_experts: int) -> bool:
    return (
        expert_indices.is_cuda
        and expert_weights.is_cuda
        and expert_indices.device == expert_weights.device
        and expert_indices.ndim == 2
        and expert_indices.shape == expert_weights.shape
        and expert_indices.dtype == torch.int32
        and expert_weights.dtype == torch.float32
        and expert_indices.shape[0] > 0
        and 0 < num_experts <= 1024
        and expert_indices.numel() < 2**31
    )


def capacity_mask(expert_indices: torch.Tensor, expert_weights: torch.Tensor, num_experts: int, capacity: int):
    """Returns ``(keep bool [T,K], kept_index int32 [T,K], accepted int32 [E])``.

    ``kept_index`` equals ``expert_indices`` where ``keep`` is set and is -1 elsewhere;
    ``accepted[e] = min(routes of e, capacity)``.  Nothing here is differentiable.
    """
    if not is_capacity_mask_supported(expert_indices, expert_weights, num_experts):
        raise RuntimeError("Unsupported tensor contract for hip capacity_mask")
    lib = _lib.load()
    idx = expert_indices.contiguous()
    w = expert_weights.detach().contiguous()
    T, K = idx.shape
    dev = idx.device
    keep = torch.empty(T, K, dtype=torch.bool, device=dev)
    kept_index = torch.empty(T, K, dtype=torch.int32, device=dev)
    accepted = torch.empty(num_experts, dtype=torch.int32, device=dev)
    ws_bytes = lib.mts_moe_capacity_workspace_bytes(T, K, num_experts)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
    _lib.check(
        lib.mts_moe_capacity_mask(
            idx.data_ptr(), w.data_ptr(), T, K, num_experts, int(capacity), keep.data_ptr(), kept_index.data_ptr(),
            accepted.data_ptr(), ws.data_ptr(), ws_bytes, _lib.stream_of(idx),
        ),
        "mts_moe_capacity_mask",
    )
    return keep, kept_index, accepted
