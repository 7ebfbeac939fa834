"""Router post-process on the GPU: one pass over the fp32 logits.

Counterpart of minitrain/kernels/triton/router.py:262-357 (autograd wrapper and
module-level entry point) with the argument checks of
minitrain/kernels/torch_ops.py:96-101.  Top-k is taken on the logits with the
lower expert index winning ties, and the statistics are reduced in a fixed
order, so the operator is deterministic and needs no deterministic-mode opt-out.
"""

import torch

from minitrain_amd import _lib
from minitrain_amd.model.ops import RouterPostprocessOutput

_MAX_EXPERTS = 1024
_MAX_TOP_K = 8
_ROUTER_WEIGHT_LDS_BYTES = 128 * 1024   # the projection kernels keep W_r [E,H] fp32 in LDS: H <= 4096 for 8 experts, 2048 for 16


def is_router_postprocess_supported(logits: torch.Tensor, top_k: int, normalize: bool) -> bool:
    del normalize  # both normalised and raw full-softmax weights are supported
    return (
        logits.is_cuda
        and logits.ndim == 2
        and logits.dtype == torch.float32
        and logits.shape[0] > 0
        and 1 <= top_k <= min(logits.shape[1], _MAX_TOP_K)
        and logits.shape[1] <= _MAX_EXPERTS
    )


class _RouterPostprocessFunction(torch.autograd.Function):
    @staticmethod
    @torch.amp.custom_fwd(device_type="cuda")
    def forward(ctx, logits: torch.Tensor, top_k: int, normalize: bool, weights_dtype):
        lib = _lib.load()
        logits = logits.contiguous()
        T, E = logits.shape
        dev = logits.device
        weights = torch.empty((T, top_k), device=dev, dtype=torch.float32)
        indices = torch.empty((T, top_k), device=dev, dtype=torch.int32)
        stats = torch.empty(2 * E + 10, device=dev, dtype=torch.float32)   # E + 3 statistics, E + 7 load statistics
        counts = torch.empty(E, device=dev, dtype=torch.int32)
        ws_bytes = lib.mts_router_workspace_bytes(T, E)
        ws = torch.empty(ws_bytes, device=dev, dtype=torch.uint8)
        prob_mean, z_loss, entropy, load_balance = stats[:E], stats[E], stats[E + 1], stats[E + 2]
        load_stats = stats[E + 3:]
        # the copy of the weights in the activation dtype, written by the same kernel (what the router
        # module otherwise makes with tensor.to(): one launch forward, one backward)
        weights_act = torch.empty((T, top_k), device=dev, dtype=weights_dtype) if weights_dtype is not None else None
        act_code = _lib.dtype_code(weights_dtype) if weights_dtype is not None else 0
        _lib.check(
            lib.mts_router_fwd(
                logits.data_ptr(), T, E, top_k, int(normalize), weights.data_ptr(), indices.data_ptr(),
                prob_mean.data_ptr(), z_loss.data_ptr(), entropy.data_ptr(), counts.data_ptr(),
                load_balance.data_ptr(), load_stats.data_ptr(), _lib.ptr(weights_act), act_code, ws.data_ptr(), ws_bytes,
                _lib.stream_of(logits),
            ),
            "mts_router_fwd",
        )
        ctx.save_for_backward(logits, weights, indices, counts)
        ctx.top_k = top_k
        ctx.normalize = normalize
        ctx.act_code = act_code
        ctx.mark_non_differentiable(indices, entropy, counts, load_stats)
        ctx.set_materialize_grads(False)   # no zero tensors for the outputs that took no part in the loss
        return weights, indices, prob_mean, z_loss, entropy, counts, load_balance, load_stats, weights_act

    @staticmethod
    @torch.amp.custom_bwd(device_type="cuda")
    def backward(ctx, grad_weights, _grad_indices, grad_probability_mean, grad_z_loss, _grad_entropy, _grad_counts,
                 grad_load_balance, _grad_load_stats, grad_weights_act):
        lib = _lib.load()
        logits, weights, indices, counts = ctx.saved_tensors
        T, E = logits.shape
        dev = logits.device

        def dense(g):   # an output that took no part in the loss comes as None and goes down as a null pointer
            return None if g is None else g.to(torch.float32).contiguous()

        g_w = dense(grad_weights)
        g_p = dense(grad_probability_mean)
        g_z = dense(grad_z_loss)
        g_lb = dense(grad_load_balance)
        g_w_act = None if grad_weights_act is None else grad_weights_act.contiguous()   # stays in the activation dtype
        grad_logits = torch.empty_like(logits)
        _lib.check(
            lib.mts_router_bwd(
                logits.data_ptr(), weights.data_ptr(), indices.data_ptr(), _lib.ptr(g_w), _lib.ptr(g_w_act), ctx.act_code,
                _lib.ptr(g_p), _lib.ptr(g_z), _lib.ptr(g_lb), counts.data_ptr(), T, E, ctx.top_k, int(ctx.normalize),
                grad_logits.data_ptr(), _lib.stream_of(logits),
            ),
            "mts_router_bwd",
        )
        return grad_logits, None, None, None


def router_postprocess(logits: torch.Tensor, top_k: int, *, normalize: bool, weights_dtype=None) -> RouterPostprocessOutput:
    """Process router logits without materialising the full probability matrix.

    ``weights_dtype`` (bf16 or fp16, an extension of the reference's signature) also asks for
    ``expert_weights_cast``, the differentiable copy of the weights in that dtype."""

    if logits.ndim != 2 or logits.dtype != torch.float32:
        raise ValueError("router logits must be a 2D fp32 tensor")
    if logits.shape[0] == 0:
        raise ValueError("router logits must contain at least one token")
    if not 1 <= top_k <= logits.shape[1]:
        raise ValueError(f"top_k must be in [1, {logits.shape[1]}], got {top_k}")
    if not is_router_postprocess_supported(logits, top_k, normalize):
        raise RuntimeError(
            "hip router postprocess requires non-empty 2D fp32 logits on the GPU, "
            f"1 <= top_k <= {_MAX_TOP_K} and at most {_MAX_EXPERTS} experts"
        )
    if weights_dtype not in (None, torch.bfloat16, torch.float16):
        raise ValueError("weights_dtype must be bfloat16 or float16")
    weights, indices, probability_mean, z_loss, entropy, counts, load_balance, load_stats, weights_cast = (
        _RouterPostprocessFunction.apply(logits, top_k, normalize, weights_dtype)
    )
    return RouterPostprocessOutput(
        expert_weights=weights,
        expert_indices=indices,
        probability_per_expert=probability_mean,
        z_loss=z_loss,
        entropy=entropy,
        expert_counts=counts,
        load_balance_loss=load_balance,
        load_stats=load_stats,
        expert_weights_cast=weights_cast,
    )


def is_router_logits_supported(hidden_states: torch.Tensor, weight: torch.Tensor) -> bool:
    return (
        hidden_states.is_cuda
        and weight.is_cuda
        and hidden_states.ndim == 2
        and weight.ndim == 2
        and hidden_states.dtype in (torch.bfloat16, torch.float16, torch.float32)
        and weight.dtype == torch.float32
        and hidden_states.shape[0] > 0
        and hidden_states.shape[1] == weight.shape[1]
        and weight.shape[0] <= 16
        and hidden_states.shape[1] % 4 == 0
        and hidden_states.shape[1] <= 4096
        and weight.shape[0] * weight.shape[1] * 4 <= _ROUTER_WEIGHT_LDS_BYTES
    )


class _RouterLogitsFunction(torch.autograd.Function):
    """logits = float(x) @ W_r^T without the fp32 copy of x; backward gives dx in x.dtype."""

    @staticmethod
    def forward(ctx, hidden_states: torch.Tensor, weight: torch.Tensor):
        lib = _lib.load()
        x = hidden_states.contiguous()
        w = weight.contiguous()
        T, H = x.shape
        E = w.shape[0]
        logits = torch.empty((T, E), device=x.device, dtype=torch.float32)
        _lib.check(
            lib.mts_router_logits_fwd(
                x.data_ptr(), w.data_ptr(), T, H, E, _lib.dtype_code(x.dtype), logits.data_ptr(), _lib.stream_of(x)
            ),
            "mts_router_logits_fwd",
        )
        ctx.save_for_backward(x, w)
        return logits

    @staticmethod
    def backward(ctx, grad_logits):
        lib = _lib.load()
        x, w = ctx.saved_tensors
        T, H = x.shape
        E = w.shape[0]
        g = grad_logits.to(torch.float32).contiguous()
        dx = torch.empty_like(x)
        dw = torch.empty_like(w)
        ws_bytes = lib.mts_router_logits_bwd_workspace_bytes(T, H, E)
        ws = torch.empty(ws_bytes, device=x.device, dtype=torch.uint8)
        _lib.check(
            lib.mts_router_logits_bwd(
                g.data_ptr(), x.data_ptr(), w.data_ptr(), T, H, E, _lib.dtype_code(x.dtype), dx.data_ptr(),
                dw.data_ptr(), ws.data_ptr(), ws_bytes, _lib.stream_of(x),
            ),
            "mts_router_logits_bwd",
        )
        return dx, dw


def router_logits(hidden_states: torch.Tensor, weight: torch.Tensor) -> torch.Tensor:
    """fp32 router logits of ``hidden_states`` [T,H] (bf16 or fp32) and ``weight`` [E,H] (fp32).

    Stands in for ``F.linear(hidden_states.float(), weight.float())`` of the reference's
    TopKRouter.forward (minitrain/model/moe_router.py:64-76).
    """

    if not is_router_logits_supported(hidden_states, weight):
        raise RuntimeError(
            "hip router_logits requires 2D bf16/fp32 activations and a 2D fp32 weight on the GPU with "
            "at most 16 experts and a hidden size that is a multiple of 4 and at most 4096 (E * H <= 32768)"
        )
    return _RouterLogitsFunction.apply(hidden_states, weight)
