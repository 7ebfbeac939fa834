"""The whole MoE layer (router projection, post-process, routing metadata, experts, combine) as one
autograd node.

The reference composes the layer from three autograd nodes (minitrain/model/moe_router.py:64-90 and
minitrain/model/blocks.py:86-102): ``F.linear`` for the router logits, ``router_postprocess`` and
``fused_moe``.  The activations feed two of them, so autograd sums two gradients for ``x`` with one more
kernel, and every node boundary is a launch boundary.  Here the forward pass starts with the chained
head (two launches: projection + post-process, then scatter + statistics) and the backward pass
forms the router's gradient before the dX combine, which adds it to the experts' gradient in the same
pass.  Same arithmetic as the separate operators; it is an extension the MoE block uses when the backend
offers it (``ops.moe_layer``) and the configuration allows it.
"""

import torch

from minitrain_amd import _lib
from minitrain_amd.kernels.hip.fused_moe import (RouterTail, expert_contract, first_violation, moe_backward, moe_forward,
                                                 needs_padding)
from minitrain_amd.kernels.hip.router import _MAX_TOP_K, is_router_logits_supported


def moe_layer_violation(x, router_weight, gate_up_proj, down_proj, top_k: int):
    """The first requirement of the layer contract that the arguments miss, or None."""
    missed = first_violation(expert_contract(x, gate_up_proj, down_proj))
    if missed is not None:
        return missed
    E = gate_up_proj.shape[0]
    return first_violation([
        (torch.is_tensor(router_weight) and router_weight.ndim == 2 and router_weight.shape[0] == E,
         "router weight is [E,H]"),
        (is_router_logits_supported(x, router_weight),
         "an fp32 router weight on the same GPU, at most 16 experts and a hidden size of at most 4096 (E * H <= 32768)"),
        (1 <= top_k <= min(E, _MAX_TOP_K), f"1 <= top_k <= min(E, {_MAX_TOP_K})"),
        (not needs_padding(x, gate_up_proj), "hidden and expert widths that are whole 16-byte chunks"),
        (x.shape[0] * top_k < 2**31, "fewer than 2^31 routes"),
    ])


class _MoELayerFunction(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, router_weight, gate_up_proj, down_proj, top_k, normalize):
        lib = _lib.load()
        x, router_weight = x.contiguous(), router_weight.contiguous()
        gate_up_proj, down_proj = gate_up_proj.contiguous(), down_proj.contiguous()
        T, H = x.shape
        E, K = router_weight.shape[0], int(top_k)
        TK = T * K
        dev = x.device
        act = _lib.dtype_code(x.dtype)
        f32, i32 = dict(dtype=torch.float32, device=dev), dict(dtype=torch.int32, device=dev)
        logits = torch.empty(T, E, **f32)
        weights = torch.empty(T, K, **f32)
        indices = torch.empty(T, K, **i32)
        narrow = x.dtype != torch.float32
        weights_act = torch.empty(T, K, dtype=x.dtype, device=dev) if narrow else None
        stats = torch.empty(2 * E + 10, **f32)   # E mean probabilities, z, entropy, load-balancing term, E + 7 load statistics
        prob_mean, z_loss, entropy, load_balance, load_stats = stats[:E], stats[E], stats[E + 1], stats[E + 2], stats[E + 3:]
        # counts, expert_start and the three permutation arrays in one allocation, each 16-byte aligned
        pad = lambda n: (n + 3) // 4 * 4
        offsets = [0, pad(E), pad(E) + pad(E + 1)]
        offsets += [offsets[2] + pad(TK), offsets[2] + 2 * pad(TK)]
        meta = torch.empty(offsets[2] + 3 * pad(TK), **i32)
        counts, expert_start = meta[:E], meta[offsets[1]:offsets[1] + E + 1]
        s_scatter, s_reverse, x_gather = (meta[o:o + TK] for o in offsets[2:])
        ws_bytes = lib.mts_moe_head_workspace_bytes(T, K, E)
        ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
        _lib.check(
            lib.mts_moe_head_fwd(
                x.data_ptr(), router_weight.data_ptr(), T, H, E, K, int(normalize), act, logits.data_ptr(),
                weights.data_ptr(), indices.data_ptr(), _lib.ptr(weights_act), prob_mean.data_ptr(), z_loss.data_ptr(),
                entropy.data_ptr(), counts.data_ptr(), load_balance.data_ptr(), load_stats.data_ptr(),
                expert_start.data_ptr(), s_scatter.data_ptr(), s_reverse.data_ptr(), x_gather.data_ptr(), ws.data_ptr(),
                ws_bytes, _lib.stream_of(x),
            ),
            "mts_moe_head_fwd",
        )
        weights_flat = (weights_act if narrow else weights).view(-1)
        out, tensors, state = moe_forward(x, gate_up_proj, down_proj, weights_flat,
                                          (expert_start, x_gather, s_scatter, s_reverse))
        ctx.n_moe = len(tensors)
        ctx.save_for_backward(*tensors, router_weight, logits, weights, indices, counts)
        ctx.state = state
        ctx.route = (K, bool(normalize), narrow)
        ctx.mark_non_differentiable(entropy, counts, load_stats, indices, weights)
        ctx.set_materialize_grads(False)
        return out, load_balance, z_loss, prob_mean, entropy, counts, load_stats, indices, weights

    @staticmethod
    def backward(ctx, g_out, g_load_balance, g_z_loss, g_prob_mean, *_unused):
        lib = _lib.load()
        tensors = ctx.saved_tensors[:ctx.n_moe]
        router_weight, logits, weights, indices, counts = ctx.saved_tensors[ctx.n_moe:]
        x = tensors[0]
        T, H = x.shape
        E = router_weight.shape[0]
        K, normalize, narrow = ctx.route
        need_x, need_wr, need_w1, need_w2 = ctx.needs_input_grad[:4]
        act = _lib.dtype_code(x.dtype)
        got = {}

        def f32(g):
            return None if g is None else g.to(torch.float32).contiguous()

        g_lb, g_z, g_p = f32(g_load_balance), f32(g_z_loss), f32(g_prob_mean)

        tail = RouterTail(router_weight, logits, weights, indices, counts, g_p, g_z, g_lb, normalize)

        def router_gradient(d_weights):
            """dS and the loss terms of the router -> the router's share of dx, and dW_r."""
            if tail.dx_r is not None:   # already formed inside the launch of the experts' backward
                got["dx_r"], got["dw_r"] = tail.dx_r, tail.dw_r
                return tail.dx_r
            dx_r = torch.empty_like(x)
            dw_r = torch.empty_like(router_weight)
            ws_bytes = lib.mts_moe_head_bwd_workspace_bytes(T, H, E)
            ws = torch.empty(ws_bytes, dtype=torch.uint8, device=x.device)
            g_w = d_weights if (d_weights is not None and not narrow) else None
            g_w_act = d_weights if (d_weights is not None and narrow) else None
            _lib.check(
                lib.mts_moe_head_bwd(
                    x.data_ptr(), router_weight.data_ptr(), logits.data_ptr(), weights.data_ptr(), indices.data_ptr(),
                    counts.data_ptr(), _lib.ptr(g_w), _lib.ptr(g_w_act), _lib.ptr(g_p), _lib.ptr(g_z), _lib.ptr(g_lb),
                    T, H, E, K, int(normalize), act, dx_r.data_ptr(), dw_r.data_ptr(), ws.data_ptr(), ws_bytes,
                    _lib.stream_of(x),
                ),
                "mts_moe_head_bwd",
            )
            got["dx_r"], got["dw_r"] = dx_r, dw_r
            return dx_r

        if g_out is None:   # only the router's loss terms reach this layer
            dx = router_gradient(None) if (need_x or need_wr) else None
            return (dx if need_x else None), (got.get("dw_r") if need_wr else None), None, None, None, None
        wants_router = need_x or need_wr
        dx, dw1, dw2, ds = moe_backward(tensors, ctx.state, g_out.contiguous(), (need_x, need_w1, need_w2, wants_router),
                                        x_addend=router_gradient if wants_router else None,
                                        router_tail=tail if wants_router else None)
        if wants_router and "dw_r" not in got:   # x needs no gradient: the combine, and with it the callback, was skipped
            router_gradient(ds)
        return dx, (got.get("dw_r") if need_wr else None), dw1, dw2, None, None


def moe_layer(x, router_weight, gate_up_proj, down_proj, top_k: int, *, normalize: bool):
    """``(hidden, load_balance_loss, z_loss, probability_per_expert, entropy, expert_counts, load_stats,
    expert_indices, expert_weights)`` of one MoE layer on ``x [T,H]``; the first four are differentiable."""
    missed = moe_layer_violation(x, router_weight, gate_up_proj, down_proj, top_k)
    if missed is not None:
        raise RuntimeError(f"Unsupported tensor contract for the hip MoE layer: it requires {missed}")
    return _MoELayerFunction.apply(x, router_weight, gate_up_proj, down_proj, top_k, normalize)
