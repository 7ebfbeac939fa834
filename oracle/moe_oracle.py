"""CPU oracle for the fused top-k MoE layer.  TEST INFRASTRUCTURE ONLY.

This module restates, on the CPU, the arithmetic of the reference's MoE path so
that the HIP kernels can be checked against it.  It is never imported by the
product package: only the test-suite, the smoke check and the benchmark's
``cpu_baseline`` leg use it, and there only as the checker.

Reference lines each function follows (paths relative to the reference root):

* ``router_postprocess``      -> minitrain/kernels/torch_ops.py:87-120 (formulas),
                                 minitrain/kernels/triton/router.py:101-126 (top-k
                                 by repeated arg-max on the LOGITS, lowest index
                                 wins a tie).
* ``router_backward_closed``  -> minitrain/kernels/triton/router.py:193-253.
* ``routing_metadata``        -> minitrain/kernels/triton/fused_moe.py:74-154 and
                                 fused_moe_kernels.py:101-119, 174-234.
* ``fused_moe``               -> minitrain/kernels/torch_ops.py:122-150.
* ``fused_moe_backward_closed`` -> minitrain/kernels/triton/fused_moe_kernels.py:
                                 567-596 (dS, dgate, dup), 627-672 (dW2),
                                 700-756 (dx), 783-828 (dW1).
* ``topk_router``             -> minitrain/model/moe_router.py:63-90, 138-144.
* ``expert_capacity``, ``capacity_mask`` -> minitrain/model/moe_router.py:29-61.
* ``apply_capacity``          -> the switched-off block at minitrain/model/moe_router.py:
                                 98-110 (mask the weights, renormalise per token).
* ``moe_feed_forward``        -> minitrain/model/blocks.py:86-96.

How each function is pinned (see tests/test_oracle_*.py):

* router forward: scipy ``logsumexp``/``softmax`` in float64, the closed form
  "normalised weights = softmax over the selected logits", constructed ties.
* router backward: float64 central finite differences and autograd of the
  forward restatement against the closed form.
* routing metadata: the worked example held by the reference
  (minitrain/kernels/triton/moe_router_scatter.md:22-26,109,162-164,202-203),
  numpy ``bincount``/``cumsum``/stable ``argsort``, permutation invariants.
* fused MoE forward: a per-route float64 brute-force loop on tiny shapes.
* fused MoE backward: float64 finite differences and autograd against the
  closed form.
* capacity mask: a per-expert Python sort on small cases, the invariants of the
  rule (kept = min(count, capacity) per expert, no dropped route outweighs a kept
  one of its expert, ties leave in descending entry order) and the all-ties case
  K=1 with normalised weights, where the first ``capacity`` tokens of an expert stay.
* dropped routes in ``fused_moe`` (expert index -1): the same outputs and
  gradients as the reference's own convention for them, a zero weight
  (minitrain/kernels/torch_ops.py:135-140).

Two behaviours of the reference's PyTorch path are library-defined and are NOT
reproduced bit for bit ("parity unpinned" at the bit level, pinned at tolerance
level): the order ``torch.topk`` returns tied probabilities in, which is replaced
here by the lowest-index rule of the reference's Triton kernel, and the bf16
rounding sequence of its expert loop, which is replaced by an fp32-accumulated
evaluation (``fused_moe`` with ``compute_dtype=torch.float32``).
"""

from __future__ import annotations

import math
from dataclasses import dataclass

import numpy as np
import torch
import torch.nn.functional as F


# ---------------------------------------------------------------------------
# Synthetic inputs (portable: numpy Philox stream, documented draw order)
# ---------------------------------------------------------------------------

def make_inputs(seed: int, T: int, H: int, E: int, I: int, *, n_layers: int = 12):
    """Draw ``x, W_r, gate_up_proj, down_proj, G`` in that order, all float32.

    x ~ N(0,1); router and expert weights ~ N(0,0.02); upstream gradient ~ N(0,1).
    The caller casts to bf16 where the configuration asks for it.
    """
    del n_layers
    rng = np.random.Generator(np.random.Philox(seed))
    x = rng.standard_normal((T, H), dtype=np.float32)
    w_r = rng.standard_normal((E, H), dtype=np.float32) * np.float32(0.02)
    gate_up = rng.standard_normal((E, 2 * I, H), dtype=np.float32) * np.float32(0.02)
    down = rng.standard_normal((E, H, I), dtype=np.float32) * np.float32(0.02)
    g = rng.standard_normal((T, H), dtype=np.float32)
    return tuple(torch.from_numpy(a) for a in (x, w_r, gate_up, down, g))


def zipf_log_bias(E: int, s: float = 1.2) -> torch.Tensor:
    """log p_e with p_e proportional to rank^-s (load-imbalanced routing)."""
    p = np.arange(1, E + 1, dtype=np.float64) ** (-s)
    p /= p.sum()
    return torch.from_numpy(np.log(p).astype(np.float32))


def inject_ties(logits: torch.Tensor, fraction: float, seed: int) -> torch.Tensor:
    """Overwrite logits on a seeded fraction of rows so that exact ties straddle
    the top-2 selection boundary: rank 1/2 two-way, rank 2/3 two-way, three-way."""
    T, E = logits.shape
    rng = np.random.Generator(np.random.Philox(seed + 1000))
    n = max(1, int(round(fraction * T))) if fraction > 0 else 0
    rows = rng.choice(T, size=n, replace=False)
    out = logits.clone()
    for j, t in enumerate(rows):
        cols = rng.choice(E, size=min(3, E), replace=False)
        row = out[t]
        top = float(row.max()) + 1.0
        kind = j % 3
        if kind == 0 or len(cols) < 3:        # two-way tie for rank 1 and 2
            row[cols[0]] = top
            row[cols[1]] = top
        elif kind == 1:                       # clear rank 1, two-way tie for rank 2/3
            row[cols[0]] = top + 1.0
            row[cols[1]] = top
            row[cols[2]] = top
        else:                                 # three-way tie across ranks 1..3
            row[cols[0]] = top
            row[cols[1]] = top
            row[cols[2]] = top
    return out


# ---------------------------------------------------------------------------
# Router post-process
# ---------------------------------------------------------------------------

@dataclass
class RouterOut:
    expert_weights: torch.Tensor
    expert_indices: torch.Tensor
    probability_per_expert: torch.Tensor
    z_loss: torch.Tensor
    entropy: torch.Tensor


def select_topk_lowest_index(logits: torch.Tensor, top_k: int) -> torch.Tensor:
    """K rounds of arg-max over the not yet selected logits; ties go to the smaller
    expert index.  A stable descending sort yields exactly that order."""
    order = torch.sort(logits, dim=-1, descending=True, stable=True).indices
    return order[:, :top_k].contiguous()


def router_postprocess(logits: torch.Tensor, top_k: int, *, normalize: bool) -> RouterOut:
    if logits.ndim != 2 or logits.dtype not in (torch.float32, torch.float64):
        raise ValueError("router logits must be a 2D fp32 tensor")
    if logits.shape[0] == 0:
        raise ValueError("router logits must contain at least one token")
    if not 1 <= top_k <= logits.shape[1]:
        raise ValueError(f"top_k must be in [1, {logits.shape[1]}], got {top_k}")
    L = torch.logsumexp(logits, dim=-1, keepdim=True)
    p = torch.exp(logits - L)
    idx = select_topk_lowest_index(logits.detach(), top_k)
    w = torch.gather(p, 1, idx)
    if normalize:
        w = w / w.sum(dim=-1, keepdim=True).clamp_min(torch.finfo(torch.float32).eps)
    entropy = -(p * p.clamp_min(1e-9).log()).sum(dim=-1).mean().detach()
    return RouterOut(w, idx.to(torch.int32), p.mean(dim=0), L.square().mean(), entropy)


def router_backward_closed(logits, indices, weights, g_w, g_p, g_z, *, normalize: bool):
    """Analytic Jacobian product of ``router_postprocess`` (numpy, float64)."""
    l = np.asarray(logits, dtype=np.float64)
    T, E = l.shape
    idx = np.asarray(indices, dtype=np.int64)
    w = np.asarray(weights, dtype=np.float64)
    g_w = np.asarray(g_w, dtype=np.float64)
    m = l.max(axis=1, keepdims=True)
    L = m + np.log(np.exp(l - m).sum(axis=1, keepdims=True))
    p = np.exp(l - L)
    dp = np.broadcast_to(np.asarray(g_p, dtype=np.float64)[None, :] / T, (T, E)).copy()
    if not normalize:
        np.add.at(dp, (np.arange(T)[:, None], idx), g_w)
    dl = p * (dp - (p * dp).sum(axis=1, keepdims=True))
    dl += float(g_z) * (2.0 / T) * L * p
    if normalize:
        dot = (w * g_w).sum(axis=1, keepdims=True)
        np.add.at(dl, (np.arange(T)[:, None], idx), w * (g_w - dot))
    return dl


# ---------------------------------------------------------------------------
# Routing metadata (integer work, numpy)
# ---------------------------------------------------------------------------

@dataclass
class RoutingMeta:
    counts: np.ndarray            # [E]   routes per expert
    expert_start: np.ndarray      # [E+1] exclusive prefix sum, last = number of kept routes (T*K without drops)
    s_scatter_idx: np.ndarray     # [TK]  sorted position -> entry (t*K+k)
    s_reverse_scatter_idx: np.ndarray  # [TK] entry -> sorted position
    x_gather_idx: np.ndarray      # [TK]  sorted position -> token
    tile_row_start: np.ndarray    # [n_tiles] first row of each block_m-row tile
    tile_expert: np.ndarray       # [n_tiles]


def routing_metadata(top_k_index, E: int, block_m: int = 64) -> RoutingMeta:
    idx = np.asarray(top_k_index)
    T, K = idx.shape
    flat = idx.reshape(-1).astype(np.int64)
    # a negative index is a dropped route of a capacity-limited dispatch: it gets no row
    kept = np.flatnonzero(flat >= 0)
    counts = np.bincount(flat[kept], minlength=E).astype(np.int32)
    expert_start = np.zeros(E + 1, dtype=np.int32)
    expert_start[1:] = np.cumsum(counts)
    order = kept[np.argsort(flat[kept], kind="stable")].astype(np.int32)
    rev = np.full(T * K, -1, dtype=np.int32)
    rev[order] = np.arange(order.size, dtype=np.int32)
    rows, experts = [], []
    for e in range(E):
        for r in range(int(expert_start[e]), int(expert_start[e + 1]), block_m):
            rows.append(r)
            experts.append(e)
    return RoutingMeta(
        counts=counts,
        expert_start=expert_start,
        s_scatter_idx=order,
        s_reverse_scatter_idx=rev,
        x_gather_idx=(order // K).astype(np.int32),
        tile_row_start=np.asarray(rows, dtype=np.int32),
        tile_expert=np.asarray(experts, dtype=np.int32),
    )


# ---------------------------------------------------------------------------
# Fused MoE (dispatch -> SwiGLU experts -> weighted combine)
# ---------------------------------------------------------------------------

def fused_moe(x, gate_up_proj, down_proj, top_k_index, top_k_weights, *, compute_dtype=None):
    """Expert loop.  With ``compute_dtype=None`` every op runs (and rounds) in the
    input dtype, as the reference's PyTorch path does; with ``torch.float32`` or
    ``torch.float64`` the inputs are widened first, nothing is rounded in between
    and the result is returned in the wide dtype ("fp32-accumulated reference")."""
    if compute_dtype is not None:
        x = x.to(compute_dtype)
        gate_up_proj = gate_up_proj.to(compute_dtype)
        down_proj = down_proj.to(compute_dtype)
        top_k_weights = top_k_weights.to(compute_dtype)
    out = torch.zeros_like(x)
    for e in torch.unique(top_k_index).tolist():
        if e < 0:   # dropped route of a capacity-limited dispatch: no contribution
            continue
        tok, kpos = torch.where(top_k_index == e)
        if tok.numel() == 0:
            continue
        cur = x[tok]
        gate, up = F.linear(cur, gate_up_proj[e]).chunk(2, dim=-1)
        cur = F.silu(gate) * up
        cur = F.linear(cur, down_proj[e])
        cur = cur * top_k_weights[tok, kpos, None]
        out.index_add_(0, tok, cur.to(out.dtype))
    return out


def fused_moe_bruteforce(x, gate_up_proj, down_proj, top_k_index, top_k_weights):
    """One route at a time, float64, plain loops; for tiny shapes only."""
    x = np.asarray(x, dtype=np.float64)
    w1 = np.asarray(gate_up_proj, dtype=np.float64)
    w2 = np.asarray(down_proj, dtype=np.float64)
    idx = np.asarray(top_k_index)
    s = np.asarray(top_k_weights, dtype=np.float64)
    T, H = x.shape
    I = w1.shape[1] // 2
    out = np.zeros((T, H))
    for t in range(T):
        for k in range(idx.shape[1]):
            e = int(idx[t, k])
            if e < 0:
                continue
            g = np.array([sum(w1[e, i, h] * x[t, h] for h in range(H)) for i in range(I)])
            u = np.array([sum(w1[e, I + i, h] * x[t, h] for h in range(H)) for i in range(I)])
            a = g / (1.0 + np.exp(-g)) * u
            y = np.array([sum(w2[e, h, i] * a[i] for i in range(I)) for h in range(H)])
            out[t] += s[t, k] * y
    return out


def fused_moe_backward_closed(x, gate_up_proj, down_proj, top_k_index, top_k_weights, d_out):
    """Closed-form gradients (numpy float64): returns dx, dW1, dW2, dS[T,K]."""
    x = np.asarray(x, dtype=np.float64)
    w1 = np.asarray(gate_up_proj, dtype=np.float64)
    w2 = np.asarray(down_proj, dtype=np.float64)
    idx = np.asarray(top_k_index)
    s = np.asarray(top_k_weights, dtype=np.float64)
    dO = np.asarray(d_out, dtype=np.float64)
    T, H = x.shape
    K = idx.shape[1]
    I = w1.shape[1] // 2
    dx = np.zeros_like(x)
    dw1 = np.zeros_like(w1)
    dw2 = np.zeros_like(w2)
    dS = np.zeros((T, K))
    for t in range(T):
        for k in range(K):
            e = int(idx[t, k])
            if e < 0:
                continue
            z = w1[e] @ x[t]
            g, u = z[:I], z[I:]
            sig = 1.0 / (1.0 + np.exp(-g))
            a = g * sig * u
            A = w2[e].T @ dO[t]
            dS[t, k] = A @ a
            da = s[t, k] * A
            dg = da * u * sig * (1.0 + g * (1.0 - sig))
            du = da * g * sig
            dz = np.concatenate([dg, du])
            dw2[e] += np.outer(dO[t], s[t, k] * a)
            dw1[e] += np.outer(dz, x[t])
            dx[t] += w1[e].T @ dz
    return dx, dw1, dw2, dS


# ---------------------------------------------------------------------------
# Capacity-limited dispatch
# ---------------------------------------------------------------------------

def expert_capacity(tokens: int, top_k: int, num_experts: int, factor: float, min_capacity: int) -> int:
    return max(min_capacity, math.ceil(factor * tokens * top_k / num_experts))


def capacity_mask(expert_indices, expert_weights, num_experts: int, capacity: int) -> torch.Tensor:
    """bool ``[T,K]``: routes ordered by descending weight (stable), then grouped by expert
    (stable); a route stays if its rank inside its expert is below ``capacity``."""
    e = np.asarray(expert_indices).reshape(-1).astype(np.int64)
    w = np.asarray(expert_weights.detach().float()).reshape(-1)
    by_weight = np.argsort(-w, kind="stable")
    route_order = by_weight[np.argsort(e[by_weight], kind="stable")]
    counts = np.bincount(e, minlength=num_experts)
    first = np.cumsum(counts) - counts
    rank = np.arange(e.size) - np.repeat(first, counts)
    keep = np.zeros(e.size, dtype=bool)
    keep[route_order] = rank < capacity
    return torch.from_numpy(keep.reshape(tuple(expert_indices.shape)))


def apply_capacity(expert_weights, keep, *, normalize: bool):
    """Weights of dropped routes become zero; with ``normalize`` the weights a token has
    left are rescaled to sum to one (a token that lost every route keeps zeros)."""
    w = expert_weights * keep
    if normalize:
        denominator = w.sum(dim=-1, keepdim=True)
        w = torch.where(denominator > 0, w / denominator.clamp_min(torch.finfo(w.dtype).eps), w)
    return w


# ---------------------------------------------------------------------------
# Callers: router module arithmetic and the MoE block
# ---------------------------------------------------------------------------

@dataclass
class RouterModuleOut:
    expert_indices: torch.Tensor
    expert_weights: torch.Tensor
    auxiliary_loss: torch.Tensor
    z_loss: torch.Tensor
    logits: torch.Tensor
    route: RouterOut


def topk_router(hidden, router_weight, top_k: int, *, normalize: bool = True,
                logit_bias=None, logits_override=None) -> RouterModuleOut:
    """fp32 router GEMM -> post-process -> assignment counts -> aux loss -> casts."""
    E = router_weight.shape[0]
    logits = F.linear(hidden.float(), router_weight.float())
    if logit_bias is not None:
        logits = logits + logit_bias
    if logits_override is not None:
        logits = logits_override
    route = router_postprocess(logits, top_k, normalize=normalize)
    counts = torch.bincount(route.expert_indices.flatten().long(), minlength=E)
    frac = counts.float() / route.expert_indices.numel()
    aux = E * torch.sum(frac * route.probability_per_expert)
    return RouterModuleOut(
        expert_indices=route.expert_indices.to(torch.int32),
        expert_weights=route.expert_weights.to(hidden.dtype),
        auxiliary_loss=aux,
        z_loss=route.z_loss,
        logits=logits,
        route=route,
    )


def moe_feed_forward(x, router_weight, gate_up_proj, down_proj, top_k: int, *,
                     normalize: bool = True, compute_dtype=None, logit_bias=None,
                     logits_override=None):
    """Router + fused MoE on a ``[T,H]`` activation; returns (hidden, router record)."""
    r = topk_router(x, router_weight, top_k, normalize=normalize,
                    logit_bias=logit_bias, logits_override=logits_override)
    hidden = fused_moe(x, gate_up_proj, down_proj, r.expert_indices, r.expert_weights,
                       compute_dtype=compute_dtype)
    return hidden, r


# ---------------------------------------------------------------------------
# Error statistics shared by the parity tests and the benchmark
# ---------------------------------------------------------------------------

def error_stats(actual: torch.Tensor, expected: torch.Tensor) -> dict:
    """max-abs, scale-normalised max error (max|a-b| / max|b|), relative L2 and
    cosine, all evaluated in float64."""
    a = actual.detach().double().cpu().flatten()
    b = expected.detach().double().cpu().flatten()
    diff = (a - b).abs()
    max_abs = float(diff.max()) if diff.numel() else 0.0
    scale = float(b.abs().max()) if b.numel() else 0.0
    sq_b = float((b * b).sum())
    sq_a = float((a * a).sum())
    rel_l2 = math.sqrt(float((diff * diff).sum()) / sq_b) if sq_b > 0 else (0.0 if max_abs == 0 else math.inf)
    den = math.sqrt(sq_a * sq_b)
    cos = float((a * b).sum()) / den if den > 0 else (1.0 if sq_a == sq_b == 0 else 0.0)
    return {
        "max_abs": max_abs,
        "max_rel_scaled": (max_abs / scale) if scale > 0 else (0.0 if max_abs == 0 else math.inf),
        "relative_l2": rel_l2,
        "cosine": cos,
    }
