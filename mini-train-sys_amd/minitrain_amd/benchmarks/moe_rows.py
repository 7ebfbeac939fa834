"""Fused-MoE operator rows in the schema of the reference's operator benchmarks
(benchmarks/operators/measurement.py:25-38, 485-496 and moe_runner.py:53,176-193):
``fwd/bwd/full_p50_ms`` and ``_p95_ms``, ``*_peak_mem_mb``, ``*_speedup`` against the PyTorch
expert loop on the same GPU, and the correctness columns ``max_abs``, ``max_rel``,
``relative_l2``, ``cosine_similarity`` with the acceptance rule
``relative_l2 <= 1e-2 and cosine_similarity >= 0.9999``.

    python -m minitrain_amd.benchmarks.moe_rows --profile layer --tokens 24576
    python -m minitrain_amd.benchmarks.moe_rows --profile mixtral --tokens 4096

    python -m minitrain_amd.benchmarks.moe_rows --tokens 24576 --zipf --capacity-factor 1.0

    python -m minitrain_amd.benchmarks.moe_rows --tokens 24576 --expert-shares 4862,12086,3507,3153,6471,5392,7811,5870 --no-torch

prints one JSON row per provider (``hip``, ``torch``).  ``--zipf`` skews the routing towards the
low expert ids (probability ~ rank^-1.2); ``--expert-shares`` draws every token's experts one after the
other with odds proportional to the given numbers (e.g. the routes per expert a trained router produced),
so that the routes per expert come out close to those proportions; with ``--capacity-factor`` every expert accepts at most
``ceil(factor*T*K/E)`` routes (minitrain/model/moe_router.py:38-42), the ``hip`` row runs the compacted
dispatch (dropped routes carry index -1), a ``hip_zero_weight`` row runs the same weights with every
route still dispatched, which is what masking the weights alone amounts to, and the selection kernel
is timed by itself (``capacity_mask_p50_ms``).  The ``torch`` provider is the expert loop
of the reference's PyTorch backend (minitrain/kernels/torch_ops.py:122-150) restated here as the
baseline of the table; it is not used by the operator.
"""

import argparse
import json
import math

import torch
import torch.nn.functional as F

PROFILES = {
    # name: (hidden, expert width, experts, top-k)
    "layer": (768, 1024, 8, 2),
    "mixtral": (4096, 14336, 8, 2),
}


def torch_expert_loop(x, gate_up, down, idx, w):
    out = torch.zeros_like(x)
    I = gate_up.shape[1] // 2
    for e in torch.unique(idx).tolist():
        tok, kpos = torch.where(idx == e)
        h = F.linear(x[tok], gate_up[e])
        y = F.linear(F.silu(h[:, :I]) * h[:, I:], down[e]) * w[tok, kpos].unsqueeze(-1)
        out.index_add_(0, tok, y)
    return out


def make_case(tokens, H, I, E, K, dtype, seed, zipf=False, shares=None):
    g = torch.Generator(device="cuda").manual_seed(seed)
    rn = lambda *s, std=1.0: (torch.randn(*s, generator=g, device="cuda") * std).to(dtype)
    x, gate_up, down = rn(tokens, H), rn(E, 2 * I, H, std=0.02), rn(E, H, I, std=0.02)
    logits = torch.randn(tokens, E, generator=g, device="cuda")
    if zipf:
        rank = torch.arange(1, E + 1, device="cuda", dtype=torch.float32)
        logits = logits + torch.log(rank ** -1.2 / (rank ** -1.2).sum())
    p, idx = torch.topk(torch.softmax(logits, dim=-1), K, dim=-1)
    if shares is not None:
        # K distinct experts per token, drawn one after the other with odds proportional to `shares`
        odds = torch.tensor(shares, dtype=torch.float64, device="cuda").expand(tokens, E).clone()
        cols = []
        for _ in range(K):
            c = torch.multinomial(odds, 1, generator=g)
            odds.scatter_(1, c, 0.0)
            cols.append(c)
        idx = torch.cat(cols, 1)
        p = torch.gather(torch.softmax(logits, dim=-1), 1, idx)
    w32 = p / p.sum(dim=-1, keepdim=True)
    grad = rn(tokens, H)
    idx = idx.int()
    return dict(x=x, gate_up=gate_up, down=down, idx=idx, idx_all=idx, w=w32.to(dtype), w32=w32, grad=grad)


def limit_capacity(case, ops, E, factor, min_capacity=4):
    """Applies the capacity limit to a case: masked and renormalised weights, and the dispatch with
    -1 on the dropped routes under ``idx`` (``idx_all`` keeps every route)."""
    tokens, K = case["idx_all"].shape
    capacity = max(min_capacity, math.ceil(factor * tokens * K / E))
    keep, kept_index, accepted = ops.capacity_mask(case["idx_all"], case["w32"], E, capacity)
    w = case["w32"] * keep
    denom = w.sum(dim=-1, keepdim=True)
    w = torch.where(denom > 0, w / denom.clamp_min(torch.finfo(w.dtype).eps), w)
    case.update(idx=kept_index, w=w.to(case["x"].dtype))
    return capacity, float(1.0 - keep.float().mean()), accepted.tolist()


def _stats(actual, expected):
    a, b = actual.double().flatten(), expected.double().flatten()
    diff = (a - b).abs()
    na, nb = float(a.norm()), float(b.norm())
    return {
        "max_abs": float(diff.max()),
        "max_rel": float((diff / b.abs().clamp_min(1e-6)).max()),
        "relative_l2": float((a - b).norm()) / nb if nb > 0 else math.inf,
        "cosine_similarity": float(torch.dot(a, b)) / (na * nb) if na * nb > 0 else -1.0,
    }


def _quantiles(samples):
    v = torch.tensor(samples, dtype=torch.float64)
    p50, p95 = torch.quantile(v, torch.tensor([0.5, 0.95], dtype=torch.float64)).tolist()
    return p50, p95


def _time(fn, iters, warmup):
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    out = []
    for _ in range(iters):
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        fn()
        b.record()
        torch.cuda.synchronize()
        out.append(a.elapsed_time(b))
    return _quantiles(out)


def _peak_mb(fn):
    torch.cuda.synchronize()
    torch.cuda.empty_cache()
    torch.cuda.reset_peak_memory_stats()
    base = torch.cuda.memory_allocated()
    fn()
    torch.cuda.synchronize()
    return max(0.0, (torch.cuda.max_memory_allocated() - base) / 2**20)


def measure(provider, op, case, iters, warmup, idx_key="idx"):
    case = {**case, "idx": case[idx_key]}
    leaves = {n: case[n].detach().clone().requires_grad_(True) for n in ("x", "gate_up", "down", "w")}

    def fwd():
        with torch.no_grad():
            op(leaves["x"], leaves["gate_up"], leaves["down"], case["idx"], leaves["w"])

    def full():
        for t in leaves.values():
            t.grad = None
        op(leaves["x"], leaves["gate_up"], leaves["down"], case["idx"], leaves["w"]).backward(case["grad"])

    held = {}

    def bwd_setup():
        for t in leaves.values():
            t.grad = None
        held["out"] = op(leaves["x"], leaves["gate_up"], leaves["down"], case["idx"], leaves["w"])

    def bwd_timed():
        samples = []
        for i in range(warmup + iters):
            bwd_setup()
            torch.cuda.synchronize()
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record()
            held["out"].backward(case["grad"])
            b.record()
            torch.cuda.synchronize()
            if i >= warmup:
                samples.append(a.elapsed_time(b))
        return _quantiles(samples)

    row = {"provider": provider}
    row["fwd_p50_ms"], row["fwd_p95_ms"] = _time(fwd, iters, warmup)
    row["bwd_p50_ms"], row["bwd_p95_ms"] = bwd_timed()
    row["full_p50_ms"], row["full_p95_ms"] = _time(full, iters, warmup)
    row["fwd_peak_mem_mb"] = _peak_mb(fwd)
    row["full_peak_mem_mb"] = _peak_mb(full)
    bwd_setup()
    row["bwd_peak_mem_mb"] = _peak_mb(lambda: held["out"].backward(case["grad"]))
    held.clear()
    return row


def correctness(op, case):
    """hip against the expert loop evaluated in fp32 on the same inputs (gradients concatenated)."""
    def run(fn, dtype):
        leaves = {n: case[n].detach().to(dtype).requires_grad_(True) for n in ("x", "gate_up", "down", "w")}
        out = fn(leaves["x"], leaves["gate_up"], leaves["down"], case["idx"], leaves["w"])
        out.backward(case["grad"].to(dtype))
        return out.detach(), [leaves[n].grad for n in ("x", "gate_up", "down", "w")]

    out_a, g_a = run(op, case["x"].dtype)
    case = {**case, "idx": case["idx_all"]}     # the expert loop dispatches every route; dropped ones weigh zero
    out_b, g_b = run(torch_expert_loop, torch.float32)
    # the gradient of a dropped route's weight is defined while it is dispatched and zero once it is not
    dropped = case["w"] == 0
    g_a[3] = torch.where(dropped, torch.zeros_like(g_a[3]), g_a[3])
    g_b[3] = torch.where(dropped, torch.zeros_like(g_b[3]), g_b[3])
    fwd = _stats(out_a, out_b)
    bwd = _stats(torch.cat([g.flatten().float() for g in g_a]), torch.cat([g.flatten() for g in g_b]))
    ok = lambda s: s["relative_l2"] <= 1e-2 and s["cosine_similarity"] >= 0.9999
    row = {f"fwd_{k}": v for k, v in fwd.items()}
    row.update({f"bwd_{k}": v for k, v in bwd.items()})
    row["fwd_correct"], row["bwd_correct"] = ok(fwd), ok(bwd)
    row["acceptance"] = "relative_l2<=1e-2_and_cosine>=0.9999"
    return row


def operator_rows(profile="layer", tokens=24576, iters=20, warmup=5, seed=1, with_torch=True, zipf=False,
                  capacity_factor=None, shares=None):
    """The benchmark rows as dictionaries: ``hip`` first, then ``hip_zero_weight`` (capacity runs) and ``torch``."""
    from minitrain_amd.model.ops import get_ops_backend

    H, I, E, K = PROFILES[profile]
    ops = get_ops_backend("hip")
    case = make_case(tokens, H, I, E, K, torch.bfloat16, seed, zipf=zipf, shares=shares)
    common = dict(op="fused_moe", profile=profile, size=tokens, hidden=H, expert_width=I, experts=E,
                  top_k=K, dtype="bf16", device=torch.cuda.get_device_name(0), timer="cuda_events",
                  routing="shares" if shares is not None else ("zipf" if zipf else "uniform"),
                  routes_per_expert=torch.bincount(case["idx"].flatten().long(), minlength=E).tolist())
    extra_rows = []
    if capacity_factor is not None:
        capacity, dropped, accepted = limit_capacity(case, ops, E, capacity_factor)
        p50, p95 = _time(lambda: ops.capacity_mask(case["idx_all"], case["w32"], E, capacity), iters, warmup)
        common.update(capacity_factor=capacity_factor, capacity=capacity, dropped_route_fraction=dropped,
                      accepted_per_expert=accepted, capacity_mask_p50_ms=p50, capacity_mask_p95_ms=p95)
        extra_rows.append(measure("hip_zero_weight", ops.fused_moe, case, iters, warmup, idx_key="idx_all"))
    hip = measure("hip", ops.fused_moe, case, iters, warmup)
    hip.update(correctness(ops.fused_moe, case))
    rows = [hip] + extra_rows
    if with_torch:
        ref = measure("torch", torch_expert_loop, case, max(3, iters // 4), 2, idx_key="idx_all")
        for m in ("fwd", "bwd", "full"):
            hip[f"{m}_speedup"] = ref[f"{m}_p50_ms"] / hip[f"{m}_p50_ms"]
            ref[f"{m}_speedup"] = 1.0
        rows.append(ref)
    return [{**common, **r} for r in rows]


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--profile", choices=sorted(PROFILES), default="layer")
    ap.add_argument("--tokens", type=int, default=24576)
    ap.add_argument("--iters", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--seed", type=int, default=1)
    ap.add_argument("--no-torch", action="store_true", help="skip the PyTorch expert-loop baseline rows")
    ap.add_argument("--zipf", action="store_true", help="routing skewed towards the low expert ids")
    ap.add_argument("--capacity-factor", type=float, default=None)
    ap.add_argument("--expert-shares", type=str, default=None,
                    help="comma-separated odds per expert: the routes per expert come out close to these proportions")
    args = ap.parse_args()
    shares = [float(v) for v in args.expert_shares.split(",")] if args.expert_shares else None
    if shares is not None and len(shares) != PROFILES[args.profile][2]:
        ap.error(f"--expert-shares needs {PROFILES[args.profile][2]} numbers")
    for row in operator_rows(args.profile, args.tokens, args.iters, args.warmup, args.seed, not args.no_torch, args.zipf,
                             args.capacity_factor, shares):
        print(json.dumps(row))


if __name__ == "__main__":
    main()
