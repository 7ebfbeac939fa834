"""The MoE layer as one autograd node (chained head, router gradient added inside the dX combine)
against the three separate operators and against the oracle."""

import numpy as np
import pytest
import torch

from oracle import moe_oracle as O
from tests.helpers import BF16_TOL, assert_close_scaled, hip_backend

pytestmark = pytest.mark.gpu


def _head(lib, x, w_r, K, normalize):
    """mts_moe_head_fwd through the C ABI; returns every output as a tensor."""
    from minitrain_amd import _lib

    T, H = x.shape
    E = w_r.shape[0]
    TK = T * K
    dev = x.device
    f32, i32 = dict(dtype=torch.float32, device=dev), dict(dtype=torch.int32, device=dev)
    o = dict(logits=torch.empty(T, E, **f32), weights=torch.empty(T, K, **f32), indices=torch.empty(T, K, **i32),
             weights_act=torch.empty(T, K, dtype=x.dtype, device=dev) if x.dtype != torch.float32 else None,
             prob_mean=torch.empty(E, **f32), z_loss=torch.empty(1, **f32), entropy=torch.empty(1, **f32),
             counts=torch.empty(E, **i32), load_balance=torch.empty(1, **f32), load_stats=torch.empty(E + 7, **f32),
             expert_start=torch.empty(E + 1, **i32), s_scatter=torch.full((TK,), -9, **i32),
             s_reverse=torch.full((TK,), -9, **i32), x_gather=torch.full((TK,), -9, **i32))
    ws_bytes = lib.mts_moe_head_workspace_bytes(T, K, E)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
    rc = lib.mts_moe_head_fwd(x.data_ptr(), w_r.data_ptr(), T, H, E, K, int(normalize), _lib.dtype_code(x.dtype),
                              *[_lib.ptr(o[k]) for k in ("logits", "weights", "indices", "weights_act", "prob_mean", "z_loss",
                                                         "entropy", "counts", "load_balance", "load_stats", "expert_start",
                                                         "s_scatter", "s_reverse", "x_gather")],
                              ws.data_ptr(), ws_bytes, _lib.stream_of(x))
    assert rc == 0, rc
    torch.cuda.synchronize()
    return o


@pytest.mark.parametrize("T,H,E,K,dtype,normalize", [
    (24576, 768, 8, 2, torch.bfloat16, True), (1, 64, 4, 1, torch.bfloat16, True), (5, 128, 8, 2, torch.float16, False),
    (257, 1024, 16, 4, torch.bfloat16, True), (3000, 192, 3, 3, torch.float32, True), (2047, 72, 12, 8, torch.float16, True),
    (98304, 768, 8, 2, torch.bfloat16, True), (700, 256, 16, 1, torch.float32, False),
    # rows wider than a wave holds in registers: column chunks forward, column ranges backward
    (4096, 4096, 8, 2, torch.bfloat16, True), (333, 2048, 16, 2, torch.float16, True), (130, 1280, 5, 2, torch.float32, True),
    # the widest rows the matrix-pipe projection takes (several register chunks per row, 104 KiB of weight terms in LDS)
    (300, 2048, 8, 2, torch.bfloat16, True), (1000, 1280, 6, 3, torch.bfloat16, False)])
def test_chained_head_equals_the_three_operators(T, H, E, K, dtype, normalize):
    print(f"head T={T} H={H} E={E} K={K} {dtype} normalize={normalize}", flush=True)
    from minitrain_amd import _lib
    from minitrain_amd.kernels.hip.fused_moe import compute_routing_metadata
    from minitrain_amd.kernels.hip.router import router_logits, router_postprocess

    lib = _lib.load()
    x, w_r, _, _, _ = O.make_inputs(300 + T + E, T, H, E, 8)
    x, w_r = x.to(dtype).cuda(), w_r.cuda()
    got = _head(lib, x, w_r, K, normalize)
    logits = router_logits(x, w_r)
    assert torch.equal(got["logits"], logits)                     # the same sums in the same order
    route = router_postprocess(logits, K, normalize=normalize, weights_dtype=None if dtype == torch.float32 else dtype)
    assert torch.equal(got["indices"], route.expert_indices)
    torch.testing.assert_close(got["weights"], route.expert_weights, rtol=2e-6, atol=1e-7)
    if E <= 8:
        assert torch.equal(got["weights"], route.expert_weights)  # one lane per row in both kernels: identical arithmetic
    if dtype != torch.float32:
        assert torch.equal(got["weights_act"], got["weights"].to(dtype))
    assert torch.equal(got["counts"], route.expert_counts)
    for name, want in (("prob_mean", route.probability_per_expert), ("z_loss", route.z_loss), ("entropy", route.entropy),
                       ("load_balance", route.load_balance_loss), ("load_stats", route.load_stats)):
        torch.testing.assert_close(got[name].flatten(), want.flatten(), rtol=2e-5, atol=2e-6, msg=name)
    # against the oracle as well
    ref = O.router_postprocess(logits.cpu(), K, normalize=normalize)
    assert torch.equal(got["indices"].cpu(), ref.expert_indices)
    torch.testing.assert_close(got["weights"].cpu(), ref.expert_weights, rtol=2e-5, atol=2e-5)
    # routing metadata: bit-exact against the stand-alone call on the same indices
    (cnt, es, xg, ss, sr, _, _, _) = compute_routing_metadata(got["indices"], E)
    assert torch.equal(got["counts"], cnt) and torch.equal(got["expert_start"], es)
    assert torch.equal(got["s_scatter"], ss) and torch.equal(got["s_reverse"], sr) and torch.equal(got["x_gather"], xg)


@pytest.mark.parametrize("T,H,E,K,dtype", [
    (1500, 768, 8, 2, torch.bfloat16),    # projection on the matrix pipe
    (1500, 256, 8, 3, torch.float16),     # 16-bit rows the matrix-pipe projection does not take: vector pipe
    (700, 192, 12, 4, torch.float32),     # more than 8 experts: several lanes per row in the post-process
    (1500, 768, 6, 2, torch.bfloat16)])
def test_ties_reach_the_chained_head_and_the_layer_node(T, H, E, K, dtype):
    """Exactly tied logits inside the chained head: experts with identical router rows tie for every
    token, all-zero tokens tie over all experts.  The lower expert index must win, in the head kernel
    and in the layer node, on the matrix-pipe and on the vector-pipe projection."""
    print(f"ties through the head T={T} H={H} E={E} K={K} {dtype}", flush=True)
    from minitrain_amd import _lib

    lib = _lib.load()
    x, w_r, w1, w2, _ = O.make_inputs(4100 + T + E, T, H, E, 64)
    w_r[1] = w_r[0]                      # experts 0 and 1 tie for every token
    w_r[E - 1] = w_r[2]                  # and so do 2 and the last one
    x[::7] = 0.0                         # every logit of these tokens is exactly 0
    x[3::11] = x[3::11].abs()            # some rows where the tied pair is likely to be on top
    x, w_r = x.to(dtype).cuda(), w_r.cuda()
    got = _head(lib, x, w_r, K, True)
    logits = got["logits"]
    assert torch.equal(logits[:, 0], logits[:, 1]) and torch.equal(logits[:, 2], logits[:, E - 1])   # the ties are real
    assert bool((logits[::7] == 0).all())
    ref = O.router_postprocess(logits.cpu(), K, normalize=True)
    assert torch.equal(got["indices"].cpu(), ref.expert_indices)
    # lowest index wins: an all-tied row selects experts 0..K-1 in that order, and the second expert of a
    # tied pair is never selected without the first
    assert torch.equal(got["indices"][::7].cpu(), torch.arange(K, dtype=torch.int32).expand(len(range(0, T, 7)), K))
    sel = torch.zeros(T, E, dtype=torch.bool).scatter_(1, ref.expert_indices.long(), True)
    assert bool((~sel[:, 1] | sel[:, 0]).all()) and bool((~sel[:, E - 1] | sel[:, 2]).all())
    torch.testing.assert_close(got["weights"].cpu(), ref.expert_weights, rtol=2e-5, atol=2e-5)
    assert torch.equal(got["counts"].cpu(), torch.bincount(ref.expert_indices.flatten().long(), minlength=E).int())
    # the layer node routes through the same head
    ops = hip_backend()
    pdt = dtype
    res = ops.moe_layer(x, w_r, w1.to(pdt).cuda(), w2.to(pdt).cuda(), K, normalize=True)
    assert res is not None
    assert torch.equal(res[7].cpu(), ref.expert_indices)


def _layer_grads(ops, case, K, normalize, dtype, fp32_params):
    pdt = torch.float32 if fp32_params else dtype
    leaves = [case["x"].to(dtype).cuda().requires_grad_(True), case["w_r"].cuda().requires_grad_(True),
              case["w1"].to(pdt).cuda().requires_grad_(True), case["w2"].to(pdt).cuda().requires_grad_(True)]
    res = ops.moe_layer(*leaves, K, normalize=normalize)
    assert res is not None
    out, aux, z = res[:3]
    torch.autograd.backward([out, aux, z], [case["g"].to(dtype).cuda(), torch.tensor(0.01, device="cuda"),
                                            torch.tensor(0.001, device="cuda")])
    torch.cuda.synchronize()
    return res, [l.grad for l in leaves]


def _separate_grads(ops, case, K, normalize, dtype, fp32_params):
    pdt = torch.float32 if fp32_params else dtype
    leaves = [case["x"].to(dtype).cuda().requires_grad_(True), case["w_r"].cuda().requires_grad_(True),
              case["w1"].to(pdt).cuda().requires_grad_(True), case["w2"].to(pdt).cuda().requires_grad_(True)]
    logits = ops.router_logits(leaves[0], leaves[1])
    route = ops.router_postprocess(logits, K, normalize=normalize, weights_dtype=None if dtype == torch.float32 else dtype)
    w = route.expert_weights_cast if dtype != torch.float32 else route.expert_weights
    out = ops.fused_moe(leaves[0], leaves[2], leaves[3], route.expert_indices, w)
    torch.autograd.backward([out, route.load_balance_loss, route.z_loss],
                            [case["g"].to(dtype).cuda(), torch.tensor(0.01, device="cuda"), torch.tensor(0.001, device="cuda")])
    torch.cuda.synchronize()
    return (out, route), [l.grad for l in leaves]


@pytest.mark.parametrize("T,H,E,I,K,dtype,fp32_params,normalize", [
    (512, 128, 8, 256, 2, torch.bfloat16, False, True), (2048, 768, 8, 1024, 2, torch.bfloat16, True, True),
    (33, 64, 4, 64, 1, torch.float16, False, True), (700, 72, 3, 40, 2, torch.bfloat16, False, False),
    (300, 64, 16, 96, 4, torch.float32, False, True), (1, 64, 4, 64, 2, torch.bfloat16, False, True),
    (200, 64, 8, 64, 5, torch.bfloat16, False, True), (300, 2048, 8, 128, 2, torch.bfloat16, False, True)])
def test_layer_node_equals_the_separate_operators_and_the_oracle(T, H, E, I, K, dtype, fp32_params, normalize):
    print(f"layer node T={T} H={H} E={E} I={I} K={K} {dtype} fp32_params={fp32_params} normalize={normalize}", flush=True)
    ops = hip_backend()
    x, w_r, w1, w2, g = O.make_inputs(400 + T, T, H, E, I)
    case = dict(x=x, w_r=w_r, w1=w1, w2=w2, g=g)
    res, grads = _layer_grads(ops, case, K, normalize, dtype, fp32_params)
    (out_s, route), grads_s = _separate_grads(ops, case, K, normalize, dtype, fp32_params)
    out = res[0]
    assert torch.equal(res[7], route.expert_indices)
    tol = 1e-5 if dtype == torch.float32 else 1e-2
    if E <= 8:   # the same kernels on the same operands (beyond 8 experts the two post-process kernels sum a row differently)
        assert torch.equal(out, out_s)
        assert torch.equal(grads[2], grads_s[2]) and torch.equal(grads[3], grads_s[3])
    else:
        for name, u, v in (("out", out, out_s), ("dW1", grads[2], grads_s[2]), ("dW2", grads[3], grads_s[3])):
            assert_close_scaled(u, v, tol, name)
    assert_close_scaled(grads[0], grads_s[0], tol, "dx, summed inside the combine vs by autograd")
    assert_close_scaled(grads[1], grads_s[1], 1e-5, "dW_r")
    # the oracle: the router module and the expert loop on the CPU, fp32-accumulated, on the same rounded values
    pdt = torch.float32 if fp32_params else dtype
    leaves = [x.to(dtype).float().requires_grad_(True), w_r.clone().requires_grad_(True),
              w1.to(pdt).float().requires_grad_(True), w2.to(pdt).float().requires_grad_(True)]
    hidden, r = O.moe_feed_forward(leaves[0].to(dtype), leaves[1], leaves[2].to(pdt), leaves[3].to(pdt), K,
                                   normalize=normalize, compute_dtype=torch.float32)
    ((hidden * g.to(dtype).float()).sum() + 0.01 * r.auxiliary_loss + 0.001 * r.z_loss).backward()
    assert torch.equal(res[7].cpu(), r.expert_indices)
    gate = 1e-5 if dtype == torch.float32 else BF16_TOL
    assert_close_scaled(out, hidden, gate, "hidden")
    torch.testing.assert_close(res[1].cpu(), r.auxiliary_loss, rtol=1e-4, atol=1e-6)
    torch.testing.assert_close(res[2].cpu(), r.z_loss, rtol=1e-4, atol=1e-6)
    for name, got, want in zip(("dx", "dW_r", "dW1", "dW2"), grads, [l.grad for l in leaves]):
        assert_close_scaled(got, want, 1e-4 if dtype == torch.float32 else gate, name)


@pytest.mark.parametrize("T,H,E,I,K,dtype,fp32_params", [
    (24576, 768, 8, 1024, 2, torch.bfloat16, False), (701, 128, 5, 128, 2, torch.float16, False),
    (1, 64, 4, 64, 2, torch.bfloat16, False), (2500, 1024, 8, 192, 3, torch.bfloat16, True)])
def test_router_backward_inside_the_joint_launch_equals_its_own_launches(T, H, E, I, K, dtype, fp32_params, monkeypatch):
    """With every gradient wanted and at most 8 experts the router's backward rides in the launch of
    dW1 + dW2 + dX as trailing blocks that form dS from the partial row sums themselves: the same
    arithmetic block for block, so every gradient equals the separate launches' bit for bit."""
    print(f"router backward in the joint launch T={T} H={H} E={E} I={I} K={K} {dtype} fp32_params={fp32_params}", flush=True)
    import importlib

    from minitrain_amd import _lib

    F = importlib.import_module("minitrain_amd.kernels.hip.fused_moe")
    assert _lib.load().mts_moe_bwd_joint_router_supported(_lib.dtype_code(dtype), T, H, I, E) == 1
    ops = hip_backend()
    x, w_r, w1, w2, g = O.make_inputs(900 + T, T, H, E, I)
    case = dict(x=x, w_r=w_r, w1=w1, w2=w2, g=g)
    monkeypatch.setattr(F.SWITCHES, "joint_bwd", True)
    monkeypatch.setattr(F.SWITCHES, "tail_in_joint", True)
    monkeypatch.setattr(F.SWITCHES, "combine_in_tail", True)   # the dX combine too (inside the library: with the partial sums
    inside = _layer_grads(ops, case, K, True, dtype, fp32_params)[1]   # for two routes per token, else one more launch)
    monkeypatch.setattr(F.SWITCHES, "combine_in_tail", False)
    own_combine = _layer_grads(ops, case, K, True, dtype, fp32_params)[1]
    monkeypatch.setattr(F.SWITCHES, "tail_in_joint", False)
    apart = _layer_grads(ops, case, K, True, dtype, fp32_params)[1]
    for other in (own_combine, apart):
        for name, a, b in zip(("dx", "dW_r", "dW1", "dW2"), inside, other):
            assert a.dtype == b.dtype and torch.equal(a, b), name


def test_layer_node_partial_gradients():
    """Only the router's loss terms reach the layer; and activations that need no gradient."""
    print("layer node partial gradients", flush=True)
    ops = hip_backend()
    T, H, E, I, K = 300, 128, 8, 128, 2
    x, w_r, w1, w2, g = O.make_inputs(77, T, H, E, I)
    mk = lambda rx: [x.bfloat16().cuda().requires_grad_(rx), w_r.cuda().requires_grad_(True),
                     w1.bfloat16().cuda().requires_grad_(True), w2.bfloat16().cuda().requires_grad_(True)]
    # (a) loss = aux + z only
    a = mk(True)
    res = ops.moe_layer(*a, K, normalize=True)
    (res[1] * 0.5 + res[2]).backward()
    b = mk(True)
    route = ops.router_postprocess(ops.router_logits(b[0], b[1]), K, normalize=True)
    (route.load_balance_loss * 0.5 + route.z_loss).backward()
    assert a[2].grad is None and a[3].grad is None
    assert_close_scaled(a[0].grad, b[0].grad, 1e-5, "dx from the router terms")
    assert_close_scaled(a[1].grad, b[1].grad, 1e-5, "dW_r from the router terms")
    # (b) x needs no gradient: the weights still get theirs
    c, d = mk(False), mk(True)
    for leaves in (c, d):
        r = ops.moe_layer(*leaves, K, normalize=True)
        torch.autograd.backward([r[0], r[1]], [g.bfloat16().cuda(), torch.tensor(0.01, device="cuda")])
    assert c[0].grad is None
    for u, v in zip(c[1:], d[1:]):
        assert torch.equal(u.grad, v.grad)


def test_block_uses_the_layer_node_and_falls_back_when_it_must():
    """MoEFeedForward takes the one-node path when the backend offers it; with a capacity limit (or a
    backend without the hook) it composes the layer from the router module and fused_moe."""
    print("block path selection", flush=True)
    from minitrain_amd.model.blocks import MoEFeedForward
    from minitrain_amd.model.config import ModelConfig

    ops = hip_backend()
    cfg = ModelConfig(hidden_size=128, n_heads=1, intermediate_size=256, num_experts=8, experts_per_token=2, n_layers=2)
    block = MoEFeedForward(cfg).cuda()
    x = torch.randn(4, 64, 128, device="cuda", dtype=torch.bfloat16, generator=torch.Generator("cuda").manual_seed(3))
    calls = []
    real = ops.moe_layer
    ops.moe_layer = lambda *a, **k: (calls.append(1), real(*a, **k))[1]
    with torch.autocast("cuda", dtype=torch.bfloat16):
        one = block(x, ops)
    assert calls == [1]
    ops.offers_moe_layer = False
    with torch.autocast("cuda", dtype=torch.bfloat16):
        three = block(x, ops)
    assert torch.equal(one.hidden_states, three.hidden_states)
    torch.testing.assert_close(one.router_aux_loss, three.router_aux_loss, rtol=2e-5, atol=1e-7)
    assert set(one.router_metrics) == set(three.router_metrics)
    for key in one.router_metrics:
        torch.testing.assert_close(one.router_metrics[key].float(), three.router_metrics[key].float(), rtol=2e-5, atol=2e-6)


def test_layer_step_replayed_from_a_graph():
    """Forward and backward of the layer node captured into one graph and replayed, with eager steps and
    synchronisations between the replays: outputs and all four gradients equal the eager step's, bit for bit.  No
    kernel of the step needs the host between launches (grids follow from the sizes, not from the routing), nothing is
    cleared with a memset, and the host side leaves the joint forward launch's status word alone while capturing."""
    ops = hip_backend()
    T, H, E, I, K = 4096, 768, 8, 1024, 2
    x, w_r, w1, w2, g = O.make_inputs(7, T, H, E, I)
    x, w1, w2, g = (t.bfloat16().cuda() for t in (x, w1, w2, g))
    w_r = w_r.cuda()
    g_aux, g_z = torch.tensor(0.01, device="cuda"), torch.tensor(0.001, device="cuda")
    leaves = [t.requires_grad_(True) for t in (x, w_r, w1, w2)]

    def step():
        for leaf in leaves:
            leaf.grad = None
        out, aux, z = ops.moe_layer(*leaves, K, normalize=True)[:3]
        torch.autograd.backward([out, aux, z], [g, g_aux, g_z])
        return out.detach(), [leaf.grad for leaf in leaves]

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(3):
            step()
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        out, grads = step()
    gen = torch.Generator().manual_seed(3)
    for replay in range(3):
        print(f"layer step graph replay {replay}", flush=True)
        with torch.no_grad():
            x.copy_(torch.randn(T, H, generator=gen).bfloat16())   # other activations, hence another routing
        graph.replay()
        torch.cuda.synchronize()
        got_out, got_grads = out.clone(), [t.clone() for t in grads]
        want_out, want_grads = step()
        torch.cuda.synchronize()
        assert torch.equal(got_out, want_out), replay
        for a, b in zip(got_grads, want_grads):
            assert torch.equal(a, b), replay
