"""HIP fused MoE (forward and backward, through the C ABI) against the oracle."""

import numpy as np
import pytest
import torch

from oracle import moe_oracle as O
from tests.helpers import BF16_TOL, assert_close_scaled, hip_backend, hip_moe_grads, oracle_moe_grads, routed_case

pytestmark = pytest.mark.gpu

NAMES = ("dx", "dW1", "dW2", "dS")


def _compare(case, *, device="cpu", tol=BF16_TOL):
    out, grads = hip_moe_grads(case["x"], case["w1"], case["w2"], case["idx"], case["w"], case["g"])
    ref_out, ref_grads = oracle_moe_grads(case["x"], case["w1"], case["w2"], case["idx"], case["w"], case["g"],
                                          device=device)
    assert out.dtype == case["x"].dtype and out.shape == case["x"].shape
    stats = {"out": assert_close_scaled(out, ref_out, tol, "out")}
    for name, got, want, leaf in zip(NAMES, grads, ref_grads, (case["x"], case["w1"], case["w2"], case["w"])):
        assert got.dtype == leaf.dtype and got.shape == leaf.shape, name
        stats[name] = assert_close_scaled(got, want, tol, name)
    # the reference's own acceptance for this operator: relative L2 and cosine
    for name, st in stats.items():
        assert st["relative_l2"] <= 1e-2 and st["cosine"] >= 0.9999, (name, st)
    return stats


@pytest.mark.parametrize("T,H,E,I,K", [(256, 64, 4, 128, 2), (33, 128, 8, 64, 2), (1, 64, 4, 64, 1),
                                       (257, 192, 8, 320, 2), (700, 72, 3, 40, 2), (129, 32, 4, 24, 3)])
def test_small_shapes(T, H, E, I, K):
    print(f"moe small T={T} H={H} E={E} I={I} K={K}", flush=True)
    _compare(routed_case(10 + T, T, H, E, I, K))


@pytest.mark.parametrize("T,H,E,I,K", [(256, 64, 4, 128, 2), (700, 72, 3, 40, 2), (2048, 768, 8, 1024, 2)])
def test_fp16_activations(T, H, E, I, K):
    """fp16 is the third activation dtype of the reference's contract (fused_moe.py:37-71)."""
    print(f"moe fp16 T={T} H={H} E={E} I={I} K={K}", flush=True)
    _compare(routed_case(60 + T, T, H, E, I, K, dtype=torch.float16))


@pytest.mark.parametrize("T,H,E,I,K,dtype", [(300, 100, 4, 52, 2, torch.bfloat16), (65, 36, 3, 20, 1, torch.float16),
                                             (200, 50, 4, 30, 2, torch.float32), (257, 64, 8, 100, 2, torch.bfloat16)])
def test_widths_that_are_not_whole_16_byte_chunks(T, H, E, I, K, dtype):
    """H or I not a multiple of 8 (4 for fp32) is legal in the reference (triton/fused_moe.py:55-70); the
    operator pads the operands with zeros, which changes no product, and cuts results and gradients back."""
    print(f"moe odd widths T={T} H={H} E={E} I={I} K={K} {dtype}", flush=True)
    _compare(routed_case(120 + T, T, H, E, I, K, dtype=dtype), tol=1e-5 if dtype == torch.float32 else BF16_TOL)


def test_fp16_activations_fp32_master_weights():
    print("moe fp16 with fp32 weights", flush=True)
    case = routed_case(61, 300, 128, 4, 192, 2, dtype=torch.float16)
    _, w_r, w1, w2, _ = O.make_inputs(61, 300, 128, 4, 192)
    case.update(w1=w1, w2=w2)
    _compare(case)


def _drawn_shapes(n, seed):
    rng = np.random.Generator(np.random.Philox(seed))
    out = []
    for i in range(n):
        E = int(rng.integers(1, 17))
        K = int(rng.integers(1, min(E, 4) + 1))
        # every other draw has whole 64-wide k-tiles (ring / specialised kernels, weights read as stored),
        # the others take the staged kernels with transposed copies
        step = 64 if i % 2 == 0 else 8
        H = int(rng.integers(1, 5)) * step if step == 64 else int(rng.integers(2, 33)) * 8
        I = int(rng.integers(1, 5)) * (32 if step == 64 else 8)
        T = int(rng.integers(1, 700))
        dtype = (torch.bfloat16, torch.float16)[int(rng.integers(0, 2))]
        out.append((T, H, E, I, K, dtype))
    return out


@pytest.mark.parametrize("T,H,E,I,K,dtype", _drawn_shapes(14, seed=2024))
def test_drawn_shapes(T, H, E, I, K, dtype):
    """Seeded draws over token counts, widths, expert counts and top-k, in both 16-bit dtypes."""
    print(f"moe drawn T={T} H={H} E={E} I={I} K={K} {dtype}", flush=True)
    _compare(routed_case(T + H + E, T, H, E, I, K, dtype=dtype))


def test_reference_edge_probe():
    """T=33, K=3, only experts {0,1} of 8 used, repeated experts inside a token and
    zero weights on [::2, -1]; zero-weight routes must still receive a gradient."""
    print("moe edge probe", flush=True)
    T, H, E, I, K = 33, 128, 8, 64, 3
    case = routed_case(5, T, H, E, I, K)
    idx = torch.stack([(torch.arange(T) + s) % 2 for s in range(K)], dim=1).to(torch.int32)
    w = torch.rand(T, K, generator=torch.Generator().manual_seed(1)).bfloat16()
    w[::2, -1] = 0
    case.update(idx=idx, w=w)
    _compare(case)
    out, grads = hip_moe_grads(case["x"], case["w1"], case["w2"], idx, w, case["g"])
    assert float(grads[3][::2, -1].float().abs().min()) > 0
    for e in range(2, E):
        assert not grads[1][e].any() and not grads[2][e].any(), "experts without routes get zero gradients"


def test_fp32_master_weights_bf16_activations():
    """Parameters stay fp32 under autocast: weight gradients come back in fp32."""
    print("moe fp32 weights", flush=True)
    case = routed_case(21, 300, 128, 4, 192, 2)
    _, w_r, w1, w2, _ = O.make_inputs(21, 300, 128, 4, 192)
    case.update(w1=w1, w2=w2)
    _compare(case)


def test_non_contiguous_inputs_and_no_grad_paths():
    print("moe non-contiguous", flush=True)
    ops = hip_backend()
    case = routed_case(31, 200, 128, 4, 128, 2)
    x = torch.zeros(200, 256, dtype=torch.bfloat16)
    x[:, ::2] = case["x"]
    xs = x.cuda()[:, ::2]
    assert not xs.is_contiguous()
    got = ops.fused_moe(xs, case["w1"].cuda(), case["w2"].cuda(), case["idx"].cuda(), case["w"].cuda())
    want = ops.fused_moe(case["x"].cuda(), case["w1"].cuda(), case["w2"].cuda(), case["idx"].cuda(), case["w"].cuda())
    assert torch.equal(got, want)
    # only x requires grad
    xg = case["x"].cuda().requires_grad_(True)
    ops.fused_moe(xg, case["w1"].cuda(), case["w2"].cuda(), case["idx"].cuda(), case["w"].cuda()).sum().backward()
    assert xg.grad is not None
    # unsupported contracts raise instead of falling back
    with pytest.raises(RuntimeError):
        ops.fused_moe(case["x"], case["w1"], case["w2"], case["idx"], case["w"])               # CPU tensors
    with pytest.raises(RuntimeError):
        ops.fused_moe(case["x"].cuda(), case["w1"].cuda(), case["w2"].cuda(), case["idx"].cuda().long(),
                      case["w"].cuda())                                                        # int64 indices
    with pytest.raises(RuntimeError):
        ops.fused_moe(case["x"].cuda(), case["w1"].cuda(), case["w2"].cuda(), case["idx"].cuda(),
                      case["w"].cuda().float())                                                # weight dtype != x dtype


def test_run_to_run_determinism():
    print("moe determinism", flush=True)
    case = routed_case(41, 1000, 128, 8, 256, 2)
    a = hip_moe_grads(case["x"], case["w1"], case["w2"], case["idx"], case["w"], case["g"])
    b = hip_moe_grads(case["x"], case["w1"], case["w2"], case["idx"], case["w"], case["g"])
    assert torch.equal(a[0], b[0])
    for u, v in zip(a[1], b[1]):
        assert torch.equal(u, v)


@pytest.mark.parametrize("T,H,E,I,skew", [(3000, 256, 8, 256, 0.7), (1500, 128, 4, 192, 0.55), (2000, 72, 16, 40, 0.4),
                                          (700, 256, 64, 256, 0.5)])
def test_weight_gradients_with_row_chunks(T, H, E, I, skew, monkeypatch):
    """Skewed routing: the weight-gradient GEMMs cut the rows of the over-full experts into chunks
    (workspace given) and must agree with the oracle and with the uncut reduction (no workspace)."""
    print(f"moe row chunks T={T} H={H} E={E} I={I} skew={skew}", flush=True)
    import importlib

    F = importlib.import_module("minitrain_amd.kernels.hip.fused_moe")
    K = 2
    case = routed_case(50 + T, T, H, E, I, K)
    rng = np.random.Generator(np.random.Philox(T))
    idx = case["idx"].clone()
    heavy = torch.from_numpy(rng.random(T) < skew)
    idx[heavy, 0] = 1                                   # expert 1 takes most first choices
    idx[heavy & (idx[:, 1] == 1), 1] = 0
    case.update(idx=idx)
    counts = np.bincount(idx.flatten().numpy(), minlength=E)
    share = (-(-T * K // E) + 31) // 32 * 32
    assert counts.max() > 1.25 * share
    _compare(case)
    cut = hip_moe_grads(case["x"], case["w1"], case["w2"], idx, case["w"], case["g"])
    monkeypatch.setattr(F, "_DW_WORKSPACE_LIMIT", 0)
    uncut = hip_moe_grads(case["x"], case["w1"], case["w2"], idx, case["w"], case["g"])
    for name, a, b in zip(NAMES, cut[1], uncut[1]):
        assert_close_scaled(a, b, 4e-3, name + " cut vs uncut")   # one bf16 rounding of fp32 sums in either order
    assert torch.equal(cut[1][0], uncut[1][0]) and torch.equal(cut[1][3], uncut[1][3])   # dx and dS do not change


@pytest.mark.parametrize("T,H,E,I,dtype,fp32_weights,skew", [
    (1000, 128, 8, 256, torch.bfloat16, False, 0.0), (257, 192, 8, 320, torch.bfloat16, False, 0.0),
    (3000, 256, 8, 256, torch.bfloat16, False, 0.7), (300, 128, 4, 192, torch.bfloat16, True, 0.0),
    (2048, 768, 8, 1024, torch.float16, False, 0.0), (1, 64, 4, 64, torch.bfloat16, False, 0.0),
    (700, 256, 64, 256, torch.float16, True, 0.5)])
def test_joint_backward_launch_equals_separate_launches(T, H, E, I, dtype, fp32_weights, skew, monkeypatch):
    """dW1, dW2, dX and the dS reduction as one launch run the same blocks as the four separate
    launches on side streams: every gradient is bit-identical, with and without row chunks."""
    print(f"moe joint backward T={T} H={H} E={E} I={I} {dtype} fp32_weights={fp32_weights} skew={skew}", flush=True)
    import importlib

    from minitrain_amd import _lib

    F = importlib.import_module("minitrain_amd.kernels.hip.fused_moe")
    assert _lib.load().mts_moe_bwd_joint_supported(_lib.dtype_code(dtype), H, I) == 1
    K = 2 if E > 1 else 1
    case = routed_case(70 + T, T, H, E, I, K, dtype=dtype)
    if fp32_weights:
        _, _, w1, w2, _ = O.make_inputs(70 + T, T, H, E, I)
        case.update(w1=w1, w2=w2)
    if skew:
        rng = np.random.Generator(np.random.Philox(T))
        idx = case["idx"].clone()
        heavy = torch.from_numpy(rng.random(T) < skew)
        idx[heavy, 0] = 1
        idx[heavy & (idx[:, 1] == 1), 1] = 0
        case.update(idx=idx)
    args = (case["x"], case["w1"], case["w2"], case["idx"], case["w"], case["g"])
    monkeypatch.setattr(F.SWITCHES, "joint_bwd", True)    # the default, whatever the environment says
    joint = hip_moe_grads(*args)
    monkeypatch.setattr(F.SWITCHES, "joint_bwd", False)
    separate = hip_moe_grads(*args)
    for name, a, b in zip(NAMES, joint[1], separate[1]):
        assert a.dtype == b.dtype and torch.equal(a, b), name
    _compare(case)   # and the separate launches against the oracle (the default path is compared everywhere else)


def test_layer_shape_subset_of_tokens():
    """293M-class layer dims at 2048 tokens: the whole oracle still runs on the CPU in seconds."""
    print("moe 2048x768x1024", flush=True)
    _compare(routed_case(1, 2048, 768, 8, 1024, 2))


@pytest.mark.parametrize("name,seed,T,imbalanced", [("config2", 1, 24576, False), ("config4", 3, 24576, True),
                                                    ("config3", 2, 98304, False)])
def test_full_size_configs(name, seed, T, imbalanced):
    """Full benchmark sizes.  The checker is the oracle's expert loop evaluated in
    fp32 on the GPU (same code, library matmuls); in addition the rows of a sample
    of tokens are checked against the oracle on the CPU (tokens are independent)."""
    print(f"moe {name} T={T}", flush=True)
    H, E, I, K = 768, 8, 1024, 2
    bias = O.zipf_log_bias(E) if imbalanced else None
    case = routed_case(seed, T, H, E, I, K, bias=bias, tie_fraction=0.01 if imbalanced else 0.0)
    if imbalanced:
        share = np.bincount(case["idx"].flatten().numpy(), minlength=E) / case["idx"].numel()
        assert share.max() > 0.3
    stats = _compare(case, device="cuda")
    print({k: (round(v["max_rel_scaled"], 5), round(v["relative_l2"], 5)) for k, v in stats.items()}, flush=True)
    # sample of tokens against the CPU oracle
    ops = hip_backend()
    out = ops.fused_moe(*(case[k].cuda() for k in ("x", "w1", "w2", "idx", "w"))).cpu()
    pick = torch.from_numpy(np.random.Generator(np.random.Philox(seed)).choice(T, size=192, replace=False))
    ref = O.fused_moe(case["x"][pick], case["w1"], case["w2"], case["idx"][pick], case["w"][pick],
                      compute_dtype=torch.float32)
    assert_close_scaled(out[pick], ref, BF16_TOL, "sampled tokens vs CPU oracle")
    # backward against the CPU oracle as well.  dX and dS of a token depend on that token alone: the sampled
    # tokens go through the oracle's autograd.  dW1 / dW2 of one expert are sums over that expert's routes:
    # float64 accumulation of the per-route outer products on the CPU, for a slice of each matrix.
    _, grads = hip_moe_grads(case["x"], case["w1"], case["w2"], case["idx"], case["w"], case["g"])
    _, ref_grads = oracle_moe_grads(case["x"][pick], case["w1"], case["w2"], case["idx"][pick], case["w"][pick],
                                    case["g"][pick])
    assert_close_scaled(grads[0].cpu()[pick], ref_grads[0], BF16_TOL, "sampled dX vs CPU oracle")
    assert_close_scaled(grads[3].cpu()[pick], ref_grads[3], BF16_TOL, "sampled dS vs CPU oracle")
    e = int(np.bincount(case["idx"].flatten().numpy(), minlength=E).argmin())   # the lightest expert: fewest rows
    dw1_ref, dw2_ref = _expert_weight_gradients_f64(case, e, rows1=slice(0, 2 * I, 61), rows2=slice(0, H, 29))
    assert_close_scaled(grads[1][e].cpu()[0:2 * I:61], dw1_ref, BF16_TOL, "dW1 slice of one expert vs float64 CPU sum")
    assert_close_scaled(grads[2][e].cpu()[0:H:29], dw2_ref, BF16_TOL, "dW2 slice of one expert vs float64 CPU sum")
    if name == "config3":
        print("peak HBM allocated (MB):", torch.cuda.max_memory_allocated() / 2**20, flush=True)


def _expert_weight_gradients_f64(case, e, rows1, rows2, wide=None):
    """Rows ``rows1`` of dW1[e] and ``rows2`` of dW2[e] from the definition (minitrain/kernels/torch_ops.py:
    122-150 differentiated by hand), accumulated in float64 on the CPU over the routes of expert ``e``."""
    x, w1, w2, idx, w, g = (case[k] for k in ("x", "w1", "w2", "idx", "w", "g"))
    tok, k = (idx == e).nonzero(as_tuple=True)
    xe, ge, se = x[tok].double(), g[tok].double(), w[tok, k].double()
    W1, W2 = w1[e].double(), w2[e].double()
    I = W2.shape[1]
    # per-row quantities: float64, or float32 products widened afterwards where the expert holds very many rows
    # (a 768-term dot product in fp32 is good to 1e-6); the sums over the rows below are always float64
    if wide is None:
        wide = torch.float64 if len(tok) <= 40000 else torch.float32
    pre = (xe.to(wide) @ W1.to(wide).T).double()
    gate, up = pre[:, :I], pre[:, I:]
    sig = torch.sigmoid(gate)
    silu = gate * sig
    act = silu * up
    d_act = (ge.to(wide) @ W2.to(wide)).double() * se[:, None]          # d loss / d act
    d_pre = torch.cat([d_act * up * (sig + silu * (1 - sig)), d_act * silu], dim=1)
    dw1 = d_pre.T[rows1] @ xe                                         # [rows1, H]
    dw2 = (ge * se[:, None]).T[rows2] @ act                           # [rows2, I]
    return dw1, dw2


def test_unweighted_post_act_path(monkeypatch):
    """The operator applies the routing weight in the gate/up epilogue and keeps post_act for dW2; the
    other route through the same C ABI (plain post_act, weighted combine, dY1 writes s*a) stays
    available to other bindings and must satisfy the same parity."""
    print("moe unweighted post_act", flush=True)
    import importlib

    F = importlib.import_module("minitrain_amd.kernels.hip.fused_moe")
    for shape in ((1000, 128, 8, 256, 2), (700, 72, 3, 40, 2)):
        case = routed_case(81, *shape)
        args = (case["x"], case["w1"], case["w2"], case["idx"], case["w"], case["g"])
        with monkeypatch.context() as m:
            m.setattr(F.SWITCHES, "weighted_post", True)    # the default, whatever the environment says
            a = hip_moe_grads(*args)
        with monkeypatch.context() as m:
            m.setattr(F.SWITCHES, "weighted_post", False)
            _compare(case)
            b = hip_moe_grads(*args)
        assert_close_scaled(a[0], b[0], 1e-2, "out, weight in the epilogue vs in the combine")
        for name, u, v in zip(NAMES, a[1], b[1]):
            assert_close_scaled(u, v, 1e-2, name)
        assert torch.equal(a[1][3], b[1][3])   # dS does not depend on where the weight is applied


def test_full_size_invariants():
    """Properties that hold at any size, checked at the benchmark size without a CPU checker.
    A row of the expert GEMMs does not depend on which rows share its tile, so permuting the tokens
    permutes the output, dX and dS bit for bit (the weight gradients add the same terms in another
    order); scaling the routing weights by two scales everything but dS by exactly two (a power of two
    commutes with every rounding on the way); renaming the experts changes nothing but the order of the
    weight gradients' leading dimension."""
    print("moe invariants at 24576 tokens", flush=True)
    T, H, E, I, K = 24576, 768, 8, 1024, 2
    case = routed_case(1, T, H, E, I, K)
    x, w1, w2, idx, w, g = (case[k] for k in ("x", "w1", "w2", "idx", "w", "g"))
    out, (dx, dw1, dw2, ds) = hip_moe_grads(x, w1, w2, idx, w, g)
    gen = torch.Generator().manual_seed(5)

    perm = torch.randperm(T, generator=gen)
    out_p, (dx_p, dw1_p, dw2_p, ds_p) = hip_moe_grads(x[perm], w1, w2, idx[perm], w[perm], g[perm])
    dev_perm = perm.cuda()
    assert torch.equal(out_p, out[dev_perm]) and torch.equal(dx_p, dx[dev_perm]) and torch.equal(ds_p, ds[dev_perm])
    assert_close_scaled(dw1_p, dw1, 5e-3, "dW1 under a token permutation")   # one bf16 rounding of another fp32 sum
    assert_close_scaled(dw2_p, dw2, 5e-3, "dW2 under a token permutation")

    out_2, (dx_2, dw1_2, dw2_2, ds_2) = hip_moe_grads(x, w1, w2, idx, w * 2, g)
    for name, a, b in (("out", out_2, out), ("dx", dx_2, dx), ("dW1", dw1_2, dw1), ("dW2", dw2_2, dw2)):
        assert torch.equal(a.float(), b.float() * 2), name
    assert torch.equal(ds_2, ds)

    sigma = torch.randperm(E, generator=gen)          # new expert j holds the weights of old expert sigma[j]
    inverse = torch.empty_like(sigma)
    inverse[sigma] = torch.arange(E)
    out_r, (dx_r, dw1_r, dw2_r, ds_r) = hip_moe_grads(x, w1[sigma], w2[sigma], inverse[idx.long()].to(idx.dtype), w, g)
    assert torch.equal(out_r, out) and torch.equal(dx_r, dx) and torch.equal(ds_r, ds)
    assert torch.equal(dw1_r, dw1[sigma.cuda()]) and torch.equal(dw2_r, dw2[sigma.cuda()])


@pytest.mark.parametrize("T,H,E,I,skew", [(600, 64, 130, 64, 0.0), (900, 64, 130, 64, 0.6), (400, 64, 1500, 32, 0.0)])
def test_more_experts_than_a_wave_holds(T, H, E, I, skew):
    """E > 64: the tile and unit lookups of the GEMM kernels take more than one round of 64 experts
    (with skew, row chunks of an over-full expert add workspace slots to the lookup)."""
    print(f"moe many experts T={T} E={E} skew={skew}", flush=True)
    case = routed_case(90 + T, T, H, E, I, 2)
    if skew:
        rng = np.random.Generator(np.random.Philox(T))
        idx = case["idx"].clone()
        heavy = torch.from_numpy(rng.random(T) < skew)
        idx[heavy, 0] = 97                                  # an expert of the second round takes most first choices
        idx[heavy & (idx[:, 1] == 97), 1] = 3
        case.update(idx=idx)
    _compare(case)


@pytest.mark.parametrize("wdtype", [torch.bfloat16, torch.float16, torch.float32])
def test_fp32_activations_with_16bit_parameters(wdtype):
    """fp32 activations take fp32, bf16 or fp16 expert parameters (widened once per call); the weight
    gradients come back in the parameter's dtype."""
    print(f"moe fp32 activations, {wdtype} parameters", flush=True)
    case = routed_case(95, 300, 64, 4, 96, 2, dtype=torch.float32)
    case.update(w1=case["w1"].to(wdtype), w2=case["w2"].to(wdtype))
    _compare(case, tol=1e-5 if wdtype == torch.float32 else 4e-3)   # 16-bit gradients: one rounding of the result


def test_intermediates_beyond_2_gib():
    """270 336 tokens at the layer shape: pre_act and d_pre_act ([T*K, 2I] bf16) are 2.2 GB each, more than
    one buffer descriptor spans, so the kernels address them tile by tile (the reference carries int64 row
    offsets for the same reason, minitrain/kernels/triton/fused_moe_kernels.py:314,413,474).  Checked on
    the CPU: forward, dX and dS of sampled tokens, and slices of dW1 / dW2 of the LAST expert, whose rows
    sit behind the 2 GiB mark."""
    print("moe intermediates beyond 2 GiB", flush=True)
    T, H, E, I, K = 270336, 768, 8, 1024, 2
    assert T * K * 2 * I * 2 > 2**31
    case = routed_case(9, T, H, E, I, K)
    out, grads = hip_moe_grads(case["x"], case["w1"], case["w2"], case["idx"], case["w"], case["g"])
    rng = np.random.Generator(np.random.Philox(9))
    last = (case["idx"] == E - 1).any(dim=1).nonzero().flatten()             # tokens with a route to the last expert
    pick = torch.cat([torch.from_numpy(rng.choice(T, size=128, replace=False)), last[torch.from_numpy(rng.choice(len(last), size=64, replace=False))]])
    ref_out, ref_grads = oracle_moe_grads(case["x"][pick], case["w1"], case["w2"], case["idx"][pick], case["w"][pick],
                                          case["g"][pick])
    assert_close_scaled(out.cpu()[pick], ref_out, BF16_TOL, "sampled tokens vs CPU oracle")
    assert_close_scaled(grads[0].cpu()[pick], ref_grads[0], BF16_TOL, "sampled dX vs CPU oracle")
    assert_close_scaled(grads[3].cpu()[pick], ref_grads[3], BF16_TOL, "sampled dS vs CPU oracle")
    dw1_ref, dw2_ref = _expert_weight_gradients_f64(case, E - 1, rows1=slice(0, 2 * I, 127), rows2=slice(0, H, 61))
    assert_close_scaled(grads[1][E - 1].cpu()[0:2 * I:127], dw1_ref, BF16_TOL, "dW1 slice of the last expert")
    assert_close_scaled(grads[2][E - 1].cpu()[0:H:61], dw2_ref, BF16_TOL, "dW2 slice of the last expert")
    assert all(torch.isfinite(t.float()).all() for t in grads)


def _skewed_indices(T, E, K, shares, seed):
    """K distinct experts per token, drawn one after the other with odds proportional to `shares`."""
    g = torch.Generator().manual_seed(seed)
    p = torch.tensor(shares, dtype=torch.float64).expand(T, E).clone()
    cols = []
    for _ in range(K):
        c = torch.multinomial(p, 1, generator=g)
        p.scatter_(1, c, 0.0)
        cols.append(c)
    return torch.cat(cols, 1).int()


def _read_schedule(table, E):
    """The used part of a schedule table as Python values: dX ranges and the units of every XCD."""
    t = table.cpu().tolist()
    slots = (2 * E + 7) // 8
    first, count, held = t[0:8], t[8:16], t[16:24]
    units = [[tuple(t[32 + (x * slots + k) * 4: 32 + (x * slots + k) * 4 + 4]) for k in range(held[x])] for x in range(8)]
    return first, count, held, units


@pytest.mark.parametrize("E,K,shares", [
    (8, 2, [4862, 12086, 3507, 3153, 6471, 5392, 7811, 5870]),      # routes per expert of a layer of the 12-layer decoder
    (8, 2, [0.48, 0.2, 0.1, 0.07, 0.05, 0.04, 0.03, 0.03]),          # Zipf-like
    (8, 2, [1] * 8), (5, 3, [5, 1, 1, 1, 0.2]), (32, 4, [1.0 / (r + 1) for r in range(32)]), (3, 1, [1, 0, 3])])
def test_joint_launch_schedule(E, K, shares):
    """The table that deals the joint backward launch's blocks out to the XCDs (written by the dO*W2 launch, or by a
    launch of its own): every unit is a row range of one expert, the units of an expert tile its rows in order, no
    XCD holds more units than the grid has room for, the dX m-tiles are split into eight consecutive ranges that
    cover them all, and the XCD with the most weight-gradient rows gets the fewest dX tiles.  Both ways of writing
    it give the same table."""
    print(f"joint launch schedule E={E} K={K}", flush=True)
    from minitrain_amd import _lib
    from minitrain_amd.kernels.hip.fused_moe import compute_routing_metadata

    lib = _lib.load()
    T, H, I = 6000, 128, 128
    idx = _skewed_indices(T, E, K, shares, 17).cuda()
    counts, es = compute_routing_metadata(idx, E)[:2]
    nbytes = lib.mts_moe_bwd_schedule_bytes(E)
    assert nbytes == 4096
    own = torch.full((nbytes // 4,), -1, dtype=torch.int32, device="cuda")
    assert lib.mts_moe_bwd_schedule(es.data_ptr(), T * K, E, own.data_ptr(), _lib.stream_of(own)) == 0
    first, count, held, units = _read_schedule(own, E)
    c = counts.cpu().tolist()
    start = es.cpu().tolist()
    slots = (2 * E + 7) // 8
    assert all(h <= slots for h in held)
    share = (-(-T * K // E) + 31) // 32 * 32
    by_expert = {}
    for x in range(8):
        for (e, rb, re_, slot) in units[x]:
            assert 0 <= e < E and start[e] <= rb <= re_ <= start[e + 1]
            by_expert.setdefault(e, []).append((rb, re_, slot))
    slot_seen = []
    for e in range(E):
        parts = sorted(by_expert.get(e, []))
        assert parts and parts[0][0] == start[e] and parts[-1][1] == start[e + 1]            # every expert is covered ...
        assert all(a[1] == b[0] for a, b in zip(parts, parts[1:]))                            # ... by consecutive ranges
        cut = c[e] > share + share * 3 // 20
        assert len(parts) == (-(-c[e] // share) if cut else 1)
        assert all((p[2] >= 0) == cut for p in parts)
        slot_seen += [p[2] for p in parts if cut]
    assert sorted(slot_seen) == list(range(len(slot_seen)))                                     # workspace slots in expert order
    m_tiles = sum(-(-n // 256) for n in c)
    assert first[0] == 0 and all(first[x + 1] == first[x] + count[x] for x in range(7)) and first[7] + count[7] == m_tiles
    loads = [sum(u[1] - u[0] for u in [(rb, re_) for (_, rb, re_, _) in units[x]]) for x in range(8)]
    if max(loads) > min(loads) and m_tiles >= 16:
        assert count[loads.index(max(loads))] <= count[loads.index(min(loads))]
    # the dO*W2 launch writes the same table on the side
    x = torch.randn(T, H, device="cuda").bfloat16()
    w2 = (torch.randn(E, H, I, device="cuda") * 0.02).bfloat16()
    pre = torch.randn(T * K, 2 * I, device="cuda").bfloat16()
    wts = torch.rand(T * K, device="cuda").bfloat16()
    _, _, xg, ss, _, _, _, _ = compute_routing_metadata(idx, E)
    dpre = torch.empty_like(pre)
    dsp = torch.empty(T * K, lib.mts_moe_ds_partials(I), device="cuda")
    side = torch.full_like(own, -1)
    rc = lib.mts_moe_bwd_dy1(x.data_ptr(), w2.data_ptr(), 1, pre.data_ptr(), wts.data_ptr(), xg.data_ptr(), ss.data_ptr(),
                             es.data_ptr(), T, K, E, H, I, _lib.MTS_BF16, dpre.data_ptr(), None, dsp.data_ptr(), side.data_ptr(),
                             _lib.stream_of(x))
    assert rc == 0
    torch.cuda.synchronize()
    assert _read_schedule(side, E) == (first, count, held, units)


@pytest.mark.parametrize("dtype,fp32_params", [(torch.bfloat16, False), (torch.float16, True)])
def test_scheduled_joint_launch_equals_the_unscheduled_one(dtype, fp32_params, monkeypatch):
    """Which XCD computes a tile does not change the tile: with the schedule and without it the operator returns
    the same gradients bit for bit under skewed routing (where the schedule moves most blocks), and they match the
    oracle."""
    print(f"scheduled joint launch {dtype} fp32_params={fp32_params}", flush=True)
    import importlib

    F = importlib.import_module("minitrain_amd.kernels.hip.fused_moe")
    T, H, E, I, K = 5000, 256, 8, 512, 2
    case = routed_case(61, T, H, E, I, K, dtype=dtype, bias=O.zipf_log_bias(E) * 0.5)
    if fp32_params:
        case["w1"], case["w2"] = case["w1"].float(), case["w2"].float()
    args = (case["x"], case["w1"], case["w2"], case["idx"], case["w"], case["g"])
    monkeypatch.setattr(F.SWITCHES, "joint_bwd", True)
    monkeypatch.setattr(F.SWITCHES, "joint_schedule", True)
    with_table = hip_moe_grads(*args)
    monkeypatch.setattr(F.SWITCHES, "joint_schedule", False)
    without = hip_moe_grads(*args)
    assert torch.equal(with_table[0], without[0])
    for name, a, b in zip(NAMES, with_table[1], without[1]):
        assert a.dtype == b.dtype and torch.equal(a, b), name
    monkeypatch.setattr(F.SWITCHES, "joint_schedule", True)
    _compare(case)


@pytest.mark.parametrize("T", [512, 8192])
def test_reference_sweep_sizes(T):
    """The smallest and a middle size of the reference's operator sweep (benchmarks/operators/moe_runner.py:135-204:
    512 ... 57 344 tokens at the layer shape) against the whole CPU oracle: at 512 tokens an expert holds fewer
    rows than one 256-row tile, so every tile of every GEMM is a partial one."""
    print(f"moe sweep size T={T}", flush=True)
    _compare(routed_case(20 + T, T, 768, 8, 1024, 2))


def test_mixtral_class_widths():
    """H = 4096, I = 14336 (the reference's `mixtral_7b` benchmark profile, moe_runner.py:53): one expert's weights
    are 224 MiB, far more than an XCD's L2, so the row-tiled GEMMs deal their tiles round-robin over the XCDs, and
    the reduction of dO*W2 is longer than the three-blocks-per-CU kernel takes, so it runs on the two-block ring.
    Checked against the CPU oracle on sampled tokens (forward, dX, dS) and on slices of one expert's dW1 / dW2
    (float64 sums over the expert's routes), and through the reference's acceptance rule on the whole operator."""
    print("moe mixtral-class widths", flush=True)
    T, H, E, I, K = 1024, 4096, 8, 14336, 2
    gen = torch.Generator(device="cuda").manual_seed(53)
    rn = lambda *shape, std=1.0: (torch.randn(*shape, generator=gen, device="cuda") * std).bfloat16().cpu()
    x, w1, w2, g = rn(T, H), rn(E, 2 * I, H, std=0.02), rn(E, H, I, std=0.02), rn(T, H)
    logits = torch.randn(T, E, generator=gen, device="cuda").cpu()
    route = O.router_postprocess(logits, K, normalize=True)
    case = dict(x=x, w1=w1, w2=w2, g=g, idx=route.expert_indices, w=route.expert_weights.bfloat16())
    out, grads = hip_moe_grads(x, w1, w2, case["idx"], case["w"], g)
    assert all(torch.isfinite(t.float()).all() for t in (out, *grads))
    pick = torch.from_numpy(np.random.Generator(np.random.Philox(53)).choice(T, size=48, replace=False))
    leaves = [t.float().requires_grad_(r) for t, r in ((x[pick], True), (w1, False), (w2, False), (case["w"][pick], True))]
    ref_out = O.fused_moe(leaves[0], leaves[1], leaves[2], case["idx"][pick], leaves[3])
    (ref_out * g[pick].float()).sum().backward()
    assert_close_scaled(out.cpu()[pick], ref_out.detach(), BF16_TOL, "sampled tokens vs CPU oracle")
    assert_close_scaled(grads[0].cpu()[pick], leaves[0].grad, BF16_TOL, "sampled dX vs CPU oracle")
    assert_close_scaled(grads[3].cpu()[pick], leaves[3].grad, BF16_TOL, "sampled dS vs CPU oracle")
    del leaves, ref_out
    e = 5
    dw1_ref, dw2_ref = _expert_weight_gradients_f64(case, e, rows1=slice(0, 2 * I, 1409), rows2=slice(0, H, 211), wide=torch.float32)
    assert_close_scaled(grads[1][e].cpu()[0:2 * I:1409], dw1_ref, BF16_TOL, "dW1 slice of one expert vs float64 CPU sum")
    assert_close_scaled(grads[2][e].cpu()[0:H:211], dw2_ref, BF16_TOL, "dW2 slice of one expert vs float64 CPU sum")
    del out, grads
    torch.cuda.empty_cache()
    # the reference's gate on the whole operator at this profile (moe_runner.py:176-193)
    from minitrain_amd.benchmarks.moe_rows import operator_rows

    hip = operator_rows("mixtral", T, iters=2, warmup=1, seed=1, with_torch=False)[0]
    for side in ("fwd", "bwd"):
        assert hip[f"{side}_relative_l2"] <= 1e-2 and hip[f"{side}_cosine_similarity"] >= 0.9999, hip
    torch.cuda.empty_cache()


def test_moe_block_end_to_end():
    """Router + fused MoE through the block that owns the parameters, with the aux and
    z losses in the objective so that all three router-gradient inlets are used."""
    print("moe block end to end", flush=True)
    from minitrain_amd.model.blocks import MoEFeedForward
    from minitrain_amd.model.config import ModelConfig

    T, H, E, I, K = 512, 128, 8, 256, 2
    cfg = ModelConfig(hidden_size=H, n_heads=1, intermediate_size=I, num_experts=E, experts_per_token=K, n_layers=12)
    x, w_r, w1, w2, g = O.make_inputs(7, T, H, E, I)
    block = MoEFeedForward(cfg).cuda()
    with torch.no_grad():
        block.router.weight.copy_(w_r)
        block.gate_up_proj.copy_(w1)
        block.down_proj.copy_(w2)
    xg = x.bfloat16().cuda().requires_grad_(True)
    with torch.autocast("cuda", dtype=torch.bfloat16):
        out = block(xg.view(4, T // 4, H), hip_backend())
    loss = (out.hidden_states.float() * g.cuda().view(4, T // 4, H)).sum() + 0.01 * out.router_aux_loss \
        + 0.001 * out.router_z_loss
    loss.backward()
    # oracle: same arithmetic on the CPU, fp32-accumulated experts
    leaves = [t.clone().requires_grad_(True) for t in (x.bfloat16().float(), w_r, w1, w2)]
    hidden, r = O.moe_feed_forward(leaves[0].bfloat16(), leaves[1], leaves[2].bfloat16(), leaves[3].bfloat16(), K,
                                   compute_dtype=torch.float32)
    ref_loss = (hidden * g).sum() + 0.01 * r.auxiliary_loss + 0.001 * r.z_loss
    ref_loss.backward()
    assert torch.equal(out.router_metrics["moe/expert_load_fraction"].cpu() * T * K,
                       torch.bincount(r.expert_indices.flatten().long(), minlength=E).float())
    assert_close_scaled(out.hidden_states.view(T, H), hidden, BF16_TOL, "hidden")
    torch.testing.assert_close(out.router_aux_loss.cpu(), r.auxiliary_loss, rtol=1e-4, atol=1e-6)
    torch.testing.assert_close(out.router_z_loss.cpu(), r.z_loss, rtol=1e-4, atol=1e-6)
    assert_close_scaled(xg.grad, leaves[0].grad, BF16_TOL, "dx")
    assert_close_scaled(block.router.weight.grad, leaves[1].grad, BF16_TOL, "dRouter")
    assert_close_scaled(block.gate_up_proj.grad, leaves[2].grad, BF16_TOL, "dW1")
    assert_close_scaled(block.down_proj.grad, leaves[3].grad, BF16_TOL, "dW2")
    for key in ("moe/router_entropy", "moe/dropped_route_fraction", "moe/max_expert_load", "moe/min_expert_load"):
        assert key in out.router_metrics
