"""mts_moe_fwd_gateup_down (gate/up + SwiGLU and the down projection as one launch) against the two launches.

Both run the same tile code on the same tiles, so every output is bit-identical; what the joint launch adds is the
hand-over of post_act rows between blocks of one launch (counters in a workspace that the launch must leave as it
found it, all zeros, and a status word that stays zero).  The cases cover whole and half tiles of the down part,
experts without rows, one-row problems, routing weights applied or not, fp16, and consecutive calls of different
sizes on one workspace."""

import os
import subprocess
import sys
from pathlib import Path

import pytest
import torch

pytestmark = pytest.mark.gpu

ROOT = Path(__file__).resolve().parents[1]


def _routing(lib, idx, E):
    from minitrain_amd.kernels.hip.fused_moe import routing_for_experts

    return routing_for_experts(idx, E)   # expert_start, x_gather, s_scatter, s_reverse


def _forward(lib, joint, x, w1, w2, weights, routing, workspace=None):
    from minitrain_amd import _lib

    expert_start, x_gather, s_scatter, _ = routing
    T, H = x.shape
    E, I = w1.shape[0], w1.shape[1] // 2
    TK = x_gather.numel()
    K = TK // T
    act = _lib.dtype_code(x.dtype)
    new = lambda *shape: torch.full(shape, 3.0, dtype=x.dtype, device=x.device)
    pre, post, y = new(TK, 2 * I), new(TK, I), new(TK, H)
    st = _lib.stream_of(x)
    wp = weights.data_ptr() if weights is not None else None
    sp = s_scatter.data_ptr() if weights is not None else None
    if joint:
        rc = lib.mts_moe_fwd_gateup_down(x.data_ptr(), w1.data_ptr(), w2.data_ptr(), x_gather.data_ptr(), expert_start.data_ptr(),
                                         wp, sp, T, K, E, H, I, act, pre.data_ptr(), post.data_ptr(), y.data_ptr(),
                                         workspace.data_ptr(), workspace.numel() * 4, st)
        assert rc == 0, rc
    else:
        rc = lib.mts_moe_fwd_gateup_swiglu(x.data_ptr(), w1.data_ptr(), x_gather.data_ptr(), expert_start.data_ptr(), wp, sp,
                                           T, K, E, H, I, act, pre.data_ptr(), post.data_ptr(), st)
        assert rc == 0, rc
        rc = lib.mts_moe_fwd_down(post.data_ptr(), w2.data_ptr(), expert_start.data_ptr(), TK, E, H, I, act, y.data_ptr(), st)
        assert rc == 0, rc
    torch.cuda.synchronize()
    return pre, post, y


def _case(seed, T, H, E, I, K, dtype, skew=0.0, empty_expert=None):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(T, H, generator=g).to(dtype).cuda()
    w1 = (torch.randn(E, 2 * I, H, generator=g) * 0.05).to(dtype).cuda()
    w2 = (torch.randn(E, H, I, generator=g) * 0.05).to(dtype).cuda()
    idx = torch.stack([torch.randperm(E, generator=g)[:K] for _ in range(T)]).int()
    if skew:
        heavy = torch.rand(T, generator=g) < skew
        idx[heavy, 0] = 1 % E
        if K > 1:
            idx[heavy & (idx[:, 1] == 1 % E), 1] = 0
    if empty_expert is not None:
        other = (empty_expert + 1) % E
        clash = (idx == other).any(1, keepdim=True) & (idx == empty_expert)
        idx[idx == empty_expert] = other
        idx[clash] = (empty_expert + 2) % E   # keep a token's experts distinct
    weights = torch.rand(T, K, generator=g).to(dtype).cuda()
    return x, w1, w2, idx.cuda(), weights


@pytest.mark.parametrize("T,H,E,I,K,dtype,skew,weighted", [
    (3000, 256, 8, 512, 2, torch.bfloat16, 0.0, True),
    (3000, 256, 8, 512, 2, torch.bfloat16, 0.7, True),      # one expert far over its share: many m-tiles on one XCD
    (777, 128, 5, 192, 3, torch.bfloat16, 0.0, False),      # ragged experts, post_act without the routing weight
    (1, 64, 4, 64, 1, torch.bfloat16, 0.0, True),           # one row: every tile is a sliver, every second half empty
    (130, 64, 3, 64, 2, torch.float16, 0.0, True),          # m-tiles of at most 128 rows cut in two: empty halves
    (2048, 768, 8, 1024, 2, torch.float16, 0.3, True),
    (5000, 192, 64, 128, 2, torch.bfloat16, 0.5, True),     # more experts than XCDs, most with a single short tile
    (4096, 64, 1, 64, 1, torch.bfloat16, 0.0, True),        # one expert, one k-tile per GEMM, one column tile each
    (9000, 512, 16, 1984, 2, torch.bfloat16, 0.2, True),    # 15.5 column tiles of gate/up: the last one half empty
    (3000, 320, 130, 64, 2, torch.float16, 0.0, True),      # more experts than a wave holds: the search walks two groups
])
def test_joint_forward_launch_equals_two_launches(T, H, E, I, K, dtype, skew, weighted):
    print(f"joint forward T={T} H={H} E={E} I={I} K={K} {dtype} skew={skew} weighted={weighted}", flush=True)
    from minitrain_amd import _lib

    lib = _lib.load()
    assert lib.mts_moe_fwd_joint_supported(_lib.dtype_code(dtype), H, I) == 1
    x, w1, w2, idx, weights = _case(11 + T, T, H, E, I, K, dtype, skew, empty_expert=2 if E > 3 else None)
    routing = _routing(lib, idx, E)
    ws = torch.zeros(lib.mts_moe_fwd_joint_workspace_bytes(T * K, E) // 4, dtype=torch.int32, device="cuda")
    want = _forward(lib, False, x, w1, w2, weights.flatten() if weighted else None, routing)
    for call in range(2):   # the second call finds the counters as the first one left them
        got = _forward(lib, True, x, w1, w2, weights.flatten() if weighted else None, routing, ws)
        assert int(ws[0]) == 0, f"status {int(ws[0])}"
        assert int((ws != 0).sum()) == 0, "the launch left counters behind"
        rows = int(routing[0][-1])   # rows behind the last expert's end (dropped routes) belong to nobody
        for name, a, b in zip(("pre_act", "post_act", "y"), got, want):
            assert torch.equal(a[:rows], b[:rows]), (name, call)


def test_joint_forward_consecutive_sizes_on_one_workspace():
    """A large problem, then smaller ones and a larger one again, on a workspace sized for the largest."""
    from minitrain_amd import _lib

    lib = _lib.load()
    H, E, I, K, dtype = 128, 8, 256, 2, torch.bfloat16
    sizes = [6000, 300, 1, 2500, 6000]
    ws = torch.zeros(lib.mts_moe_fwd_joint_workspace_bytes(max(sizes) * K, E) // 4, dtype=torch.int32, device="cuda")
    for n, T in enumerate(sizes):
        print(f"joint forward on a shared workspace: T={T}", flush=True)
        x, w1, w2, idx, weights = _case(500 + n, T, H, E, I, K, dtype, skew=0.4 if n % 2 else 0.0)
        routing = _routing(lib, idx, E)
        want = _forward(lib, False, x, w1, w2, weights.flatten(), routing)
        got = _forward(lib, True, x, w1, w2, weights.flatten(), routing, ws)
        assert int((ws != 0).sum()) == 0
        for a, b in zip(got, want):
            assert torch.equal(a, b), T


def test_joint_forward_while_another_stream_keeps_the_chip_busy():
    """Blocks of other kernels take CUs and cache lines while the launch runs (large copies and GEMMs on a second stream):
    the hand-over of rows between the launch's blocks does not depend on having the chip to itself."""
    from minitrain_amd import _lib

    lib = _lib.load()
    T, H, E, I, K = 24576, 768, 8, 1024, 2
    side = torch.cuda.Stream()
    a = torch.randn(4096, 4096, device="cuda", dtype=torch.bfloat16)
    big = torch.empty(128 * 2**20, device="cuda", dtype=torch.uint8)
    big2 = torch.empty_like(big)
    ws = torch.zeros(lib.mts_moe_fwd_joint_workspace_bytes(T * K, E) // 4, dtype=torch.int32, device="cuda")
    for seed in range(4):
        print(f"joint forward beside another stream: seed {seed}", flush=True)
        x, w1, w2, idx, weights = _case(2000 + seed, T, H, E, I, K, torch.bfloat16, skew=0.2 * seed)
        routing = _routing(lib, idx, E)
        want = _forward(lib, False, x, w1, w2, weights.flatten(), routing)
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for _ in range(8):
                if seed % 2:
                    torch.mm(a, a)
                else:
                    big2.copy_(big)
        for _ in range(3):
            got = _forward(lib, True, x, w1, w2, weights.flatten(), routing, ws)
            assert int((ws != 0).sum()) == 0, f"status {int(ws[0])}"
            for u, v in zip(got, want):
                assert torch.equal(u, v)
        torch.cuda.synchronize()


def test_operator_forward_replayed_from_a_graph():
    """The operator's forward pass captured into a graph and replayed with other activations and another routing in
    the same buffers, with eager calls and synchronisations between the replays: every replay gives what the eager call
    gives.  (The launch's counters are cleared by a fill kernel inside the graph and left clear by the launch; the host
    side does not look at the status word while a stream is being captured.)"""
    from tests.helpers import hip_backend, routed_case
    from minitrain_amd.kernels.hip.fused_moe import joint_forward_status

    ops = hip_backend()
    T, H, E, I, K = 4096, 768, 8, 1024, 2
    case = routed_case(5, T, H, E, I, K)
    x, w1, w2, idx, w = (case[k].cuda() for k in ("x", "w1", "w2", "idx", "w"))
    gen = torch.Generator().manual_seed(17)
    with torch.no_grad():
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for _ in range(3):
                ops.fused_moe(x, w1, w2, idx, w)
        torch.cuda.current_stream().wait_stream(side)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            out = ops.fused_moe(x, w1, w2, idx, w)
        for replay in range(4):
            print(f"graph replay {replay}", flush=True)
            x.copy_(torch.randn(T, H, generator=gen).to(x.dtype))
            idx.copy_(torch.stack([torch.randperm(E, generator=gen)[:K] for _ in range(T)]).int())
            graph.replay()
            torch.cuda.synchronize()
            eager = ops.fused_moe(x, w1, w2, idx, w)
            assert torch.equal(out, eager), replay
    assert joint_forward_status() == 0


@pytest.mark.parametrize("dtype,fp32_weights", [(torch.bfloat16, False), (torch.float16, True)])
def test_operator_with_and_without_the_joint_forward_launch(dtype, fp32_weights, monkeypatch):
    """The operator's output and every gradient are bit-identical whichever way the forward GEMMs are launched."""
    import importlib

    from tests.helpers import hip_moe_grads, routed_case
    from oracle import moe_oracle as O

    F = importlib.import_module("minitrain_amd.kernels.hip.fused_moe")
    T, H, E, I, K = 1500, 192, 8, 320, 2
    case = routed_case(333, T, H, E, I, K, dtype=dtype)
    if fp32_weights:
        _, _, w1, w2, _ = O.make_inputs(333, T, H, E, I)
        case.update(w1=w1, w2=w2)
    args = (case["x"], case["w1"], case["w2"], case["idx"], case["w"], case["g"])
    monkeypatch.setattr(F.SWITCHES, "joint_fwd", True)
    one = hip_moe_grads(*args)
    assert F.joint_forward_status() == 0
    monkeypatch.setattr(F.SWITCHES, "joint_fwd", False)
    two = hip_moe_grads(*args)
    assert torch.equal(one[0], two[0])
    for a, b in zip(one[1], two[1]):
        assert torch.equal(a, b)


def test_host_side_raises_on_a_status_word(monkeypatch):
    """The host side looks at the status word of an earlier call without waiting for the GPU; a word that is not
    zero raises and the counters are dropped.  The word is written by the test: no launch is made to fail."""
    import importlib

    F = importlib.import_module("minitrain_amd.kernels.hip.fused_moe")
    ws = F._JointForwardWorkspace(torch.device("cuda", torch.cuda.current_device()))
    buf = ws.get(64)
    ws.before_launch()
    ws.after_launch()            # call 1: the word (zero) is copied to the host
    torch.cuda.synchronize()
    ws.before_launch()           # ... and found to be zero
    buf[0] = 1
    for _ in range(F._JointForwardWorkspace.CHECK_EVERY):
        ws.after_launch()        # the next copy is due CHECK_EVERY calls after the first
    torch.cuda.synchronize()
    with pytest.raises(RuntimeError, match="status 1"):
        ws.before_launch()
    assert ws.buf is None and ws.status() == 0


def test_a_wait_that_is_given_up_ends_the_launch_and_is_reported(tmp_path):
    """With a wait limit of zero (set from the host, read when the library is loaded) a down block that finds its rows
    unfinished gives up at once instead of waiting: the launch still ends and the status word says 1."""
    env = dict(os.environ, MTS_FWD_JOINT_SPIN_US="0")
    run = subprocess.run([sys.executable, str(ROOT / "tests" / "joint_forward_child.py")], env=env, capture_output=True, text=True,
                         timeout=300, cwd=str(ROOT))
    assert run.returncode == 0, run.stderr[-2000:]
    # at the child's size every down block comes early, so with no time to wait the word must say so
    assert "status after a limit of zero: 1" in run.stdout and "cleared workspace: equal" in run.stdout, run.stdout
