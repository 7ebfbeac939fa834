"""Child process of tests/test_gpu_joint_forward.py: the joint gate/up + down launch at a size whose tiles all fit the
chip at once, so that every down block starts while the gate/up tiles it reads from are still running, with whatever
wait limit the environment holds (it is read once per process).  Prints the status word; the outputs are compared
with the two launches when the status is zero."""

import sys
from pathlib import Path

import torch

ROOT = Path(__file__).resolve().parents[1]
sys.path.insert(0, str(ROOT))
sys.path.insert(0, str(ROOT / "mini-train-sys_amd"))

from tests import test_gpu_joint_forward as J   # noqa: E402
from minitrain_amd import _lib   # noqa: E402

if __name__ == "__main__":
    lib = _lib.load()
    T, H, E, I, K, dtype = 2000, 768, 8, 1024, 2, torch.bfloat16
    x, w1, w2, idx, weights = J._case(5, T, H, E, I, K, dtype)
    routing = J._routing(lib, idx, E)
    ws = torch.zeros(lib.mts_moe_fwd_joint_workspace_bytes(T * K, E) // 4, dtype=torch.int32, device="cuda")
    want = J._forward(lib, False, x, w1, w2, weights.flatten(), routing)
    print("joint forward child: launching", flush=True)
    got = J._forward(lib, True, x, w1, w2, weights.flatten(), routing, ws)
    status = int(ws[0])
    print(f"status after a limit of zero: {status}", flush=True)
    assert status in (0, 1), status
    if status == 0:
        assert all(torch.equal(a, b) for a, b in zip(got, want))
    # what the host does after a failed launch: the counters are cleared (or dropped) before the workspace is used again
    ws.zero_()
    torch.cuda.synchronize()
    print("cleared workspace: equal" if int((ws != 0).sum()) == 0 else "cleared workspace: not zero", flush=True)
