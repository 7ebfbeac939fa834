"""Child process of tests/test_gpu_tile_choices.py: one layer step (forward and backward) of the hip backend on
seeded inputs, with whatever tile-choice overrides the environment holds, written to the .npz file named in
argv[1].  The overrides are read once per process, which is why this runs in a process of its own."""

import sys
from pathlib import Path

import numpy as np
import torch

ROOT = Path(__file__).resolve().parents[1]
sys.path.insert(0, str(ROOT))
sys.path.insert(0, str(ROOT / "mini-train-sys_amd"))

from oracle import moe_oracle as O   # noqa: E402  (test infrastructure: the seeded inputs)

SHAPES = {"layer": (3000, 256, 8, 512, 2), "ragged": (777, 128, 5, 192, 3)}   # T, H, E, I, K


def layer_step(name):
    from minitrain_amd.model.ops import get_ops_backend

    ops = get_ops_backend("hip")
    T, H, E, I, K = SHAPES[name]
    x, w_r, w1, w2, g = O.make_inputs(4100 + T, T, H, E, I)
    leaves = [x.bfloat16().cuda().requires_grad_(True), w_r.cuda().requires_grad_(True),
              w1.bfloat16().cuda().requires_grad_(True), w2.bfloat16().cuda().requires_grad_(True)]
    out, aux, z = ops.moe_layer(*leaves, K, normalize=True)[:3]
    torch.autograd.backward([out, aux, z], [g.bfloat16().cuda(), torch.tensor(0.01, device="cuda"),
                                            torch.tensor(0.001, device="cuda")])
    torch.cuda.synchronize()
    named = dict(out=out, dx=leaves[0].grad, dw_r=leaves[1].grad, dw1=leaves[2].grad, dw2=leaves[3].grad)
    return {f"{name}_{k}": v.detach().float().cpu().numpy() for k, v in named.items()}


if __name__ == "__main__":
    results = {}
    for shape in SHAPES:
        print(f"tile choice child: {shape}", flush=True)
        results.update(layer_step(shape))
    np.savez(sys.argv[1], **results)
