"""Writes tests/golden/config1_fp32.npz: the 256-token fp32 debug configuration of the
MoE layer (batch 2 x seq 128, d_model 64, 4 experts, top-2, d_ff 128, seed 0) evaluated
by the CPU oracle in float64 (inputs are the fp32 draws of ``make_inputs``).

The vectors come from this repository's oracle, not from the reference implementation,
which was read but not executed; the oracle itself is pinned by tests/test_oracle_*.py.
Run from the repository root:  python tests/golden/make_config1_golden.py
"""

import os
import sys

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import moe_oracle as O  # noqa: E402

CONFIG1 = dict(seed=0, T=256, H=64, E=4, I=128, K=2)


def evaluate():
    c = CONFIG1
    x, w_r, w1, w2, g = O.make_inputs(c["seed"], c["T"], c["H"], c["E"], c["I"])
    leaves = [t.double().requires_grad_(True) for t in (x, w_r, w1, w2)]
    hidden, r = O.moe_feed_forward(leaves[0], leaves[1], leaves[2], leaves[3], c["K"], compute_dtype=torch.float64)
    loss = (hidden * g.double()).sum() + 0.01 * r.auxiliary_loss + 0.001 * r.z_loss
    loss.backward()
    return dict(
        expert_indices=r.expert_indices.numpy(),
        expert_weights=r.route.expert_weights.detach().numpy(),
        probability_per_expert=r.route.probability_per_expert.detach().numpy(),
        z_loss=r.z_loss.detach().numpy(),
        auxiliary_loss=r.auxiliary_loss.detach().numpy(),
        hidden=hidden.detach().numpy(),
        dx=leaves[0].grad.numpy(),
        d_router=leaves[1].grad.numpy(),
        d_gate_up=leaves[2].grad.numpy(),
        d_down=leaves[3].grad.numpy(),
        x_head=x[:4, :8].numpy(),          # guards the input stream itself
    )


if __name__ == "__main__":
    out = {k: (v.astype(np.float32) if v.dtype == np.float64 else v) for k, v in evaluate().items()}
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "config1_fp32.npz")
    np.savez_compressed(path, **out)
    print("wrote", path, {k: v.shape for k, v in out.items()})
