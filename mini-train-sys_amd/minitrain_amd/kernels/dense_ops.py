"""The six operators that stay on stock PyTorch-ROCm.

The `hip` backend replaces only the two MoE operators; like the reference's
Triton backend (minitrain/kernels/triton/__init__.py:36) it inherits the rest
from a plain PyTorch class.  This base class deliberately has NO
``router_postprocess`` and NO ``fused_moe``: there is nothing for the MoE path to
fall back to.
"""

import torch
import torch.nn.functional as F


class DenseTorchOps:
    name = "torch-dense"

    def rmsnorm(self, x, weight, eps):
        x32 = x.float()
        y = x32 * torch.rsqrt(x32.pow(2).mean(dim=-1, keepdim=True) + eps)
        return (y * weight.float()).to(x.dtype)

    def rope(self, q, k, cos, sin):
        def rot(t):
            t1, t2 = t[..., : t.shape[-1] // 2], t[..., t.shape[-1] // 2 :]
            return torch.cat((-t2, t1), dim=-1)

        cos = cos.to(q.dtype)
        sin = sin.to(q.dtype)
        return q * cos + rot(q) * sin, k * cos + rot(k) * sin

    def swiglu(self, gate, up):
        return F.silu(gate) * up

    def attention(self, q, k, v, *, is_causal, dropout_p):
        return F.scaled_dot_product_attention(q, k, v, is_causal=is_causal, dropout_p=dropout_p)

    def cross_entropy(self, logits, targets):
        return F.cross_entropy(logits.float(), targets)

    def fused_linear_cross_entropy(self, x, weight, targets):
        return F.cross_entropy(F.linear(x, weight).float(), targets)
