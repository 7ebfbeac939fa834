"""HIP router projection (fp32 logits straight from the activation dtype) against float64.

The reference computes ``F.linear(hidden_states.float(), weight.float())``
(minitrain/model/moe_router.py:64-76); the conversion of bf16 to fp32 is exact, so the
float64 product of the same values is the checker: fp32 sums must agree with it at 1e-5
of the tensor's scale, whatever order they run in.
"""

import numpy as np
import pytest
import torch

from tests.helpers import hip_backend

pytestmark = pytest.mark.gpu

F32_TOL = 1e-5    # max|a-b| / max|b| for fp32 results (logits, dW_r)
BF16_ULP = 2.0 ** -8   # dx is rounded to bf16 once


def _scaled_err(a, b):
    return float((a.double() - b.double()).abs().max() / b.double().abs().max().clamp_min(1e-30))


def _case(T, H, E, dtype, seed):
    rng = np.random.Generator(np.random.Philox(seed))
    x = torch.from_numpy(rng.standard_normal((T, H), dtype=np.float32)).to(dtype)
    w = torch.from_numpy(rng.standard_normal((E, H), dtype=np.float32) * np.float32(0.02))
    g = torch.from_numpy(rng.standard_normal((T, E), dtype=np.float32))
    return x, w, g


@pytest.mark.parametrize("T,H,E", [(1, 64, 4), (5, 64, 3), (257, 768, 8), (1000, 1024, 16), (4096, 768, 8), (24576, 768, 8),
                                   (300, 4096, 8), (1000, 2048, 16), (513, 1280, 8), (100, 3072, 5), (64, 2052, 8),
                                   # bf16 rows, up to 8 experts, H % 64 == 0 and H <= 2048: the projection on the matrix pipe;
                                   # several register chunks per row, more groups of 16 rows than waves
                                   (40000, 1024, 7), (333, 2048, 8)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
def test_router_logits_forward_backward(T, H, E, dtype):
    ops = hip_backend()
    x, w, g = _case(T, H, E, dtype, seed=T + H + E)
    xd, wd = x.cuda().requires_grad_(True), w.cuda().requires_grad_(True)
    logits = ops.router_logits(xd, wd)
    assert logits is not None and logits.dtype == torch.float32 and logits.shape == (T, E)
    ref = x.double() @ w.double().T
    assert _scaled_err(logits.detach().cpu(), ref) <= F32_TOL
    logits.backward(g.cuda())
    dx_ref = g.double() @ w.double()
    dw_ref = g.double().T @ x.double()
    assert xd.grad.dtype == dtype and wd.grad.dtype == torch.float32
    assert _scaled_err(xd.grad.cpu(), dx_ref) <= (F32_TOL if dtype == torch.float32 else BF16_ULP)   # one 16-bit rounding
    assert _scaled_err(wd.grad.cpu(), dw_ref) <= F32_TOL


def test_router_logits_is_deterministic_and_matches_torch_path():
    ops = hip_backend()
    x, w, g = _case(24576, 768, 8, torch.bfloat16, seed=11)
    xd, wd = x.cuda(), w.cuda()
    outs = []
    for _ in range(2):
        a, b = xd.clone().requires_grad_(True), wd.clone().requires_grad_(True)
        y = ops.router_logits(a, b)
        y.backward(g.cuda())
        outs.append((y.detach().clone(), a.grad.clone(), b.grad.clone()))
    for p, q in zip(outs[0], outs[1]):
        assert torch.equal(p, q)
    # the reference's own formulation on the same device
    a, b = xd.clone().requires_grad_(True), wd.clone().requires_grad_(True)
    y = torch.nn.functional.linear(a.float(), b)
    y.backward(g.cuda())
    assert _scaled_err(outs[0][0].cpu(), y.detach().cpu()) <= F32_TOL
    assert _scaled_err(outs[0][1].cpu(), a.grad.cpu()) <= BF16_ULP
    assert _scaled_err(outs[0][2].cpu(), b.grad.cpu()) <= F32_TOL


def test_router_logits_unsupported_contract_returns_none():
    ops = hip_backend()
    x = torch.randn(8, 8192, device="cuda", dtype=torch.bfloat16)     # hidden size above the kernel's range
    w = torch.randn(8, 8192, device="cuda")
    assert ops.router_logits(x, w) is None
    x = torch.randn(8, 4096, device="cuda", dtype=torch.bfloat16)     # 16 x 4096 fp32 weights do not fit the LDS
    w = torch.randn(16, 4096, device="cuda")
    assert ops.router_logits(x, w) is None
    x = torch.randn(8, 64, device="cuda", dtype=torch.float64)        # unsupported activation dtype
    assert ops.router_logits(x, torch.randn(8, 64, device="cuda")) is None
    from minitrain_amd.kernels.hip import router_logits
    with pytest.raises(RuntimeError):
        router_logits(x, torch.randn(8, 64, device="cuda"))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])   # bf16: matrix-pipe projection; fp16: vector pipe
def test_router_logits_with_weights_that_are_not_finite_or_round_to_infinity(dtype):
    """An infinite weight gives infinite logits of the product's sign (NaN where the activation is zero), a NaN
    weight gives NaN, and a finite weight beyond the largest bf16 value stays finite: what the fp32 dot product
    of the reference (`F.linear(x.float(), w)`) gives, on both projections, and the other experts do not notice."""
    ops = hip_backend()
    T, H, E = 600, 256, 8
    x, w, _ = _case(T, H, E, dtype, seed=77)
    x[5] = 0.0                                  # 0 * inf
    w[2, 17] = float("inf")
    w[4, 200] = float("nan")
    w[6, 3] = -float("inf")
    w[1, 9] = 3.4e38                            # finite in fp32, above the largest bf16 value
    x[:, 9] = x[:, 9] * 1e-3                    # keeps expert 1's logits finite
    got = ops.router_logits(x.cuda(), w.cuda()).cpu()
    want = torch.nn.functional.linear(x.float(), w)
    assert torch.equal(torch.isnan(got), torch.isnan(want))
    assert torch.equal(torch.isinf(got), torch.isinf(want))
    inf = torch.isinf(want)
    assert torch.equal(torch.sign(got[inf]), torch.sign(want[inf]))
    fin = torch.isfinite(want)
    assert bool(fin[:, 1].all())
    ref64 = (x.double()[:, None, :] * w.double()[None, :, :]).nan_to_num(0.0, 0.0, 0.0).sum(-1)
    for e in (0, 1, 3, 5, 7):
        assert _scaled_err(got[:, e], ref64[:, e]) <= F32_TOL, e
