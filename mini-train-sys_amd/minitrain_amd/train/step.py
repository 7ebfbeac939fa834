"""One optimizer update, as the reference's ``Trainer.train_step`` runs it
(minitrain/train/trainer.py:85-159): forward under autocast with fp32 parameters, backward,
global-norm clipping, AdamW with weight decay on matrices only
(minitrain/train/optim.py:30-47), ``zero_grad(set_to_none=True)``.
"""

import contextlib

import torch


def build_optimizer(model: torch.nn.Module, *, lr: float = 3e-4, weight_decay: float = 0.1, betas=(0.9, 0.95),
                    eps: float = 1e-8) -> torch.optim.Optimizer:
    decay = [p for p in model.parameters() if p.requires_grad and p.ndim >= 2]
    no_decay = [p for p in model.parameters() if p.requires_grad and p.ndim < 2]
    groups = [{"params": decay, "weight_decay": weight_decay}, {"params": no_decay, "weight_decay": 0.0}]
    fused = any(p.is_cuda for p in model.parameters())
    return torch.optim.AdamW(groups, lr=lr, betas=betas, eps=eps, fused=fused)


def train_step(model: torch.nn.Module, optimizer: torch.optim.Optimizer, batch: dict, *,
               autocast_dtype: torch.dtype | None = torch.bfloat16, grad_clip_norm: float | None = 1.0,
               use_fused_loss: bool = False, check_finite: bool = True) -> torch.Tensor:
    """Forward, backward, clipping and the optimizer update, exactly once; returns the loss.

    A non-finite loss or gradient norm raises ``FloatingPointError`` from the host before the optimizer
    runs (the conditions the reference tests, minitrain/train/trainer.py:77-78,101-106).  The test is one flag
    computed on the device and read once per step; nothing on the device asserts or traps.
    ``check_finite=False`` skips the read (and its synchronisation) for callers that check at their own
    interval."""
    model.train()
    device = next(model.parameters()).device
    input_ids = batch["input_ids"].to(device, non_blocking=True)
    targets = batch["targets"].to(device, non_blocking=True)
    ctx = (
        torch.autocast(device_type=device.type, dtype=autocast_dtype)
        if autocast_dtype is not None and device.type == "cuda"
        else contextlib.nullcontext()
    )
    with ctx:
        loss, _ = model(input_ids, targets=targets, use_fused_loss=use_fused_loss)
    finite = torch.isfinite(loss.detach())
    loss.backward()
    if grad_clip_norm is not None:
        norm = torch.nn.utils.clip_grad_norm_(model.parameters(), grad_clip_norm)
        finite = finite & torch.isfinite(norm)
    if check_finite and not bool(finite):   # one host read per step
        optimizer.zero_grad(set_to_none=True)
        raise FloatingPointError("non-finite training loss or global gradient norm")
    optimizer.step()
    optimizer.zero_grad(set_to_none=True)
    return loss.detach()
