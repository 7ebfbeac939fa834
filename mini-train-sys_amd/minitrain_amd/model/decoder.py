"""Host model of the MoE path: a causal decoder whose feed-forward blocks are MoE layers.

Same constructor, parameter names, forward signature and loss composition as the
reference's ``MiniTransformer`` (minitrain/model/transformer.py:10-170) with its blocks
(minitrain/model/blocks.py:19-60, 105-135) and rotary cache (minitrain/model/rotary.py), so a
state dict of one loads into the other.  Every operator goes through the ``ops`` backend: the
``hip`` backend supplies the two MoE operators (and the router projection and route counts the
router module asks for), the other six stay on stock PyTorch-ROCm.
"""

import math

import torch
from torch import nn

from minitrain_amd.model.blocks import MoEFeedForward
from minitrain_amd.model.config import ModelConfig
from minitrain_amd.model.ops import OpsBackend


def rotary_tables(head_dim: int, seq_len: int, theta: float, dtype: torch.dtype):
    """cos/sin of the rotary angles, ``[seq_len, head_dim]``: computed in fp32, cast once."""
    if head_dim % 2:
        raise ValueError("RoPE requires an even head_dim")
    inv_freq = theta ** (-torch.arange(0, head_dim, 2, dtype=torch.float32) / head_dim)
    angles = torch.outer(torch.arange(seq_len, dtype=torch.float32), inv_freq).repeat(1, 2)
    return angles.cos().to(dtype), angles.sin().to(dtype)


class RotaryEmbedding(nn.Module):
    def __init__(self, head_dim: int, max_seq_len: int, theta: float, *, cache_dtype: torch.dtype) -> None:
        super().__init__()
        cos, sin = rotary_tables(head_dim, max_seq_len, theta, cache_dtype)
        self.register_buffer("cos", cos, persistent=False)
        self.register_buffer("sin", sin, persistent=False)

    def forward(self, seq_len: int):
        if seq_len > self.cos.size(0):
            raise ValueError(f"seq_len={seq_len} exceeds configured max seq_len={self.cos.size(0)}")
        return self.cos[:seq_len], self.sin[:seq_len]


class RMSNorm(nn.Module):
    def __init__(self, hidden_size: int, eps: float) -> None:
        super().__init__()
        self.weight = nn.Parameter(torch.ones(hidden_size))
        self.eps = eps

    def forward(self, x: torch.Tensor, ops: OpsBackend) -> torch.Tensor:
        return ops.rmsnorm(x, self.weight, self.eps)


class CausalSelfAttention(nn.Module):
    def __init__(self, cfg: ModelConfig) -> None:
        super().__init__()
        self.n_heads, self.head_dim, self.p_drop = cfg.n_heads, cfg.head_dim, cfg.dropout
        self.qkv = nn.Linear(cfg.hidden_size, 3 * cfg.hidden_size, bias=False)
        self.out = nn.Linear(cfg.hidden_size, cfg.hidden_size, bias=False)
        self.resid_dropout = nn.Dropout(cfg.dropout)
        nn.init.normal_(self.qkv.weight, mean=0.0, std=0.02)
        nn.init.normal_(self.out.weight, mean=0.0, std=0.02 / math.sqrt(2 * cfg.n_layers))

    def forward(self, x, ops: OpsBackend, rope_cos, rope_sin):
        B, S, H = x.shape
        q, k, v = (t.view(B, S, self.n_heads, self.head_dim).transpose(1, 2) for t in self.qkv(x).chunk(3, dim=-1))
        q, k = ops.rope(q, k, rope_cos, rope_sin)
        ctx = ops.attention(q, k, v, is_causal=True, dropout_p=self.p_drop if self.training else 0.0)
        return self.resid_dropout(self.out(ctx.transpose(1, 2).reshape(B, S, H)))


class TransformerBlock(nn.Module):
    def __init__(self, cfg: ModelConfig) -> None:
        super().__init__()
        if not cfg.is_moe:
            raise ValueError("this host model carries MoE feed-forward blocks only (ffn_type='moe')")
        self.attn_norm = RMSNorm(cfg.hidden_size, cfg.norm_eps)
        self.attn = CausalSelfAttention(cfg)
        self.ffn_norm = RMSNorm(cfg.hidden_size, cfg.norm_eps)
        self.ffn = MoEFeedForward(cfg)

    def forward(self, x, ops: OpsBackend, rope_cos, rope_sin):
        x = x + self.attn(self.attn_norm(x, ops), ops, rope_cos, rope_sin)
        ffn = self.ffn(self.ffn_norm(x, ops), ops)
        return x + ffn.hidden_states, ffn


class MiniTransformer(nn.Module):
    """Causal LM with MoE feed-forward blocks; ``forward`` returns ``(loss, logits-or-hidden)``."""

    def __init__(self, cfg: ModelConfig, ops: OpsBackend, *, activation_dtype: torch.dtype = torch.float32) -> None:
        super().__init__()
        if activation_dtype not in (torch.float32, torch.bfloat16, torch.float16):
            raise ValueError(f"Unsupported activation dtype: {activation_dtype}")
        self.cfg, self.ops, self.activation_dtype = cfg, ops, activation_dtype
        self.embed = nn.Embedding(cfg.vocab_size, cfg.hidden_size)
        self.dropout = nn.Dropout(cfg.dropout)
        self.rotary = RotaryEmbedding(cfg.head_dim, cfg.seq_len, cfg.rope_theta, cache_dtype=activation_dtype)
        self.blocks = nn.ModuleList(TransformerBlock(cfg) for _ in range(cfg.n_layers))
        self.norm = RMSNorm(cfg.hidden_size, cfg.norm_eps)
        self.lm_head = nn.Linear(cfg.hidden_size, cfg.vocab_size, bias=False)
        nn.init.normal_(self.embed.weight, mean=0.0, std=0.02)
        if cfg.tie_word_embeddings:
            self.lm_head.weight = self.embed.weight
        else:
            nn.init.normal_(self.lm_head.weight, mean=0.0, std=0.02)
        self.last_training_metrics: dict[str, torch.Tensor] = {}
        self._router_aux = None
        self._router_z = None

    def hidden_states(self, input_ids: torch.Tensor) -> torch.Tensor:
        hidden = self.dropout(self.embed(input_ids).to(self.activation_dtype))
        cos, sin = self.rotary(hidden.size(1))
        if cos.device != hidden.device or cos.dtype != hidden.dtype:
            raise RuntimeError("RoPE cache must match the residual device and dtype")
        aux, z, per_layer = [], [], {}
        for block in self.blocks:
            hidden, ffn = block(hidden, self.ops, cos, sin)
            aux.append(ffn.router_aux_loss)
            z.append(ffn.router_z_loss)
            for name, value in ffn.router_metrics.items():
                per_layer.setdefault(name, []).append(value)
        metrics = {}
        for name, values in per_layer.items():
            stacked = torch.stack(values)
            if stacked.ndim == 1:
                metrics[name] = stacked.float().mean()
            else:   # per-expert vectors: one entry per expert, averaged over layers
                for i, v in enumerate(stacked.detach().mean(dim=0)):
                    metrics[f"{name}/expert_{i:02d}"] = v
        self._router_aux = torch.stack(aux).mean()
        self._router_z = torch.stack(z).mean()
        metrics["moe/aux_loss"] = self._router_aux.detach()
        metrics["moe/z_loss"] = self._router_z.detach()
        self.last_training_metrics = metrics
        return self.norm(hidden, self.ops)

    def forward(self, input_ids: torch.Tensor, targets: torch.Tensor | None = None, use_fused_loss: bool = False):
        hidden = self.hidden_states(input_ids)
        if targets is None:
            return None, self.lm_head(hidden)
        if use_fused_loss:
            lm_loss = self.ops.fused_linear_cross_entropy(
                hidden.reshape(-1, hidden.size(-1)), self.lm_head.weight, targets.reshape(-1)
            )
            output = hidden
        else:
            output = self.lm_head(hidden)
            lm_loss = self.ops.cross_entropy(output.reshape(-1, output.size(-1)), targets.reshape(-1))
        weighted_aux = self.cfg.router_aux_loss_coef * self._router_aux
        weighted_z = self.cfg.router_z_loss_coef * self._router_z
        loss = lm_loss + weighted_aux + weighted_z
        m = self.last_training_metrics
        m["loss/lm_cross_entropy"] = lm_loss.detach()
        m["loss/moe_aux_weighted"] = weighted_aux.detach()
        m["loss/moe_z_weighted"] = weighted_z.detach()
        m["loss/moe_regularization_total"] = (weighted_aux + weighted_z).detach()
        m["loss/total"] = loss.detach()
        return loss, output
