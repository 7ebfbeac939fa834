"""The fields of the reference's ``ModelConfig`` (minitrain/model/config.py:4-27)
that the MoE block reads, with the same names and defaults."""

from dataclasses import dataclass


@dataclass(frozen=True)
class ModelConfig:
    n_layers: int = 12
    hidden_size: int = 768
    intermediate_size: int = 2048
    dropout: float = 0.0
    ffn_type: str = "moe"
    num_experts: int = 8
    experts_per_token: int = 2
    router_aux_loss_coef: float = 1e-2
    router_z_loss_coef: float = 1e-3
    router_normalize_topk: bool = True
    router_jitter_noise: float = 0.0

    def __post_init__(self) -> None:
        if min(self.n_layers, self.hidden_size, self.intermediate_size) <= 0:
            raise ValueError("all model dimensions must be positive")
        if not 0 <= self.dropout < 1:
            raise ValueError("dropout must be in [0, 1)")
        if self.num_experts <= 0:
            raise ValueError("num_experts must be positive")
        if not 0 < self.experts_per_token <= self.num_experts:
            raise ValueError("experts_per_token must be in [1, num_experts]")
        if not 0 <= self.router_jitter_noise < 1:
            raise ValueError("router_jitter_noise must be in [0, 1)")
