"""Model configuration: the fields, names and defaults of the reference's ``ModelConfig``
(minitrain/model/config.py:4-63) that the decoder and its MoE blocks read.  The reference
reserves ``expert_capacity_factor`` / ``expert_min_capacity`` for a compacted dispatch and
ignores them (config.py:24-28); here a factor other than None switches that dispatch on."""

from dataclasses import dataclass


@dataclass(frozen=True)
class ModelConfig:
    vocab_size: int = 32000
    seq_len: int = 2048
    n_layers: int = 12
    n_heads: int = 12
    hidden_size: int = 768
    intermediate_size: int = 2048
    norm_eps: float = 1e-5
    rope_theta: float = 10000.0
    dropout: float = 0.0
    tie_word_embeddings: bool = False
    ffn_type: str = "moe"
    num_experts: int = 8
    experts_per_token: int = 2
    router_aux_loss_coef: float = 1e-2
    router_z_loss_coef: float = 1e-3
    router_normalize_topk: bool = True
    router_jitter_noise: float = 0.0
    expert_capacity_factor: float | None = None
    expert_min_capacity: int = 4

    def __post_init__(self) -> None:
        sizes = (self.vocab_size, self.seq_len, self.n_layers, self.n_heads, self.hidden_size, self.intermediate_size)
        if min(sizes) <= 0:
            raise ValueError("all model dimensions must be positive")
        if not 0 <= self.dropout < 1:
            raise ValueError("dropout must be in [0, 1)")
        if self.norm_eps <= 0 or self.rope_theta <= 0:
            raise ValueError("norm_eps and rope_theta must be positive")
        if self.ffn_type not in {"dense", "moe"}:
            raise ValueError("ffn_type must be either 'dense' or 'moe'")
        if self.hidden_size % self.n_heads != 0:
            raise ValueError("hidden_size must be divisible by n_heads")
        if self.num_experts <= 0:
            raise ValueError("num_experts must be positive")
        if not 0 < self.experts_per_token <= self.num_experts:
            raise ValueError("experts_per_token must be in [1, num_experts]")
        if self.router_aux_loss_coef < 0 or self.router_z_loss_coef < 0:
            raise ValueError("router loss coefficients must be non-negative")
        if not 0 <= self.router_jitter_noise < 1:
            raise ValueError("router_jitter_noise must be in [0, 1)")
        if self.expert_capacity_factor is not None and self.expert_capacity_factor <= 0:
            raise ValueError("expert_capacity_factor must be positive or null")
        if self.expert_min_capacity <= 0:
            raise ValueError("expert_min_capacity must be positive")

    @property
    def head_dim(self) -> int:
        return self.hidden_size // self.n_heads

    @property
    def is_moe(self) -> bool:
        return self.ffn_type == "moe"
