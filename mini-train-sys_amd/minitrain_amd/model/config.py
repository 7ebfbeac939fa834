"""Model configuration.

Field names and defaults are those of the reference's ``ModelConfig``
(minitrain/model/config.py:4-63), since configs written for it must load here; the checks raise
``ValueError`` for the same conditions.  One deliberate difference: the reference reserves
``expert_capacity_factor`` / ``expert_min_capacity`` for a compacted dispatch and ignores them
(config.py:24-28); here a factor other than None switches that dispatch on.
"""

from dataclasses import dataclass, fields


@dataclass(frozen=True)
class ModelConfig:
    # decoder geometry
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
    # feed-forward flavour and router
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
        problem = self._first_problem()
        if problem:
            raise ValueError(problem)

    def _first_problem(self) -> str | None:
        sizes = ("vocab_size", "seq_len", "n_layers", "n_heads", "hidden_size", "intermediate_size", "num_experts",
                 "expert_min_capacity")
        for name in sizes:
            if getattr(self, name) <= 0:
                return f"{name} must be positive"
        unit_interval = ("dropout", "router_jitter_noise")
        for name in unit_interval:
            if not 0 <= getattr(self, name) < 1:
                return f"{name} must be in [0, 1)"
        for name in ("norm_eps", "rope_theta"):
            if getattr(self, name) <= 0:
                return f"{name} must be positive"
        for name in ("router_aux_loss_coef", "router_z_loss_coef"):
            if getattr(self, name) < 0:
                return f"{name} must be non-negative"
        if self.ffn_type not in ("dense", "moe"):
            return "ffn_type must be either 'dense' or 'moe'"
        if self.hidden_size % self.n_heads:
            return "hidden_size must be divisible by n_heads"
        if not 1 <= self.experts_per_token <= self.num_experts:
            return "experts_per_token must be in [1, num_experts]"
        if self.expert_capacity_factor is not None and self.expert_capacity_factor <= 0:
            return "expert_capacity_factor must be positive or null"
        return None

    @property
    def head_dim(self) -> int:
        return self.hidden_size // self.n_heads

    @property
    def is_moe(self) -> bool:
        return self.ffn_type == "moe"

    @classmethod
    def field_names(cls) -> tuple[str, ...]:
        return tuple(f.name for f in fields(cls))
