"""The part of RustingBrain's ``TransformerLm`` builder surface that selects and
sizes the sparse layers (reference src/transformer.rs:60-227, :278-447).

Only the mixture-of-experts feed-forward of a block is built here; attention,
embeddings and the rest of the model are outside this package.  The builder
keeps the reference's method names — ``.experts(n, k)``, ``.moe_layers(..)``,
``.shared_expert(b)``, ``.moe_d_ff(f)``, ``.aux_loss_weight(w)``,
``.router_z_loss_weight(w)`` — validates like ``TransformerConfig::validate``
and hands out one ``MoeLayer`` per index in ``moe_layers``.
"""
from __future__ import annotations

from dataclasses import dataclass, field, replace
from typing import Dict, Iterable, List, Optional

from .moe import (DEFAULT_AUX_LOSS_WEIGHT, DEFAULT_ROUTER_Z_LOSS_WEIGHT, Device, InvalidConfig, MoeConfig,
                  MoeLayer)


@dataclass(frozen=True)
class ParameterCounts:
    total: int
    active: int


@dataclass(frozen=True)
class TransformerConfig:
    """Defaults are the reference's roughly 55M-total / 36M-active model
    (src/transformer.rs:100-126)."""
    vocab_size: int = 32_000
    d_model: int = 512
    n_layers: int = 8
    n_heads: int = 8
    n_kv_heads: int = 2
    head_dim: int = 64
    d_ff: int = 1408
    moe_d_ff: int = 352
    num_experts: int = 8
    experts_per_token: int = 2
    moe_layers: tuple = tuple(range(2, 8))
    shared_expert: bool = True
    max_seq_len: int = 2048
    tie_embeddings: bool = True
    aux_loss_weight: float = DEFAULT_AUX_LOSS_WEIGHT
    router_z_loss_weight: float = DEFAULT_ROUTER_Z_LOSS_WEIGHT

    def moe_config(self) -> MoeConfig:
        return MoeConfig(self.num_experts, self.experts_per_token, self.moe_d_ff, self.shared_expert,
                         self.aux_loss_weight, self.router_z_loss_weight)

    def is_moe_layer(self, layer: int) -> bool:
        return layer in self.moe_layers

    def validate(self) -> None:
        for name in ("vocab_size", "d_model", "n_layers", "n_heads", "n_kv_heads", "head_dim", "d_ff",
                     "max_seq_len"):
            if getattr(self, name) == 0:
                raise InvalidConfig(f"{name} must be non-zero")
        if self.n_heads % self.n_kv_heads != 0 or self.n_kv_heads > self.n_heads:
            raise InvalidConfig(f"n_heads ({self.n_heads}) must be a multiple of n_kv_heads ({self.n_kv_heads})")
        if self.head_dim % 2 != 0:
            raise InvalidConfig(f"head_dim must be even for rotary embeddings, got {self.head_dim}")
        for layer in self.moe_layers:
            if layer >= self.n_layers:
                raise InvalidConfig(f"moe_layers names layer {layer}, but the model has {self.n_layers} layers")
        if self.moe_layers:
            self.moe_config().validate()

    def parameter_counts(self) -> ParameterCounts:
        """src/transformer.rs:194-227."""
        query = self.d_model * self.n_heads * self.head_dim
        key_value = 2 * self.d_model * self.n_kv_heads * self.head_dim
        attention = 2 * query + key_value
        norms = 2 * self.d_model
        dense_ffn = 3 * self.d_model * self.d_ff
        expert = 3 * self.d_model * self.moe_d_ff
        shared = expert if self.shared_expert else 0
        router = self.num_experts * self.d_model
        moe_total = router + self.num_experts * expert + shared
        moe_active = router + self.experts_per_token * expert + shared
        total = self.vocab_size * self.d_model + self.d_model
        if not self.tie_embeddings:
            total += self.vocab_size * self.d_model
        active = total
        for layer in range(self.n_layers):
            total += attention + norms
            active += attention + norms
            if self.is_moe_layer(layer):
                total += moe_total
                active += moe_active
            else:
                total += dense_ffn
                active += dense_ffn
        return ParameterCounts(total, active)


class TransformerBuilder:
    def __init__(self) -> None:
        self._config = TransformerConfig()

    def config(self, config: TransformerConfig) -> "TransformerBuilder":
        self._config = config
        return self

    def _with(self, **kw) -> "TransformerBuilder":
        self._config = replace(self._config, **kw)
        return self

    def vocab_size(self, v: int): return self._with(vocab_size=v)
    def d_model(self, v: int): return self._with(d_model=v)
    def n_layers(self, v: int): return self._with(n_layers=v)
    def heads(self, n_heads: int, n_kv_heads: int, head_dim: int):
        return self._with(n_heads=n_heads, n_kv_heads=n_kv_heads, head_dim=head_dim)
    def d_ff(self, v: int): return self._with(d_ff=v)
    def moe_d_ff(self, v: int): return self._with(moe_d_ff=v)
    def experts(self, num_experts: int, experts_per_token: int):
        return self._with(num_experts=num_experts, experts_per_token=experts_per_token)
    def moe_layers(self, layers: Iterable[int]): return self._with(moe_layers=tuple(layers))
    def shared_expert(self, shared_expert: bool): return self._with(shared_expert=shared_expert)
    def max_seq_len(self, v: int): return self._with(max_seq_len=v)
    def tie_embeddings(self, v: bool): return self._with(tie_embeddings=v)
    def aux_loss_weight(self, w: float): return self._with(aux_loss_weight=w)
    def router_z_loss_weight(self, w: float): return self._with(router_z_loss_weight=w)

    def parameter_counts(self) -> ParameterCounts:
        return self._config.parameter_counts()

    def build_moe_layers(self, device: Device, *, act_dtype: str = "f32", weight_dtype: str = "f32",
                         max_tokens: Optional[int] = None) -> Dict[int, MoeLayer]:
        """Validates (before any allocation, as the reference does) and returns
        ``{layer index: MoeLayer}`` for every index in ``moe_layers``."""
        self._config.validate()
        cfg = self._config
        tokens = max_tokens if max_tokens is not None else cfg.max_seq_len
        return {i: MoeLayer(cfg.d_model, cfg.moe_config(), device, act_dtype=act_dtype,
                            weight_dtype=weight_dtype, max_tokens=tokens) for i in cfg.moe_layers}
