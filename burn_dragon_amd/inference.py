"""build_model_config (reference: src/inference.rs:4-40; ModelOverrides: src/config/core.rs:43-53)."""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional

from .model.config import BDHConfig
from .positional import RotaryEmbedding


@dataclass
class ModelOverrides:
    n_layer: Optional[int] = None
    n_embd: Optional[int] = None
    n_head: Optional[int] = None
    mlp_internal_dim_multiplier: Optional[int] = None
    relu_threshold: Optional[float] = None
    dropout: Optional[float] = None
    fused_kernels: Optional[bool] = None
    block_size: Optional[int] = None
    rotary_embedding: Optional[RotaryEmbedding] = None


def build_model_config(overrides: ModelOverrides, training_block_size: int) -> BDHConfig:
    cfg = BDHConfig()
    if overrides.n_layer is not None:
        cfg.n_layer = overrides.n_layer
    if overrides.n_embd is not None:
        cfg.n_embd = overrides.n_embd
    if overrides.n_head is not None:
        cfg.n_head = overrides.n_head
    if overrides.mlp_internal_dim_multiplier is not None:
        cfg.mlp_internal_dim_multiplier = overrides.mlp_internal_dim_multiplier
    if overrides.relu_threshold is not None:
        cfg.fused_kernels.relu_threshold = overrides.relu_threshold
    if overrides.dropout is not None:
        cfg.dropout = overrides.dropout
    if overrides.fused_kernels is not None:
        cfg.fused_kernels.enabled = overrides.fused_kernels
    block = max(overrides.block_size if overrides.block_size is not None else training_block_size, 1)
    cfg.fused_kernels.set_block_sizes(block, block)  # always dense patterns (:28-32)
    if overrides.rotary_embedding is not None:
        cfg.fused_kernels.set_rotary_embedding(overrides.rotary_embedding)
    return cfg
