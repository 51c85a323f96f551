"""BDHConfig / FusedKernelConfig (reference: src/model/config.rs:10-164)."""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import List, Optional

from ..kernel.block_sparse import BlockPattern1d, BlockPattern2d, BlockSparseConfig
from ..positional import RotaryEmbedding


@dataclass
class FusedKernelConfig:
    """src/model/config.rs:10-31 (defaults :20-31)."""

    enabled: bool = False
    block_sparse: BlockSparseConfig = field(default_factory=lambda: BlockSparseConfig.dense(64, 64))
    rope_theta: float = 65_536.0
    relu_threshold: float = 0.0
    alibi_slopes: Optional[List[float]] = None
    rotary_embedding: RotaryEmbedding = RotaryEmbedding.ALIBI

    def set_block_sizes(self, latent: int, time: int) -> None:
        self.block_sparse = BlockSparseConfig(BlockPattern1d.dense(latent), BlockPattern2d.dense(time))

    def with_block_sizes(self, latent: int, time: int) -> "FusedKernelConfig":
        self.set_block_sizes(latent, time)
        return self

    def set_alibi_slopes(self, slopes: List[float]) -> None:
        self.alibi_slopes = list(slopes)

    def set_rotary_embedding(self, rotary_embedding: RotaryEmbedding) -> None:
        self.rotary_embedding = RotaryEmbedding.parse(rotary_embedding)


@dataclass
class BDHConfig:
    """src/model/config.rs:113-164 (defaults :125-137)."""

    n_layer: int = 6
    n_embd: int = 256
    dropout: float = 0.1
    n_head: int = 4
    mlp_internal_dim_multiplier: int = 4
    n_expert: int = 1
    vocab_size: int = 256
    fused_kernels: FusedKernelConfig = field(default_factory=FusedKernelConfig)

    def latent_per_head(self) -> int:
        total = self.mlp_internal_dim_multiplier * self.n_embd
        assert total % self.n_head == 0, "latent size must be divisible by the number of heads"
        latent_per_head = total // self.n_head
        assert latent_per_head % self.n_expert == 0, (
            f"latent per head {latent_per_head} must be divisible by experts {self.n_expert}")
        return latent_per_head

    def latent_total(self) -> int:
        return self.latent_per_head() * self.n_head

    def latent_per_expert(self) -> int:
        return self.latent_per_head() // self.n_expert
