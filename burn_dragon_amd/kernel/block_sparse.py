"""Block patterns (reference: src/kernel/block_sparse.rs:11-133)."""
from __future__ import annotations

from dataclasses import dataclass
from typing import FrozenSet, Iterable, List, Optional, Tuple


@dataclass(frozen=True)
class BlockPattern1d:
    """Latent-axis block mask (src/kernel/block_sparse.rs:11-63)."""

    block_size: int
    active_blocks: Optional[FrozenSet[int]] = None

    @classmethod
    def dense(cls, block_size: int) -> "BlockPattern1d":
        return cls(max(block_size, 1), None)

    @classmethod
    def from_blocks(cls, block_size: int, blocks: Iterable[int]) -> "BlockPattern1d":
        return cls(block_size, frozenset(blocks))

    def is_sparse(self) -> bool:
        return self.active_blocks is not None

    def is_block_active(self, block_idx: int) -> bool:
        return True if self.active_blocks is None else block_idx in self.active_blocks

    def block_bytes(self, elements: int) -> bytes:
        """One byte per latent block: the form the C ABI takes."""
        size = max(self.block_size, 1)
        total = -(-elements // size)
        return bytes(1 if self.is_block_active(i) else 0 for i in range(total))


@dataclass(frozen=True)
class BlockPattern2d:
    """Time-block pair pattern (src/kernel/block_sparse.rs:66-117); dense = col <= row."""

    block_size: int
    active_pairs: Optional[FrozenSet[Tuple[int, int]]] = None

    @classmethod
    def dense(cls, block_size: int) -> "BlockPattern2d":
        return cls(max(block_size, 1), None)

    @classmethod
    def from_pairs(cls, block_size: int, pairs: Iterable[Tuple[int, int]]) -> "BlockPattern2d":
        return cls(block_size, frozenset(pairs))

    def is_sparse(self) -> bool:
        return self.active_pairs is not None

    def is_active(self, row: int, col: int) -> bool:
        return col <= row if self.active_pairs is None else (row, col) in self.active_pairs

    def iter_cols(self, row: int, total_blocks: int) -> List[int]:
        if self.active_pairs is None:
            return list(range(0, min(row, max(total_blocks - 1, 0)) + 1)) if total_blocks > 0 else []
        return sorted(c for (r, c) in self.active_pairs if r == row and c < total_blocks)


@dataclass(frozen=True)
class BlockSparseConfig:
    latent: BlockPattern1d
    time: BlockPattern2d

    @classmethod
    def dense(cls, latent_block: int, time_block: int) -> "BlockSparseConfig":
        return cls(BlockPattern1d.dense(latent_block), BlockPattern2d.dense(time_block))
