"""Host-side mirror of the reference's `kernel` module (src/kernel/mod.rs)."""
from . import block_sparse, linear_attention, relu_lowrank
from .block_sparse import BlockPattern1d, BlockPattern2d, BlockSparseConfig

__all__ = ["block_sparse", "linear_attention", "relu_lowrank", "BlockPattern1d", "BlockPattern2d",
           "BlockSparseConfig"]
