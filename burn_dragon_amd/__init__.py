"""burn_dragon_amd — the BDH cached-inference hot path of mosure/burn_dragon on MI355X.

The package is a thin host-side mirror of the reference's interface for that path
(`kernel`, `model`, `positional`, `inference`, `generation`, `tokenizer`, `record`) over the C ABI of libbdh_mi355x.so
(include/bdh_mi355x.h).  All computation happens in hand-written HIP kernels; there is
no CPU or framework fallback.
"""
from . import ffi
from .inference import ModelOverrides, build_model_config
from .kernel import BlockPattern1d, BlockPattern2d, BlockSparseConfig
from .model import BDH, BDHConfig, FusedKernelConfig, LayerState, ModelState
from .positional import RotaryEmbedding
from .tokenizer import ByteTokenizer, CharVocab, Tokenizer

__all__ = ["ffi", "ModelOverrides", "build_model_config", "BlockPattern1d", "BlockPattern2d", "BlockSparseConfig",
           "BDH", "BDHConfig", "FusedKernelConfig", "LayerState", "ModelState", "RotaryEmbedding",
           "ByteTokenizer", "CharVocab", "Tokenizer"]
