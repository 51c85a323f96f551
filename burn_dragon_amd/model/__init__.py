from .attention import Attention
from .bdh import BDH, DecodeGraph
from .config import BDHConfig, FusedKernelConfig
from .state import LayerState, LayerVizState, ModelState

__all__ = ["Attention", "BDH", "DecodeGraph", "BDHConfig", "FusedKernelConfig", "LayerState", "LayerVizState", "ModelState"]
