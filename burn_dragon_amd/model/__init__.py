from .bdh import BDH, DecodeGraph
from .config import BDHConfig, FusedKernelConfig
from .state import LayerState, ModelState

__all__ = ["BDH", "DecodeGraph", "BDHConfig", "FusedKernelConfig", "LayerState", "ModelState"]
