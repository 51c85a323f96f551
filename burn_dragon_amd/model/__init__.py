from .bdh import BDH
from .config import BDHConfig, FusedKernelConfig
from .state import LayerState, ModelState

__all__ = ["BDH", "BDHConfig", "FusedKernelConfig", "LayerState", "ModelState"]
