"""LayerState / ModelState (reference: src/model/state.rs:5-57)."""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import List, Optional

import torch


@dataclass
class LayerVizState:
    """src/model/state.rs:17-24 (the reference's "viz" feature): [h,N] maps of the first sequence's last
    token, and the energy map of the layer's state."""

    x_last: torch.Tensor
    y_last: torch.Tensor
    xy_last: torch.Tensor
    rho_last: torch.Tensor


@dataclass
class LayerState:
    rho: Optional[torch.Tensor] = None  # [B,h,Nq,d]
    viz: Optional[LayerVizState] = None  # filled by BDH.forward_with_state(..., viz=True)

    def take_viz(self) -> Optional[LayerVizState]:
        """src/model/state.rs:76-80."""
        viz, self.viz = self.viz, None
        return viz


@dataclass
class ModelState:
    layers: List[LayerState] = field(default_factory=list)
    position: int = 0
    # all layers share one allocation [L,B,h,Nq,d]; layers[i].rho are views into it
    storage: Optional[torch.Tensor] = None
    # ALiBi with lazy decay only: [L,B,h,N] int32, the token count at which each state row was last brought
    # up to date (see BDH(alibi_lazy=True)); None for an eagerly decayed state
    stamps: Optional[torch.Tensor] = None
    # a model built with defer_updates only: the update logs of its layers (BDH.flush_state applies them)
    logs: Optional[object] = None

    @classmethod
    def new(cls, num_layers: int) -> "ModelState":
        return cls(layers=[LayerState() for _ in range(num_layers)], position=0)

    def reset(self) -> None:
        for layer in self.layers:
            layer.rho = None
        self.storage = None
        self.stamps = None
        self.logs = None
        self.position = 0

    def len(self) -> int:
        return self.position

    def __len__(self) -> int:
        return self.position

    def is_empty(self) -> bool:
        return self.position == 0

    def take_viz(self) -> List[Optional[LayerVizState]]:
        """src/model/state.rs:59-65."""
        return [layer.take_viz() for layer in self.layers]

    def clear_viz(self) -> None:
        """src/model/state.rs:67-72."""
        for layer in self.layers:
            layer.viz = None

    def trim(self, max_len: int) -> None:
        """A no-op, as in the reference (src/model/state.rs:55-57)."""
        _ = max_len
