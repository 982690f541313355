"""Operations on the residual stream between layers (a model's run order may name one in front of
a layer call).  ``forward(hidden, pending, first) -> hidden``: ``pending`` are branch outputs not
yet added to the stream, ``first`` is the stream as the embedding left it."""
from __future__ import annotations

from typing import Dict, Optional

import torch

from ..config.registry import STREAM_OPS
from ..models.spec import TensorSpec
from ..ops import kernels as K
from .base import Part
from .linear import Linear


@STREAM_OPS.register("reinject")
class Reinject(Part):
    """``h <- W [h ; h0]``: the stream joined with the embedding output and projected back to its
    width (``W`` is ``[width, 2 width]``, the stream's columns first).  The product takes the
    weights' type; its result goes into the stream in the stream's type."""

    graph_safe = True

    def __init__(self, prefix: str = "", *, width: int, weight_name: str = "weight"):
        super().__init__(prefix)
        self.width = int(width)
        self.weight_name = prefix + weight_name
        self.linear: Optional[Linear] = None

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        return {self.weight_name: TensorSpec((self.width, 2 * self.width))}

    def load(self, tensors: Dict[str, torch.Tensor]) -> None:
        self.linear = Linear(tensors[self.weight_name])

    def activation_elements(self) -> int:
        return 3 * self.width

    def forward(self, hidden: torch.Tensor, pending, first: torch.Tensor) -> torch.Tensor:
        joined = torch.empty((hidden.shape[0], 2 * self.width), dtype=self.linear.weight.dtype, device=hidden.device)
        K.stream_join(hidden, first, joined, deltas=pending)
        return self.linear(joined, out=hidden)
