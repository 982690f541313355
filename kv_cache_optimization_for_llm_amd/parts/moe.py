"""A routed feed-forward: every token is sent to ``top`` of ``experts`` small feed-forward layers
``W_down act(W_up x)`` and takes the weighted sum of what they return.

Router: ``scores = softmax(W_router x)`` in fp32 over all router outputs.  The ``top`` outputs with
the largest ``scores + correction`` (a stored vector that shifts the choice but not the weights)
are chosen; their weights are the plain scores (``renormalise``: divided by their sum).  The last
``identity`` router outputs stand for experts that return their input: they have no tensors.

Everything from the router's logits to the sum stays on the device (``csrc/moe.hip``): the chosen
(token, choice) slots are sorted by expert into tiles of 16 rows, one kernel runs the first
product of every tile with its activation, a second the other product times the slot's weight,
and a third adds a token's rows up - no count of tokens per expert reaches the host, so a step
with this layer can be captured into a graph.  The experts' matrices are stacked at load time
(``[experts, ff, hidden]`` and ``[experts, hidden, ff]``).
"""
from __future__ import annotations

from typing import Dict, Optional

import torch

from ..config.registry import FEED_FORWARDS
from ..models.spec import TensorSpec
from ..ops import kernels as K
from .base import FeedForward, MixerContext


@FEED_FORWARDS.register("routed_experts")
class RoutedExperts(FeedForward):
    graph_safe = True
    # a function ``(part, idx [T, top] on the device)`` called after every routing of an eager step:
    # for whoever wants to see which experts the tokens were sent to (tests do); None: nothing is called
    on_route = None

    def __init__(self, prefix: str, *, hidden_size: int, intermediate_size: int, experts: int, top: int,
                 identity: int = 0, activation: str = "gelu", correction: bool = True, renormalise: bool = False,
                 tensor_names: Optional[Dict[str, str]] = None):
        """``tensor_names`` maps ``router``, ``correction``, ``up``, ``down`` to names behind ``prefix``;
        the experts' names hold ``{e}`` for the expert's number."""
        super().__init__(prefix)
        self.hidden_size, self.intermediate_size = int(hidden_size), int(intermediate_size)
        self.experts, self.top, self.identity = int(experts), int(top), int(identity)
        if self.experts < 0 or self.identity < 0 or not 0 < self.top <= self.experts + self.identity:
            raise ValueError(f"{prefix}: top {top} of {experts} experts and {identity} identity experts")
        if activation not in K.EXPERT_ACTIVATIONS:
            raise ValueError(f"activation {activation!r} is not one of {sorted(K.EXPERT_ACTIVATIONS)}")
        self.activation, self.has_correction, self.renormalise = activation, bool(correction), bool(renormalise)
        names = dict(router="router", correction="correction", up="e{e}.up", down="e{e}.down")
        names.update(tensor_names or {})
        self.names = {key: prefix + name for key, name in names.items()}
        self.outputs = self.experts + self.identity

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        n, W, I = self.names, self.hidden_size, self.intermediate_size
        specs = {n["router"]: TensorSpec((self.outputs, W))}
        if self.has_correction:
            specs[n["correction"]] = TensorSpec((self.outputs,), init="zeros", role="vector")
        for e in range(self.experts):
            specs[n["up"].format(e=e)] = TensorSpec((I, W))
            specs[n["down"].format(e=e)] = TensorSpec((W, I))
        return specs

    def load(self, tensors: Dict[str, torch.Tensor]) -> None:
        n = self.names
        self.router = tensors[n["router"]].contiguous()             # its logits are formed in 32-bit (ops.kernels.small_product_f32)
        self.correction = tensors[n["correction"]].float().contiguous() if self.has_correction else None
        if self.experts:
            self.w_up = torch.stack([tensors[n["up"].format(e=e)] for e in range(self.experts)]).contiguous()
            self.w_down = torch.stack([tensors[n["down"].format(e=e)] for e in range(self.experts)]).contiguous()
        else:
            self.w_up = self.w_down = None

    def activation_elements(self) -> int:
        return self.outputs + self.top * (2 * self.intermediate_size + 2 * self.hidden_size) + self.hidden_size

    def forward(self, x, ctx: MixerContext, tail=None):
        T, dev = x.shape[0], x.device
        logits = K.small_product_f32(x, self.router, torch.empty((T, self.outputs), dtype=torch.float32, device=dev))
        idx = torch.empty((T, self.top), dtype=torch.int32, device=dev)
        wgt = torch.empty((T, self.top), dtype=torch.float32, device=dev)
        K.moe_route(logits, self.correction, self.top, idx, wgt, self.renormalise)
        if RoutedExperts.on_route is not None and not torch.cuda.is_current_stream_capturing():
            RoutedExperts.on_route(self, idx)
        slots = T * self.top
        rows = torch.empty((slots, self.hidden_size), dtype=torch.float32, device=dev)
        if self.experts:
            tiles = K.moe_tiles(slots, self.experts)
            sorted_slot = torch.empty(tiles * K.MOE_TILE, dtype=torch.int32, device=dev)
            tile_expert = torch.empty(tiles, dtype=torch.int32, device=dev)
            K.moe_align(idx, self.experts, sorted_slot, tile_expert)
            act = torch.empty((tiles * K.MOE_TILE, self.intermediate_size), dtype=x.dtype, device=dev)
            K.moe_expert_rows(x, self.w_up, act, sorted_slot, tile_expert, self.top, activation=self.activation)
            K.moe_expert_rows(act, self.w_down, rows, sorted_slot, tile_expert, self.top, slot_weight=wgt)
        out = torch.empty_like(x)
        return K.moe_combine(x, rows, idx, wgt, self.experts, out)
