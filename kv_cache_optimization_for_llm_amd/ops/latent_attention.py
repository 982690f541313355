"""Kernel choice for attention over low-rank entries and for the per-head products around it."""
from __future__ import annotations

import torch

from . import kernels as K


def heads_product(x: torch.Tensor, w: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    """``out[t, h] = w[h] @ x[t, h]`` for ``w`` ``[heads, N, K]``; ``x`` and ``out`` may be views into
    wider buffers."""
    return K.heads_matmul(x, w, out)


def latent_attention(q_lat: torch.Tensor, out: torch.Tensor, kv, batch, scale: float, window: int = 0,
                     keep_first: int = 0, sinks=None) -> torch.Tensor:
    """Causal attention of the step's tokens over the rows of ``kv.arrays["latent"]``
    (``[pages, page_size, key_dim]``): ``q_lat`` ``[T, heads, key_dim]``, ``out`` ``[T, heads, rank]``."""
    if window <= 0:
        keep_first = 0
    return K.latent_attention_rowwise(q_lat, out, kv.arrays["latent"], kv.block_table, batch.tok_seat,
                                      batch.positions, scale, window, keep_first, sinks)
