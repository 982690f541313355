"""Kernel choice for attention over low-rank entries and for the per-head products around it."""
from __future__ import annotations

import torch

from . import kernels as K


def heads_product(x: torch.Tensor, w: torch.Tensor, out: torch.Tensor, gates=None) -> torch.Tensor:
    """``out[t, h] = w[h] @ x[t, h]`` for ``w`` ``[heads, N, K]``; ``x`` and ``out`` may be views into
    wider buffers.  ``gates`` ``[T, heads]``: head h of row t times ``sigmoid(gates[t, h])``."""
    return K.heads_matmul(x, w, out, gates)


TRANSPOSED = "latent_t"         # name of the cache array that holds the latent part a second time, [rank, page_size]
_TARGET_WAVES = 1024            # wavefronts a launch should have before keys stop being cut into ranges
_MIN_KEYS_PER_RANGE = 128


def mfma_supported(rank: int, key_dim: int, page_size: int = 16) -> bool:
    """Whether the matrix-core kernel has an instance for these sizes (it then wants the transposed
    copy of the latent in the cache entry)."""
    return K.latent_attention_mfma_supported(rank, key_dim, page_size)


def choose_ranges(items: int, max_context: int, visible: int = 0) -> tuple:
    """(ranges, keys per range) for ``items`` work items over at most ``max_context`` keys: ranges
    of at least 128 keys until the launch has about four wavefronts a compute unit.  ``visible``
    > 0: a row sees at most so many keys (a window and the kept first positions), wherever they
    lie: the ranges are sized as if the context were that long, and most of them stay empty."""
    want = max(1, _TARGET_WAVES // max(1, items))
    span = min(max_context, visible) if visible > 0 else max_context
    ranges = max(1, min(want, span // _MIN_KEYS_PER_RANGE))
    if ranges == 1:
        return 1, 0
    per = (-(-span // ranges) + 31) // 32 * 32
    return -(-max_context // per), per


def latent_attention(q_lat: torch.Tensor, out: torch.Tensor, kv, batch, scale: float, window: int = 0,
                     keep_first: int = 0, sinks=None) -> torch.Tensor:
    """Causal attention of the step's tokens over the rows of ``kv.arrays["latent"]``
    (``[pages, page_size, key_dim]``): ``q_lat`` ``[T, heads, key_dim]``, ``out`` ``[T, heads, rank]``."""
    if window <= 0:
        keep_first = 0
    cache = kv.arrays["latent"]
    if q_lat.dtype == torch.bfloat16 and TRANSPOSED in kv.arrays \
            and mfma_supported(out.shape[2], q_lat.shape[2], cache.shape[1]):
        item_entry, item_row0, _ = batch.attention_items(q_lat.shape[1], 1, "all")
        ranges, per = choose_ranges(item_entry.shape[0], batch.max_context, window + keep_first if window > 0 else 0)
        return K.latent_attention_mfma(q_lat, out, cache, kv.arrays[TRANSPOSED], kv.block_table, item_entry, item_row0,
                                       batch.entry_seat, batch.entry_q_start, batch.entry_start_pos, scale, window,
                                       keep_first, sinks, ranges, per)
    return K.latent_attention_rowwise(q_lat, out, kv.arrays["latent"], kv.block_table, batch.tok_seat,
                                      batch.positions, scale, window, keep_first, sinks)
