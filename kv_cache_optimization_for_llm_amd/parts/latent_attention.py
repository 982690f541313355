"""Attention over a low-rank key/value entry (latent attention).

Per token the cache holds ONE row for all heads: a latent vector ``c`` of ``rank`` elements (the
down-projected input, RMS-normed with a weight) and a rotated key part ``k_r`` of ``rot_dim``
elements that every head shares.  Head ``h`` has an unrotated key ``U_k[h] c``, a value
``U_v[h] c`` and a query ``[q_p[h] ; q_r[h]]`` (``dim`` unrotated and ``rot_dim`` rotated
elements):

    score_h(i, j) = (q_p[h]_i . U_k[h] c_j + q_r[h]_i . k_r_j) * scale
    out_h(i)      = sum_j p_h(i, j) U_v[h] c_j

Keys and values are never expanded.  The key expansion moves to the query side,
``q_p . U_k c = (U_k^T q_p) . c``, so a head's query becomes a row ``[U_k[h]^T q_p[h] ; q_r[h]]`` of
the cache's own layout and every head attends over the same rows (one shared "kv head" of
``rank + rot_dim`` elements whose first ``rank`` are also the value); the value expansion moves
behind the attention, ``sum_j p U_v c_j = U_v (sum_j p c_j)``.  What a step costs per cached token
is then independent of the number of heads' key and value sizes, and a prompt cut anywhere
continues from the rows alone.

Options: a softmax sink per head (``exp(sink_h)`` added to the denominator; no key, no value,
not scaled), a sigmoid output gate per head read from the mixer's input, a window with kept first
positions.  Softmax, the latent's norm and the rotation are fp32.
"""
from __future__ import annotations

from typing import Dict, Optional

import torch

from ..config.registry import MIXERS, POSITION_ENCODINGS
from ..models.spec import PartSpec, TensorSpec
from ..ops import kernels as K
from ..ops import latent_attention as lat_ops
from .base import CacheArray, KVCacheSpec, Mixer, MixerContext, NormedRows
from .linear import Linear


def latent_cache_spec(rank: int, rot_dim: int, kind: str = "full", window: int = 0, keep_first: int = 0,
                      transposed: bool = False) -> KVCacheSpec:
    """One row ``[latent (rank) ; rotated key part (rot_dim)]`` per token, pages ``[page_size, rank +
    rot_dim]``; with ``transposed`` the latent a second time in pages ``[rank, page_size]``, the
    layout in which the matrix-core kernel reads it as the values' operand."""
    arrays = (CacheArray("latent", (int(rank) + int(rot_dim),), token_axis=0),)
    if transposed:
        arrays += (CacheArray(lat_ops.TRANSPOSED, (int(rank),), token_axis=1),)
    return KVCacheSpec(arrays, kind, int(window), int(keep_first) if kind == "window" else 0)


@MIXERS.register("latent_attention")
class LatentAttention(Mixer):
    graph_safe = True

    def __init__(self, prefix: str, *, hidden_size: int, num_heads: int, head_dim: int, rot_dim: int,
                 value_dim: int, rank: int, scale: float, norm_eps: float, position: PartSpec, sink: bool = False,
                 gate: bool = False, window: int = 0, keep_first: int = 0,
                 tensor_names: Optional[Dict[str, str]] = None):
        """``head_dim``: unrotated query/key elements per head; ``rot_dim``: rotated ones (the
        ``position`` encoding must rotate exactly these); ``rank``: size of the latent.
        ``tensor_names`` maps ``q``, ``down``, ``down_norm``, ``up_k``, ``up_v``, ``sink``, ``gate``,
        ``o`` to the tensors' names behind ``prefix``."""
        super().__init__(prefix)
        self.hidden_size, self.num_heads, self.head_dim = int(hidden_size), int(num_heads), int(head_dim)
        self.rot_dim, self.value_dim, self.rank = int(rot_dim), int(value_dim), int(rank)
        self.scale, self.norm_eps = float(scale), float(norm_eps)
        self.has_sink, self.has_gate = bool(sink), bool(gate)
        self.window = int(window)
        self.keep_first = int(keep_first) if self.window > 0 else 0
        names = dict(q="q_proj.weight", down="kv_down.weight", down_norm="kv_norm.weight", up_k="k_up.weight",
                     up_v="v_up.weight", sink="sinks", gate="gate.weight", o="o_proj.weight")
        names.update(tensor_names or {})
        self.names = {key: prefix + name for key, name in names.items()}
        self.position = POSITION_ENCODINGS.get(position.kind)(**position.params)
        if getattr(self.position, "rotary_dim", None) != self.rot_dim or getattr(self.position, "unit_norm_eps", None) is not None:
            raise ValueError("latent attention needs a rotary encoding over exactly its rot_dim elements")
        self.key_dim = self.rank + self.rot_dim
        self.proj: Optional[Linear] = None          # [q ; down ; gate] joined
        self.o: Optional[Linear] = None
        self.up_k_t = self.up_v = self.norm_weight = self.sinks = None

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        n, H, W = self.names, self.num_heads, self.hidden_size
        specs = {
            n["q"]: TensorSpec((H * (self.head_dim + self.rot_dim), W)),
            n["down"]: TensorSpec((self.key_dim, W)),
            n["down_norm"]: TensorSpec((self.rank,), init="norm", role="vector"),
            n["up_k"]: TensorSpec((H * self.head_dim, self.rank)),
            n["up_v"]: TensorSpec((H * self.value_dim, self.rank)),
            n["o"]: TensorSpec((W, H * self.value_dim)),
        }
        if self.has_sink:
            specs[n["sink"]] = TensorSpec((H,), init="normal", role="vector")
        if self.has_gate:
            specs[n["gate"]] = TensorSpec((H, W))
        return specs

    def load(self, tensors: Dict[str, torch.Tensor]) -> None:
        n, H = self.names, self.num_heads
        mats = [tensors[n["q"]], tensors[n["down"]]] + ([tensors[n["gate"]]] if self.has_gate else [])
        if len({m.dtype for m in mats}) != 1:
            raise ValueError(f"{self.prefix}: the input projections are stored in different dtypes")
        self.proj = Linear(torch.cat(mats, dim=0))
        self.kv_off = H * (self.head_dim + self.rot_dim)
        self.gate_off = self.kv_off + self.key_dim
        self.o = Linear(tensors[n["o"]])
        # U_k per head, transposed: the query-side product reads [heads, rank, dim]
        self.up_k_t = tensors[n["up_k"]].view(H, self.head_dim, self.rank).transpose(1, 2).contiguous()
        self.up_v = tensors[n["up_v"]].view(H, self.value_dim, self.rank).contiguous()
        self.norm_weight = tensors[n["down_norm"]].contiguous()
        self.sinks = tensors[n["sink"]].to(torch.float32).contiguous() if self.has_sink else None

    def kv_cache_spec(self) -> KVCacheSpec:
        # a bf16 model at sizes the matrix-core kernel has an instance for keeps the transposed copy
        # it reads (asked after load(): the weights' type is the compute type)
        fast = self.proj is not None and self.proj.weight.dtype == torch.bfloat16 and self.proj.weight.is_cuda \
            and lat_ops.mfma_supported(self.rank, self.key_dim)
        return latent_cache_spec(self.rank, self.rot_dim, kind="window" if self.window > 0 else "full",
                                 window=self.window, keep_first=self.keep_first, transposed=fast)

    def activation_elements(self) -> int:
        H = self.num_heads
        return (self.proj.out_features if self.proj is not None else 0) + H * (self.key_dim + self.rank + self.value_dim) \
            + self.hidden_size

    def forward(self, x, ctx: MixerContext, tail=None):
        if isinstance(x, NormedRows):
            x = x.materialize()
        batch, kv = ctx.batch, ctx.kv
        if kv is None:
            raise K.KernelError("latent attention: the mixer has no cache view")
        T, H = x.shape[0], self.num_heads
        y = self.proj(x)                                                    # [T, q | entry | gates]
        q_lat = torch.empty((T, H, self.key_dim), dtype=x.dtype, device=x.device)
        cos, sin = self.position.tables(x.device)
        write = kv.writes
        K.latent_encode_cache(y, self.kv_off, q_lat, kv.arrays["latent"] if write else None, self.norm_weight,
                              self.norm_eps, cos, sin, batch.positions, kv.slot_mapping if write else None, H,
                              self.head_dim, self.rank, interleaved=self.position.pairing == "interleaved",
                              cache_t=kv.arrays.get(lat_ops.TRANSPOSED) if write else None)
        # the key expansion on the query side: q_lat[:, h, :rank] = U_k[h]^T q_p[h]
        q_plain = y[:, :self.kv_off].view(T, H, self.head_dim + self.rot_dim)[:, :, :self.head_dim]
        lat_ops.heads_product(q_plain, self.up_k_t, q_lat[:, :, :self.rank])
        o_lat = torch.empty((T, H, self.rank), dtype=x.dtype, device=x.device)
        lat_ops.latent_attention(q_lat, o_lat, kv, batch, self.scale, self.window, self.keep_first, self.sinks)
        out = torch.empty((T, H * self.value_dim), dtype=x.dtype, device=x.device)
        # the value expansion behind the attention, the head's output gate in the same pass
        lat_ops.heads_product(o_lat, self.up_v, out.view(T, H, self.value_dim),
                              gates=y[:, self.gate_off:self.gate_off + H] if self.has_gate else None)
        return self.o(out)
