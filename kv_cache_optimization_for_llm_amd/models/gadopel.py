"""The Gadopel decoder as data: its ``config.json`` -> ModelSpec.

A decoder whose layers are parallel blocks (both branches read the same layer-normed stream:
``h += mixer(LN_1(h)) + ffn(LN_2(h))``) over a residual stream kept in 32-bit.  A layer's mixer is
latent attention (one low-rank key/value row per token for all heads, rotate-half rotation of a
separate rotated part, a softmax sink and a sigmoid output gate per head) or grouped-query
attention with an interleaved, YaRN-scaled partial rotation, unit-RMS queries and keys, and a
sliding window that keeps a request's first positions; its feed-forward is gated with a ReLU, or
absent.  A run of layers may be repeated with the same weights (each pass has cache slots of its
own); in front of every pass the stream is joined with the embedding output and projected back
(``loop.in``).  Layer norm at the end, then the output matrix ``head``.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Mapping, Optional, Tuple

from ..config.model_config import ConfigError
from ..config.registry import register_architecture
from ..parts.rotary import yarn_magnitude
from .spec import LayerCall, LayerSpec, ModelSpec, PartSpec

MIXER_TYPES = ("latent_attention", "attention")
FEED_FORWARD_KINDS = ("dense",)


def _need(d: Mapping[str, Any], key: str, where: str, kind=int):
    if not isinstance(d, Mapping) or key not in d or d[key] is None:
        raise ConfigError(f"config.json: {where} needs '{key}'")
    v = d[key]
    if isinstance(v, bool) or not isinstance(v, (int, float) if kind is float else kind):
        raise ConfigError(f"config.json: {where}.{key} must be {'a number' if kind is float else kind.__name__}, got {v!r}")
    return kind(v)


@dataclass(frozen=True)
class GadopelConfig:
    """``config.json`` of a Gadopel model, checked: ``vocab``, ``width``, ``norm.eps``, ``layers``
    (per layer ``type``, ``mixer`` sizes and ``mlp`` or null) and the optional ``loop``
    (``start``, ``stop``, ``times``)."""

    vocab: int
    width: int
    norm_eps: float
    layers: Tuple[Mapping[str, Any], ...]
    loop: Optional[Tuple[int, int, int]]
    max_positions: int

    @staticmethod
    def from_dict(d: Mapping[str, Any]) -> "GadopelConfig":
        vocab, width = _need(d, "vocab", "the model"), _need(d, "width", "the model")
        eps = _need(d.get("norm"), "eps", "norm", float)
        layers = d.get("layers")
        if not isinstance(layers, (list, tuple)) or not layers:
            raise ConfigError("config.json: 'layers' must be a non-empty list")
        for i, layer in enumerate(layers):
            where = f"layers[{i}]"
            if not isinstance(layer, Mapping) or layer.get("type") not in MIXER_TYPES:
                raise ConfigError(f"config.json: {where}.type must be one of {MIXER_TYPES}")
            m = layer.get("mixer")
            for key in ("heads", "dim", "vdim"):
                _need(m, key, where + ".mixer")
            _need(m, "scale", where + ".mixer", float)
            rot = m.get("rot")
            _need(rot, "dims", where + ".mixer.rot")
            _need(rot, "base", where + ".mixer.rot", float)
            if rot["dims"] % 2:
                raise ConfigError(f"config.json: {where}.mixer.rot.dims must be even")
            if rot.get("scaling") is not None:
                for key in ("factor", "original", "fast", "slow"):
                    _need(rot["scaling"], key, where + ".mixer.rot.scaling", float)
            if layer["type"] == "latent_attention":
                for key in ("kv_rank", "rot_dim"):
                    _need(m, key, where + ".mixer")
                if rot["dims"] != m["rot_dim"]:
                    raise ConfigError(f"config.json: {where}: the rotation covers rot.dims = {rot['dims']} elements, "
                                      f"the rotated part has rot_dim = {m['rot_dim']}")
            else:
                g = _need(m, "kv_heads", where + ".mixer")
                if g <= 0 or m["heads"] % g:
                    raise ConfigError(f"config.json: {where}: {m['heads']} heads is not a multiple of {g} kv heads")
                if rot["dims"] > m["dim"]:
                    raise ConfigError(f"config.json: {where}: rot.dims {rot['dims']} exceeds dim {m['dim']}")
                if m["dim"] % 4:
                    raise ConfigError(f"config.json: {where}: dim {m['dim']} must be a multiple of 4 (keys lie in the "
                                      "cache in chunks of 4 or 8 elements)")
                if m.get("mask") is not None:
                    _need(m["mask"], "size", where + ".mixer.mask")
            mlp = layer.get("mlp")
            if mlp is not None:
                if mlp.get("kind", "dense") not in FEED_FORWARD_KINDS:
                    raise ConfigError(f"config.json: {where}.mlp.kind must be one of {FEED_FORWARD_KINDS}")
                _need(mlp, "ff", where + ".mlp")
        loop = d.get("loop")
        if loop is not None:
            a, b, n = (_need(loop, k, "loop") for k in ("start", "stop", "times"))
            if not (0 <= a < b <= len(layers)) or n < 1:
                raise ConfigError(f"config.json: loop {a}..{b} x {n} does not fit {len(layers)} layers")
            loop = (a, b, n)
        return GadopelConfig(vocab=vocab, width=width, norm_eps=eps, layers=tuple(layers), loop=loop,
                             max_positions=int(d.get("max_positions", 1 << 17)))


def _rotary(rot: Mapping[str, Any], head_dim: int, max_positions: int, **more) -> PartSpec:
    scaling = rot.get("scaling")
    params = dict(head_dim=head_dim, rotary_dim=int(rot["dims"]), max_positions=max_positions, theta=float(rot["base"]),
                  frequencies="plain_f64", **more)
    if scaling is not None:
        params.update(frequencies="yarn", magnitude=yarn_magnitude(scaling["factor"]),
                      frequency_params=dict(factor=float(scaling["factor"]), original=float(scaling["original"]),
                                            fast=float(scaling["fast"]), slow=float(scaling["slow"])))
    return PartSpec("rotary", params)


def gadopel_spec(cfg: GadopelConfig) -> ModelSpec:
    W, eps = cfg.width, cfg.norm_eps
    layers, ignorable = [], []
    for i, layer in enumerate(cfg.layers):
        p, m = f"l{i}.", layer["mixer"]
        if layer["type"] == "latent_attention":
            mixer = PartSpec("latent_attention", dict(
                prefix=p + "mix.", hidden_size=W, num_heads=int(m["heads"]), head_dim=int(m["dim"]),
                rot_dim=int(m["rot_dim"]), value_dim=int(m["vdim"]), rank=int(m["kv_rank"]), scale=float(m["scale"]),
                norm_eps=eps, sink=True, gate=True,
                position=_rotary(m["rot"], int(m["rot_dim"]), cfg.max_positions, pairing="half"),
                tensor_names=dict(q="q", down="dkv", down_norm="dkv.norm", up_k="uk", up_v="uv", sink="sink",
                                  gate="g", o="o")))
        else:
            mask = m.get("mask") or {}
            mixer = PartSpec("gqa_attention", dict(
                prefix=p + "mix.", hidden_size=W, num_heads=int(m["heads"]), num_kv_heads=int(m["kv_heads"]),
                head_dim=int(m["dim"]), value_dim=int(m["vdim"]), scale=float(m["scale"]),
                window=int(mask.get("size", 0)), keep_first=int(mask.get("keep_first", 0)),
                position=_rotary(m["rot"], int(m["dim"]), cfg.max_positions, pairing="interleaved", unit_norm_eps=eps),
                tensor_names=dict(q="q", k="k", v="v", o="o")))
        norms = {"mixer": PartSpec("layernorm", dict(prefix=p, width=W, eps=eps, weight_name="norm1"))}
        mlp = layer.get("mlp")
        if mlp is not None:
            ffn = PartSpec("gated", dict(prefix=p + "mlp.", hidden_size=W, intermediate_size=int(mlp["ff"]),
                                         activation="relu", tensor_names=dict(gate="gate", up="up", down="down")))
            norms["feed_forward"] = PartSpec("layernorm", dict(prefix=p, width=W, eps=eps, weight_name="norm2"))
        else:
            ffn = PartSpec("none")
            ignorable.append(p + "norm2")       # a layer without a feed-forward has nothing to normalise for it
        layers.append(LayerSpec(block=PartSpec("parallel"), mixer=mixer, feed_forward=ffn, norms=norms, prefix=p))
    # run order: layers before the loop, the looped run `times` times (each pass its own cache
    # slots, the stream re-joined with the embedding output in front of each), the rest
    n = len(layers)
    a, b, times = cfg.loop if cfg.loop is not None else (n, n, 0)
    order, slot = [], 0
    for i in range(a):
        order.append(LayerCall(layer=i, cache=slot))
        slot += 1
    for _ in range(times):
        for i in range(a, b):
            order.append(LayerCall(layer=i, cache=slot, before=0 if i == a else None))
            slot += 1
    for i in range(b, n):
        order.append(LayerCall(layer=i, cache=slot))
        slot += 1
    stream_ops = (PartSpec("reinject", dict(prefix="loop.", width=W, weight_name="in")),) if cfg.loop is not None else ()
    return ModelSpec(
        architecture="Gadopel", hidden_size=W, vocab_size=cfg.vocab, embedding_name="embed",
        layers=tuple(layers), order=tuple(order),
        final_norm=PartSpec("layernorm", dict(prefix="final.", width=W, eps=eps, weight_name="norm")),
        final_norm_prefix="final.", head_name="head", max_positions=cfg.max_positions,
        stream_ops=stream_ops, residual_dtype="float32", ignorable_tensors=tuple(ignorable))


register_architecture("Gadopel", GadopelConfig.from_dict, gadopel_spec, replace=True)
