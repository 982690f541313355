"""The Radilix decoder as data: its ``config.json`` -> ModelSpec.

A decoder over a residual stream kept in 32-bit whose layers have ONE norm (RMS, the weight
stored around zero: ``x / rms(x) * (1 + w)``) that both branches read, and whose branches enter the
stream times a constant: ``h += m (mixer(n(h)) + ffn(n(h)))``.  A layer's mixer is

* ``gla``: gated linear attention - a state per head with a decay per key channel; or
* ``parallel``: two mixers side by side on the same input, added with two constants - grouped-query
  softmax attention with biases, a rotate-half rotation of a head's first elements and a sigmoid
  output gate (``left``), and a gated delta rule with short convolutions (``right``).

Its feed-forward is a mixture of experts (erf-gelu experts without biases, a softmax router
with a correction of the choice, identity experts at the end of the router's outputs), or
absent.  A layer may run with another layer's weights (``weights_of``) over a cache and state of
its own.  The model's norm at the end, then the output matrix ``head``.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Mapping, Optional, Tuple

from ..config.model_config import ConfigError
from ..config.registry import register_architecture
from .gadopel import _need
from .spec import LayerCall, LayerSpec, ModelSpec, PartSpec

LAYER_TYPES = ("gla", "parallel")
FEED_FORWARD_KINDS = ("moe",)


def _heads(m: Mapping[str, Any], where: str, kv: bool) -> None:
    for key in ("heads", "dim", "vdim"):
        if _need(m, key, where) <= 0:
            raise ConfigError(f"config.json: {where}.{key} must be positive")
    if kv:
        g = _need(m, "kv_heads", where)
        if g <= 0 or m["heads"] % g:
            raise ConfigError(f"config.json: {where}: {m['heads']} heads is not a multiple of {g} kv heads")


def _check_mixer(kind: str, m: Mapping[str, Any], where: str) -> None:
    if kind == "gla":
        _heads(m, where, kv=False)
        if _need(m, "tau", where, float) <= 0:
            raise ConfigError(f"config.json: {where}.tau must be positive")
        return
    left, right = m.get("left"), m.get("right")
    _heads(left, where + ".left", kv=True)
    _need(left, "scale", where + ".left", float)
    rot = left.get("rot")
    if rot is not None:
        dims = _need(rot, "dims", where + ".left.rot")
        _need(rot, "base", where + ".left.rot", float)
        if dims % 2 or not 0 <= dims <= left["dim"]:
            raise ConfigError(f"config.json: {where}.left.rot.dims {dims} must be even and at most dim {left['dim']}")
    if left["dim"] % 4:
        raise ConfigError(f"config.json: {where}.left.dim {left['dim']} must be a multiple of 4 (keys lie in the "
                          "cache in chunks of 4 or 8 elements)")
    _heads(right, where + ".right", kv=True)
    if not 1 <= _need(right, "conv", where + ".right") <= 17:
        raise ConfigError(f"config.json: {where}.right.conv must lie in 1..17")
    _need(m, "left_scale", where, float)
    _need(m, "right_scale", where, float)


def _check_mlp(mlp: Mapping[str, Any], where: str) -> None:
    if mlp.get("kind") not in FEED_FORWARD_KINDS:
        raise ConfigError(f"config.json: {where}.kind must be one of {FEED_FORWARD_KINDS}")
    _need(mlp.get("expert"), "ff", where + ".expert")
    r = mlp.get("router")
    experts, top = _need(r, "experts", where + ".router"), _need(r, "top", where + ".router")
    identity = int(r.get("identity", 0) or 0)
    if experts < 0 or identity < 0 or not 0 < top <= experts + identity:
        raise ConfigError(f"config.json: {where}.router: top {top} of {experts} experts and {identity} identity experts")


@dataclass(frozen=True)
class RadilixConfig:
    """``config.json`` of a Radilix model, checked: ``vocab``, ``width``, ``norm.eps``, ``residual_mult``
    and ``layers`` (per layer ``type``, ``mixer``, ``mlp`` or null, optionally ``weights_of``)."""

    vocab: int
    width: int
    norm_eps: float
    residual_mult: float
    layers: Tuple[Mapping[str, Any], ...]
    max_positions: int

    @staticmethod
    def from_dict(d: Mapping[str, Any]) -> "RadilixConfig":
        vocab, width = _need(d, "vocab", "the model"), _need(d, "width", "the model")
        eps = _need(d.get("norm"), "eps", "norm", float)
        layers = d.get("layers")
        if not isinstance(layers, (list, tuple)) or not layers:
            raise ConfigError("config.json: 'layers' must be a non-empty list")
        for i, layer in enumerate(layers):
            where = f"layers[{i}]"
            if not isinstance(layer, Mapping) or layer.get("type") not in LAYER_TYPES:
                raise ConfigError(f"config.json: {where}.type must be one of {LAYER_TYPES}")
            _check_mixer(layer["type"], layer.get("mixer"), where + ".mixer")
            if layer.get("mlp") is not None:
                _check_mlp(layer["mlp"], where + ".mlp")
            j = layer.get("weights_of")
            if j is not None:
                if isinstance(j, bool) or not isinstance(j, int) or not 0 <= j < len(layers) or j == i \
                        or layers[j].get("weights_of") is not None:
                    raise ConfigError(f"config.json: {where}.weights_of must name another layer that has weights of its own")
                if layers[j]["type"] != layer["type"] or layers[j].get("mixer") != layer.get("mixer") \
                        or layers[j].get("mlp") != layer.get("mlp"):
                    raise ConfigError(f"config.json: {where} uses the weights of layer {j} but is of another make")
        return RadilixConfig(vocab=vocab, width=width, norm_eps=eps,
                             residual_mult=float(d.get("residual_mult", 1.0)), layers=tuple(layers),
                             max_positions=int(d.get("max_positions", 1 << 17)))


def _norm(prefix: str, name: str, width: int, eps: float) -> PartSpec:
    return PartSpec("layernorm", dict(prefix=prefix, width=width, eps=eps, weight_name=name, center=False,
                                      weight_offset=1.0))


def _mixer(kind: str, m: Mapping[str, Any], p: str, W: int, eps: float, max_positions: int) -> PartSpec:
    if kind == "gla":
        return PartSpec("gated_linear_attention", dict(
            prefix=p, hidden_size=W, num_heads=int(m["heads"]), head_dim=int(m["dim"]), value_dim=int(m["vdim"]),
            tau=float(m["tau"]), norm_eps=eps, decay_rank=m.get("decay_rank")))
    left, right = m["left"], m["right"]
    rot = left.get("rot")
    if rot is not None and int(rot["dims"]) > 0:
        position = PartSpec("rotary", dict(head_dim=int(left["dim"]), rotary_dim=int(rot["dims"]),
                                           max_positions=max_positions, theta=float(rot["base"]),
                                           frequencies="plain_f64", pairing="half"))
    else:
        position = PartSpec("none")
    attention = PartSpec("gated_gqa_attention", dict(
        prefix=p + "left.", hidden_size=W, num_heads=int(left["heads"]), num_kv_heads=int(left["kv_heads"]),
        head_dim=int(left["dim"]), value_dim=int(left["vdim"]), scale=float(left["scale"]), position=position,
        bias=True, gate="sigmoid"))
    delta = PartSpec("gated_delta_rule", dict(
        prefix=p + "right.", hidden_size=W, num_heads=int(right["heads"]), num_kv_heads=int(right["kv_heads"]),
        head_dim=int(right["dim"]), value_dim=int(right["vdim"]), conv_taps=int(right["conv"]), norm_eps=eps))
    return PartSpec("side_by_side", dict(prefix=p, hidden_size=W, children=(attention, delta),
                                         scales=(float(m["left_scale"]), float(m["right_scale"]))))


def radilix_spec(cfg: RadilixConfig) -> ModelSpec:
    W, eps = cfg.width, cfg.norm_eps
    layers, index_of, order = [], {}, []
    for i, layer in enumerate(cfg.layers):
        if layer.get("weights_of") is not None:
            continue
        p = f"l{i}."
        mlp = layer.get("mlp")
        if mlp is not None:
            r = mlp["router"]
            ffn = PartSpec("routed_experts", dict(
                prefix=p + "mlp.", hidden_size=W, intermediate_size=int(mlp["expert"]["ff"]), experts=int(r["experts"]),
                top=int(r["top"]), identity=int(r.get("identity", 0) or 0), activation="gelu", correction=True))
        else:
            ffn = PartSpec("none")
        index_of[i] = len(layers)
        layers.append(LayerSpec(
            block=PartSpec("parallel", dict(shared_norm=True, residual_mult=cfg.residual_mult)),
            mixer=_mixer(layer["type"], layer["mixer"], p + "mix.", W, eps, cfg.max_positions), feed_forward=ffn,
            norms={"mixer": _norm(p, "norm1", W, eps)}, prefix=p))
    # every layer of the list is one call with a cache and state slot of its own, whoever's weights it runs with
    for i, layer in enumerate(cfg.layers):
        j = layer.get("weights_of")
        order.append(LayerCall(layer=index_of[i if j is None else j], cache=i))
    return ModelSpec(
        architecture="Radilix", hidden_size=W, vocab_size=cfg.vocab, embedding_name="embed",
        layers=tuple(layers), order=tuple(order), final_norm=_norm("final.", "norm", W, eps),
        final_norm_prefix="final.", head_name="head", max_positions=cfg.max_positions, residual_dtype="float32")


register_architecture("Radilix", RadilixConfig.from_dict, radilix_spec, replace=True)
