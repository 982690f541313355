"""A plain, slow implementation of the Gadopel decoder, one function per mechanism, on the CPU.

It shares no code with the engine: it reads ``config.json``'s dictionary and a name -> tensor
mapping directly and works on whole sequences with dense matrices (no cache, no pages, no
batching).  Everything is computed in ``dtype`` (float64 by default) from the stored values.

Notation.  ``x`` [T, W] is the residual stream of one sequence, positions 0..T-1.

* layer:    ``x <- x + mix(LN1(x)) + ff(LN2(x))`` (both branches read the same ``x``)
* LN:       ``(x - mean) / sqrt(var + eps) * w``, biased variance
* looping:  layers ``start..stop-1`` run ``times`` times; in front of every pass
            ``x <- W_in [x ; x0]`` with ``x0`` the token embeddings
* head:     ``logits = W_head LN_final(x)``
"""
from __future__ import annotations

import math
from typing import Dict, List, Mapping, Optional

import torch


def unit_rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)


def layer_norm(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    mu = x.mean(dim=-1, keepdim=True)
    var = ((x - mu) ** 2).mean(dim=-1, keepdim=True)
    return (x - mu) / torch.sqrt(var + eps) * w


def rotary_frequencies(dims: int, base: float, scaling: Optional[Mapping] = None):
    """(frequencies [dims / 2], magnitude): plain ``base^(-2i/dims)``, or blended between the plain
    and the ``factor``-times slower frequency by a linear ramp over the pair index (YaRN), with the
    rotation's cos and sin scaled by ``0.1 ln(factor) + 1``."""
    f = [base ** (-2.0 * i / dims) for i in range(dims // 2)]
    if not scaling:
        return f, 1.0
    factor, orig = float(scaling["factor"]), float(scaling["original"])

    def turn_index(turns: float) -> float:
        return dims * math.log(orig / (2.0 * math.pi * turns)) / (2.0 * math.log(base))

    lo = max(math.floor(turn_index(float(scaling["fast"]))), 0)
    hi = min(math.ceil(turn_index(float(scaling["slow"]))), dims - 1)
    out = []
    for i, fi in enumerate(f):
        ramp = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
        out.append(fi / factor * ramp + fi * (1.0 - ramp))
    return out, 0.1 * math.log(factor) + 1.0


def rotate(x: torch.Tensor, positions: torch.Tensor, freqs: List[float], magnitude: float,
           interleaved: bool) -> torch.Tensor:
    """Rotates the first ``2 len(freqs)`` elements of the last axis of ``x`` [T, ..., d]; pair i is
    (2i, 2i + 1) when ``interleaved`` and (i, i + n) otherwise."""
    n = len(freqs)
    ang = positions.to(x.dtype)[:, None] * torch.tensor(freqs, dtype=x.dtype)[None, :]
    cos, sin = torch.cos(ang) * magnitude, torch.sin(ang) * magnitude
    while cos.dim() < x.dim():
        cos, sin = cos.unsqueeze(1), sin.unsqueeze(1)
    out = x.clone()
    if interleaved:
        u, v = x[..., 0:2 * n:2], x[..., 1:2 * n:2]
        out[..., 0:2 * n:2] = u * cos - v * sin
        out[..., 1:2 * n:2] = v * cos + u * sin
    else:
        u, v = x[..., :n], x[..., n:2 * n]
        out[..., :n] = u * cos - v * sin
        out[..., n:2 * n] = v * cos + u * sin
    return out


def visible(T: int, window: int = 0, keep_first: int = 0) -> torch.Tensor:
    """[T, T] bool: query i sees key j when j <= i and (no window, or i - j < window, or j < keep_first)."""
    i = torch.arange(T)[:, None]
    j = torch.arange(T)[None, :]
    ok = j <= i
    if window > 0:
        ok = ok & ((i - j < window) | (j < keep_first))
    return ok


def softmax_rows(scores: torch.Tensor, mask: torch.Tensor, sink: Optional[torch.Tensor] = None) -> torch.Tensor:
    """scores [H, T, T]; masked keys weigh nothing; ``sink`` [H] adds exp(sink) to each denominator."""
    s = scores.masked_fill(~mask[None], float("-inf"))
    m = s.max(dim=-1, keepdim=True).values
    if sink is not None:
        m = torch.maximum(m, sink[:, None, None])
    e = torch.exp(s - m)
    den = e.sum(dim=-1, keepdim=True)
    if sink is not None:
        den = den + torch.exp(sink[:, None, None] - m)
    return e / den


def latent_attention(h: torch.Tensor, w: Mapping[str, torch.Tensor], p: str, mc: Mapping, eps: float) -> torch.Tensor:
    T = h.shape[0]
    H, d, r, dv, rank = mc["heads"], mc["dim"], mc["rot_dim"], mc["vdim"], mc["kv_rank"]
    pos = torch.arange(T)
    freqs, mag = rotary_frequencies(mc["rot"]["dims"], mc["rot"]["base"], mc["rot"].get("scaling"))
    q = (h @ w[p + "q"].T).view(T, H, d + r)
    q_plain, q_rot = q[..., :d], rotate(q[..., d:], pos, freqs, mag, interleaved=False)
    down = h @ w[p + "dkv"].T
    c = unit_rms(down[:, :rank], eps) * w[p + "dkv.norm"]
    k_rot = rotate(down[:, rank:], pos, freqs, mag, interleaved=False)          # one for all heads
    k_plain = (c @ w[p + "uk"].T).view(T, H, d)
    v = (c @ w[p + "uv"].T).view(T, H, dv)
    scores = (torch.einsum("ihd,jhd->hij", q_plain, k_plain) + torch.einsum("ihd,jd->hij", q_rot, k_rot)) * mc["scale"]
    prob = softmax_rows(scores, visible(T), w[p + "sink"])
    out = torch.einsum("hij,jhd->ihd", prob, v)
    gate = torch.sigmoid(h @ w[p + "g"].T)                                       # [T, H]
    return (out * gate[..., None]).reshape(T, H * dv) @ w[p + "o"].T


def windowed_attention(h: torch.Tensor, w: Mapping[str, torch.Tensor], p: str, mc: Mapping, eps: float) -> torch.Tensor:
    T = h.shape[0]
    H, G, d, dv = mc["heads"], mc["kv_heads"], mc["dim"], mc["vdim"]
    pos = torch.arange(T)
    freqs, mag = rotary_frequencies(mc["rot"]["dims"], mc["rot"]["base"], mc["rot"].get("scaling"))
    q = unit_rms(rotate((h @ w[p + "q"].T).view(T, H, d), pos, freqs, mag, interleaved=True), eps)
    k = unit_rms(rotate((h @ w[p + "k"].T).view(T, G, d), pos, freqs, mag, interleaved=True), eps)
    v = (h @ w[p + "v"].T).view(T, G, dv)
    k = k.repeat_interleave(H // G, dim=1)
    v = v.repeat_interleave(H // G, dim=1)
    scores = torch.einsum("ihd,jhd->hij", q, k) * mc["scale"]
    mask_cfg = mc.get("mask") or {}
    prob = softmax_rows(scores, visible(T, int(mask_cfg.get("size", 0)), int(mask_cfg.get("keep_first", 0))))
    return torch.einsum("hij,jhd->ihd", prob, v).reshape(T, H * dv) @ w[p + "o"].T


def dense_relu_glu(h: torch.Tensor, w: Mapping[str, torch.Tensor], p: str) -> torch.Tensor:
    return (torch.relu(h @ w[p + "gate"].T) * (h @ w[p + "up"].T)) @ w[p + "down"].T


MIXERS = {"latent_attention": latent_attention, "attention": windowed_attention}


def run_order(cfg: Mapping) -> List[tuple]:
    """[(layer index, True when a new pass starts in front of it)]"""
    n = len(cfg["layers"])
    loop = cfg.get("loop")
    if not loop:
        return [(i, False) for i in range(n)]
    a, b, times = loop["start"], loop["stop"], loop["times"]
    order = [(i, False) for i in range(a)]
    for _ in range(times):
        order += [(i, i == a) for i in range(a, b)]
    return order + [(i, False) for i in range(b, n)]


def forward(cfg: Mapping, weights: Mapping[str, torch.Tensor], tokens, dtype=torch.float64,
            residuals: Optional[list] = None) -> torch.Tensor:
    """Logits [T, vocab] of one whole sequence; ``residuals`` collects the stream after every layer run."""
    w: Dict[str, torch.Tensor] = {k: (v.to(dtype) if v.is_floating_point() else v) for k, v in weights.items()}
    eps = cfg["norm"]["eps"]
    x0 = w["embed"][torch.as_tensor(tokens, dtype=torch.long)]
    x = x0
    for i, new_pass in run_order(cfg):
        if new_pass:
            x = torch.cat([x, x0], dim=-1) @ w["loop.in"].T
        layer, p = cfg["layers"][i], f"l{i}."
        branch = MIXERS[layer["type"]](layer_norm(x, w[p + "norm1"], eps), w, p + "mix.", layer["mixer"], eps)
        if layer.get("mlp"):
            branch = branch + dense_relu_glu(layer_norm(x, w[p + "norm2"], eps), w, p + "mlp.")
        x = x + branch
        if residuals is not None:
            residuals.append(x)
    return layer_norm(x, w["final.norm"], eps) @ w["head"].T
