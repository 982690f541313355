"""A plain, slow implementation of the Radilix decoder: one function per mechanism, whole
sequences, dense matrices, float64, token-by-token recurrences.  It shares no code with the engine.

Notation: ``x`` is the residual stream ``[T, W]``, ``h`` a normed copy of it, ``W_*`` matrices
stored ``[out, in]``.  A layer is ``x <- x + m (mixer(h) + ff(h))`` with ``h = norm(x)``: one norm,
both branches read it.  Mixers: ``gla`` (a linear-attention state with a decay per key channel),
``parallel`` (softmax attention beside a gated delta rule, added with two constants).  The
feed-forward is a mixture of experts whose last router outputs stand for identity experts.
"""
import math
from typing import Dict, List, Optional

import torch

F = torch.float64


def rms_norm_offset(x, w, eps):
    """x / sqrt(mean(x^2) + eps) * (1 + w): the weight is stored around zero."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * (1.0 + w)


def rms_norm_plain(x, w, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * w


def silu(z):
    return z * torch.sigmoid(z)


def gelu_erf(z):
    return 0.5 * z * (1.0 + torch.erf(z / math.sqrt(2.0)))


def rotate_first_dims(x, positions, dims, base):
    """x [T, heads, d]; the first ``dims`` elements of every head are rotated, element i with
    element i + dims/2, by the angle position * base^(-2i/dims); the rest pass."""
    half = dims // 2
    i = torch.arange(half, dtype=F)
    freq = torch.pow(torch.tensor(float(base), dtype=F), -2.0 * i / dims)
    ang = positions.to(F)[:, None] * freq[None, :]
    c, s = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
    u, v = x[..., :half], x[..., half:dims]
    return torch.cat([u * c - v * s, v * c + u * s, x[..., dims:]], dim=-1)


def _same(t):
    return t


def softmax_attention(W: Dict[str, torch.Tensor], p: str, m: dict, h, positions, rounded=_same):
    """Causal grouped-query softmax attention with biases on q, k, v, a rotation of the first
    ``rot.dims`` elements and a sigmoid gate on the concatenated heads."""
    T = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = (rounded(h @ W[p + "q"].T) + W[p + "q.b"]).view(T, H, d)
    k = (rounded(h @ W[p + "k"].T) + W[p + "k.b"]).view(T, G, d)
    v = rounded(rounded(h @ W[p + "v"].T) + W[p + "v.b"]).view(T, G, dv)
    q = rounded(rotate_first_dims(q, positions, m["rot"]["dims"], m["rot"]["base"]))
    k = rounded(rotate_first_dims(k, positions, m["rot"]["dims"], m["rot"]["base"]))
    out = torch.zeros(T, H, dv, dtype=F)
    causal = positions[:, None] >= positions[None, :]
    for head in range(H):
        g = head // (H // G)
        score = (q[:, head] @ k[:, g].T) * m["scale"]
        score = score.masked_fill(~causal, float("-inf"))
        out[:, head] = torch.softmax(score, dim=-1) @ v[:, g]
    gate = torch.sigmoid(rounded(h @ W[p + "g"].T))
    return rounded(rounded(out).reshape(T, H * dv) * gate) @ W[p + "o"].T


def causal_conv_silu(x, w):
    """x [T, C], w [C, taps]: y_t = silu(sum_j w[:, j] x_(t - taps + 1 + j)), zeros before the start."""
    T, C = x.shape
    taps = w.shape[1]
    padded = torch.cat([torch.zeros(taps - 1, C, dtype=F), x], dim=0)
    y = torch.zeros(T, C, dtype=F)
    for j in range(taps):
        y = y + padded[j:j + T] * w[:, j][None, :]
    return silu(y)


def delta_rule_recurrence(q, k, v, beta, decay):
    """q, k [T, d] (already unit vectors, q scaled), v [T, dv], beta, decay [T]: per token
    S <- decay S; u = beta (v - S^T k); S <- S + k u^T; o = S^T q, from S = 0.  Returns o [T, dv] and S."""
    T, d = q.shape
    S = torch.zeros(d, v.shape[1], dtype=F)
    out = torch.zeros(T, v.shape[1], dtype=F)
    for t in range(T):
        S = decay[t] * S
        u = beta[t] * (v[t] - S.T @ k[t])
        S = S + torch.outer(k[t], u)
        out[t] = S.T @ q[t]
    return out, S


def unit_vectors(x, eps=1e-6):
    return x / torch.sqrt((x * x).sum(-1, keepdim=True) + eps)


def gated_delta_rule(W: Dict[str, torch.Tensor], p: str, m: dict, h, eps, rounded=_same):
    """Short convolutions with silu on q, k, v; unit-norm q (times d^-1/2) and k; a step size
    beta = sigmoid(.) and a decay exp(-exp(A_log) softplus(. + dt_bias)) per head; the recurrence; every
    head's read-out divided by its root mean square, times a weight, times silu(gate); output matrix."""
    T = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = causal_conv_silu(rounded(h @ W[p + "q"].T), W[p + "q.conv"]).view(T, G, d)
    k = causal_conv_silu(rounded(h @ W[p + "k"].T), W[p + "k.conv"]).view(T, G, d)
    v = causal_conv_silu(rounded(h @ W[p + "v"].T), W[p + "v.conv"]).view(T, H, dv)
    q = unit_vectors(q) * d ** -0.5
    k = unit_vectors(k)
    beta = torch.sigmoid(rounded(h @ W[p + "b"].T))                                   # [T, H]
    decay = torch.exp(-torch.exp(W[p + "A_log"]) * torch.nn.functional.softplus(rounded(h @ W[p + "a"].T) + W[p + "dt_bias"]))
    out = torch.zeros(T, H, dv, dtype=F)
    for head in range(H):
        g = head // (H // G)
        out[:, head], _ = delta_rule_recurrence(q[:, g], k[:, g], v[:, head], beta[:, head], decay[:, head])
    out = out / torch.sqrt((out * out).mean(-1, keepdim=True) + eps) * W[p + "norm"]
    out = out.reshape(T, H * dv) * silu(rounded(h @ W[p + "g"].T))
    return rounded(out) @ W[p + "o"].T


def parallel_mixer(W, p, m, h, positions, eps, rounded=_same):
    left = softmax_attention(W, p + "left.", m["left"], h, positions, rounded)
    right = gated_delta_rule(W, p + "right.", m["right"], h, eps, rounded)
    return m["left_scale"] * left + m["right_scale"] * right


def decayed_outer_recurrence(q, k, v, alpha):
    """q, k, alpha [T, d], v [T, dv]: S_t = diag(alpha_t) S_(t-1) + k_t v_t^T, o_t = S_t^T q_t from S = 0."""
    T, d = q.shape
    S = torch.zeros(d, v.shape[1], dtype=F)
    out = torch.zeros(T, v.shape[1], dtype=F)
    for t in range(T):
        S = alpha[t][:, None] * S + torch.outer(k[t], v[t])
        out[t] = S.T @ q[t]
    return out, S


def gla_mixer(W: Dict[str, torch.Tensor], p: str, m: dict, h, eps, rounded=_same):
    """Gated linear attention: alpha = sigmoid(z)^(1/tau) per key channel, z a low-rank projection with a bias."""
    T = h.shape[0]
    H, d, dv = m["heads"], m["dim"], m["vdim"]
    q = rounded(h @ W[p + "q"].T).view(T, H, d) * d ** -0.5
    k = rounded(h @ W[p + "k"].T).view(T, H, d)
    v = rounded(h @ W[p + "v"].T).view(T, H, dv)
    z = rounded(h @ W[p + "a1"].T) @ W[p + "a2"].T + W[p + "a2.b"]
    alpha = torch.exp(torch.nn.functional.logsigmoid(z) / m["tau"]).view(T, H, d)
    out = torch.zeros(T, H, dv, dtype=F)
    for head in range(H):
        out[:, head], _ = decayed_outer_recurrence(q[:, head], k[:, head], v[:, head], alpha[:, head])
    out = rms_norm_plain(out, W[p + "norm"], eps).reshape(T, H * dv)
    return rounded(out * silu(rounded(h @ W[p + "g"].T))) @ W[p + "o"].T


def route(logits, correction, top):
    """scores = softmax(logits); the ``top`` largest of scores + correction are chosen (of equal ones
    the lowest index first).  Returns scores, the choice [T, top] and, per token, the margin between
    the last chosen and the best left-out choice score (inf when nothing is left out)."""
    s = torch.softmax(logits, dim=-1)
    choice = s + correction if correction is not None else s
    order = torch.sort(choice, dim=-1, descending=True, stable=True).indices
    chosen = order[:, :top]
    if top < choice.shape[1]:
        margin = choice.gather(1, order[:, top - 1:top]) - choice.gather(1, order[:, top:top + 1])
        margin = margin[:, 0]
    else:
        margin = torch.full((logits.shape[0],), float("inf"), dtype=F)
    return s, chosen, margin


def mixture_of_experts(W: Dict[str, torch.Tensor], p: str, mlp: dict, h, forced=None, margins: Optional[list] = None):
    """``forced`` [T, top]: experts to use instead of the router's own choice (their weights are still
    this router's scores).  ``margins`` collects (choice, margin) of the router's own choice."""
    r = mlp["router"]
    E, top = r["experts"], r["top"]
    s, chosen, margin = route(h @ W[p + "router"].T, W.get(p + "correction"), top)
    if margins is not None:
        margins.append((chosen, margin))
    if forced is not None:
        chosen = forced
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for e in chosen[t].tolist():
            y = h[t] if e >= E else gelu_erf(h[t] @ W[f"{p}e{e}.up"].T) @ W[f"{p}e{e}.down"].T
            out[t] = out[t] + s[t, e] * y
    return out


def layer_prefix(cfg: dict, i: int) -> str:
    j = cfg["layers"][i].get("weights_of")
    return f"l{i if j is None else j}."


def forward(cfg: dict, W: Dict[str, torch.Tensor], tokens: List[int], layers_out: Optional[list] = None,
            forced: Optional[dict] = None, margins: Optional[dict] = None, rounded=None):
    """Logits [T, vocab] (float64) of one sequence from position 0.  ``W`` holds float64 tensors.
    ``layers_out`` collects the stream after every layer; ``forced`` {layer: [T, top]} replaces routers'
    choices; ``margins`` {layer: (choice, margin)} collects the routers' own.  ``rounded`` (a function on
    tensors) is applied to every norm's output, the mixers' projections and every branch's output: with a rounding to a
    shorter format it shows how far such rounding moves the logits at each position."""
    rounded = rounded or (lambda t: t)
    eps, mult = cfg["norm"]["eps"], cfg["residual_mult"]
    positions = torch.arange(len(tokens))
    x = W["embed"][torch.tensor(tokens)]
    for i, layer in enumerate(cfg["layers"]):
        p = layer_prefix(cfg, i)
        h = rounded(rms_norm_offset(x, W[p + "norm1"], eps))
        if layer["type"] == "gla":
            a = gla_mixer(W, p + "mix.", layer["mixer"], h, eps, rounded)
        elif layer["type"] == "parallel":
            a = parallel_mixer(W, p + "mix.", layer["mixer"], h, positions, eps, rounded)
        else:
            raise ValueError(layer["type"])
        f = 0.0
        if layer.get("mlp"):
            got = []
            f = mixture_of_experts(W, p + "mlp.", layer["mlp"], h, None if forced is None else forced.get(i), got)
            if margins is not None:
                margins[i] = got[0]
        x = x + mult * (rounded(a) + (rounded(f) if layer.get("mlp") else 0.0))
        if layers_out is not None:
            layers_out.append(x.clone())
    return rounded(rms_norm_offset(x, W["final.norm"], eps)) @ W["head"].T


def to_f64(tensors: Dict[str, torch.Tensor]) -> Dict[str, torch.Tensor]:
    return {k: (v.to(F) if v.is_floating_point() else v) for k, v in tensors.items()}
