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


def softmax_attention(W: Dict[str, torch.Tensor], p: str, m: dict, h, positions):
    """Causal grouped-query softmax attention with biases on q, k, v, a rotation of the first
    ``rot.dims`` elements and a sigmoid gate on the concatenated heads."""
    T = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = (h @ W[p + "q"].T + W[p + "q.b"]).view(T, H, d)
    k = (h @ W[p + "k"].T + W[p + "k.b"]).view(T, G, d)
    v = (h @ W[p + "v"].T + W[p + "v.b"]).view(T, G, dv)
    q = rotate_first_dims(q, positions, m["rot"]["dims"], m["rot"]["base"])
    k = rotate_first_dims(k, positions, m["rot"]["dims"], m["rot"]["base"])
    out = torch.zeros(T, H, dv, dtype=F)
    causal = positions[:, None] >= positions[None, :]
    for head in range(H):
        g = head // (H // G)
        score = (q[:, head] @ k[:, g].T) * m["scale"]
        score = score.masked_fill(~causal, float("-inf"))
        out[:, head] = torch.softmax(score, dim=-1) @ v[:, g]
    gate = torch.sigmoid(h @ W[p + "g"].T)
    return (out.reshape(T, H * dv) * gate) @ W[p + "o"].T


def causal_conv_silu(x, w):
    """x [T, C], w [C, taps]: y_t = silu(sum_j w[:, j] x_(t - taps + 1 + j)), zeros before the start."""
    T, C = x.shape
    taps = w.shape[1]
    padded = torch.cat([torch.zeros(taps - 1, C, dtype=F), x], dim=0)
    y = torch.zeros(T, C, dtype=F)
    for j in range(taps):
        y = y + padded[j:j + T] * w[:, j][None, :]
    return silu(y)


def gated_delta_rule(W: Dict[str, torch.Tensor], p: str, m: dict, h, eps):
    """Per head: S <- g S; u = beta (v - S^T k); S <- S + k u^T; o = S^T q."""
    T = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = causal_conv_silu(h @ W[p + "q"].T, W[p + "q.conv"]).view(T, G, d)
    k = causal_conv_silu(h @ W[p + "k"].T, W[p + "k.conv"]).view(T, G, d)
    v = causal_conv_silu(h @ W[p + "v"].T, W[p + "v.conv"]).view(T, H, dv)
    q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * d ** -0.5
    k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    beta = torch.sigmoid(h @ W[p + "b"].T)                                            # [T, H]
    decay = torch.exp(-torch.exp(W[p + "A_log"]) * torch.nn.functional.softplus(h @ W[p + "a"].T + W[p + "dt_bias"]))
    out = torch.zeros(T, H, dv, dtype=F)
    for head in range(H):
        g = head // (H // G)
        S = torch.zeros(d, dv, dtype=F)
        for t in range(T):
            S = decay[t, head] * S
            u = beta[t, head] * (v[t, head] - S.T @ k[t, g])
            S = S + torch.outer(k[t, g], u)
            out[t, head] = S.T @ q[t, g]
    out = out / torch.sqrt((out * out).mean(-1, keepdim=True) + eps) * W[p + "norm"]
    out = out.reshape(T, H * dv) * silu(h @ W[p + "g"].T)
    return out @ W[p + "o"].T


def parallel_mixer(W, p, m, h, positions, eps):
    left = softmax_attention(W, p + "left.", m["left"], h, positions)
    right = gated_delta_rule(W, p + "right.", m["right"], h, eps)
    return m["left_scale"] * left + m["right_scale"] * right


def gla_mixer(W: Dict[str, torch.Tensor], p: str, m: dict, h, eps):
    """S_t = diag(alpha_t) S_(t-1) + k_t v_t^T, o_t = S_t^T q_t, alpha = sigmoid(z)^(1/tau)."""
    T = h.shape[0]
    H, d, dv = m["heads"], m["dim"], m["vdim"]
    q = (h @ W[p + "q"].T).view(T, H, d) * d ** -0.5
    k = (h @ W[p + "k"].T).view(T, H, d)
    v = (h @ W[p + "v"].T).view(T, H, dv)
    z = (h @ W[p + "a1"].T) @ W[p + "a2"].T + W[p + "a2.b"]
    alpha = torch.exp(torch.nn.functional.logsigmoid(z) / m["tau"]).view(T, H, d)
    out = torch.zeros(T, H, dv, dtype=F)
    for head in range(H):
        S = torch.zeros(d, dv, dtype=F)
        for t in range(T):
            S = alpha[t, head][:, None] * S + torch.outer(k[t, head], v[t, head])
            out[t, head] = S.T @ q[t, head]
    out = rms_norm_plain(out, W[p + "norm"], eps).reshape(T, H * dv)
    return (out * silu(h @ W[p + "g"].T)) @ W[p + "o"].T


def mixture_of_experts(W: Dict[str, torch.Tensor], p: str, mlp: dict, h):
    r = mlp["router"]
    E, I, top = r["experts"], r.get("identity", 0), r["top"]
    s = torch.softmax(h @ W[p + "router"].T, dim=-1)                                  # [T, E + I]
    choice = s + W[p + "correction"] if (p + "correction") in W else s
    chosen = torch.topk(choice, top, dim=-1).indices
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for e in chosen[t].tolist():
            y = h[t] if e >= E else gelu_erf(h[t] @ W[f"{p}e{e}.up"].T) @ W[f"{p}e{e}.down"].T
            out[t] = out[t] + s[t, e] * y
    return out


def layer_prefix(cfg: dict, i: int) -> str:
    j = cfg["layers"][i].get("weights_of")
    return f"l{i if j is None else j}."


def forward(cfg: dict, W: Dict[str, torch.Tensor], tokens: List[int], layers_out: Optional[list] = None):
    """Logits [T, vocab] (float64) of one sequence from position 0.  ``W`` holds float64 tensors.
    ``layers_out`` collects the stream after every layer."""
    eps, mult = cfg["norm"]["eps"], cfg["residual_mult"]
    positions = torch.arange(len(tokens))
    x = W["embed"][torch.tensor(tokens)]
    for i, layer in enumerate(cfg["layers"]):
        p = layer_prefix(cfg, i)
        h = rms_norm_offset(x, W[p + "norm1"], eps)
        if layer["type"] == "gla":
            a = gla_mixer(W, p + "mix.", layer["mixer"], h, eps)
        elif layer["type"] == "parallel":
            a = parallel_mixer(W, p + "mix.", layer["mixer"], h, positions, eps)
        else:
            raise ValueError(layer["type"])
        f = mixture_of_experts(W, p + "mlp.", layer["mlp"], h) if layer.get("mlp") else 0.0
        x = x + mult * (a + f)
        if layers_out is not None:
            layers_out.append(x.clone())
    return rms_norm_offset(x, W["final.norm"], eps) @ W["head"].T


def to_f64(tensors: Dict[str, torch.Tensor]) -> Dict[str, torch.Tensor]:
    return {k: (v.to(F) if v.is_floating_point() else v) for k, v in tensors.items()}
