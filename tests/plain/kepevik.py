"""A plain, slow implementation of the Kepevik decoder: whole sequences, no cache, no state carried
between calls, one function per mechanism, only ``torch`` tensor arithmetic.  It shares no code with
``torchllms_amd``; the tests compare the engine against it.

Conventions: one sequence at a time; activations are [S, ...]; ``weights`` maps the checkpoint's own
tensor names (``l3.mix.q``, ``l1.mix.left.k``, ``l2.mlp.e0.up``, ``final.norm`` ...) to tensors;
``config`` is the dictionary of config.json.  Everything is computed in the dtype the weights are
given in (the tests pass 32-bit or 64-bit copies), so the functions state the formulas and nothing
about rounding.
"""

from __future__ import annotations

import math
from typing import Dict, List, Optional

import torch


# ----------------------------------------------------------------------------- small functions
def gelu_erf(z: torch.Tensor) -> torch.Tensor:
    return 0.5 * z * (1.0 + torch.erf(z / math.sqrt(2.0)))


def silu(z: torch.Tensor) -> torch.Tensor:
    return z / (1.0 + torch.exp(-z))


def sigmoid(z: torch.Tensor) -> torch.Tensor:
    return 1.0 / (1.0 + torch.exp(-z))


def log_sigmoid(z: torch.Tensor) -> torch.Tensor:
    return torch.minimum(z, torch.zeros_like(z)) - torch.log1p(torch.exp(-z.abs()))


def softplus(z: torch.Tensor) -> torch.Tensor:
    return torch.clamp(z, min=0.0) + torch.log1p(torch.exp(-z.abs()))


def rms_unit(x: torch.Tensor, eps: float) -> torch.Tensor:
    """x over its root mean square along the last axis, eps under the root."""
    return x / torch.sqrt((x ** 2).mean(-1, keepdim=True) + eps)


def offset_norm(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    """RMS norm whose stored weight lies around zero: the factor is 1 + w."""
    return rms_unit(x, eps) * (1.0 + w)


def causal_conv(x: torch.Tensor, taps: torch.Tensor) -> torch.Tensor:
    """x [S, C]; taps [C, K]: the last column multiplies the current token, the one before it the
    previous token, and so on; inputs before the sequence's start are zero."""
    S, C = x.shape
    K = taps.shape[1]
    out = torch.zeros_like(x)
    for t in range(S):
        for j in range(K):
            src = t - (K - 1 - j)
            if src >= 0:
                out[t] += taps[:, j] * x[src]
    return out


def rotate_half_split(x: torch.Tensor, positions: torch.Tensor, dims: int, base: float) -> torch.Tensor:
    """x [S, heads, dim]: channel i of the first ``dims`` is paired with channel i + dims/2 and the pair is
    turned by the angle position * base^(-2i/dims); the channels behind ``dims`` pass unchanged."""
    if dims == 0:
        return x
    half = dims // 2
    freq = torch.tensor([base ** (-2.0 * i / dims) for i in range(half)], dtype=torch.float64)
    ang = positions.to(torch.float64)[:, None] * freq[None, :]
    c = torch.cos(ang).to(x.dtype)[:, None, :]
    s = torch.sin(ang).to(x.dtype)[:, None, :]
    a, b = x[..., :half], x[..., half:dims]
    return torch.cat([a * c - b * s, b * c + a * s, x[..., dims:]], dim=-1)


# ----------------------------------------------------------------------------- mixers
def matrix_memory(h: torch.Tensor, w: Dict[str, torch.Tensor], p: str, m: dict, eps: float) -> torch.Tensor:
    """The mLSTM cell with a matrix memory per head, written as the recurrence itself."""
    S = h.shape[0]
    H, dk, dv, cap = m["heads"], m["dim"], m["vdim"], float(m["gate_cap"])
    q = (h @ w[p + "q"].T).reshape(S, H, dk) * dk ** -0.5
    k = (h @ w[p + "k"].T).reshape(S, H, dk)
    v = (h @ w[p + "v"].T).reshape(S, H, dv)
    gi = cap * torch.tanh((h @ w[p + "i"].T + w[p + "i.b"]) / cap)
    gf = log_sigmoid(cap * torch.tanh((h @ w[p + "f"].T + w[p + "f.b"]) / cap))
    out = torch.zeros(S, H, dv, dtype=h.dtype)
    for a in range(H):
        C = torch.zeros(dk, dv, dtype=h.dtype)
        n = torch.zeros(dk, dtype=h.dtype)
        mx = torch.zeros((), dtype=h.dtype)
        for t in range(S):
            new = torch.maximum(gf[t, a] + mx, gi[t, a])
            keep = torch.exp(gf[t, a] + mx - new)
            take = torch.exp(gi[t, a] - new)
            C = keep * C + take * torch.outer(k[t, a], v[t, a])
            n = keep * n + take * k[t, a]
            mx = new
            den = torch.maximum((n @ q[t, a]).abs(), torch.exp(-mx)) + 1e-6
            out[t, a] = (C.T @ q[t, a]) / den
    out = rms_unit(out, eps).reshape(S, H * dv) * w[p + "norm"]
    out = out * sigmoid(h @ w[p + "g"].T)
    return out @ w[p + "o"].T


def softmax_branch(h: torch.Tensor, w: Dict[str, torch.Tensor], p: str, m: dict) -> torch.Tensor:
    """Causal attention whose values are the keys as projected (before the rotation)."""
    S = h.shape[0]
    H, G, dk = m["heads"], m["kv_heads"], m["dim"]
    pos = torch.arange(S)
    q = (h @ w[p + "q"].T).reshape(S, H, dk)
    k = (h @ w[p + "k"].T).reshape(S, G, dk)
    v = k.clone()
    q = rotate_half_split(q, pos, m["rot"]["dims"], float(m["rot"]["base"]))
    k = rotate_half_split(k, pos, m["rot"]["dims"], float(m["rot"]["base"]))
    out = torch.zeros(S, H, dk, dtype=h.dtype)
    for a in range(H):
        g = a // (H // G)
        for t in range(S):
            sc = (k[: t + 1, g] @ q[t, a]) * float(m["scale"])
            pr = torch.exp(sc - sc.max())
            pr = pr / pr.sum()
            out[t, a] = pr @ v[: t + 1, g]
    return out.reshape(S, H * dk) @ w[p + "o"].T


def delta_branch(h: torch.Tensor, w: Dict[str, torch.Tensor], p: str, m: dict, eps: float) -> torch.Tensor:
    """The gated delta rule with a decay for every key channel."""
    S = h.shape[0]
    H, G, dk, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = silu(causal_conv(h @ w[p + "q"].T, w[p + "q.conv"])).reshape(S, G, dk)
    k = silu(causal_conv(h @ w[p + "k"].T, w[p + "k.conv"])).reshape(S, G, dk)
    v = silu(causal_conv(h @ w[p + "v"].T, w[p + "v.conv"])).reshape(S, H, dv)
    q = q / torch.sqrt((q ** 2).sum(-1, keepdim=True) + 1e-6) * dk ** -0.5
    k = k / torch.sqrt((k ** 2).sum(-1, keepdim=True) + 1e-6)
    beta = sigmoid(h @ w[p + "b"].T)
    rate = torch.exp(w[p + "A_log"])[None, :, None]
    step = softplus(((h @ w[p + "a1"].T) @ w[p + "a2"].T + w[p + "dt_bias"]).reshape(S, H, dk))
    decay = torch.exp(-rate * step)
    out = torch.zeros(S, H, dv, dtype=h.dtype)
    for a in range(H):
        g = a // (H // G)
        M = torch.zeros(dk, dv, dtype=h.dtype)
        for t in range(S):
            M = decay[t, a][:, None] * M
            u = beta[t, a] * (v[t, a] - M.T @ k[t, g])
            M = M + torch.outer(k[t, g], u)
            out[t, a] = M.T @ q[t, g]
    out = rms_unit(out, eps) * w[p + "norm"]
    gate = sigmoid((h @ w[p + "g1"].T) @ w[p + "g2"].T).reshape(S, H, dv)
    return (out * gate).reshape(S, H * dv) @ w[p + "o"].T


def mixer(h, w, p, layer, eps):
    m = layer["mixer"]
    if layer["type"] == "mlstm":
        return matrix_memory(h, w, p, m, eps)
    if layer["type"] == "parallel":
        left = softmax_branch(h, w, p + "left.", m["left"])
        right = delta_branch(h, w, p + "right.", m["right"], eps)
        return float(m["left_scale"]) * left + float(m["right_scale"]) * right
    raise ValueError(layer["type"])


# ----------------------------------------------------------------------------- feed-forwards
def gated_expert(h, w, p):
    return (silu(h @ w[p + "gate"].T) * (h @ w[p + "up"].T)) @ w[p + "down"].T


def routed(h: torch.Tensor, w: Dict[str, torch.Tensor], p: str, mlp: dict) -> torch.Tensor:
    r = mlp["router"]
    E, ident, top = r["experts"], int(r.get("identity", 0) or 0), r["top"]
    z = h @ w[p + "router"].T
    s = torch.softmax(z, dim=-1)
    choice = s + w[p + "correction"]
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        chosen = torch.topk(choice[t], top).indices.tolist()
        for e in chosen:
            if e >= E:
                out[t] += s[t, e] * h[t]
            else:
                out[t] += s[t, e] * gated_expert(h[t : t + 1], w, f"{p}e{e}.")[0]
    if mlp.get("shared"):
        out = out + sigmoid(h @ w[p + "shared.sg"].T) * gated_expert(h, w, p + "shared.")
    return out


def feed_forward(h, w, p, mlp):
    if mlp["kind"] == "dense":
        return gelu_erf(h @ w[p + "up"].T + w[p + "up.b"]) @ w[p + "down"].T + w[p + "down.b"]
    if mlp["kind"] == "moe":
        return routed(h, w, p, mlp)
    raise ValueError(mlp["kind"])


# ----------------------------------------------------------------------------- the model
def forward(config: dict, weights: Dict[str, torch.Tensor], tokens: List[int], streams: Optional[list] = None) -> torch.Tensor:
    """Logits [S, vocab] of one sequence; ``streams`` (a list) receives the residual stream after every layer."""
    eps = float(config["norm"]["eps"])
    x = weights["embed"][torch.tensor(tokens)] * float(config["embedding"]["scale"])
    for i, layer in enumerate(config["layers"]):
        L = f"l{i}."
        y = mixer(offset_norm(x, weights[L + "norm1"], eps), weights, L + "mix.", layer, eps)
        x = x + offset_norm(y, weights[L + "norm1b"], eps) * weights[L + "ls1"]
        if layer.get("mlp") is not None:
            y = feed_forward(offset_norm(x, weights[L + "norm2"], eps), weights, L + "mlp.", layer["mlp"])
            x = x + offset_norm(y, weights[L + "norm2b"], eps) * weights[L + "ls2"]
        if streams is not None:
            streams.append(x.clone())
    return offset_norm(x, weights["final.norm"], eps) @ weights["embed"].T
