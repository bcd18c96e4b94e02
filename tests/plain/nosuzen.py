"""A plain, slow Nosuzen: whole sequences at once, no cache, one function per mechanism, in the precision of the
tensors it is given (tests hand it 64-bit ones).  It shares no code with the engine.

Notation: ``h`` [T, D] rows of one sequence, positions 0..T-1; a layer's tensors under their checkpoint names in a
dict ``w``; a layer's description ``cfg`` as config.json gives it."""

from __future__ import annotations

import math
from typing import Dict, List, Optional

import torch


# ----------------------------------------------------------------------------- small pieces
def dyt(x, w: Dict[str, torch.Tensor], name: str):
    """Dynamic tanh: ``tanh(alpha x) * weight + bias``, no statistics."""
    return torch.tanh(w[name + ".alpha"] * x) * w[name] + w[name + ".b"]


def over_rms(x, eps: float):
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def silu(z):
    return z * torch.sigmoid(z)


def rotary_frequencies(rot: Dict, dtype=torch.float64):
    """``(frequency of every pair, factor on cosines and sines)`` of a ``rot`` entry; with ``scaling`` the
    frequencies of long wavelengths are divided by ``factor`` behind a linear ramp over the pair index."""
    dims, base = rot["dims"], float(rot["base"])
    i = torch.arange(dims // 2, dtype=torch.float64)
    f = base ** (-2.0 * i / dims)
    mag = 1.0
    sc = rot.get("scaling")
    if sc:
        def turn_at(t):
            return dims * math.log(sc["original"] / (2 * math.pi * t)) / (2 * math.log(base))
        lo = max(math.floor(turn_at(sc["fast"])), 0)
        hi = min(math.ceil(turn_at(sc["slow"])), dims - 1)
        ramp = ((i - lo) / max(hi - lo, 0.001)).clamp(0, 1)
        f = f / sc["factor"] * ramp + f * (1 - ramp)
        mag = 0.1 * math.log(sc["factor"]) + 1.0
    return f.to(dtype), mag


def rotate(x, positions, rot: Dict, layout: str):
    """Rotate the first ``rot.dims`` channels of the last axis of ``x`` [T, ..., d]; ``layout`` "half" pairs channel
    i with i + dims/2, "interleaved" 2i with 2i+1."""
    dims = rot["dims"]
    if dims == 0:
        return x
    f, mag = rotary_frequencies(rot, x.dtype)
    ang = positions.to(x.dtype)[:, None] * f[None, :]          # [T, dims/2]
    shape = [x.shape[0]] + [1] * (x.dim() - 2) + [dims // 2]
    c, s = (torch.cos(ang) * mag).view(shape), (torch.sin(ang) * mag).view(shape)
    out = x.clone()
    if layout == "half":
        a, b = x[..., : dims // 2], x[..., dims // 2 : dims]
        out[..., : dims // 2] = a * c - b * s
        out[..., dims // 2 : dims] = b * c + a * s
    else:
        a, b = x[..., 0:dims:2], x[..., 1:dims:2]
        out[..., 0:dims:2] = a * c - b * s
        out[..., 1:dims:2] = b * c + a * s
    return out


def short_conv(u, taps):
    """``y_t = sum_j taps[:, j] u_(t - K + 1 + j)`` channel by channel, zeros before the start; u [T, C], taps [C, K]."""
    K = taps.shape[1]
    T = u.shape[0]
    padded = torch.cat([u.new_zeros(K - 1, u.shape[1]), u], dim=0)
    y = u.new_zeros(u.shape)
    for j in range(K):
        y = y + padded[j : j + T] * taps[:, j][None, :]
    return y


def visible(T: int, size: int, keep_first: int = 0):
    """bool [T, T]: query i sees key j when j <= i and (i - j < size or j < keep_first)."""
    i = torch.arange(T)[:, None]
    j = torch.arange(T)[None, :]
    return (j <= i) & ((i - j < size) | (j < keep_first))


def softmax_attention(q, k, v, mask, scale: float):
    """q [T, H, d], k [T, H, d], v [T, H, dv] (already one key/value head per query head) -> [T, H, dv]."""
    s = torch.einsum("ihd,jhd->hij", q, k) * scale
    s = s.masked_fill(~mask[None], float("-inf"))
    return torch.einsum("hij,jhd->ihd", torch.softmax(s, dim=-1), v)


# ----------------------------------------------------------------------------- mixers
def differential_attention(h, w, p: str, m: Dict, eps: float, borrowed=None):
    """Two softmax maps per head over the same values, ``a1 - lambda a2``, each head over its root mean square and
    times ``1 - diff``.  Returns ``(output, (keys, values))``; ``borrowed``: another layer's (keys, values)."""
    T = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    pos = torch.arange(T)
    q = h @ w[p + "q"].T
    if m.get("conv"):
        q = short_conv(q, w[p + "q.conv"])
    q = rotate(q.view(T, H, 2, d), pos, m["rot"], "half")
    if borrowed is None:
        k, v = h @ w[p + "k"].T, h @ w[p + "v"].T
        if m.get("conv"):
            k, v = short_conv(k, w[p + "k.conv"]), short_conv(v, w[p + "v.conv"])
        k = rotate(k.view(T, G, 2, d), pos, m["rot"], "half")
        v = v.view(T, G, dv)
    else:
        k, v = borrowed
    rep = H // G
    kk, vv = k.repeat_interleave(rep, dim=1), v.repeat_interleave(rep, dim=1)
    mask = visible(T, m["mask"]["size"], m["mask"].get("keep_first", 0))
    a1 = softmax_attention(q[:, :, 0], kk[:, :, 0], vv, mask, m["scale"])
    a2 = softmax_attention(q[:, :, 1], kk[:, :, 1], vv, mask, m["scale"])
    lam = torch.exp((w[p + "lq1"] * w[p + "lk1"]).sum()) - torch.exp((w[p + "lq2"] * w[p + "lk2"]).sum()) + m["diff"]
    o = over_rms(a1 - lam * a2, eps) * (1.0 - m["diff"])
    return o.reshape(T, H * dv) @ w[p + "o"].T, (k, v)


def grouped_attention(h, w, p: str, m: Dict, eps: float):
    """Grouped-query attention with a weighted RMS norm of queries and keys before the rotation."""
    T = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    pos = torch.arange(T)
    q = over_rms((h @ w[p + "q"].T).view(T, H, d), eps) * w[p + "q.norm"]
    k = over_rms((h @ w[p + "k"].T).view(T, G, d), eps) * w[p + "k.norm"]
    v = (h @ w[p + "v"].T).view(T, G, dv)
    q, k = rotate(q, pos, m["rot"], "half"), rotate(k, pos, m["rot"], "half")
    rep = H // G
    mask = visible(T, m["mask"]["size"], m["mask"].get("keep_first", 0))
    o = softmax_attention(q, k.repeat_interleave(rep, dim=1), v.repeat_interleave(rep, dim=1), mask, m["scale"])
    return o.reshape(T, H * dv) @ w[p + "o"].T


def gated_linear_attention(h, w, p: str, m: Dict, eps: float):
    """Per head ``S <- diag(alpha_t) S + k_t v_t^T; o_t = S^T q_t`` with a decay per key channel."""
    T = h.shape[0]
    H, d, dv = m["heads"], m["dim"], m["vdim"]
    q = (h @ w[p + "q"].T).view(T, H, d) * d ** -0.5
    k = (h @ w[p + "k"].T).view(T, H, d)
    v = (h @ w[p + "v"].T).view(T, H, dv)
    z = (h @ w[p + "a1"].T) @ w[p + "a2"].T + w[p + "a2.b"]
    alpha = torch.sigmoid(z).pow(1.0 / m["tau"]).view(T, H, d)
    S = h.new_zeros(H, d, dv)
    outs = []
    for t in range(T):
        S = alpha[t][:, :, None] * S + k[t][:, :, None] * v[t][:, None, :]
        outs.append(torch.einsum("hdv,hd->hv", S, q[t]))
    o = over_rms(torch.stack(outs), eps) * w[p + "norm"]
    return (o.reshape(T, H * dv) * silu(h @ w[p + "g"].T)) @ w[p + "o"].T


def latent_attention(h, w, p: str, m: Dict, eps: float):
    """Keys and values of all heads expanded from one normed latent per token; one rotated key part for all heads."""
    T = h.shape[0]
    H, d, r, dv, R = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    pos = torch.arange(T)
    q = (h @ w[p + "q"].T).view(T, H, d + r)
    down = h @ w[p + "dkv"].T
    c = over_rms(down[:, :R], eps) * w[p + "dkv.norm"]
    shared = rotate(down[:, R:], pos, m["rot"], "interleaved")                    # [T, r]
    q_rot = rotate(q[:, :, d:], pos, m["rot"], "interleaved")
    k_plain = (c @ w[p + "uk"].T).view(T, H, d)
    v = (c @ w[p + "uv"].T).view(T, H, dv)
    qq = torch.cat([q[:, :, :d], q_rot], dim=-1)
    kk = torch.cat([k_plain, shared[:, None, :].expand(T, H, r)], dim=-1)
    o = softmax_attention(qq, kk, v, visible(T, m["mask"]["size"]), m["scale"])
    return o.reshape(T, H * dv) @ w[p + "o"].T


def mixer(h, w, i: int, layer: Dict, eps: float, kept: Dict[int, tuple]):
    p, m = f"l{i}.mix.", layer["mixer"]
    if layer["type"] == "attention":
        src = m.get("kv_from")
        y, kv = differential_attention(h, w, p, m, eps, borrowed=None if src is None else kept[src])
        if src is None:
            kept[i] = kv
        return y
    if layer["type"] == "latent_attention":
        return latent_attention(h, w, p, m, eps)
    left = grouped_attention(h, w, p + "left.", m["left"], eps)
    right = gated_linear_attention(h, w, p + "right.", m["right"], eps)
    return m["left_scale"] * left + m["right_scale"] * right


# ----------------------------------------------------------------------------- feed-forward
def gated_expert(h, w, p: str):
    return (silu(h @ w[p + "gate"].T) * (h @ w[p + "up"].T)) @ w[p + "down"].T


def routed_choice(z, router: Dict):
    """``(chosen experts [T, top], their weights)`` from the router's outputs z [T, E]."""
    E, top = router["experts"], router["top"]
    s = torch.softmax(z, dim=-1)
    allowed = s
    groups = router.get("groups")
    if groups:
        per = E // groups["count"]
        best = s.view(-1, groups["count"], per).max(dim=-1).values
        kept = best.topk(groups["keep"], dim=-1).indices
        open_ = torch.zeros_like(best, dtype=torch.bool).scatter_(1, kept, True)
        allowed = s.masked_fill(~open_.repeat_interleave(per, dim=1), float("-inf"))
    ids = allowed.topk(top, dim=-1).indices
    chosen = s.gather(1, ids)
    return ids, chosen / (chosen.sum(dim=-1, keepdim=True) + 1e-20) * router.get("scale", 1.0)


def mixture(h, w, p: str, mlp: Dict):
    z = h.float() @ w[p + "router"].float().T if h.dtype != torch.float64 else h @ w[p + "router"].T
    ids, weights = routed_choice(z.to(h.dtype), mlp["router"])
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for e, g in zip(ids[t].tolist(), weights[t]):
            out[t] += g * gated_expert(h[t : t + 1], w, f"{p}e{e}.")[0]
    if mlp.get("shared"):
        out = out + gated_expert(h, w, p + "shared.")
    return out


# ----------------------------------------------------------------------------- the model
def hyper_sublayer(streams, w, p: str, norm_name: str, branch):
    """``u = sum_s in[s] x_s; y = branch(norm(u)); x_t <- sum_s mix[s, t] x_s + out[t] y`` for streams [S, T, D]."""
    u = torch.einsum("s,std->td", w[p + ".in"], streams)
    y = branch(dyt(u, w, norm_name))
    return torch.einsum("sr,std->rtd", w[p + ".mix"], streams) + w[p + ".out"][:, None, None] * y[None]


def forward(config: Dict, tensors: Dict[str, torch.Tensor], tokens: List[int], dtype=torch.float64, layer_outputs: Optional[list] = None):
    """Logits [T, vocab] of one sequence."""
    w = {k: (v.to(dtype) if v.is_floating_point() else v) for k, v in tensors.items()}
    eps = float(config["norm"]["eps"])
    x = w["embed"][torch.tensor(tokens, dtype=torch.long)] * config["embedding"]["scale"]
    streams = x[None].repeat(config["streams"], 1, 1)
    kept: Dict[int, tuple] = {}
    for i, layer in enumerate(config["layers"]):
        streams = hyper_sublayer(streams, w, f"l{i}.hc1", f"l{i}.norm1", lambda h: mixer(h, w, i, layer, eps, kept))
        if layer.get("mlp") is not None:
            streams = hyper_sublayer(streams, w, f"l{i}.hc2", f"l{i}.norm2", lambda h: mixture(h, w, f"l{i}.mlp.", layer["mlp"]))
        if layer_outputs is not None:
            layer_outputs.append(streams.sum(dim=0))
    return dyt(streams.sum(dim=0), w, "final.norm") @ w["head"].T
