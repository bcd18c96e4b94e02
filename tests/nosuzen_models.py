"""Small Nosuzen configurations for the tests, and model folders with random weights made from them.

The configurations differ from each other in every size and constant, and in what a single model may happen to make
equal or one: streams (one among them), heads and kv heads, sizes of keys and values, rotated channels (all, some,
none), windows and kept first positions (none among them), taps of the convolutions (one, none), a layer that reads
the keys and values of the layer right before it or of one further back, with a smaller and with a larger window
than the owner's, YaRN on any kind of layer or on none, groups of experts (none, one, as many as experts), one
choice and several, a shared expert or none, layers without a feed-forward, every kind of layer first and last."""

from __future__ import annotations

from pathlib import Path
from typing import Dict

import torch


def rot(dims, base=10000.0, scaling=None):
    d = {"dims": dims, "base": base}
    if scaling is not None:
        factor, original, fast, slow = scaling
        d["scaling"] = {"factor": factor, "original": original, "fast": fast, "slow": slow}
    return d


def diff_attention(heads, kv_heads, dim, vdim, scale, diff, rotation, size, keep_first=0, conv=None, kv_from=None):
    d = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale, "diff": diff, "rot": rotation,
         "mask": {"size": size, "keep_first": keep_first}}
    if conv is not None:
        d["conv"] = conv
    if kv_from is not None:
        d["kv_from"] = kv_from
    return d


def latent(heads, dim, rot_dim, vdim, kv_rank, scale, size, base=10000.0, scaling=None):
    return {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank, "scale": scale,
            "rot": rot(rot_dim, base, scaling), "mask": {"size": size}}


def left(heads, kv_heads, dim, vdim, scale, rotation, size, keep_first=0):
    return {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale, "rot": rotation,
            "mask": {"size": size, "keep_first": keep_first}}


def right(heads, dim, vdim, tau, decay_rank=None):
    d = {"heads": heads, "dim": dim, "vdim": vdim, "tau": tau}
    if decay_rank is not None:
        d["decay_rank"] = decay_rank
    return d


def pair(lf, rt, left_scale, right_scale):
    return {"left": lf, "right": rt, "left_scale": left_scale, "right_scale": right_scale}


def moe(ff, experts, top, scale=1.0, groups=None, shared=None):
    router = {"experts": experts, "top": top, "scale": scale}
    if groups is not None:
        router["groups"] = {"count": groups[0], "keep": groups[1]}
    d = {"kind": "moe", "expert": {"ff": ff}, "router": router}
    if shared is not None:
        d["shared"] = {"ff": shared}
    return d


def layer(kind, mixer, mlp=None):
    return {"type": kind, "mixer": mixer, "mlp": mlp}


def model(vocab, width, streams, scale, eps, layers):
    return {"architecture": "Nosuzen", "vocab": vocab, "width": width, "streams": streams, "embedding": {"scale": scale},
            "norm": {"eps": eps}, "layers": layers}


CONFIG_A = model(131, 64, 2, 2.0, 1e-5, [
    layer("attention", diff_attention(4, 2, 16, 24, 0.3, 0.4, rot(16, 10000.0), 24, keep_first=5, conv=4), moe(40, 6, 2, 1.5, groups=(3, 2), shared=24)),
    layer("latent_attention", latent(2, 16, 8, 24, 40, 0.2, 30, scaling=(4.0, 32, 8.0, 1.0)), None),
    layer("parallel", pair(left(4, 2, 32, 32, 0.2, rot(16, 1000.0, (2.0, 16, 4.0, 1.0)), 20, keep_first=3), right(2, 16, 24, 8.0, 6), 0.7, 0.4),
          moe(24, 4, 1, 2.0)),
    layer("attention", diff_attention(4, 2, 16, 24, 0.25, 0.7, rot(8, 500.0), 40, keep_first=0, conv=2, kv_from=0), moe(32, 4, 4, 1.0, groups=(1, 1), shared=16)),
])
CONFIG_B = model(77, 96, 1, 1.0, 1e-6, [
    layer("parallel", pair(left(6, 1, 64, 64, 0.125, rot(64, 250000.0), 48, keep_first=0), right(3, 32, 16, 16.0, 5), 0.5, 0.5), None),
    layer("attention", diff_attention(2, 2, 32, 16, 0.2, 0.5, rot(32, 1e6, (8.0, 24, 16.0, 2.0)), 33, keep_first=16), moe(48, 6, 3, 2.5, groups=(6, 4), shared=32)),
    layer("attention", diff_attention(4, 2, 32, 16, 0.15, 0.3, rot(32, 1e6, (8.0, 24, 16.0, 2.0)), 17, keep_first=20, conv=1, kv_from=1), None),
    layer("latent_attention", latent(3, 24, 16, 20, 112, 0.15, 64, base=300.0), moe(16, 3, 2, 1.0)),
])
CONFIG_C = model(200, 128, 4, 6.0, 1e-5, [
    layer("latent_attention", latent(4, 40, 32, 24, 224, 0.11, 50, scaling=(4.0, 64, 16.0, 2.0)), moe(56, 10, 3, 1.75, groups=(2, 1), shared=72)),
    layer("attention", diff_attention(2, 1, 40, 80, 0.16, 0.35, rot(40, 5e5), 36, keep_first=8, conv=3), moe(32, 5, 2, 0.5)),
    layer("parallel", pair(left(2, 1, 128, 128, 0.09, rot(64, 1000.0), 28, keep_first=9), right(4, 64, 32, 4.0, 16), 0.8, 0.2), moe(32, 7, 2, 1.0, shared=8)),
    layer("attention", diff_attention(4, 1, 40, 80, 0.16, 0.2, rot(0, 1e4), 60, keep_first=2, conv=5, kv_from=1), None),
    layer("parallel", pair(left(4, 4, 16, 8, 0.3, rot(0, 100.0), 100, keep_first=0), right(1, 128, 128, 32.0, 3), 0.3, 0.9), moe(24, 2, 2, 3.0, groups=(2, 2))),
])
CONFIGS = {"A": CONFIG_A, "B": CONFIG_B, "C": CONFIG_C}
PAGE_SIZE = {"A": 8, "B": 16, "C": 4}


def single_layer(entry: dict, width: int = 64, vocab: int = 61, streams: int = 2) -> dict:
    """A model of one layer, for a mechanism alone."""
    return model(vocab, width, streams, 2.0, 1e-5, [entry])


def make_folder(path, cfg_dict: dict, seed: int = 0, dtype=torch.bfloat16, sharpen: float = 3.0, decisive_router: bool = False) -> Path:
    """A model folder written by the package's random-weights mode, then made harder on faults: the projections of the
    mixers are scaled up so that their outputs depend on their inputs; the q and k projections of the softmax layers
    so that scores have about the spread ``sharpen`` and every query looks at a few keys, near and far; the norms get
    weights, biases and alphas with a spread, the streams' weights too; the linear attention's decays reach from a
    few tokens to hundreds; the vectors behind lambda make it differ from ``diff``.  ``decisive_router``: the router's
    outputs are led by what the norm's bias gives every expert, two apart from expert to expert, so that rounding
    cannot change a choice (what a bfloat16 run is compared on); without it the choice changes from token to token."""
    from safetensors.torch import save_file

    from torchllms_amd.config.nosuzen import NosuzenConfig
    from torchllms_amd.weights import write_model_folder

    folder = write_model_folder(path, NosuzenConfig.from_dict(cfg_dict), seed=seed, dtype=dtype)
    _, tensors = read_folder(folder)
    gen = torch.Generator().manual_seed(seed + 1)
    width = cfg_dict["width"]
    for name in list(tensors):
        t = tensors[name].float()
        leaf = name.split(".", 1)[-1] if name.startswith("l") else name
        last = leaf.rsplit(".", 1)[-1]
        li = int(name[1 : name.index(".")]) if name[0] == "l" and name[1].isdigit() else None
        if leaf in ("norm1", "norm2") or name == "final.norm":
            t = 1.0 + 0.3 * torch.randn(t.shape, generator=gen)
        elif leaf in ("norm1.b", "norm2.b", "final.norm.b"):
            t = 0.3 * torch.randn(t.shape, generator=gen)
        elif last == "alpha":
            # (a steep tanh over a sum of several streams acts like a sign: channels near zero would turn rounding into
            # whole steps, in the plain model as in the engine; steepness and read weights shrink with the streams)
            t = (0.5 + 2.0 * torch.rand(t.shape, generator=gen)) / cfg_dict["streams"]
        elif leaf.startswith("hc") and last == "in":
            t = (0.4 + 0.8 * torch.rand(t.shape, generator=gen)) / cfg_dict["streams"]
        elif leaf.startswith("hc") and last == "out":
            t = 0.4 + 0.8 * torch.rand(t.shape, generator=gen)
        elif leaf.startswith("hc") and last == "mix":
            # (well inside what keeps the streams from growing layer after layer: rounding would grow with them)
            t = torch.eye(t.shape[0]) * 0.6 + (0.3 / t.shape[0]) * torch.randn(t.shape, generator=gen)
        elif last == "norm":
            t = 1.0 + 0.2 * torch.randn(t.shape, generator=gen)
        elif last in ("lq1", "lk1", "lq2", "lk2"):
            t = 0.25 * torch.randn(t.shape, generator=gen)
        elif leaf == "mix.right.a2.b":
            t = 2.0 + 3.0 * torch.randn(t.shape, generator=gen)
        elif leaf in ("mix.right.q", "mix.right.k", "mix.right.v", "mix.right.g", "mix.right.o", "mix.right.a1"):
            t = t * 5.0
        elif last in ("q", "k") and leaf.startswith("mix.") and "right" not in leaf and sharpen > 0:
            # a score is scale * sum over dim of q_i k_i with q_i, k_i ~ N(0, 0.02^2 width) as drawn (inputs of size one)
            m = cfg_dict["layers"][li]["mixer"]
            m = m["left"] if "left" in leaf else m
            t = t * (sharpen / (m["scale"] * m["dim"] ** 0.5 * 0.0004 * width)) ** 0.5
        elif last in ("dkv", "uk") and sharpen > 0:
            t = t * 4.0
        elif leaf.startswith("mix.") and last in ("v", "o", "uv"):
            t = t * 5.0
        elif last == "conv":
            t = 0.6 * torch.randn(t.shape, generator=gen)
        elif leaf.startswith("mlp.") and last in ("up", "gate", "down"):
            t = t * 3.0
        elif leaf == "mlp.router":
            t = 2.0 * torch.randn(t.shape, generator=gen)
        tensors[name] = t
    if decisive_router:
        for name in list(tensors):
            if name.endswith("mlp.router"):
                # (a bias well above what the tanh adds to it, so that bias . row stays near |bias|^2 for every token)
                bias = tensors[name.replace("mlp.router", "norm2.b")] * 5.0
                tensors[name.replace("mlp.router", "norm2.b")] = bias
                lead = 2.0 * torch.randperm(tensors[name].shape[0], generator=gen).float()
                tensors[name] = 0.02 * tensors[name] + lead[:, None] * bias[None, :] / bias.pow(2).sum()
    tensors = {k: v.to(dtype).contiguous() for k, v in tensors.items()}
    save_file(tensors, str(folder / "model.safetensors"), metadata={"format": "pt"})
    return folder


def read_folder(folder) -> (dict, Dict[str, torch.Tensor]):
    """config.json as a dict and the tensors by their checkpoint names, read with safetensors
    directly (not through the package's loader)."""
    import json

    from safetensors import safe_open

    folder = Path(folder)
    with open(folder / "config.json") as f:
        cfg = json.load(f)
    tensors = {}
    with safe_open(str(folder / "model.safetensors"), framework="pt", device="cpu") as f:
        for name in f.keys():
            tensors[name] = f.get_tensor(name)
    return cfg, tensors
