"""Typed configuration of the Nosuzen decoder, read from ``config.json``, and the model it describes.

A Nosuzen model is a list of layers over several 32-bit residual streams (hyper-connections): every sublayer reads a
weighted sum of the streams through a norm without statistics (dynamic tanh) and writes its result back into all of
them.  A layer's mixer is differential attention (two softmax maps per head over the same values, queries, keys and
values through a short convolution, a sliding window that keeps the first positions; a layer may read an earlier
layer's keys and values instead of making its own), attention through a latent (one normed latent and one rotated
key part per token, YaRN-scaled rotation of interleaved pairs, a sliding window), or two mixers side by side whose
results are added with two weights: grouped-query attention with a weighted norm of queries and keys and gated linear
attention with a decay per key channel.  The feed-forward is a mixture of experts whose router keeps the best groups
of experts, renormalises the chosen scores and scales them, beside a shared expert; a layer may have none.  Every
size and constant comes from config.json (the number of values between the two matrices of the linear attention's
decay from the tensors' shapes); nothing here knows a particular model.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Dict, List, Optional, Tuple

from .llama import ConfigError
from .spec import LayerRun, LayerSpec, ModelSpec, PartSpec

ARCHITECTURE = "Nosuzen"
LAYER_TYPES = ("attention", "latent_attention", "parallel")
#: config.json names no longest context: angles and states are computed from positions, so the bound is a matter
#: of memory alone; an engine is given its own ``max_model_len`` or pool size
DEFAULT_MAX_POSITIONS = 1 << 20

_ATTENTION_KEYS = ("heads", "kv_heads", "dim", "vdim", "scale", "diff", "rot", "mask")
_LATENT_KEYS = ("heads", "dim", "rot_dim", "vdim", "kv_rank", "scale", "rot", "mask")
_LEFT_KEYS = ("heads", "kv_heads", "dim", "vdim", "scale", "rot", "mask")
_RIGHT_KEYS = ("heads", "dim", "vdim", "tau")
_NUMBERS = ("scale", "diff", "tau")


def _positive_int(where: str, name: str, v) -> int:
    if not isinstance(v, int) or isinstance(v, bool) or v <= 0:
        raise ConfigError(f"{where}: {name} must be a positive integer, got {v!r}")
    return v


def _count(where: str, name: str, v) -> int:
    if not isinstance(v, int) or isinstance(v, bool) or v < 0:
        raise ConfigError(f"{where}: {name} must be an integer that is not negative, got {v!r}")
    return v


def _number(where: str, name: str, v) -> float:
    if not isinstance(v, (int, float)) or isinstance(v, bool):
        raise ConfigError(f"{where}: {name} must be a number, got {v!r}")
    return float(v)


def _sizes(where: str, d, keys) -> Dict[str, Any]:
    if not isinstance(d, dict):
        raise ConfigError(f"{where}: no sizes")
    lacking = [k for k in keys if k not in d]
    if lacking:
        raise ConfigError(f"{where}: lacks {lacking}")
    for k in keys:
        if k in _NUMBERS:
            _number(where, k, d[k])
        elif k == "rot_dim":
            _count(where, k, d[k])  # (a latent layer may rotate nothing)
        elif k not in ("rot", "mask"):
            _positive_int(where, k, d[k])
    return dict(d)


def _rotation(where: str, rot, most: int) -> Dict[str, Any]:
    if not isinstance(rot, dict) or "dims" not in rot or "base" not in rot:
        raise ConfigError(f"{where}: rot needs 'dims' and 'base'")
    dims = _count(where, "rot.dims", rot["dims"])
    if dims % 2 or dims > most:
        raise ConfigError(f"{where}: rot.dims={dims} must be even and at most {most}")
    if not _number(where, "rot.base", rot["base"]) > 0:
        raise ConfigError(f"{where}: rot.base must be positive")
    scaling = rot.get("scaling")
    if scaling is not None:
        if not isinstance(scaling, dict) or any(k not in scaling for k in ("factor", "original", "fast", "slow")):
            raise ConfigError(f"{where}: rot.scaling needs 'factor', 'original', 'fast' and 'slow'")
        for k in ("factor", "original", "fast", "slow"):
            if not _number(where, "rot.scaling." + k, scaling[k]) > 0:
                raise ConfigError(f"{where}: rot.scaling.{k} must be positive")
    return dict(rot)


def _mask(where: str, mask, keeps: bool) -> Dict[str, int]:
    if not isinstance(mask, dict) or "size" not in mask:
        raise ConfigError(f"{where}: mask needs 'size'")
    out = {"size": _positive_int(where, "mask.size", mask["size"])}
    if keeps:
        out["keep_first"] = _count(where, "mask.keep_first", mask.get("keep_first", 0))
    return out


@dataclass(frozen=True)
class NosuzenLayer:
    """One entry of ``layers``: the mixer's type and sizes and the feed-forward's description (None: none)."""

    type: str
    mixer: Dict[str, Any]
    mlp: Optional[Dict[str, Any]] = None

    def to_dict(self) -> Dict[str, Any]:
        return {"type": self.type, "mixer": self.mixer, "mlp": self.mlp}


@dataclass(frozen=True)
class NosuzenConfig:
    vocab: int
    width: int
    streams: int
    layers: Tuple[NosuzenLayer, ...]
    norm_eps: float
    embedding_scale: float = 1.0
    eos_token_id: Any = None
    architectures: tuple = (ARCHITECTURE,)

    # ------------------------------------------------------------------ reading / writing
    @classmethod
    def from_dict(cls, d: Dict[str, Any]) -> "NosuzenConfig":
        missing = [k for k in ("vocab", "width", "layers", "norm", "streams") if k not in d]
        if missing:
            raise ConfigError(f"config.json lacks required keys {missing}")
        _positive_int("config", "vocab", d["vocab"])
        _positive_int("config", "width", d["width"])
        _positive_int("config", "streams", d["streams"])
        if not isinstance(d["layers"], list) or not d["layers"]:
            raise ConfigError("config.json: 'layers' must be a list with at least one layer")
        eps = d["norm"].get("eps") if isinstance(d["norm"], dict) else None
        if not isinstance(eps, (int, float)) or not eps > 0:
            raise ConfigError(f"config.json: norm.eps must be positive, got {eps!r}")
        emb = d.get("embedding") or {}
        layers = tuple(cls._layer_from_dict(i, entry) for i, entry in enumerate(d["layers"]))
        for i, layer in enumerate(layers):
            src = layer.mixer.get("kv_from") if layer.type == "attention" else None
            if src is None:
                continue
            if not isinstance(src, int) or isinstance(src, bool) or not 0 <= src < i or layers[src].type != "attention" \
                    or layers[src].mixer.get("kv_from") is not None:
                raise ConfigError(f"layers[{i}]: kv_from={src!r} must name an earlier attention layer with keys and values of its own")
            theirs = layers[src].mixer
            for k in ("kv_heads", "dim", "vdim"):
                if theirs[k] != layer.mixer[k]:
                    raise ConfigError(f"layers[{i}]: {k}={layer.mixer[k]} differs from that of layer {src}, whose keys and values it reads")
        return cls(
            vocab=d["vocab"],
            width=d["width"],
            streams=d["streams"],
            layers=layers,
            norm_eps=float(eps),
            embedding_scale=_number("embedding", "scale", emb.get("scale", 1.0)),
            eos_token_id=d.get("eos_token_id"),
        )

    @staticmethod
    def _layer_from_dict(i: int, entry: Dict[str, Any]) -> NosuzenLayer:
        where = f"layers[{i}]"
        kind = entry.get("type") if isinstance(entry, dict) else None
        if kind not in LAYER_TYPES:
            raise ConfigError(f"{where}: type {kind!r} is not one of {list(LAYER_TYPES)}")
        mixer = entry.get("mixer")
        if kind == "attention":
            mixer = _sizes(where + ".mixer", mixer, _ATTENTION_KEYS)
            if mixer["heads"] % mixer["kv_heads"]:
                raise ConfigError(f"{where}: {mixer['heads']} heads are not a multiple of {mixer['kv_heads']} kv_heads")
            mixer["rot"] = _rotation(where, mixer["rot"], mixer["dim"])
            mixer["mask"] = _mask(where, mixer["mask"], keeps=True)
            mixer["conv"] = _count(where, "conv", mixer.get("conv", 0) or 0)
        elif kind == "latent_attention":
            mixer = _sizes(where + ".mixer", mixer, _LATENT_KEYS)
            mixer["rot"] = _rotation(where, mixer["rot"], mixer["rot_dim"])
            if mixer["rot"]["dims"] != mixer["rot_dim"]:
                raise ConfigError(f"{where}: the rotated part has rot_dim={mixer['rot_dim']} channels, so rot.dims must be that")
            mixer["mask"] = _mask(where, mixer["mask"], keeps=False)
        else:
            if not isinstance(mixer, dict):
                raise ConfigError(f"{where}: no 'mixer' sizes")
            lacking = [k for k in ("left", "right", "left_scale", "right_scale") if k not in mixer]
            if lacking:
                raise ConfigError(f"{where}: the parallel mixer lacks {lacking}")
            left = _sizes(where + ".mixer.left", mixer["left"], _LEFT_KEYS)
            right = _sizes(where + ".mixer.right", mixer["right"], _RIGHT_KEYS)
            if left["heads"] % left["kv_heads"]:
                raise ConfigError(f"{where}.left: {left['heads']} heads are not a multiple of {left['kv_heads']} kv_heads")
            left["rot"] = _rotation(where + ".left", left["rot"], left["dim"])
            left["mask"] = _mask(where + ".left", left["mask"], keeps=True)
            if not right["tau"] > 0:
                raise ConfigError(f"{where}.right: tau must be positive, got {right['tau']!r}")
            mixer = dict(mixer, left=left, right=right, left_scale=_number(where, "left_scale", mixer["left_scale"]),
                         right_scale=_number(where, "right_scale", mixer["right_scale"]))
        mlp = entry.get("mlp")
        if mlp is not None:
            mlp = NosuzenConfig._mlp_from_dict(where + ".mlp", mlp)
        return NosuzenLayer(type=kind, mixer=mixer, mlp=mlp)

    @staticmethod
    def _mlp_from_dict(where: str, mlp) -> Dict[str, Any]:
        if not isinstance(mlp, dict) or mlp.get("kind") != "moe":
            raise ConfigError(f"{where}: kind {mlp.get('kind') if isinstance(mlp, dict) else mlp!r} is not 'moe'")
        expert, router = mlp.get("expert"), mlp.get("router")
        if not isinstance(expert, dict) or not isinstance(router, dict):
            raise ConfigError(f"{where}: a mixture of experts needs 'expert' and 'router'")
        _positive_int(where + ".expert", "ff", expert.get("ff"))
        experts = _positive_int(where + ".router", "experts", router.get("experts"))
        top = _positive_int(where + ".router", "top", router.get("top"))
        if top > experts:
            raise ConfigError(f"{where}.router: {top} choices among {experts} experts")
        _number(where + ".router", "scale", router.get("scale", 1.0))
        groups = router.get("groups")
        if groups is not None:
            if not isinstance(groups, dict):
                raise ConfigError(f"{where}.router: groups must give 'count' and 'keep'")
            count = _positive_int(where + ".router.groups", "count", groups.get("count"))
            keep = _positive_int(where + ".router.groups", "keep", groups.get("keep"))
            if experts % count or keep > count or keep * (experts // count) < top:
                raise ConfigError(f"{where}.router: {count} groups of which {keep} stay do not fit {experts} experts and {top} choices")
        shared = mlp.get("shared")
        if shared is not None:
            if not isinstance(shared, dict):
                raise ConfigError(f"{where}: shared must give the shared expert's sizes")
            _positive_int(where + ".shared", "ff", shared.get("ff"))
        return dict(mlp)

    def to_dict(self) -> Dict[str, Any]:
        d: Dict[str, Any] = {
            "architecture": ARCHITECTURE,
            "vocab": self.vocab,
            "width": self.width,
            "streams": self.streams,
            "embedding": {"scale": self.embedding_scale},
            "norm": {"eps": self.norm_eps},
            "layers": [layer.to_dict() for layer in self.layers],
        }
        if self.eos_token_id is not None:
            d["eos_token_id"] = self.eos_token_id
        return d


def decay_rank(right: Dict[str, Any]) -> int:
    """How many numbers lie between the two matrices of the linear attention's decay.  The tensors' shapes say it
    (``nosuzen_sizes_from_tensors`` writes it into the configuration as ``decay_rank``, and a configuration may name it
    itself); a configuration that says nothing, as one made for random weights may, gets 16."""
    return int(right.get("decay_rank") or 16)


def nosuzen_sizes_from_tensors(cfg: NosuzenConfig, shapes: Dict[str, tuple]) -> NosuzenConfig:
    """The configuration with the size that config.json leaves to the tensors: of every parallel layer's linear
    attention the first size of ``l<i>.mix.right.a1``."""
    layers = []
    for i, layer in enumerate(cfg.layers):
        if layer.type == "parallel":
            shape = shapes.get(f"l{i}.mix.right.a1")
            if shape is not None and len(shape) == 2:
                right = dict(layer.mixer["right"], decay_rank=int(shape[0]))
                layer = NosuzenLayer(type=layer.type, mixer=dict(layer.mixer, right=right), mlp=layer.mlp)
        layers.append(layer)
    return NosuzenConfig(vocab=cfg.vocab, width=cfg.width, streams=cfg.streams, layers=tuple(layers), norm_eps=cfg.norm_eps,
                         embedding_scale=cfg.embedding_scale, eos_token_id=cfg.eos_token_id)


def _rope(rot: Dict[str, Any], head_dim: int, pairing: str) -> PartSpec:
    if rot["dims"] == 0:
        return PartSpec("none", {})
    scaling = dict(rot["scaling"], rope_type="yarn") if rot.get("scaling") else None
    return PartSpec("rope", dict(head_dim=head_dim, rotary_dim=rot["dims"], theta=float(rot["base"]), scaling=scaling, pairing=pairing,
                                 precise=True))


def _feed_forward_spec(cfg: NosuzenConfig, mlp: Dict[str, Any]) -> PartSpec:
    router = mlp["router"]
    groups = router.get("groups") or {}
    return PartSpec("routed", dict(
        hidden_size=cfg.width, expert_size=mlp["expert"]["ff"], num_experts=router["experts"], top=router["top"],
        shared_size=(mlp.get("shared") or {}).get("ff", 0), shared_gate=False, correction=False,
        groups=int(groups.get("count", 0) or 0), keep_groups=int(groups.get("keep", 0) or 0), normalize=True,
        route_scale=float(router.get("scale", 1.0)),
    ))


def nosuzen_model_spec(cfg: NosuzenConfig) -> ModelSpec:
    """The model as data: one ``LayerSpec`` per layer, named ``l<i>`` as its tensors are."""
    from ..parts.attention import covering_window

    def norm():
        return PartSpec("dynamic_tanh", dict(size=cfg.width))

    # what the pages of a layer with keys and values of its own must serve: its mask and those of the layers that read them
    readers: Dict[int, List[tuple]] = {}
    for i, layer in enumerate(cfg.layers):
        if layer.type == "attention":
            m = layer.mixer
            owner = i if m.get("kv_from") is None else m["kv_from"]
            readers.setdefault(owner, []).append((m["mask"]["size"], m["mask"].get("keep_first", 0)))
    specs: List[LayerSpec] = []
    order: List[LayerRun] = []
    for i, layer in enumerate(cfg.layers):
        m = layer.mixer
        parts = {"norm1": norm()}
        params: Dict[str, Any] = {"streams": cfg.streams}
        cache_from = None
        if layer.type == "attention":
            block = "hyper"
            shares = m.get("kv_from") is not None
            cache_from = m.get("kv_from")
            window, keep = covering_window(readers[i]) if not shares else (m["mask"]["size"], m["mask"].get("keep_first", 0))
            parts["mix"] = PartSpec("differential_attention", dict(
                hidden_size=cfg.width, num_heads=m["heads"], num_kv_heads=m["kv_heads"], head_dim=m["dim"], v_head_dim=m["vdim"],
                softmax_scale=float(m["scale"]), diff=float(m["diff"]), norm_eps=cfg.norm_eps, window=m["mask"]["size"],
                keep_first=m["mask"].get("keep_first", 0), conv_taps=m.get("conv", 0), shares_kv=shares,
                position=_rope(m["rot"], m["dim"], "half"), cache_window=window, cache_keep_first=keep))
        elif layer.type == "latent_attention":
            block = "hyper"
            parts["mix"] = PartSpec("latent_attention", dict(
                hidden_size=cfg.width, num_heads=m["heads"], head_dim=m["dim"], rot_dim=m["rot_dim"], v_head_dim=m["vdim"],
                q_rank=None, kv_rank=m["kv_rank"], softmax_scale=float(m["scale"]), norm_eps=cfg.norm_eps,
                position=_rope(m["rot"], m["rot_dim"], "interleaved"), window=m["mask"]["size"]))
        else:
            block = "hyper_pair"
            left, right = m["left"], m["right"]
            parts["left"] = PartSpec("attention", dict(
                hidden_size=cfg.width, num_heads=left["heads"], num_kv_heads=left["kv_heads"], head_dim=left["dim"], qkv_bias=False,
                softmax_scale=float(left["scale"]), window=left["mask"]["size"], keep_first=left["mask"].get("keep_first", 0),
                position=_rope(left["rot"], left["dim"], "half"), v_head_dim=left["vdim"], qk_norm_eps=cfg.norm_eps,
                qk_norm_weight=True))
            parts["right"] = PartSpec("gated_linear", dict(
                hidden_size=cfg.width, num_heads=right["heads"], head_dim=right["dim"], v_head_dim=right["vdim"], tau=float(right["tau"]),
                decay_rank=decay_rank(right), norm_eps=cfg.norm_eps))
            params.update(left_scale=m["left_scale"], right_scale=m["right_scale"])
        if layer.mlp is not None:
            parts["norm2"] = norm()
            parts["mlp"] = _feed_forward_spec(cfg, layer.mlp)
        else:
            block += "_mixer"
        specs.append(LayerSpec(name=f"l{i}", block=block, parts=parts, block_params=params))
        order.append(LayerRun(i, cache_from=cache_from))
    spec = ModelSpec(
        architecture=ARCHITECTURE,
        hidden_size=cfg.width,
        vocab_size=cfg.vocab,
        max_positions=DEFAULT_MAX_POSITIONS,
        embedding=PartSpec("embedding", dict(vocab_size=cfg.vocab, hidden_size=cfg.width, scale=cfg.embedding_scale,
                                             stream_dtype="float32")),
        layers=specs,
        order=order,
        final_norm=norm(),
        head=PartSpec("lm_head", dict(vocab_size=cfg.vocab, hidden_size=cfg.width, tied=False)),
    )
    spec.validate()
    return spec
