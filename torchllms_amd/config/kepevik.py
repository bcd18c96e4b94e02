"""Typed configuration of the Kepevik decoder, read from ``config.json``, and the model it describes.

A Kepevik model is a list of layers over a 32-bit residual stream.  Every layer has a token mixer and a
feed-forward (or none), each between a norm before and a norm behind it, the normed result times a layer scale:
``x <- x + ls * post(branch(pre(x)))``.  The mixer is a matrix memory (mLSTM) or two mixers side by side that read
the same rows: softmax attention whose values are its keys before the rotation, and a gated delta rule with a
decay per key channel; their results are added with two weights.  The feed-forward is dense (biases, exact gelu)
or a mixture of experts (softmax router, a correction for the choice, experts that hand their input through, a
gated shared expert).  Norm weights are stored around zero.  The output head is the embedding table.  Every size
and constant comes from config.json; nothing here knows a particular model.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Dict, List, Optional, Tuple

from .llama import ConfigError
from .spec import LayerRun, LayerSpec, ModelSpec, PartSpec

ARCHITECTURE = "Kepevik"
LAYER_TYPES = ("mlstm", "parallel")
#: config.json names no longest context: angles and states are computed from positions, so the bound is a matter
#: of memory alone; an engine is given its own ``max_model_len`` or pool size
DEFAULT_MAX_POSITIONS = 1 << 20

_MLSTM_KEYS = ("heads", "dim", "vdim", "gate_cap")
_LEFT_KEYS = ("heads", "kv_heads", "dim", "vdim", "scale", "rot")
_RIGHT_KEYS = ("heads", "kv_heads", "dim", "vdim", "conv")


def _positive_int(where: str, name: str, v) -> int:
    if not isinstance(v, int) or isinstance(v, bool) or v <= 0:
        raise ConfigError(f"{where}: {name} must be a positive integer, got {v!r}")
    return v


def _number(where: str, name: str, v) -> float:
    if not isinstance(v, (int, float)) or isinstance(v, bool):
        raise ConfigError(f"{where}: {name} must be a number, got {v!r}")
    return float(v)


def _sizes(where: str, d, keys, numbers=()) -> Dict[str, Any]:
    if not isinstance(d, dict):
        raise ConfigError(f"{where}: no sizes")
    lacking = [k for k in keys if k not in d]
    if lacking:
        raise ConfigError(f"{where}: lacks {lacking}")
    for k in keys:
        if k in numbers:
            _number(where, k, d[k])
        elif k != "rot":
            _positive_int(where, k, d[k])
    return dict(d)


@dataclass(frozen=True)
class KepevikLayer:
    """One entry of ``layers``: the mixer's type and sizes and the feed-forward's description (None: none)."""

    type: str
    mixer: Dict[str, Any]
    mlp: Optional[Dict[str, Any]] = None

    def to_dict(self) -> Dict[str, Any]:
        return {"type": self.type, "mixer": self.mixer, "mlp": self.mlp}


@dataclass(frozen=True)
class KepevikConfig:
    vocab: int
    width: int
    layers: Tuple[KepevikLayer, ...]
    norm_eps: float
    embedding_scale: float = 1.0
    eos_token_id: Any = None
    architectures: tuple = (ARCHITECTURE,)

    # ------------------------------------------------------------------ reading / writing
    @classmethod
    def from_dict(cls, d: Dict[str, Any]) -> "KepevikConfig":
        missing = [k for k in ("vocab", "width", "layers", "norm") if k not in d]
        if missing:
            raise ConfigError(f"config.json lacks required keys {missing}")
        _positive_int("config", "vocab", d["vocab"])
        _positive_int("config", "width", d["width"])
        if not isinstance(d["layers"], list) or not d["layers"]:
            raise ConfigError("config.json: 'layers' must be a list with at least one layer")
        eps = d["norm"].get("eps") if isinstance(d["norm"], dict) else None
        if not isinstance(eps, (int, float)) or not eps > 0:
            raise ConfigError(f"config.json: norm.eps must be positive, got {eps!r}")
        emb = d.get("embedding") or {}
        return cls(
            vocab=d["vocab"],
            width=d["width"],
            layers=tuple(cls._layer_from_dict(i, entry) for i, entry in enumerate(d["layers"])),
            norm_eps=float(eps),
            embedding_scale=_number("embedding", "scale", emb.get("scale", 1.0)),
            eos_token_id=d.get("eos_token_id"),
        )

    @staticmethod
    def _layer_from_dict(i: int, entry: Dict[str, Any]) -> KepevikLayer:
        where = f"layers[{i}]"
        kind = entry.get("type") if isinstance(entry, dict) else None
        if kind not in LAYER_TYPES:
            raise ConfigError(f"{where}: type {kind!r} is not one of {list(LAYER_TYPES)}")
        mixer = entry.get("mixer")
        if kind == "mlstm":
            mixer = _sizes(where + ".mixer", mixer, _MLSTM_KEYS, numbers=("gate_cap",))
            if not mixer["gate_cap"] > 0:
                raise ConfigError(f"{where}: gate_cap must be positive, got {mixer['gate_cap']!r}")
        else:
            if not isinstance(mixer, dict):
                raise ConfigError(f"{where}: no 'mixer' sizes")
            lacking = [k for k in ("left", "right", "left_scale", "right_scale") if k not in mixer]
            if lacking:
                raise ConfigError(f"{where}: the parallel mixer lacks {lacking}")
            left = _sizes(where + ".mixer.left", mixer["left"], _LEFT_KEYS, numbers=("scale",))
            right = _sizes(where + ".mixer.right", mixer["right"], _RIGHT_KEYS)
            for side, m in (("left", left), ("right", right)):
                if m["heads"] % m["kv_heads"]:
                    raise ConfigError(f"{where}.{side}: {m['heads']} heads are not a multiple of {m['kv_heads']} kv_heads")
            if left["vdim"] != left["dim"]:
                raise ConfigError(f"{where}.left: the values are the keys, so vdim={left['vdim']} must be dim={left['dim']}")
            rot = left["rot"]
            if not isinstance(rot, dict) or "dims" not in rot or "base" not in rot:
                raise ConfigError(f"{where}.left: rot needs 'dims' and 'base'")
            if not isinstance(rot["dims"], int) or isinstance(rot["dims"], bool) or rot["dims"] < 0 or rot["dims"] % 2 or rot["dims"] > left["dim"]:
                raise ConfigError(f"{where}.left: rot.dims={rot['dims']!r} must be even and at most dim={left['dim']}")
            if not _number(where + ".left", "rot.base", rot["base"]) > 0:
                raise ConfigError(f"{where}.left: rot.base must be positive")
            mixer = dict(mixer, left=left, right=right, left_scale=_number(where, "left_scale", mixer["left_scale"]),
                         right_scale=_number(where, "right_scale", mixer["right_scale"]))
        mlp = entry.get("mlp")
        if mlp is not None:
            mlp = KepevikConfig._mlp_from_dict(where + ".mlp", mlp)
        return KepevikLayer(type=kind, mixer=mixer, mlp=mlp)

    @staticmethod
    def _mlp_from_dict(where: str, mlp) -> Dict[str, Any]:
        if not isinstance(mlp, dict) or mlp.get("kind") not in ("dense", "moe"):
            raise ConfigError(f"{where}: kind {mlp.get('kind') if isinstance(mlp, dict) else mlp!r} is not 'dense' or 'moe'")
        if mlp["kind"] == "dense":
            _positive_int(where, "ff", mlp.get("ff"))
            return dict(mlp)
        expert, router = mlp.get("expert"), mlp.get("router")
        if not isinstance(expert, dict) or not isinstance(router, dict):
            raise ConfigError(f"{where}: a mixture of experts needs 'expert' and 'router'")
        _positive_int(where + ".expert", "ff", expert.get("ff"))
        _positive_int(where + ".router", "experts", router.get("experts"))
        _positive_int(where + ".router", "top", router.get("top"))
        identity = router.get("identity", 0) or 0
        if not isinstance(identity, int) or isinstance(identity, bool) or identity < 0:
            raise ConfigError(f"{where}.router: identity must be an integer that is not negative, got {identity!r}")
        if router["top"] > router["experts"] + identity:
            raise ConfigError(f"{where}.router: {router['top']} choices among {router['experts']} + {identity} outputs")
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
            "embedding": {"scale": self.embedding_scale},
            "norm": {"eps": self.norm_eps},
            "layers": [layer.to_dict() for layer in self.layers],
        }
        if self.eos_token_id is not None:
            d["eos_token_id"] = self.eos_token_id
        return d


def low_ranks(right: Dict[str, Any]) -> Tuple[int, int]:
    """How many numbers lie between the two matrices of the delta rule's decay and of its output gate.  The tensors'
    shapes say it (``kepevik_sizes_from_tensors`` writes them into the configuration as ``decay_rank`` and
    ``gate_rank``, and a configuration may name them itself); a configuration that says nothing, as one made for
    random weights may, gets the keys' head size over four, at least 8."""
    default = max(8, right["dim"] // 4)
    return int(right.get("decay_rank") or default), int(right.get("gate_rank") or default)


def kepevik_sizes_from_tensors(cfg: KepevikConfig, shapes: Dict[str, tuple]) -> KepevikConfig:
    """The configuration with the sizes that config.json leaves to the tensors: of every parallel layer's delta rule
    the first size of ``l<i>.mix.right.a1`` (decay) and of ``l<i>.mix.right.g1`` (output gate)."""
    layers = []
    for i, layer in enumerate(cfg.layers):
        if layer.type == "parallel":
            right = dict(layer.mixer["right"])
            for tensor, key in (("a1", "decay_rank"), ("g1", "gate_rank")):
                shape = shapes.get(f"l{i}.mix.right.{tensor}")
                if shape is not None and len(shape) == 2:
                    right[key] = int(shape[0])
            layer = KepevikLayer(type=layer.type, mixer=dict(layer.mixer, right=right), mlp=layer.mlp)
        layers.append(layer)
    return KepevikConfig(vocab=cfg.vocab, width=cfg.width, layers=tuple(layers), norm_eps=cfg.norm_eps,
                         embedding_scale=cfg.embedding_scale, eos_token_id=cfg.eos_token_id)


def _feed_forward_spec(cfg: KepevikConfig, mlp: Dict[str, Any]) -> PartSpec:
    if mlp["kind"] == "dense":
        return PartSpec("dense_gelu", dict(hidden_size=cfg.width, intermediate_size=mlp["ff"]))
    router = mlp["router"]
    return PartSpec("routed", dict(
        hidden_size=cfg.width, expert_size=mlp["expert"]["ff"], num_experts=router["experts"], top=router["top"],
        num_identity=int(router.get("identity", 0) or 0), shared_size=(mlp.get("shared") or {}).get("ff", 0),
    ))


def kepevik_model_spec(cfg: KepevikConfig) -> ModelSpec:
    """The model as data: one ``LayerSpec`` per layer, named ``l<i>`` as its tensors are."""
    def norm(offset=1.0, scaled=False):
        return PartSpec("rmsnorm", dict(size=cfg.width, eps=cfg.norm_eps, stream_dtype="float32", offset=offset, scaled=scaled))

    specs: List[LayerSpec] = []
    for i, layer in enumerate(cfg.layers):
        m = layer.mixer
        parts = {"norm1": norm(), "norm1b": norm(scaled=True)}
        params: Dict[str, Any] = {}
        if layer.type == "mlstm":
            block = "sandwich"
            parts["mix"] = PartSpec("matrix_memory", dict(
                hidden_size=cfg.width, num_heads=m["heads"], head_dim=m["dim"], v_head_dim=m["vdim"], gate_cap=float(m["gate_cap"]),
                norm_eps=cfg.norm_eps))
        else:
            block = "sandwich_pair"
            left, right = m["left"], m["right"]
            rot = left["rot"]
            position = PartSpec("rope", dict(head_dim=left["dim"], rotary_dim=rot["dims"], theta=float(rot["base"]), scaling=None,
                                             pairing="half")) if rot["dims"] > 0 else PartSpec("none", {})
            parts["left"] = PartSpec("attention", dict(
                hidden_size=cfg.width, num_heads=left["heads"], num_kv_heads=left["kv_heads"], head_dim=left["dim"], qkv_bias=False,
                softmax_scale=float(left["scale"]), window=0, position=position, values_from_keys=True))
            decay_rank, gate_rank = low_ranks(right)
            parts["right"] = PartSpec("gated_delta", dict(
                hidden_size=cfg.width, num_heads=right["heads"], num_key_heads=right["kv_heads"], head_dim=right["dim"],
                v_head_dim=right["vdim"], conv_taps=right["conv"], norm_eps=cfg.norm_eps, decay="channel", decay_rank=decay_rank,
                gate_rank=gate_rank, gate_act="sigmoid"))
            params = dict(left_scale=m["left_scale"], right_scale=m["right_scale"])
        if layer.mlp is not None:
            parts["norm2"] = norm()
            parts["norm2b"] = norm(scaled=True)
            parts["mlp"] = _feed_forward_spec(cfg, layer.mlp)
        else:
            block += "_mixer"
        specs.append(LayerSpec(name=f"l{i}", block=block, parts=parts, block_params=params))
    spec = ModelSpec(
        architecture=ARCHITECTURE,
        hidden_size=cfg.width,
        vocab_size=cfg.vocab,
        max_positions=DEFAULT_MAX_POSITIONS,
        embedding=PartSpec("embedding", dict(vocab_size=cfg.vocab, hidden_size=cfg.width, scale=cfg.embedding_scale,
                                             stream_dtype="float32")),
        layers=specs,
        order=[LayerRun(i) for i in range(len(specs))],
        final_norm=norm(),
        head=PartSpec("lm_head", dict(vocab_size=cfg.vocab, hidden_size=cfg.width, tied=True)),
    )
    spec.validate()
    return spec
