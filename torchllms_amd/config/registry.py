"""One registry from an architecture's name (``config.json["architectures"][0]``) to
everything the engine needs to run it.

The reference picks its model class with if/elif on flags of ``ModelParams``
(reference: torchllms/models/networks.py:779-788) and sniffs the architecture name
while converting checkpoints (torchllms/models/checkpoint_converter.py:323-327); here the
name in config.json is the only key.
"""

from __future__ import annotations

import json
from dataclasses import dataclass
from pathlib import Path
from typing import Any, Callable, Dict, List, Optional, Sequence

from .llama import ConfigError, LlamaConfig, llama_model_spec
from .spec import ModelSpec
from .taluvik import ARCHITECTURE as TALUVIK, TaluvikConfig, taluvik_model_spec
from .vobolorn import ARCHITECTURE as VOBOLORN, VobolornConfig, vobolorn_model_spec
from .kepevik import ARCHITECTURE as KEPEVIK, KepevikConfig, kepevik_model_spec, kepevik_sizes_from_tensors
from .nosuzen import ARCHITECTURE as NOSUZEN, NosuzenConfig, nosuzen_model_spec, nosuzen_sizes_from_tensors


@dataclass(frozen=True)
class ArchSpec:
    """What an architecture registers.

    ``config_from_dict``  config.json contents -> typed configuration
    ``model_spec``        typed configuration  -> ``ModelSpec`` (parts, sizes, order)
    ``weight_rules``      typed configuration  -> list of ``weights.names.NameRule`` that map
                          checkpoint tensor names to the parts' own names
    """

    name: str
    config_from_dict: Callable[[Dict[str, Any]], Any]
    model_spec: Callable[[Any], ModelSpec]
    weight_rules: Callable[[Any], List[Any]]
    #: typed configuration -> the token ids that end a generation when the caller names none
    #: (the checkpoint's end-of-sequence ids); None: the architecture has none to offer
    stop_token_ids: Optional[Callable[[Any], Sequence[int]]] = None
    #: the class of the typed configuration, so that a configuration alone (no folder, no
    #: config.json) finds its architecture: ``architecture_of``
    config_type: Optional[type] = None

    #: typed configuration -> the contents of a config.json that ``config_from_dict`` reads back
    #: (None: the configuration's own ``to_dict()``, or its fields if it is a dataclass)
    config_to_dict: Optional[Callable[[Any], Dict[str, Any]]] = None

    #: (typed configuration, tensor name -> shape of the folder's tensors) -> typed configuration: for an
    #: architecture some of whose sizes config.json leaves to the tensors' shapes (None: config.json says all)
    sizes_from_tensors: Optional[Callable[[Any, Dict[str, tuple]], Any]] = None

    def config_json(self, config) -> Dict[str, Any]:
        """What a model folder's config.json holds for this configuration; it names this architecture."""
        if self.config_to_dict is not None:
            d = dict(self.config_to_dict(config))
        elif hasattr(config, "to_dict"):
            d = dict(config.to_dict())
        else:
            import dataclasses

            d = dataclasses.asdict(config)
        if not d.get("architectures") and not d.get("architecture"):
            d["architectures"] = [self.name]
        return d

    def default_stop_token_ids(self, config) -> List[int]:
        return [] if self.stop_token_ids is None else [int(t) for t in self.stop_token_ids(config)]


ARCHITECTURES: Dict[str, ArchSpec] = {}


def register_architecture(arch: ArchSpec) -> ArchSpec:
    ARCHITECTURES[arch.name] = arch
    return arch


def get_architecture(name: str) -> ArchSpec:
    try:
        return ARCHITECTURES[name]
    except KeyError:
        raise ConfigError(
            f"architecture {name!r} is not registered; registered: {sorted(ARCHITECTURES)}"
        ) from None


def architecture_of(config) -> ArchSpec:
    """The registered architecture of a typed configuration: the one whose ``config_type`` is the
    configuration's class.  Where several share a class (or none names one) the configuration has
    to say which it is, by an ``architectures`` attribute as config.json has."""
    matches = [a for a in ARCHITECTURES.values() if a.config_type is not None and type(config) is a.config_type]
    if len(matches) == 1:
        return matches[0]
    names = getattr(config, "architectures", None)
    if names:
        return get_architecture(names[0])
    raise ConfigError(
        f"no registered architecture names {type(config).__name__} as its config_type, and the configuration "
        f"has no 'architectures' entry; registered: {sorted(ARCHITECTURES)}"
    )


def architecture_name(config_dict: Dict[str, Any]) -> str:
    """The architecture a config.json names: the first of "architectures", or the string "architecture"."""
    archs = config_dict.get("architectures")
    if archs:
        return archs[0]
    one = config_dict.get("architecture")
    if isinstance(one, str) and one:
        return one
    raise ConfigError('config.json names no architecture ("architectures" or "architecture")')


def load_config(folder) -> tuple:
    """Read ``folder/config.json``; return ``(ArchSpec, typed configuration)``."""
    path = Path(folder) / "config.json"
    if not path.is_file():
        raise FileNotFoundError(f"{path} not found")
    with open(path) as f:
        d = json.load(f)
    arch = get_architecture(architecture_name(d))
    config = arch.config_from_dict(d)
    if arch.sizes_from_tensors is not None:
        from ..weights.loader import safetensors_files, tensor_shapes

        try:
            safetensors_files(folder)
        except FileNotFoundError:
            return arch, config  # a folder with a configuration alone: the sizes stay as config.json and defaults give them
        config = arch.sizes_from_tensors(config, tensor_shapes(folder))
    return arch, config


def _llama_rules(cfg: LlamaConfig):
    from ..weights.names import llama_name_rules

    return llama_name_rules(cfg)


def _llama_stop_ids(cfg: LlamaConfig):
    """config.json's ``eos_token_id``: one id or a list (reference: llm.py:188-200 falls back to the
    tokenizer's eos id, which is this id for the checkpoints it loads)."""
    eos = cfg.eos_token_id
    return [] if eos is None else (list(eos) if isinstance(eos, (list, tuple)) else [eos])


register_architecture(
    ArchSpec(
        name="LlamaForCausalLM",
        config_from_dict=LlamaConfig.from_dict,
        model_spec=llama_model_spec,
        weight_rules=_llama_rules,
        stop_token_ids=_llama_stop_ids,
        config_type=LlamaConfig,
    )
)


def _taluvik_rules(cfg: TaluvikConfig):
    from ..weights.names import taluvik_name_rules

    return taluvik_name_rules(cfg)


def _taluvik_stop_ids(cfg: TaluvikConfig):
    eos = cfg.eos_token_id
    return [] if eos is None else (list(eos) if isinstance(eos, (list, tuple)) else [eos])


register_architecture(
    ArchSpec(
        name=TALUVIK,
        config_from_dict=TaluvikConfig.from_dict,
        model_spec=taluvik_model_spec,
        weight_rules=_taluvik_rules,
        stop_token_ids=_taluvik_stop_ids,
        config_type=TaluvikConfig,
    )
)


def _vobolorn_rules(cfg: VobolornConfig):
    from ..weights.names import vobolorn_name_rules

    return vobolorn_name_rules(cfg)


def _vobolorn_stop_ids(cfg: VobolornConfig):
    eos = cfg.eos_token_id
    return [] if eos is None else (list(eos) if isinstance(eos, (list, tuple)) else [eos])


register_architecture(
    ArchSpec(
        name=VOBOLORN,
        config_from_dict=VobolornConfig.from_dict,
        model_spec=vobolorn_model_spec,
        weight_rules=_vobolorn_rules,
        stop_token_ids=_vobolorn_stop_ids,
        config_type=VobolornConfig,
    )
)


def _kepevik_rules(cfg: KepevikConfig):
    from ..weights.names import kepevik_name_rules

    return kepevik_name_rules(cfg)


def _kepevik_stop_ids(cfg: KepevikConfig):
    eos = cfg.eos_token_id
    return [] if eos is None else (list(eos) if isinstance(eos, (list, tuple)) else [eos])


register_architecture(
    ArchSpec(
        name=KEPEVIK,
        config_from_dict=KepevikConfig.from_dict,
        model_spec=kepevik_model_spec,
        weight_rules=_kepevik_rules,
        stop_token_ids=_kepevik_stop_ids,
        config_type=KepevikConfig,
        sizes_from_tensors=kepevik_sizes_from_tensors,
    )
)


def _nosuzen_rules(cfg: NosuzenConfig):
    from ..weights.names import nosuzen_name_rules

    return nosuzen_name_rules(cfg)


def _nosuzen_stop_ids(cfg: NosuzenConfig):
    eos = cfg.eos_token_id
    return [] if eos is None else (list(eos) if isinstance(eos, (list, tuple)) else [eos])


register_architecture(
    ArchSpec(
        name=NOSUZEN,
        config_from_dict=NosuzenConfig.from_dict,
        model_spec=nosuzen_model_spec,
        weight_rules=_nosuzen_rules,
        stop_token_ids=_nosuzen_stop_ids,
        config_type=NosuzenConfig,
        sizes_from_tensors=nosuzen_sizes_from_tensors,
    )
)
