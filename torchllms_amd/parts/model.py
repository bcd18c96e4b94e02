"""Puts a model together from a ``ModelSpec`` and runs it over one step's tokens."""

from __future__ import annotations

from typing import Dict, List, Tuple

import torch

from ..config.spec import ModelSpec
from .base import BLOCKS, EMBEDDINGS, HEADS, NORMS, SLOT_KINDS, Block, ParamSpec, Part

# importing the modules registers the built-in parts
from . import attention as _attention  # noqa: F401
from . import blocks as _blocks  # noqa: F401
from . import embedding as _embedding  # noqa: F401
from . import feed_forward as _feed_forward  # noqa: F401
from . import latent as _latent  # noqa: F401
from . import norms as _norms  # noqa: F401
from . import positions as _positions  # noqa: F401
from . import recurrent as _recurrent  # noqa: F401


class Model:
    """Embedding, layers in the order the spec lists, final norm, output head.

    Tensor names: ``embed.<tensor>``, ``<layer name>.<slot>.<tensor>`` with the slots of the layer's
    block arrangement (``mixer_norm``, ``mixer``, ``ffn_norm``, ``ffn`` for a pre-norm block), then
    ``final_norm.<tensor>`` and ``head.<tensor>``.
    """

    def __init__(self, spec: ModelSpec):
        spec.validate()
        self.spec = spec
        self.embedding = EMBEDDINGS.build(spec.embedding)
        self.blocks: List[Block] = []
        for layer in spec.layers:
            if layer.block not in BLOCKS:
                raise KeyError(f"no block arrangement named {layer.block!r}; registered: {sorted(BLOCKS)}")
            block_cls = BLOCKS[layer.block]
            missing = [s for s in block_cls.SLOTS if s not in layer.parts]
            extra = [s for s in layer.parts if s not in block_cls.SLOTS]
            if missing or extra:
                raise ValueError(
                    f"{layer.name}: the arrangement {layer.block!r} has the parts {list(block_cls.SLOTS)}; "
                    f"the layer lacks {missing} and names {extra} that the arrangement does not have"
                )
            parts = {slot: SLOT_KINDS[kind].build(layer.parts[slot]) for slot, kind in block_cls.SLOTS.items()}
            self.blocks.append(block_cls(parts, **layer.block_params))
        self.final_norm = NORMS.build(spec.final_norm)
        self.head = HEADS.build(spec.head)
        # every arrangement learns which one follows it, where that is the same in all of its runs
        followers: Dict[int, set] = {}
        for pos, run in enumerate(spec.order):
            nxt = spec.order[pos + 1].layer if pos + 1 < len(spec.order) else None
            followers.setdefault(run.layer, set()).add(nxt)
        for layer, nexts in followers.items():
            only = next(iter(nexts)) if len(nexts) == 1 else None
            self.blocks[layer].expects(self.blocks[only] if only is not None else None)
        # per run: (slot of a mixer, name of one of the things it keeps or None, key of the cache entry, whether the run owns the entry)
        self._run_caches: List[List[tuple]] = []
        for run_id, run in enumerate(spec.order):
            src = run_id if run.cache_from is None else run.cache_from
            if run.cache_from is not None:
                theirs = set(self.blocks[spec.order[src].layer].mixers())
                mine = set(self.blocks[run.layer].mixers())
                if not mine <= theirs:
                    raise ValueError(
                        f"order[{run_id}] borrows the cache of order[{src}], whose layer has no mixer in the "
                        f"slots {sorted(mine - theirs)}"
                    )
            entries = []
            for slot, mixer in self.blocks[run.layer].mixers().items():
                need = mixer.cache_need()
                if not isinstance(need, dict):
                    entries.append((slot, None, (src, slot), run.cache_from is None))
                    continue
                # a mixer that keeps several things: in a run that borrows, the pages are the other run's and what
                # else the mixer keeps (state) is its own; what only the other run's mixer has is borrowed too
                names = dict(need)
                theirs = {}
                if run.cache_from is not None:
                    other = self.blocks[spec.order[src].layer].mixers()[slot].cache_need()
                    theirs = dict(other) if isinstance(other, dict) else {}
                for name in list(names) + [n for n in theirs if n not in names]:
                    borrowed = run.cache_from is not None and name in theirs and (name not in names or hasattr(names[name], "num_kv_heads"))
                    entries.append((slot, name, (src if borrowed else run_id, slot, name), not borrowed))
            self._run_caches.append(entries)

    def all_parts(self) -> List[Part]:
        """Every part of the model, blocks and their sub-parts included."""
        parts: List[Part] = [self.embedding, self.final_norm, self.head]
        for b in self.blocks:
            parts.append(b)
            parts.extend(b.sub_parts().values())
        return parts

    # ------------------------------------------------------------------ tensors
    def param_specs(self) -> Dict[str, ParamSpec]:
        out: Dict[str, ParamSpec] = {}
        for name, spec in self.embedding.param_specs().items():
            out[f"embed.{name}"] = spec
        for layer, block in zip(self.spec.layers, self.blocks):
            for name, spec in block.param_specs().items():
                out[f"{layer.name}.{name}"] = spec
        for name, spec in self.final_norm.param_specs().items():
            out[f"final_norm.{name}"] = spec
        for name, spec in self.head.param_specs().items():
            out[f"head.{name}"] = spec
        return out

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        """Hand every part its tensors (already on the device, in their final dtypes)."""

        def sub(prefix: str) -> Dict[str, torch.Tensor]:
            prefix = prefix + "."
            return {k[len(prefix):]: v for k, v in tensors.items() if k.startswith(prefix)}

        self.embedding.bind(sub("embed"))
        for layer, block in zip(self.spec.layers, self.blocks):
            block.bind(sub(layer.name))
        self.final_norm.bind(sub("final_norm"))
        self.head.bind(sub("head"))
        if getattr(self.head, "tied", False):
            self.head.tie(self.embedding)

    def ignorable_tensors(self) -> List[str]:
        """Names a checkpoint may hold without the model using them (``Part.ignorable_params``)."""
        out = [f"embed.{n}" for n in self.embedding.ignorable_params()]
        for layer, block in zip(self.spec.layers, self.blocks):
            for slot, part in block.sub_parts().items():
                out += [f"{layer.name}.{slot}.{n}" for n in part.ignorable_params()]
        out += [f"final_norm.{n}" for n in self.final_norm.ignorable_params()]
        out += [f"head.{n}" for n in self.head.ignorable_params()]
        return out

    def linear_weights(self):
        """All matrices of the model, grouped by (shape, use, result dtype or None): see
        ``Part.linear_weights``."""
        groups = {}
        for part in self.all_parts():
            for item in part.linear_weights():
                item = item if isinstance(item, tuple) else (item,)
                w = item[0]
                use = item[1] if len(item) > 1 else "plain"
                out_dtype = item[2] if len(item) > 2 else None
                if w is not None:
                    groups.setdefault((tuple(w.shape), use, out_dtype), []).append(w)
        return groups

    def check_sizes(self, dtype: torch.dtype) -> None:
        """Every part says whether kernels exist for its sizes (``Part.check_sizes``)."""
        for part in self.all_parts():
            part.check_sizes(dtype)

    # ------------------------------------------------------------------ cache
    def cache_needs(self) -> List[Tuple[Tuple[int, str], object]]:
        """``((run id, slot), need)`` for every mixer of every run that owns a cache entry."""
        needs = []
        for run_id, run in enumerate(self.spec.order):
            mixers = self.blocks[run.layer].mixers()
            for slot, name, key, owns in self._run_caches[run_id]:
                if not owns or key[0] != run_id:
                    continue
                need = mixers[slot].cache_need()
                needs.append((key, need if name is None else need[name]))
        return needs

    # ------------------------------------------------------------------ one step
    def forward(self, ctx, cache) -> torch.Tensor:
        """Run this step's tokens; returns float32 logits [len(ctx.logit_rows), vocab]."""
        h = self.embedding.forward(ctx.tokens)
        delta = None
        for run, entries in zip(self.spec.order, self._run_caches):
            views = {}
            for slot, name, key, writes in entries:
                if name is None:
                    views[slot] = cache.view(key, writes)
                else:
                    views.setdefault(slot, {})[name] = cache.view(key, writes)
            h, delta = self.blocks[run.layer].forward(h, delta, ctx, views)
        if ctx.logit_rows.numel() == 0:
            return torch.empty((0, self.spec.vocab_size), dtype=torch.float32, device=h.device)
        x = self.final_norm.forward_rows(h, self.final_norm.delta(delta), ctx.logit_rows)
        return self.head.forward(x)
