"""Tensor-name rules: checkpoint names -> the parts' own names, with re-layouts.

Two spellings of the Llama 3 decoder are accepted:

* the checkpoint's own (``model.layers.3.self_attn.q_proj.weight`` ...), whose q/k rows are
  laid out for half-split rotary pairs ``(i, i + head_dim/2)``;
* the reference's internal one (``layers.3.attention.wq.weight`` ...), whose q/k rows are
  already laid out for interleaved pairs ``(2i, 2i+1)``.

The name table and the row permutation restate
reference: torchllms/models/checkpoint_converter.py:96-108 (permute), 124-141 (names),
199-229 (inverse).  The engine rotates interleaved pairs (reference:
torchllms/models/networks.py:332-352), so checkpoint-spelled q/k tensors are permuted on load.
"""

from __future__ import annotations

import re
from dataclasses import dataclass
from typing import Callable, List, Optional, Tuple

import torch


def half_split_to_interleaved(w: torch.Tensor, n_heads: int, head_dim: int) -> torch.Tensor:
    """Reorder rows of a q/k projection (or entries of its bias) so that the element that sat
    at offset ``i`` / ``i + head_dim/2`` of each head sits at ``2i`` / ``2i + 1``."""
    if w.shape[0] != n_heads * head_dim:
        raise ValueError(f"expected leading size {n_heads * head_dim}, got {tuple(w.shape)}")
    rest = w.shape[1:]
    return w.reshape(n_heads, 2, head_dim // 2, *rest).transpose(1, 2).reshape(n_heads * head_dim, *rest)


def interleaved_to_half_split(w: torch.Tensor, n_heads: int, head_dim: int) -> torch.Tensor:
    """Inverse of :func:`half_split_to_interleaved`."""
    if w.shape[0] != n_heads * head_dim:
        raise ValueError(f"expected leading size {n_heads * head_dim}, got {tuple(w.shape)}")
    rest = w.shape[1:]
    return w.reshape(n_heads, head_dim // 2, 2, *rest).transpose(1, 2).reshape(n_heads * head_dim, *rest)


@dataclass(frozen=True)
class NameRule:
    """``external`` and ``internal`` are patterns in which ``{}`` stands for a layer index.

    ``load`` re-lays a tensor out on the way in, ``save`` on the way out (both None: as is).
    ``internal=None`` means: a tensor of this name is known and dropped.
    """

    external: str
    internal: Optional[str]
    load: Optional[Callable[[torch.Tensor], torch.Tensor]] = None
    save: Optional[Callable[[torch.Tensor], torch.Tensor]] = None

    def _regex(self, pattern: str) -> "re.Pattern":
        return re.compile("^" + re.escape(pattern).replace(re.escape("{}"), r"(\d+)") + "$")

    def match_external(self, name: str) -> Optional[Tuple[Optional[str]]]:
        m = self._regex(self.external).match(name)
        if m is None:
            return None
        if self.internal is None:
            return (None,)
        return (self.internal.format(*m.groups()),)

    def match_internal(self, name: str) -> Optional[str]:
        if self.internal is None:
            return None
        m = self._regex(self.internal).match(name)
        if m is None:
            return None
        return self.external.format(*m.groups())


def llama_name_rules(cfg) -> List[NameRule]:
    """Rules for both spellings.  The checkpoint spelling comes first, so it is the one
    used when a model folder is written."""
    hq, hkv, dh = cfg.num_attention_heads, cfg.num_key_value_heads, cfg.head_dim

    def perm(h):
        return (
            lambda w: half_split_to_interleaved(w, h, dh),
            lambda w: interleaved_to_half_split(w, h, dh),
        )

    q_in, q_out = perm(hq)
    k_in, k_out = perm(hkv)
    L = "model.layers.{}."
    I = "layers.{}."
    rules = [
        NameRule("model.embed_tokens.weight", "embed.weight"),
        NameRule(L + "self_attn.q_proj.weight", I + "mixer.wq.weight", q_in, q_out),
        NameRule(L + "self_attn.q_proj.bias", I + "mixer.wq.bias", q_in, q_out),
        NameRule(L + "self_attn.k_proj.weight", I + "mixer.wk.weight", k_in, k_out),
        NameRule(L + "self_attn.k_proj.bias", I + "mixer.wk.bias", k_in, k_out),
        NameRule(L + "self_attn.v_proj.weight", I + "mixer.wv.weight"),
        NameRule(L + "self_attn.v_proj.bias", I + "mixer.wv.bias"),
        NameRule(L + "self_attn.o_proj.weight", I + "mixer.wo.weight"),
        NameRule(L + "self_attn.rotary_emb.inv_freq", None),
        NameRule(L + "mlp.gate_proj.weight", I + "ffn.w1.weight"),
        NameRule(L + "mlp.up_proj.weight", I + "ffn.w3.weight"),
        NameRule(L + "mlp.down_proj.weight", I + "ffn.w2.weight"),
        NameRule(L + "input_layernorm.weight", I + "mixer_norm.weight"),
        NameRule(L + "post_attention_layernorm.weight", I + "ffn_norm.weight"),
        NameRule("model.norm.weight", "final_norm.weight"),
        NameRule("lm_head.weight", "head.weight"),
        # the reference's internal spelling, taken as is
        NameRule("tok_embeddings.weight", "embed.weight"),
        NameRule(I + "attention.wq.weight", I + "mixer.wq.weight"),
        NameRule(I + "attention.wq.bias", I + "mixer.wq.bias"),
        NameRule(I + "attention.wk.weight", I + "mixer.wk.weight"),
        NameRule(I + "attention.wk.bias", I + "mixer.wk.bias"),
        NameRule(I + "attention.wv.weight", I + "mixer.wv.weight"),
        NameRule(I + "attention.wv.bias", I + "mixer.wv.bias"),
        NameRule(I + "attention.wo.weight", I + "mixer.wo.weight"),
        NameRule(I + "feed_forward.w1.weight", I + "ffn.w1.weight"),
        NameRule(I + "feed_forward.w3.weight", I + "ffn.w3.weight"),
        NameRule(I + "feed_forward.w2.weight", I + "ffn.w2.weight"),
        NameRule(I + "attention_norm.weight", I + "mixer_norm.weight"),
        NameRule(I + "ffn_norm.weight", I + "ffn_norm.weight"),
        NameRule("norm.weight", "final_norm.weight"),
        NameRule("output.weight", "head.weight"),
    ]
    return rules


def taluvik_name_rules(cfg) -> List[NameRule]:
    """Taluvik checkpoints name a layer's tensors ``l<i>.norm1[.b]``, ``l<i>.mix.<tensor>`` and
    ``l<i>.mlp.{gate,up,down}``; the parts' own names differ only where a part is shared with other
    architectures (the norm, the attention, the gated feed-forward)."""
    L = "l{}."
    rules = [
        NameRule("embed", "embed.weight"),
        NameRule("final.norm", "final_norm.weight"),
        NameRule("final.norm.b", "final_norm.bias"),
        NameRule("head", "head.weight"),
        NameRule(L + "norm1", L + "norm1.weight"),
        NameRule(L + "norm1.b", L + "norm1.bias"),
        NameRule(L + "mlp.gate", L + "mlp.w1.weight"),
        NameRule(L + "mlp.up", L + "mlp.w3.weight"),
        NameRule(L + "mlp.down", L + "mlp.w2.weight"),
    ]
    kinds = {layer.type for layer in cfg.layers}
    attention = {"q": "wq.weight", "k": "wk.weight", "v": "wv.weight", "o": "wo.weight", "sink": "sinks"}
    recurrent = ["in", "conv", "conv.b", "x", "dt", "dt.b", "A_log", "D", "o", "q", "q.conv", "k", "k.conv", "v", "v.conv",
                 "b", "a", "dt_bias", "norm", "g"]
    # a tensor's name alone does not say which mixer it belongs to (every mixer has an "o"): the rules are
    # written per layer, from the layer's type
    for i, layer in enumerate(cfg.layers):
        if layer.weights_of is not None:
            continue
        p = f"l{i}.mix."
        if layer.type == "attention":
            rules += [NameRule(p + ext, p + own) for ext, own in attention.items()]
        else:
            rules += [NameRule(p + n, p + n) for n in recurrent]
    return rules


def vobolorn_name_rules(cfg) -> List[NameRule]:
    """Vobolorn checkpoints name a layer's tensors ``l<i>.norm1``, ``l<i>.norm2``, ``l<i>.mix.<tensor>`` (a bias
    is the tensor's name with ``.b``, a norm inside the mixer ``<tensor>.norm``) and ``l<i>.mlp.{gate,up,down}``.
    The rules are written per layer, from the layer's type: the mixers share names (every one has an ``o``)."""
    L = "l{}."
    rules = [
        NameRule("embed", "embed.weight"),
        NameRule("final.norm", "final_norm.weight"),
        NameRule("head", "head.weight"),
        NameRule(L + "norm1", L + "norm1.weight"),
        NameRule(L + "norm2", L + "norm2.weight"),
        NameRule(L + "mlp.gate", L + "mlp.w1.weight"),
        NameRule(L + "mlp.up", L + "mlp.w3.weight"),
        NameRule(L + "mlp.down", L + "mlp.w2.weight"),
    ]
    grouped = {"q": "wq.weight", "k": "wk.weight", "v": "wv.weight", "o": "wo.weight", "q.b": "wq.bias", "k.b": "wk.bias",
               "v.b": "wv.bias", "q.norm": "q_norm.weight", "k.norm": "k_norm.weight", "vmix": "vmix", "g": "wg.weight"}
    latent = {"dq": "dq.weight", "dq.norm": "dq_norm.weight", "uq": "uq.weight", "dkv": "dkv.weight", "dkv.norm": "dkv_norm.weight",
              "uk": "uk.weight", "uv": "uv.weight", "g": "wg.weight", "o": "wo.weight"}
    for i, layer in enumerate(cfg.layers):
        p = f"l{i}.mix."
        names = latent if layer.type == "latent_attention" else grouped
        rules += [NameRule(p + ext, p + own) for ext, own in names.items()]
    return rules


def kepevik_name_rules(cfg) -> List[NameRule]:
    """Kepevik checkpoints name a layer's tensors ``l<i>.norm1``, ``norm1b``, ``norm2``, ``norm2b`` (the norms before
    and behind the two branches), ``l<i>.ls1`` and ``ls2`` (the layer scales, which belong to the norms behind the
    branches here), ``l<i>.mix.<tensor>`` (a parallel layer: ``l<i>.mix.left.<tensor>`` and ``mix.right.<tensor>``) and
    ``l<i>.mlp.<tensor>`` (a mixture: ``mlp.e<j>.{gate,up,down}``, ``mlp.router``, ``mlp.correction``,
    ``mlp.shared.{gate,up,down,sg}``); a bias is the tensor's name with ``.b``.  The output head is the embedding."""
    L = "l{}."
    rules = [
        NameRule("embed", "embed.weight"),
        NameRule("final.norm", "final_norm.weight"),
        NameRule(L + "norm1", L + "norm1.weight"),
        NameRule(L + "norm1b", L + "norm1b.weight"),
        NameRule(L + "ls1", L + "norm1b.scale"),
        NameRule(L + "norm2", L + "norm2.weight"),
        NameRule(L + "norm2b", L + "norm2b.weight"),
        NameRule(L + "ls2", L + "norm2b.scale"),
        NameRule(L + "mlp.up", L + "mlp.up.weight"),
        NameRule(L + "mlp.up.b", L + "mlp.up.bias"),
        NameRule(L + "mlp.down", L + "mlp.down.weight"),
        NameRule(L + "mlp.down.b", L + "mlp.down.bias"),
        NameRule(L + "mlp.router", L + "mlp.router.weight"),
        NameRule(L + "mlp.correction", L + "mlp.correction"),
        NameRule(L + "mlp.e{}.gate", L + "mlp.experts.{}.w1.weight"),
        NameRule(L + "mlp.e{}.up", L + "mlp.experts.{}.w3.weight"),
        NameRule(L + "mlp.e{}.down", L + "mlp.experts.{}.w2.weight"),
        NameRule(L + "mlp.shared.gate", L + "mlp.shared.w1.weight"),
        NameRule(L + "mlp.shared.up", L + "mlp.shared.w3.weight"),
        NameRule(L + "mlp.shared.down", L + "mlp.shared.w2.weight"),
        NameRule(L + "mlp.shared.sg", L + "mlp.shared.gate.weight"),
    ]
    memory = ["q", "k", "v", "g", "o", "norm", "i", "i.b", "f", "f.b"]
    left = {"q": "wq.weight", "k": "wk.weight", "o": "wo.weight"}
    right = ["q", "q.conv", "k", "k.conv", "v", "v.conv", "b", "A_log", "norm", "a1", "a2", "dt_bias", "g1", "g2", "o"]
    for i, layer in enumerate(cfg.layers):
        p = f"l{i}.mix."
        if layer.type == "mlstm":
            rules += [NameRule(p + n, p + n) for n in memory]
        else:
            rules += [NameRule(p + "left." + ext, f"l{i}.left." + own) for ext, own in left.items()]
            rules += [NameRule(p + "right." + n, f"l{i}.right." + n) for n in right]
    return rules


def nosuzen_name_rules(cfg) -> List[NameRule]:
    """Nosuzen checkpoints name a layer's tensors ``l<i>.norm1`` and ``l<i>.norm2`` (with ``.b`` and ``.alpha`` beside the
    weight), ``l<i>.hc1.{in,out,mix}`` and ``hc2`` (the streams' read, write and mixing weights of the two sublayers),
    ``l<i>.mix.<tensor>`` (a parallel layer: ``mix.left.<tensor>`` and ``mix.right.<tensor>``; a convolution's taps are
    ``<tensor>.conv``, a norm inside a mixer ``<tensor>.norm``, a bias ``<tensor>.b``) and ``l<i>.mlp.e<j>.{gate,up,down}``,
    ``mlp.router``, ``mlp.shared.{gate,up,down}``; beside them ``embed``, ``final.norm`` (+ ``.b``, ``.alpha``) and ``head``."""
    L = "l{}."
    rules = [
        NameRule("embed", "embed.weight"),
        NameRule("head", "head.weight"),
        NameRule("final.norm", "final_norm.weight"),
        NameRule("final.norm.b", "final_norm.bias"),
        NameRule("final.norm.alpha", "final_norm.alpha"),
        NameRule(L + "mlp.router", L + "mlp.router.weight"),
        NameRule(L + "mlp.e{}.gate", L + "mlp.experts.{}.w1.weight"),
        NameRule(L + "mlp.e{}.up", L + "mlp.experts.{}.w3.weight"),
        NameRule(L + "mlp.e{}.down", L + "mlp.experts.{}.w2.weight"),
        NameRule(L + "mlp.shared.gate", L + "mlp.shared.w1.weight"),
        NameRule(L + "mlp.shared.up", L + "mlp.shared.w3.weight"),
        NameRule(L + "mlp.shared.down", L + "mlp.shared.w2.weight"),
    ]
    for q in ("1", "2"):
        rules += [NameRule(L + "norm" + q, L + "norm" + q + ".weight"), NameRule(L + "norm" + q + ".b", L + "norm" + q + ".bias"),
                  NameRule(L + "norm" + q + ".alpha", L + "norm" + q + ".alpha")]
        rules += [NameRule(L + "hc" + q + "." + n, L + "hc" + q + "." + n) for n in ("in", "out", "mix")]
    differential = ["q", "k", "v", "q.conv", "k.conv", "v.conv", "lq1", "lk1", "lq2", "lk2", "o"]
    latent = {"q": "q.weight", "dkv": "dkv.weight", "dkv.norm": "dkv_norm.weight", "uk": "uk.weight", "uv": "uv.weight", "o": "wo.weight"}
    left = {"q": "wq.weight", "k": "wk.weight", "v": "wv.weight", "q.norm": "q_norm.weight", "k.norm": "k_norm.weight", "o": "wo.weight"}
    right = ["q", "k", "v", "g", "o", "norm", "a1", "a2", "a2.b"]
    for i, layer in enumerate(cfg.layers):
        p = f"l{i}.mix."
        if layer.type == "attention":
            rules += [NameRule(p + n, p + n) for n in differential]
        elif layer.type == "latent_attention":
            rules += [NameRule(p + ext, p + own) for ext, own in latent.items()]
        else:
            rules += [NameRule(p + "left." + ext, f"l{i}.left." + own) for ext, own in left.items()]
            rules += [NameRule(p + "right." + n, f"l{i}.right." + n) for n in right]
    return rules
