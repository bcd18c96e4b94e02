"""Grouped-query attention over paged keys and values."""

from __future__ import annotations

import logging
from typing import Dict, Optional

import torch

from ..config.spec import PartSpec
from ..kernels import ops
from ..kernels.attention import paged_attention
from .base import MIXERS, POSITIONS, KVNeed, Mixer, ParamSpec


#: (heads, kv heads, head size) whose fall to the plain attention kernel has been reported
_SAID_SLOW: set = set()


@MIXERS.register("attention")
class Attention(Mixer):
    """q/k/v projections, position encoding on q and k, keys and values appended to the cache,
    causal attention of the new queries over everything cached for their request, output
    projection (reference: torchllms/models/networks.py:460-558; plain formula 355-397).

    Query head h reads key/value head ``h // (num_heads / num_kv_heads)``.  ``window`` w > 0
    limits a query at position p to keys p-w+1..p.  ``shares_kv``: this layer has no k/v
    projections and reads the cache of the run named by the execution order.  ``kv_page_size``:
    tokens per page of this layer's keys and values, when not the engine's own (layers that ask for
    the same form a group of pages of their own).  ``v_head_dim``: the values' head size when it is
    not the keys'.  ``qk_norm_eps`` > 0: after the rotation every query and key head is divided by its
    root mean square (eps under the root, no weight).  ``softcap`` c > 0: scores become
    c tanh(score / c).  ``chunk`` n > 0: a query sees only the keys of its own chunk of n positions,
    chunks counted from position 0.  ``sinks``: a learned number per query head (tensor ``sinks``)
    whose exponential joins the softmax's denominator, with no value behind it.

    Heads prepared before the scores (any of these takes the layer through ``ops.head_prepare``):
    ``qk_norm_weight``: the norm of queries and keys has a weight per channel (tensors ``q_norm.weight`` and
    ``k_norm.weight`` of the head size, shared by the heads) and stands before the rotation;
    ``q_temp_coef`` c != 0: the query at position p is multiplied by ``1 + c ln(floor((p + 1) / q_temp_every) + 1)``;
    ``value_mix``: "source" leaves this step's values where later layers find them (under ``value_mix_key``),
    "mix" turns its values into ``(1 - m) v + m v_source`` of the same token before they are cached (``m``: the
    tensor ``vmix``, one number); ``out_gate``: the heads' outputs are multiplied by the sigmoid of a projection of
    the layer's input (tensor ``wg.weight``), "channel" by channel or "head" by head.

    ``values_from_keys``: there is no value projection; a token's values are its keys as projected, before the
    rotation (the key rows of the fused projection stand in it a second time as value rows).
    """

    #: every launch is fixed by the step's shape: a decode step may be recorded in a HIP graph
    graph_safe = True
    takes_normed_rows = True

    def __init__(
        self,
        hidden_size: int,
        num_heads: int,
        num_kv_heads: int,
        head_dim: int,
        qkv_bias: bool,
        softmax_scale: float,
        window: int,
        position: PartSpec,
        shares_kv: bool = False,
        kv_page_size: Optional[int] = None,
        v_head_dim: Optional[int] = None,
        qk_norm_eps: float = 0.0,
        softcap: float = 0.0,
        chunk: int = 0,
        sinks: bool = False,
        qk_norm_weight: bool = False,
        q_temp_coef: float = 0.0,
        q_temp_every: int = 1,
        value_mix: Optional[str] = None,
        value_mix_key: str = "values",
        out_gate: Optional[str] = None,
        values_from_keys: bool = False,
    ):
        self.values_from_keys = bool(values_from_keys)
        if self.values_from_keys and (shares_kv or (v_head_dim and v_head_dim != head_dim) or qkv_bias):
            raise ValueError("attention: values that are the keys have the keys' head size, no bias, and a cache of their own")
        if num_heads % num_kv_heads:
            raise ValueError(f"{num_heads} heads are not a multiple of {num_kv_heads} kv heads")
        self.hidden_size = hidden_size
        self.num_heads = num_heads
        self.num_kv_heads = num_kv_heads
        self.head_dim = head_dim
        self.qkv_bias = qkv_bias
        self.softmax_scale = float(softmax_scale)
        self.window = int(window)
        self.shares_kv = shares_kv
        self.kv_page_size = kv_page_size
        self.v_head_dim = int(v_head_dim) if v_head_dim else head_dim
        self.qk_norm_eps = float(qk_norm_eps)
        self.softcap = float(softcap)
        self.chunk = int(chunk)
        self.has_sinks = bool(sinks)
        if self.qk_norm_eps < 0 or self.softcap < 0 or self.chunk < 0:
            raise ValueError("attention: qk_norm_eps, softcap and chunk must not be negative")
        self.qk_norm_weight = bool(qk_norm_weight)
        self.q_temp_coef = float(q_temp_coef)
        self.q_temp_every = int(q_temp_every)
        self.value_mix = value_mix
        self.value_mix_key = value_mix_key
        self.out_gate = out_gate
        if value_mix not in (None, "source", "mix") or out_gate not in (None, "channel", "head"):
            raise ValueError("attention: value_mix is None, \"source\" or \"mix\"; out_gate is None, \"channel\" or \"head\"")
        if self.qk_norm_weight and not self.qk_norm_eps > 0:
            raise ValueError("attention: a weighted norm of queries and keys needs qk_norm_eps > 0")
        if self.q_temp_coef != 0.0 and self.q_temp_every <= 0:
            raise ValueError("attention: q_temp_every must be positive")
        if value_mix is not None and shares_kv:
            raise ValueError("attention: a layer without values of its own cannot mix them")
        self.q_norm: Optional[torch.Tensor] = None
        self.k_norm: Optional[torch.Tensor] = None
        self.vmix: Optional[torch.Tensor] = None
        if qkv_bias and self.extended and not self.prepared:
            raise ValueError("attention: q/k/v biases together with a unit norm, capped scores, chunks, sinks or values of their own size are not built")
        self.sinks: Optional[torch.Tensor] = None
        self.position = POSITIONS.build(position)
        self.wqkv: Optional[torch.Tensor] = None
        self.bqkv: Optional[torch.Tensor] = None
        self.wo: Optional[torch.Tensor] = None

    @property
    def prepared(self) -> bool:
        """Whether the heads go through ``ops.head_prepare`` (weighted norm, query factor, mixed values, gate)."""
        return self.qk_norm_weight or self.q_temp_coef != 0.0 or self.value_mix is not None or self.out_gate is not None

    @property
    def gate_rows(self) -> int:
        return 0 if self.out_gate is None else (self.num_heads * self.v_head_dim if self.out_gate == "channel" else self.num_heads)

    @property
    def extended(self) -> bool:
        """Whether the layer needs what only the unfused path and the plain attention kernel do."""
        return (self.v_head_dim != self.head_dim or self.qk_norm_eps > 0 or self.softcap > 0 or self.chunk > 0 or self.has_sinks)

    def param_specs(self) -> Dict[str, ParamSpec]:
        q = self.num_heads * self.head_dim
        kv = self.num_kv_heads * self.head_dim
        specs = {"wq.weight": ParamSpec((q, self.hidden_size)),
                 "wo.weight": ParamSpec((self.hidden_size, self.num_heads * self.v_head_dim))}
        if not self.shares_kv:
            specs["wk.weight"] = ParamSpec((kv, self.hidden_size))
            if not self.values_from_keys:
                specs["wv.weight"] = ParamSpec((self.num_kv_heads * self.v_head_dim, self.hidden_size))
        if self.has_sinks:
            specs["sinks"] = ParamSpec((self.num_heads,), kind="vector", init="zeros")
        if self.qkv_bias:
            specs["wq.bias"] = ParamSpec((q,), init="zeros")
            if not self.shares_kv:
                specs["wk.bias"] = ParamSpec((kv,), init="zeros")
                specs["wv.bias"] = ParamSpec((self.num_kv_heads * self.v_head_dim,), init="zeros")
        if self.qk_norm_weight:
            specs["q_norm.weight"] = ParamSpec((self.head_dim,), kind="vector", init="ones")
            if not self.shares_kv:
                specs["k_norm.weight"] = ParamSpec((self.head_dim,), kind="vector", init="ones")
        if self.value_mix == "mix":
            specs["vmix"] = ParamSpec((), kind="vector", init="fraction")
        if self.out_gate is not None:
            specs["wg.weight"] = ParamSpec((self.gate_rows, self.hidden_size))
        return specs

    def ignorable_params(self):
        # the layer whose values the others lean on may carry a mixing factor that it has no use for
        return ["vmix"] if self.value_mix == "source" else []

    def check_sizes(self, dtype: torch.dtype) -> None:
        if not 0 < self.v_head_dim <= ops.ATTENTION_MAX_HEAD_DIM:
            raise ValueError(f"attention: values of head size {self.v_head_dim}; the attention kernels take up to {ops.ATTENTION_MAX_HEAD_DIM}")
        if not 0 < self.head_dim <= ops.ATTENTION_MAX_HEAD_DIM:
            raise ValueError(
                f"attention: head size {self.head_dim}; the attention kernels take head sizes up to "
                f"{ops.ATTENTION_MAX_HEAD_DIM} (any number of heads and of query heads per kv head)"
            )
        if dtype == torch.bfloat16 and not self.extended:
            fast = (ops.decode_attention_supported(dtype, self.num_heads, self.num_kv_heads, self.head_dim),
                    ops.prefill_attention_supported(dtype, self.num_heads, self.num_kv_heads, self.head_dim))
            said = (self.num_heads, self.num_kv_heads, self.head_dim)
            if not all(fast) and said not in _SAID_SLOW:
                _SAID_SLOW.add(said)
                logging.getLogger("torchllms_amd").warning(
                    "attention with %d heads in %d groups of head size %d: the matrix-core kernels take head sizes %s with at "
                    "most 16 query heads per kv head (8 at head size 256 in decode steps); %s run the plain kernel (right, and several times slower)",
                    self.num_heads, self.num_kv_heads, self.head_dim, "/".join(str(d) for d in ops.DECODE_HEAD_DIMS),
                    "decode steps and prompts" if not any(fast) else "decode steps" if not fast[0] else "prompts",
                )
        rot = self.position.rotary_args()
        if rot is not None and (rot.rotary_dim % 2 or rot.rotary_dim > self.head_dim):
            raise ValueError(f"attention: {rot.rotary_dim} rotated channels of a head of {self.head_dim} (even, at most the head size)")

    def cache_need(self):
        if self.shares_kv:
            return None
        return KVNeed(num_kv_heads=self.num_kv_heads, head_dim=self.head_dim, window=self.window, page_size=self.kv_page_size,
                      v_head_dim=self.v_head_dim if self.v_head_dim != self.head_dim else None)

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        names = ["wq"] if self.shares_kv else ["wq", "wk", "wk" if self.values_from_keys else "wv"]
        # one fused projection [q rows | k rows | v rows | gate rows]: a single matrix product per token batch
        self.wqkv = torch.cat([tensors[f"{n}.weight"] for n in names + (["wg"] if self.out_gate else [])], dim=0).contiguous()
        if self.qk_norm_weight:
            self.q_norm = tensors["q_norm.weight"].float().contiguous()
            self.k_norm = None if self.shares_kv else tensors["k_norm.weight"].float().contiguous()
        if self.value_mix == "mix":
            self.vmix = tensors["vmix"].float().reshape(1).contiguous()
        if self.qkv_bias:
            self.bqkv = torch.cat([tensors[f"{n}.bias"] for n in names], dim=0).contiguous()
        self.wo = tensors["wo.weight"].contiguous()
        if self.has_sinks:
            self.sinks = tensors["sinks"].float().contiguous()
        self.position.to(self.wo.device)

    def linear_weights(self):
        return [(self.wqkv, "plain" if self.prepared else "qkv"), (self.wo, "sum")]

    def forward(self, x, ctx, cache):
        n_kv_in_row = 0 if self.shares_kv else self.num_kv_heads
        rot = self.position.rotary_args()
        g = cache.group
        store = cache.writes and not self.shares_kv
        # cosines and sines of this step's positions: made once per step and shared by every layer
        # whose position encoding has the same frequencies
        table = None
        if rot is not None and rot.rotary_dim > 0:
            key = ("rope_table", rot.inv_freq.data_ptr())
            table = ctx.scratch.get(key)
            if table is None:
                table = ctx.scratch[key] = ops.rope_table(ctx.positions, rot.inv_freq)
        if self.prepared:
            return self._forward_prepared(x, ctx, cache, n_kv_in_row, rot, table, store)
        if self.extended:
            return self._forward_extended(x, ctx, cache, n_kv_in_row, rot, table, store)
        qkv = ops.qkv_rope_store(
            x,
            self.wqkv,
            self.bqkv,
            self.num_heads,
            n_kv_in_row,
            self.head_dim,
            ctx.positions,
            rot.inv_freq if rot else None,
            rot.rotary_dim if rot else 0,
            rot.pairing if rot else 0,
            table,
            cache.k_pages if store else None,
            cache.v_pages if store else None,
            ctx.slot_mappings[g] if store else None,
            cache.page_size if store else 0,
        )
        attn = paged_attention(
            qkv, self.num_heads, self.num_kv_heads, self.head_dim, cache.k_pages, cache.v_pages,
            ctx, g, self.window, self.softmax_scale,
        )
        return ops.linear_to_sum(attn, self.wo, may_wait=True)

    def _forward_extended(self, x, ctx, cache, n_kv_in_row, rot, table, store):
        """The layer with a unit norm on queries and keys, capped scores, chunks, sinks or values of their
        own head size: the projection, then rotation, norm and cache write in one kernel, then the plain
        attention kernel, which takes all of these."""
        g = cache.group
        qkv = ops.linear(ops.resolved(x), self.wqkv)
        ops.rope_norm_kv_write(
            qkv, self.num_heads, n_kv_in_row, self.head_dim, self.v_head_dim, table, rot.rotary_dim if rot else 0,
            rot.pairing if rot else 0, self.qk_norm_eps,
            cache.k_pages if store else None, cache.v_pages if store else None,
            ctx.slot_mappings[g] if store else None, cache.page_size if store else 0,
        )
        attn = paged_attention(
            qkv, self.num_heads, self.num_kv_heads, self.head_dim, cache.k_pages, cache.v_pages, ctx, g, self.window,
            self.softmax_scale, softcap=self.softcap, chunk=self.chunk, sinks=self.sinks, v_head_dim=self.v_head_dim,
        )
        return ops.linear_to_sum(attn, self.wo, may_wait=True)

    def _forward_prepared(self, x, ctx, cache, n_kv_in_row, rot, table, store):
        """The layer whose heads are prepared before the scores: one product for q | k | v | gate, one kernel
        for the weighted norm, the rotation, the query factor, the mixed values and the cache write, the
        attention kernel that takes the sizes, the gate, the output product."""
        g = cache.group
        H, dk, dv = self.num_heads, self.head_dim, self.v_head_dim
        rows = ops.linear(ops.resolved(x), self.wqkv)
        v_at = (H + n_kv_in_row) * dk
        v_first = None
        if self.value_mix == "mix":
            v_first = ctx.scratch.get(("value_mix", self.value_mix_key))
            if v_first is None:
                raise RuntimeError(f"attention: no earlier layer of this step has left values under {self.value_mix_key!r}")
        ops.head_prepare(
            rows, H, n_kv_in_row, dk, dv if n_kv_in_row else 0, bias=self.bqkv,
            q_norm=self.q_norm, k_norm=self.k_norm if n_kv_in_row else None, norm_dims=dk if self.qk_norm_weight else 0,
            eps=self.qk_norm_eps, cos_sin=table, rot_offset=0, rot_dims=rot.rotary_dim if rot else 0,
            pairing=rot.pairing if rot else 0, positions=ctx.positions, temp_coef=self.q_temp_coef, temp_every=self.q_temp_every,
            v_first=v_first, v_mix=self.vmix if v_first is not None else None,
            k_pages=cache.k_pages if store else None, v_pages=cache.v_pages if store else None,
            slot_mapping=ctx.slot_mappings[g] if store else None, page_size=cache.page_size if store else 0,
        )
        if self.value_mix == "source":
            ctx.scratch[("value_mix", self.value_mix_key)] = rows[:, v_at : v_at + n_kv_in_row * dv]
        attn = paged_attention(
            rows, H, self.num_kv_heads, dk, cache.k_pages, cache.v_pages, ctx, g, self.window, self.softmax_scale,
            softcap=self.softcap, chunk=self.chunk, sinks=self.sinks, v_head_dim=dv,
        )
        if self.out_gate is not None:
            gate_at = v_at + n_kv_in_row * dv
            ops.sigmoid_gate_(attn, rows[:, gate_at : gate_at + self.gate_rows], per=1 if self.out_gate == "channel" else dv)
        return ops.linear_to_sum(attn, self.wo, may_wait=True)
