"""Grouped-query attention over paged keys and values."""

from __future__ import annotations

import logging
from typing import Dict, Optional

import torch

from ..config.spec import PartSpec
from ..kernels import ops
from ..kernels.attention import paged_attention
from .base import MIXERS, POSITIONS, KVNeed, Mixer, ParamSpec, StateNeed
from .positions import step_table


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

    ``keep_first`` n > 0 (with a window): a query also sees the first n positions of its request, at their true
    positions; their pages are never given back.
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
        keep_first: int = 0,
    ):
        self.values_from_keys = bool(values_from_keys)
        self.keep_first = int(keep_first)
        if self.keep_first < 0:
            raise ValueError("attention: keep_first must not be negative")
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
                      v_head_dim=self.v_head_dim if self.v_head_dim != self.head_dim else None,
                      keep_first=self.keep_first if self.window > 0 else 0)

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
            table = step_table(rot, ctx)
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
            ctx, g, self.window, self.softmax_scale, keep_first=self.keep_first,
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
            keep_first=self.keep_first,
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
            softcap=self.softcap, chunk=self.chunk, sinks=self.sinks, v_head_dim=dv, keep_first=self.keep_first,
        )
        if self.out_gate is not None:
            gate_at = v_at + n_kv_in_row * dv
            ops.sigmoid_gate_(attn, rows[:, gate_at : gate_at + self.gate_rows], per=1 if self.out_gate == "channel" else dv)
        return ops.linear_to_sum(attn, self.wo, may_wait=True)


def covering_window(masks) -> tuple:
    """``(window, keep_first)`` of the pages that serve every one of ``masks`` (pairs ``(window, keep_first)``, window 0:
    every key stays): what the layer that owns keys and values asks of the cache when other layers read them too."""
    masks = list(masks)
    if any(w <= 0 for w, _ in masks):
        return 0, 0
    return max(w for w, _ in masks), max(k for _, k in masks)


@MIXERS.register("differential_attention")
class DifferentialAttention(Mixer):
    """Differential attention: every head has two softmax maps over the same values, each with queries and keys of its
    own (``head_dim`` channels a map), and the head's output is ``a_1 - lambda a_2`` divided by its root mean square
    over ``v_head_dim`` (eps under the root, no weight), times ``1 - diff``; ``lambda = exp(lq1 . lk1) - exp(lq2 . lk2) +
    diff`` is one number of the layer.  Query head h reads key/value head ``h // (num_heads / num_kv_heads)``.

    Tensors ``q`` [H * 2 * d, hidden], ``k`` [G * 2 * d, hidden] (head by head as [map 1, map 2]), ``v`` [G * dv, hidden],
    ``o``, ``lq1``, ``lk1``, ``lq2``, ``lk2`` [d]; ``conv_taps`` K > 0: a causal convolution over K taps on every channel
    of q, k and v right behind the projection (tensors ``q.conv`` ... [channels, K], no bias, no activation), whose last
    K - 1 inputs per request are state.  Then the rotation of every map (``position``), the cache write, causal softmax
    attention inside ``window`` (0: none) plus the first ``keep_first`` positions.

    In the cache the two maps are heads of their own: keys lie as ``2 G`` heads, map 1 of all kv heads and then map 2,
    so that the grouped mapping of query heads to key heads holds for each map, and the values as ``G`` heads that
    both maps read (``KVNeed.num_v_heads``).  The weights are put into that order when they arrive.  ``shares_kv``: no
    k and v tensors; the run reads the pages of the run that the execution order names, with its own queries, their
    convolution and its own mask; ``cache_window`` / ``cache_keep_first``: what the pages must serve when other layers
    read them too (default: this layer's own mask)."""

    graph_safe = True

    def __init__(self, hidden_size: int, num_heads: int, num_kv_heads: int, head_dim: int, v_head_dim: int, softmax_scale: float,
                 diff: float, norm_eps: float, window: int, position: PartSpec, keep_first: int = 0, conv_taps: int = 0,
                 shares_kv: bool = False, kv_page_size: Optional[int] = None, cache_window: Optional[int] = None,
                 cache_keep_first: Optional[int] = None):
        if num_heads % num_kv_heads:
            raise ValueError(f"differential attention: {num_heads} heads are not a multiple of {num_kv_heads} kv heads")
        if window < 0 or keep_first < 0 or conv_taps < 0:
            raise ValueError("differential attention: window, keep_first and conv_taps must not be negative")
        self.hidden_size, self.H, self.G, self.d, self.dv = hidden_size, num_heads, num_kv_heads, head_dim, v_head_dim
        self.softmax_scale, self.diff, self.norm_eps = float(softmax_scale), float(diff), float(norm_eps)
        self.window, self.keep_first, self.taps = int(window), int(keep_first), int(conv_taps)
        self.shares_kv, self.kv_page_size = bool(shares_kv), kv_page_size
        self.cache_window = self.window if cache_window is None else int(cache_window)
        self.cache_keep_first = self.keep_first if cache_keep_first is None else int(cache_keep_first)
        self.position = POSITIONS.build(position)
        self.wqkv = self.wo = self.conv_w = None
        self.lam = 0.0

    @property
    def q_cols(self) -> int:
        return 2 * self.H * self.d

    @property
    def channels(self) -> int:
        """Columns of the fused projection (and channels of the convolution)."""
        return self.q_cols + (0 if self.shares_kv else 2 * self.G * self.d + self.G * self.dv)

    def param_specs(self) -> Dict[str, ParamSpec]:
        D, d = self.hidden_size, self.d
        sizes = {"q": self.q_cols} if self.shares_kv else {"q": self.q_cols, "k": 2 * self.G * d, "v": self.G * self.dv}
        specs = {name: ParamSpec((rows, D)) for name, rows in sizes.items()}
        if self.taps > 0:
            specs.update({f"{name}.conv": ParamSpec((rows, self.taps), init="conv") for name, rows in sizes.items()})
        for name in ("lq1", "lk1", "lq2", "lk2"):
            specs[name] = ParamSpec((d,), kind="vector", init="normal")
        specs["o"] = ParamSpec((D, self.H * self.dv))
        return specs

    def check_sizes(self, dtype: torch.dtype) -> None:
        if not 0 < self.dv <= ops.ATTENTION_MAX_HEAD_DIM or not 0 < self.d <= min(ops.ATTENTION_MAX_KEY_DIM, ops.HEAD_PREPARE_MAX_DIM):
            raise ValueError(f"differential attention: heads of {self.d} channels with values of {self.dv}; the kernels take "
                             f"{min(ops.ATTENTION_MAX_KEY_DIM, ops.HEAD_PREPARE_MAX_DIM)} and {ops.ATTENTION_MAX_HEAD_DIM}")
        if self.taps > 64:
            raise ValueError(f"differential attention: a convolution over {self.taps} taps; the kernel takes up to 64")
        rotated = getattr(self.position, "rotary_dim", 0)
        if rotated % 2 or rotated > self.d:
            raise ValueError(f"differential attention: {rotated} rotated channels of a map of {self.d}")

    def cache_need(self):
        needs = {}
        if not self.shares_kv:
            needs["kv"] = KVNeed(num_kv_heads=2 * self.G, head_dim=self.d, window=self.cache_window, page_size=self.kv_page_size,
                                 v_head_dim=self.dv, keep_first=self.cache_keep_first if self.cache_window > 0 else 0, num_v_heads=self.G)
        if self.taps > 0:  # (one tap has no history; the row is never empty, so that there is a tensor to point at)
            needs["conv"] = StateNeed(shape=(max((self.taps - 1) * self.channels, 1),), dtype="float32")
        return needs

    def _maps_first(self, t: torch.Tensor, heads: int) -> torch.Tensor:
        """Rows stored head by head as [map 1, map 2] -> map 1 of all heads, then map 2."""
        return t.reshape(heads, 2, self.d, *t.shape[1:]).transpose(0, 1).reshape(t.shape).contiguous()

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        parts = [("q", self.H)] if self.shares_kv else [("q", self.H), ("k", self.G), ("v", 0)]

        def ordered(name, heads, suffix=""):
            """Rows of q and k with the maps first; the values' rows as they are (heads 0)."""
            t = tensors[name + suffix]
            return self._maps_first(t, heads) if heads else t

        self.wqkv = torch.cat([ordered(n, h) for n, h in parts], dim=0).contiguous()
        if self.taps > 0:
            self.conv_w = torch.cat([ordered(n, h, ".conv") for n, h in parts], dim=0).float().t().contiguous()  # [taps, channels]
        self.wo = tensors["o"].contiguous()
        f = {n: tensors[n].float() for n in ("lq1", "lk1", "lq2", "lk2")}
        self.lam = float(torch.exp((f["lq1"] * f["lk1"]).sum()) - torch.exp((f["lq2"] * f["lk2"]).sum())) + self.diff
        self.position.to(self.wo.device)

    def linear_weights(self):
        return [self.wqkv, (self.wo, "sum")]

    def forward(self, x, ctx, cache):
        H, G, d, dv = self.H, self.G, self.d, self.dv
        kv = cache["kv"]
        g = kv.group
        store = kv.writes and not self.shares_kv
        rows = ops.linear(ops.resolved(x), self.wqkv)
        if self.taps > 0:
            rows = ops.causal_conv(rows, self.conv_w, None, cache["conv"].tensor, 0, ctx.token_seq, ctx.qo_indptr, ctx.slot_ids, silu=False)
        rot = self.position.rotary_args()
        table = step_table(rot, ctx) if rot is not None and rot.rotary_dim > 0 else None
        n_k = 0 if self.shares_kv else 2 * G
        # every map is a head of its own for the rotation and in the pages
        ops.head_prepare(
            rows, 2 * H, n_k, d, 0, cos_sin=table, rot_offset=0, rot_dims=rot.rotary_dim if table is not None else 0,
            pairing=rot.pairing if rot else 0, k_pages=kv.k_pages if store else None,
            slot_mapping=ctx.slot_mappings[g] if store else None, page_size=kv.page_size if store else 0,
        )
        if store:
            # the values go to their pages as they are (to the kernel they are heads without norm or rotation)
            ops.head_prepare(rows[:, (2 * H + n_k) * d :], 0, G, dv, 0, k_pages=kv.v_pages, slot_mapping=ctx.slot_mappings[g],
                             page_size=kv.page_size)
        maps = paged_attention(rows, 2 * H, 2 * G, d, kv.k_pages, kv.v_pages, ctx, g, self.window, self.softmax_scale,
                               v_head_dim=dv, keep_first=self.keep_first, value_heads=G)
        out = ops.maps_join(maps, H, dv, self.lam, self.norm_eps, 1.0 - self.diff)
        return ops.linear_to_sum(out, self.wo, may_wait=True)
