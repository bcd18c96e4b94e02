"""Arrangements of a layer's parts."""

from __future__ import annotations

from typing import Dict, Optional

import torch

from ..kernels import ops
from .base import BLOCKS, Block, ParamSpec


@BLOCKS.register("pre_norm")
class PreNormBlock(Block):
    """``h = x + mixer(norm(x)); out = h + ffn(norm(h))``
    (reference: torchllms/models/networks.py:635-644).  Each residual sum is fused into the
    norm that reads it; the last one is handed on as ``delta``."""

    graph_safe = True
    SLOTS = {"mixer_norm": "norm", "mixer": "mixer", "ffn_norm": "norm", "ffn": "feed_forward"}

    def forward(self, h, delta, ctx, cache):
        h, y = self.mixer_norm.forward_add_for(self.mixer, h, delta)
        a = self.mixer.forward(y, ctx, cache["mixer"])
        h, y = self.ffn_norm.forward_add_for(self.ffn, h, a)
        f = self.ffn.forward(y, ctx)
        return h, f


class _Parallel(Block):
    """One norm whose output every branch of the layer reads: ``x <- x + mult * (sum of the branches)``.
    The sum is handed on unapplied (``ops.ScaledSum``), so that the next norm's kernel adds it."""

    graph_safe = True

    def __init__(self, parts, residual_mult: float = 1.0):
        super().__init__(parts)
        self.residual_mult = float(residual_mult)

    def branches(self, y, ctx, cache):
        raise NotImplementedError

    def forward(self, h, delta, ctx, cache):
        h, y = self.norm1.forward_add(h, self.norm1.delta(delta))
        return h, ops.ScaledSum(self.branches(y, ctx, cache), self.residual_mult)


@BLOCKS.register("parallel")
class ParallelBlock(_Parallel):
    """``h = norm1(x); x <- x + mult * (mix(h) + mlp(h))``."""

    SLOTS = {"norm1": "norm", "mix": "mixer", "mlp": "feed_forward"}

    def branches(self, y, ctx, cache):
        return [self.mix.forward(y, ctx, cache["mix"]), self.mlp.forward(y, ctx)]


@BLOCKS.register("parallel_mixer")
class ParallelMixerBlock(_Parallel):
    """The same layer without a feed-forward: ``x <- x + mult * mix(norm1(x))``."""

    SLOTS = {"norm1": "norm", "mix": "mixer"}

    def branches(self, y, ctx, cache):
        return [self.mix.forward(y, ctx, cache["mix"])]


class _BranchNorm(Block):
    """Layers whose norms stand behind the branches: every branch reads the residual stream itself and its
    output is normed on the way into the stream, ``x <- x + norm(branch(x))``, one branch after the other.
    The stream is 32-bit whatever the model's dtype (an embedding with ``stream_dtype="float32"`` opens it, norms
    with ``stream_dtype="float32"`` keep it); the rows a branch reads are the stream rounded to the model's
    dtype, which the norm's kernel leaves beside the sum.  Nothing is handed on unapplied."""

    graph_safe = True
    _ROWS = "stream_rows"  # in ctx.scratch: (the stream the rows were made from, the rows in the model's dtype)

    def __init__(self, parts):
        super().__init__(parts)
        self.dtype = None

    def bind(self, tensors):
        super().bind(tensors)
        matrices = [v for v in tensors.values() if v.dim() == 2]
        self.dtype = matrices[0].dtype if matrices else next(iter(tensors.values())).dtype

    def rows_of(self, h, ctx):
        kept = ctx.scratch.get(self._ROWS)
        if kept is not None and kept[0] is h:
            return kept[1]
        return h if h.dtype == self.dtype else h.to(self.dtype)

    def keep_rows(self, h, rows, ctx):
        ctx.scratch[self._ROWS] = (h, rows)


@BLOCKS.register("branch_norm")
class BranchNormBlock(_BranchNorm):
    """``x <- x + norm1(mix(x)); x <- x + norm2(mlp(x))``."""

    SLOTS = {"norm1": "norm", "norm2": "norm", "mix": "mixer", "mlp": "feed_forward"}

    def forward(self, h, delta, ctx, cache):
        if delta is not None:
            h = h + ops.resolved(delta).float()
        h, x = self.norm1.forward_branch(h, self.mix.forward(self.rows_of(h, ctx), ctx, cache["mix"]))
        h, x = self.norm2.forward_branch(h, self.mlp.forward(x, ctx))
        self.keep_rows(h, x, ctx)
        return h, None


@BLOCKS.register("branch_norm_mixer")
class BranchNormMixerBlock(_BranchNorm):
    """The same layer without a feed-forward: ``x <- x + norm1(mix(x))``."""

    SLOTS = {"norm1": "norm", "mix": "mixer"}

    def forward(self, h, delta, ctx, cache):
        if delta is not None:
            h = h + ops.resolved(delta).float()
        h, x = self.norm1.forward_branch(h, self.mix.forward(self.rows_of(h, ctx), ctx, cache["mix"]))
        self.keep_rows(h, x, ctx)
        return h, None


class _Sandwich(Block):
    """Layers with a norm before and a norm behind every branch, over a 32-bit residual stream:
    ``x <- x + post(branch(pre(x)))``, one branch after the other.  The norm behind a branch and the norm before the
    next one (of this layer or of the next layer of this kind) run as one kernel over the rows: a layer hands the
    rows that the next layer's first norm would make on, under ``_ROWS`` of the step's scratch, when the next layer
    has said (``expects``) which norm that is."""

    graph_safe = True
    _ROWS = "sandwich_rows"  # in ctx.scratch: (the stream the rows were made from, the norm that made them, the rows)

    def first_norm(self):
        return self.norm1

    def __init__(self, parts):
        super().__init__(parts)
        self.next_first_norm = None  # the first norm of the layer that runs after this one, if that is known

    def expects(self, following: "Block") -> None:
        """Told once, when the model is put together: ``following`` runs right after this layer."""
        self.next_first_norm = following.first_norm() if isinstance(following, _Sandwich) else None

    def rows_for(self, norm, h, ctx):
        kept = ctx.scratch.get(self._ROWS)
        if kept is not None and kept[0] is h and kept[1] is norm:
            return kept[2]
        return norm.forward(h)

    def mix_branch(self, y, ctx, cache):
        raise NotImplementedError

    def forward(self, h, delta, ctx, cache):
        if delta is not None:
            h = h + ops.resolved(delta).float()
        a = self.mix_branch(self.rows_for(self.norm1, h, ctx), ctx, cache)
        has_mlp = "mlp" in self.parts
        after = self.norm2 if has_mlp else self.next_first_norm
        h, y = self.norm1b.forward_branch_then(h, a, after)
        if has_mlp:
            after = self.next_first_norm
            h, y = self.norm2b.forward_branch_then(h, self.mlp.forward(y, ctx), after)
        if after is not None:
            ctx.scratch[self._ROWS] = (h, after, y)
        return h, None


@BLOCKS.register("sandwich")
class SandwichBlock(_Sandwich):
    """``x <- x + norm1b(mix(norm1(x))); x <- x + norm2b(mlp(norm2(x)))``."""

    SLOTS = {"norm1": "norm", "mix": "mixer", "norm1b": "norm", "norm2": "norm", "mlp": "feed_forward", "norm2b": "norm"}

    def mix_branch(self, y, ctx, cache):
        return self.mix.forward(y, ctx, cache["mix"])


@BLOCKS.register("sandwich_mixer")
class SandwichMixerBlock(_Sandwich):
    """The same layer without a feed-forward: ``x <- x + norm1b(mix(norm1(x)))``."""

    SLOTS = {"norm1": "norm", "mix": "mixer", "norm1b": "norm"}

    def mix_branch(self, y, ctx, cache):
        return self.mix.forward(y, ctx, cache["mix"])


class _SandwichPair(_Sandwich):
    """Two mixers side by side that read the same normed rows; the branch is
    ``left_scale * left(h) + right_scale * right(h)``.  Each keeps a cache entry of its own."""

    def __init__(self, parts, left_scale: float = 1.0, right_scale: float = 1.0):
        super().__init__(parts)
        self.left_scale, self.right_scale = float(left_scale), float(right_scale)

    def mix_branch(self, y, ctx, cache):
        a = ops.resolved(self.left.forward(y, ctx, cache["left"]))
        b = ops.resolved(self.right.forward(y, ctx, cache["right"]))
        return ops.weighted_pair(a, self.left_scale, b, self.right_scale)


@BLOCKS.register("sandwich_pair")
class SandwichPairBlock(_SandwichPair):
    """``x <- x + norm1b(s_l left(norm1(x)) + s_r right(norm1(x))); x <- x + norm2b(mlp(norm2(x)))``."""

    SLOTS = {"norm1": "norm", "left": "mixer", "right": "mixer", "norm1b": "norm", "norm2": "norm", "mlp": "feed_forward",
             "norm2b": "norm"}


@BLOCKS.register("sandwich_pair_mixer")
class SandwichPairMixerBlock(_SandwichPair):
    """The same layer without a feed-forward."""

    SLOTS = {"norm1": "norm", "left": "mixer", "right": "mixer", "norm1b": "norm"}


class _Hyper(Block):
    """Layers over several residual streams (hyper-connections).  Instead of one stream there are ``streams`` 32-bit
    copies ``x_1 .. x_S`` (all equal to the embedding's rows when the first such layer opens them).  Sublayer q
    (1: the mixer, 2: the feed-forward) reads ``u = sum_s in_q[s] x_s``, works on ``norm_q(u)``, and its result y goes
    back into all streams at once, ``x_r <- sum_s mix_q[s, r] x_s + out_q[r] y``: the tensors ``hc<q>.in`` [S],
    ``hc<q>.out`` [S] and ``hc<q>.mix`` [S, S] (indexed [from, to]) are the arrangement's own.  A sublayer's write, the
    next sublayer's read and its norm are one kernel over the rows (also across layers, when the next layer is of
    this kind: ``expects``).  The norms take several streams (``dynamic_tanh``); whoever reads the model's last
    streams (the final norm) takes their plain sum."""

    graph_safe = True
    _ROWS = "hyper_rows"  # in ctx.scratch: (the streams the rows were made from, the norm that made them, the rows)

    def __init__(self, parts, streams: int):
        super().__init__(parts)
        if not isinstance(streams, int) or not 0 < streams <= ops.MAX_STREAMS:
            raise ValueError(f"hyper-connections: {streams!r} streams (1 to {ops.MAX_STREAMS})")
        self.streams = streams
        self.has_mlp = "mlp" in self.parts
        self.hc: Dict[str, torch.Tensor] = {}
        self.next_block: Optional["_Hyper"] = None

    def own_specs(self) -> Dict[str, ParamSpec]:
        S, specs = self.streams, {}
        for q in ("hc1", "hc2") if self.has_mlp else ("hc1",):
            specs[f"{q}.in"] = ParamSpec((S,), kind="matrix", init="fraction")
            specs[f"{q}.out"] = ParamSpec((S,), kind="matrix", init="fraction")
            specs[f"{q}.mix"] = ParamSpec((S, S), kind="matrix", init="near_identity")
        return specs

    def param_specs(self) -> Dict[str, ParamSpec]:
        specs = super().param_specs()
        specs.update(self.own_specs())
        return specs

    def bind(self, tensors) -> None:
        super().bind(tensors)
        self.hc = {name: tensors[name].float().contiguous() for name in self.own_specs()}

    def expects(self, following) -> None:
        self.next_block = following if isinstance(following, _Hyper) and following.streams == self.streams else None

    def mix_branch(self, y, ctx, cache):
        raise NotImplementedError

    def forward(self, h, delta, ctx, cache):
        if delta is not None:
            if h.dim() == 3:
                raise ValueError("hyper-connections: a sum that is not applied yet cannot be added to several streams")
            h = h + ops.resolved(delta).float()
        if h.dim() == 2:
            h = ops.streams_open(h if h.dtype == torch.float32 else h.float(), self.streams)
        kept = ctx.scratch.get(self._ROWS)
        if kept is not None and kept[0] is h and kept[1] is self.norm1:
            y = kept[2]
        else:
            y = self.norm1.read(h, self.hc["hc1.in"])
        a = ops.resolved(self.mix_branch(y, ctx, cache))
        last, mix, out = a, self.hc["hc1.mix"], self.hc["hc1.out"]
        if self.has_mlp:
            y = self.norm2.read(h, self.hc["hc2.in"], branch=a, mix=mix, out_weights=out)
            last, mix, out = ops.resolved(self.mlp.forward(y, ctx)), self.hc["hc2.mix"], self.hc["hc2.out"]
        nxt = self.next_block
        if nxt is not None:
            y = nxt.norm1.read(h, nxt.hc["hc1.in"], branch=last, mix=mix, out_weights=out)
            ctx.scratch[self._ROWS] = (h, nxt.norm1, y)
        else:
            ops.streams_update(h, branch=last, mix=mix, out_weights=out)
        return h, None


@BLOCKS.register("hyper")
class HyperBlock(_Hyper):
    """A mixer and a feed-forward over several streams."""

    SLOTS = {"norm1": "norm", "mix": "mixer", "norm2": "norm", "mlp": "feed_forward"}

    def mix_branch(self, y, ctx, cache):
        return self.mix.forward(y, ctx, cache["mix"])


@BLOCKS.register("hyper_mixer")
class HyperMixerBlock(_Hyper):
    """The same layer without a feed-forward."""

    SLOTS = {"norm1": "norm", "mix": "mixer"}

    def mix_branch(self, y, ctx, cache):
        return self.mix.forward(y, ctx, cache["mix"])


class _HyperPair(_Hyper):
    """Two mixers side by side that read the same normed rows; the mixer's result is
    ``left_scale * left(h) + right_scale * right(h)``.  Each keeps a cache entry of its own."""

    def __init__(self, parts, streams: int, left_scale: float = 1.0, right_scale: float = 1.0):
        super().__init__(parts, streams)
        self.left_scale, self.right_scale = float(left_scale), float(right_scale)

    def mix_branch(self, y, ctx, cache):
        a = ops.resolved(self.left.forward(y, ctx, cache["left"]))
        b = ops.resolved(self.right.forward(y, ctx, cache["right"]))
        return ops.weighted_pair(a, self.left_scale, b, self.right_scale)


@BLOCKS.register("hyper_pair")
class HyperPairBlock(_HyperPair):
    SLOTS = {"norm1": "norm", "left": "mixer", "right": "mixer", "norm2": "norm", "mlp": "feed_forward"}


@BLOCKS.register("hyper_pair_mixer")
class HyperPairMixerBlock(_HyperPair):
    SLOTS = {"norm1": "norm", "left": "mixer", "right": "mixer"}
