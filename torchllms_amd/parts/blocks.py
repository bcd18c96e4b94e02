"""Arrangements of a layer's parts."""

from __future__ import annotations

from ..kernels import ops
from .base import BLOCKS, Block


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
