"""Normalisations."""

from __future__ import annotations

from typing import Dict, Optional

import torch

from ..kernels import ops
from .base import NORMS, Norm, ParamSpec


@NORMS.register("rmsnorm")
class RMSNorm(Norm):
    """``y = cast(x32 * rsqrt(mean(x32^2) + eps)) * weight``: statistics and scaling in 32-bit,
    the weight multiply after the cast back (reference: torchllms/models/networks.py:186-200).

    ``stream_dtype`` "float32": the norm works beside a 32-bit residual stream whatever the model's dtype.
    Then ``y = cast(x32 * rsqrt(mean(x32^2) + eps) * weight32)``, rounded once; it reads rows of the stream or of
    the model's dtype and hands on rows of the model's dtype, and ``forward_branch`` adds a normed branch to the
    stream (``stream += norm(branch)``), which is what a block that norms its branches' outputs calls.

    Beside a 32-bit stream the weight may be stored around another number than one (``offset`` c: the factor is
    ``c + weight``) and a second vector may follow it (``scaled``: the tensor ``scale``, a layer's scale on a normed
    branch): ``y = x32 * rsqrt(mean(x32^2) + eps) * (c + weight32) * scale32``.  Both are folded into one 32-bit
    vector when the tensors arrive (``factor``).  ``forward_branch_then`` adds a normed branch to the stream and
    hands on what another norm makes of the new stream, in one pass."""

    graph_safe = True
    takes_split_sums = True  # ops.rmsnorm adds the slices of a split product while it reads them

    def __init__(self, size: int, eps: float, stream_dtype: Optional[str] = None, offset: float = 0.0, scaled: bool = False):
        if stream_dtype not in (None, "float32"):
            raise ValueError(f"rmsnorm: stream_dtype {stream_dtype!r} (None: the model's dtype, or \"float32\")")
        if stream_dtype is None and (float(offset) != 0.0 or scaled):
            raise ValueError("rmsnorm: an offset of the weight or a second scale needs the 32-bit residual stream (stream_dtype=\"float32\")")
        self.size = size
        self.eps = float(eps)
        self.stream_dtype = stream_dtype
        self.offset = float(offset)
        self.scaled = bool(scaled)
        self.takes_split_sums = stream_dtype is None
        self.weight: Optional[torch.Tensor] = None
        self.out_dtype: Optional[torch.dtype] = None

    def param_specs(self) -> Dict[str, ParamSpec]:
        # (beside a 32-bit stream the vector follows the model's dtype, which is the dtype of the normed rows)
        specs = {"weight": ParamSpec((self.size,), kind="vector" if self.stream_dtype is None else "matrix",
                                     init="ones" if self.offset == 0.0 else "normal")}
        if self.scaled:
            specs["scale"] = ParamSpec((self.size,), kind="matrix", init="fraction")
        return specs

    def check_sizes(self, dtype: torch.dtype) -> None:
        if not 0 < self.size <= ops.rmsnorm_max_hidden():
            raise ValueError(f"rmsnorm: rows of {self.size} elements; the kernel takes 1 to {ops.rmsnorm_max_hidden()}")

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        self.weight = tensors["weight"].contiguous()
        if self.stream_dtype is not None:
            self.out_dtype = self.weight.dtype
            self.weight = self.weight.float()
            if self.offset != 0.0:
                self.weight = self.weight + self.offset
            if self.scaled:
                self.weight = self.weight * tensors["scale"].float()
            self.weight = self.weight.contiguous()

    @property
    def factor(self) -> torch.Tensor:
        """Beside a 32-bit stream: the 32-bit vector a normed row is multiplied by (offset and scale folded in)."""
        return self.weight

    def forward_branch_then(self, stream: torch.Tensor, branch, then: Optional["RMSNorm"]):
        """``stream += norm(branch)`` in place, and ``then.forward(stream)`` of the new stream from the same pass
        over the rows (None when ``then`` is None: nobody reads them).  Returns ``(stream, rows)``."""
        if self.stream_dtype is None or (then is not None and (not isinstance(then, RMSNorm) or then.stream_dtype is None)):
            raise ValueError("rmsnorm: forward_branch_then joins two RMS norms beside the 32-bit residual stream")
        rows = ops.post_norm_add_norm(stream, ops.resolved(branch), self.weight, self.eps,
                                      then.weight if then is not None else None, then.eps if then is not None else 0.0)
        return stream, rows

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        if self.stream_dtype is not None:
            return ops.rmsnorm_columns(x, self.weight, self.eps, self.out_dtype)
        return ops.rmsnorm(x, self.weight, self.eps)

    def forward_branch(self, stream: torch.Tensor, branch, want_rows: bool = True):
        """``stream += norm(branch)`` in place and in 32-bit; returns ``(stream, its new rows in the model's dtype)``
        (the rows are None with ``want_rows`` False: nobody reads them)."""
        if self.stream_dtype is None:
            raise ValueError("rmsnorm: forward_branch needs the 32-bit residual stream (stream_dtype=\"float32\")")
        return stream, ops.branch_norm_add(stream, ops.resolved(branch), self.weight, self.eps, want_rows=want_rows)

    def forward_add(self, h: torch.Tensor, delta: Optional[torch.Tensor]):
        if self.stream_dtype is not None:
            if delta is not None:
                h = h + ops.resolved(delta).float()
            return h, self.forward(h)
        if delta is None:
            return h, ops.rmsnorm(h, self.weight, self.eps)
        return ops.rmsnorm(h, self.weight, self.eps, delta=delta, return_sum=True)

    def forward_add_for(self, reader, h: torch.Tensor, delta):
        if (isinstance(delta, ops.PendingProduct) and getattr(reader, "takes_normed_rows", False)
                and self.weight.dtype == torch.bfloat16 and self.size <= ops.NORMED_ROWS_MAX_WIDTH):
            # the product's own kernel adds it to h and leaves the rows' statistics, which the reader's kernel applies
            return delta.added_to(h, self.weight, self.eps)
        return self.forward_add(h, delta)

    def forward_rows(self, h: torch.Tensor, delta: Optional[torch.Tensor], rows: torch.Tensor) -> torch.Tensor:
        if self.stream_dtype is not None:
            if delta is not None:
                h = h + ops.resolved(delta).float()
            return ops.rmsnorm_columns(h, self.weight, self.eps, self.out_dtype, rows=rows)
        return ops.rmsnorm(h, self.weight, self.eps, delta=delta, rows=rows)


@NORMS.register("layernorm")
class LayerNorm(Norm):
    """``y = (x - mean) / sqrt(mean((x - mean)^2) + eps) * weight + bias``, statistics in 32-bit.  The
    residual stream it reads may be 32-bit in a bfloat16 model; what it hands on has the model's dtype.
    Its kernel adds a ``ScaledSum`` (a factor times the sum of a layer's branches) to the stream on the way."""

    graph_safe = True

    def __init__(self, size: int, eps: float):
        self.size = size
        self.eps = float(eps)
        self.weight: Optional[torch.Tensor] = None
        self.bias: Optional[torch.Tensor] = None
        self.out_dtype: Optional[torch.dtype] = None

    def param_specs(self) -> Dict[str, ParamSpec]:
        # (kind "matrix": the vectors follow the model's dtype, which is the dtype of the normed rows)
        return {"weight": ParamSpec((self.size,), kind="matrix", init="ones"), "bias": ParamSpec((self.size,), kind="matrix", init="zeros")}

    def check_sizes(self, dtype: torch.dtype) -> None:
        if not 0 < self.size <= ops.rmsnorm_max_hidden():
            raise ValueError(f"layernorm: rows of {self.size} elements; the kernel takes 1 to {ops.rmsnorm_max_hidden()}")

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        self.out_dtype = tensors["weight"].dtype
        self.weight = tensors["weight"].float().contiguous()
        self.bias = tensors["bias"].float().contiguous()

    def delta(self, delta):
        if delta is None or isinstance(delta, ops.ScaledSum):
            return delta
        return ops.ScaledSum([ops.resolved(delta)], 1.0)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return ops.layernorm(x, self.weight, self.bias, self.eps, self.out_dtype)

    def forward_add(self, h: torch.Tensor, delta):
        delta = self.delta(delta)
        if delta is None:
            return h, ops.layernorm(h, self.weight, self.bias, self.eps, self.out_dtype)
        return ops.layernorm(h, self.weight, self.bias, self.eps, self.out_dtype, delta=delta, return_sum=True)

    def forward_rows(self, h: torch.Tensor, delta, rows: torch.Tensor) -> torch.Tensor:
        return ops.layernorm(h, self.weight, self.bias, self.eps, self.out_dtype, delta=self.delta(delta), rows=rows)


@NORMS.register("dynamic_tanh")
class DynamicTanh(Norm):
    """``y = tanh(alpha x) * weight + bias`` with one learned number ``alpha``: a norm that takes no mean and no
    variance.  It reads a 32-bit residual stream, or several (``[S, n, D]``: hyper-connections), of which it takes a
    weighted sum first, and hands on rows of the model's dtype; everything is worked out in 32-bit.  A block over
    several streams calls ``read`` (the weighted sum and the norm, optionally behind a branch's write into the
    streams: one kernel); everybody else ``forward`` / ``forward_rows``, which take several streams as their plain sum."""

    graph_safe = True

    def __init__(self, size: int):
        self.size = size
        self.weight: Optional[torch.Tensor] = None
        self.bias: Optional[torch.Tensor] = None
        self.alpha: Optional[torch.Tensor] = None
        self.out_dtype: Optional[torch.dtype] = None

    def param_specs(self) -> Dict[str, ParamSpec]:
        # (kind "matrix": the vectors follow the model's dtype, which is the dtype of the normed rows)
        return {"weight": ParamSpec((self.size,), kind="matrix", init="ones"), "bias": ParamSpec((self.size,), kind="matrix", init="zeros"),
                "alpha": ParamSpec((), kind="matrix", init="fraction")}

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        self.out_dtype = tensors["weight"].dtype
        self.weight = tensors["weight"].float().contiguous()
        self.bias = tensors["bias"].float().contiguous()
        self.alpha = tensors["alpha"].float().reshape(1).contiguous()

    def read(self, streams: torch.Tensor, read_weights: Optional[torch.Tensor], branch=None, mix=None, out_weights=None,
             rows: Optional[torch.Tensor] = None) -> torch.Tensor:
        """The normed weighted sum of ``streams`` [S, n, D] (``read_weights`` None: the plain sum; ``rows``: of those
        tokens only), taken after ``branch`` has gone into the streams through ``mix`` and ``out_weights``, if given."""
        return ops.streams_update(streams, branch=branch, mix=mix, out_weights=out_weights, read_weights=read_weights,
                                  alpha=self.alpha, weight=self.weight, bias=self.bias, rows=rows, out_dtype=self.out_dtype)

    @staticmethod
    def _streams(h: torch.Tensor) -> torch.Tensor:
        if h.dtype != torch.float32:
            raise ValueError("dynamic_tanh: the residual stream is 32-bit")
        return h if h.dim() == 3 else h.unsqueeze(0)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return self.read(self._streams(x), None)

    def forward_add(self, h: torch.Tensor, delta):
        if delta is not None:
            if h.dim() == 3:
                raise ValueError("dynamic_tanh: a sum that is not applied yet cannot be added to several streams")
            h = h + ops.resolved(delta).float()
        return h, self.forward(h)

    def forward_rows(self, h: torch.Tensor, delta, rows: torch.Tensor) -> torch.Tensor:
        if delta is not None:
            h, _ = self.forward_add(h, delta)
        return self.read(self._streams(h), None, rows=rows)
