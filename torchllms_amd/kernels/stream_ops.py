"""Kernels of layers over several residual streams (hyper-connections) with a norm that takes no statistics
(dynamic tanh), and the joining of the two softmax maps of differential attention."""

from __future__ import annotations

from typing import Optional

import torch

from .base import F32, KernelError, _gpu, _i32, _ptr, _stream, check, core, dtype_code

#: the most residual streams the kernels take
MAX_STREAMS = 16


def _f32(v: Optional[torch.Tensor], shape, what: str) -> None:
    if v is not None and (tuple(v.shape) != tuple(shape) or v.dtype != torch.float32 or not v.is_contiguous()):
        raise KernelError(f"{what} must be contiguous float32 of shape {tuple(shape)}")


def streams_open(rows: torch.Tensor, n_streams: int) -> torch.Tensor:
    """float32 [S, n, D]: every stream a copy of ``rows`` (float32 [n, D])."""
    _gpu(rows)
    if rows.dim() != 2 or rows.dtype != torch.float32 or not rows.is_contiguous():
        raise KernelError("streams_open: the rows must be a contiguous float32 matrix")
    if not 0 < n_streams <= MAX_STREAMS:
        raise KernelError(f"streams_open: {n_streams} streams (1 to {MAX_STREAMS})")
    out = torch.empty((n_streams,) + tuple(rows.shape), dtype=torch.float32, device=rows.device)
    check(core().tl_streams_open(rows.data_ptr(), out.data_ptr(), n_streams, rows.numel(), _stream()))
    return out


def streams_update(
    streams: torch.Tensor,
    branch: Optional[torch.Tensor] = None,
    mix: Optional[torch.Tensor] = None,
    out_weights: Optional[torch.Tensor] = None,
    read_weights: Optional[torch.Tensor] = None,
    alpha: Optional[torch.Tensor] = None,
    weight: Optional[torch.Tensor] = None,
    bias: Optional[torch.Tensor] = None,
    rows: Optional[torch.Tensor] = None,
    out_dtype: Optional[torch.dtype] = None,
) -> Optional[torch.Tensor]:
    """One trip over the streams ``x`` (float32 [S, n, D], changed in place), everything in 32-bit, sums over s ascending.

    With ``branch`` [n, D] (32-bit or of ``out_dtype``): ``x_r <- sum_s mix[s, r] x_s + out_weights[r] * branch`` for all
    r at once (``mix`` float32 [S, S] indexed [from, to], ``out_weights`` float32 [S]).
    With ``weight``: returns ``tanh(alpha u) * weight + bias`` in ``out_dtype`` for ``u = sum_s read_weights[s] x_s`` of
    the streams as they then are (``read_weights`` None: the plain sum; ``alpha`` one float32 on the device, ``weight`` and
    ``bias`` float32 [D]); ``rows`` (int32, only without a branch): of those tokens only."""
    _gpu(streams, branch, mix, out_weights, read_weights, alpha, weight, bias, rows)
    _i32(rows, "rows")
    if streams.dim() != 3 or streams.dtype != torch.float32 or not streams.is_contiguous():
        raise KernelError("streams_update: the streams must be a contiguous float32 [S, n, D] tensor")
    S, n_all, D = streams.shape
    if S > MAX_STREAMS:
        raise KernelError(f"streams_update: {S} streams, at most {MAX_STREAMS}")
    if branch is None and weight is None:
        raise KernelError("streams_update: neither a branch to add nor a norm to read through")
    if branch is not None:
        if rows is not None or tuple(branch.shape) != (n_all, D) or not branch.is_contiguous():
            raise KernelError("streams_update: the branch must be contiguous [n, D], for all tokens")
        _f32(mix, (S, S), "streams_update: mix")
        _f32(out_weights, (S,), "streams_update: out_weights")
        if mix is None or out_weights is None:
            raise KernelError("streams_update: a branch needs mix and out_weights")
        if out_dtype is None:
            out_dtype = branch.dtype
        if branch.dtype not in (torch.float32, out_dtype):
            raise KernelError("streams_update: the branch is 32-bit or of the rows' dtype")
    out = None
    n = n_all if rows is None else rows.numel()
    if weight is not None:
        _f32(weight, (D,), "streams_update: weight")
        _f32(bias, (D,), "streams_update: bias")
        _f32(read_weights, (S,), "streams_update: read_weights")
        if bias is None or alpha is None or alpha.dtype != torch.float32 or alpha.numel() != 1 or out_dtype is None:
            raise KernelError("streams_update: a normed read needs weight, bias, one float32 alpha and the rows' dtype")
        out = torch.empty((n, D), dtype=out_dtype, device=streams.device)
    check(core().tl_streams_update(
        streams.data_ptr(), S, n_all * D, n, D, _ptr(branch), dtype_code(branch.dtype) if branch is not None else F32, _ptr(mix),
        _ptr(out_weights), _ptr(read_weights), _ptr(alpha), _ptr(weight), _ptr(bias), _ptr(rows), _ptr(out),
        dtype_code(out_dtype if out_dtype is not None else torch.float32), _stream()))
    return out


def maps_join(maps: torch.Tensor, n_heads: int, v_head_dim: int, lam: float, eps: float, gain: float) -> torch.Tensor:
    """Differential attention's join.  ``maps`` [n, 2 * H * dv]: the first map's output of all heads, then the second's.
    Returns [n, H * dv]: per head ``o = a_1 - lam * a_2`` divided by its root mean square (``eps`` under the root), times
    ``gain``, in 32-bit."""
    _gpu(maps)
    if maps.dim() != 2 or maps.stride(1) != 1 or maps.shape[1] != 2 * n_heads * v_head_dim:
        raise KernelError(f"maps_join: the maps must be [n, {2 * n_heads * v_head_dim}] with contiguous rows")
    n = maps.shape[0]
    out = torch.empty((n, n_heads * v_head_dim), dtype=maps.dtype, device=maps.device)
    check(core().tl_maps_join(maps.data_ptr(), maps.stride(0), out.data_ptr(), n, n_heads, v_head_dim, float(lam), float(eps), float(gain),
                              dtype_code(maps.dtype), _stream()))
    return out
