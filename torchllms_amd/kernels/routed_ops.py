"""Kernels of a routed feed-forward (router with softmax scores and a correction for the choice, the (token, choice)
pairs gathered in the order of their experts, experts over their rows, experts that hand their input through, a
shared expert with a gate), of a dense
feed-forward with biases and the exact gelu, and of layers with a norm on either side of every branch."""

from __future__ import annotations

from typing import Optional, Tuple

import torch

from .base import F32, KernelError, _gpu, _ptr, _stream, check, core, dtype_code

#: the most outputs a router may have (experts and experts that hand their input through together)
ROUTER_MAX_OUTPUTS = 512


def router_topk(z: torch.Tensor, n_out: int, correction: Optional[torch.Tensor], top: int, groups: int = 0, keep_groups: int = 0,
                normalize: bool = False, scale: float = 1.0) -> Tuple[torch.Tensor, torch.Tensor]:
    """``z`` float32 [n, >= n_out]: the router's outputs in the first ``n_out`` columns.  ``s = softmax(z)``; the
    ``top`` outputs with the largest ``s + correction`` are chosen (of equal ones the lower index).  Returns
    ``(ids int32 [n, top], weights float32 [n, top])``, the weights being the chosen outputs' ``s``.  ``correction``
    None: the largest ``s``.  ``groups`` g > 0: the outputs form g equal groups of neighbours, a group's score is the
    largest ``s`` in it, and only outputs of the ``keep_groups`` best groups can be chosen.  ``normalize``: the weights
    are divided by their sum (+ 1e-20); ``scale`` then multiplies them."""
    _gpu(z, correction)
    if z.dim() != 2 or z.dtype != torch.float32 or z.stride(1) != 1 or z.shape[1] < n_out:
        raise KernelError(f"router_topk: z must be float32 [n, >= {n_out}] with contiguous rows")
    if correction is not None and (tuple(correction.shape) != (n_out,) or correction.dtype != torch.float32 or not correction.is_contiguous()):
        raise KernelError(f"router_topk: correction must be a float32 vector of {n_out} entries")
    if not 0 < top <= n_out:
        raise KernelError(f"router_topk: {top} choices among {n_out} outputs")
    if groups and (groups < 0 or groups > 64 or n_out % groups or not 0 < keep_groups <= groups or keep_groups * (n_out // groups) < top):
        raise KernelError(f"router_topk: {groups} groups of which {keep_groups} stay do not fit {n_out} outputs and {top} choices (at most 64 groups)")
    n = z.shape[0]
    ids = torch.empty((n, top), dtype=torch.int32, device=z.device)
    weights = torch.empty((n, top), dtype=torch.float32, device=z.device)
    check(core().tl_router_topk(z.data_ptr(), z.stride(0), _ptr(correction), n, n_out, top, ids.data_ptr(), weights.data_ptr(),
                                int(groups), int(keep_groups), 1 if normalize else 0, float(scale), _stream()))
    return ids, weights


def _pairs(x, ids, n_experts):
    if x.dim() != 2 or not x.is_contiguous():
        raise KernelError("routed experts: x must be a contiguous [n, D] matrix")
    if ids.dim() != 2 or ids.shape[0] != x.shape[0] or ids.dtype != torch.int32 or not ids.is_contiguous():
        raise KernelError("routed experts: ids must be contiguous int32 [n, top]")
    if n_experts < 0:
        raise KernelError("routed experts: a negative number of experts")


def _expert_rows(rows, weights, offsets, what):
    if rows.dim() != 2 or not rows.is_contiguous():
        raise KernelError(f"{what}: the rows must be a contiguous matrix")
    if weights.dim() != 3 or weights.shape[2] != rows.shape[1] or weights.dtype != rows.dtype or not weights.is_contiguous():
        raise KernelError(f"{what}: weights must be contiguous [E, outputs, {rows.shape[1]}] of the rows' dtype")
    if offsets.dtype != torch.int32 or offsets.dim() != 1 or offsets.numel() < weights.shape[0] + 1 or not offsets.is_contiguous():
        raise KernelError(f"{what}: offsets must be contiguous int32 with an entry per expert and one more")


def expert_glu_rows(rows: torch.Tensor, w_gate_up: torch.Tensor, offsets: torch.Tensor) -> torch.Tensor:
    """``mid[r] = silu(Wg[e] rows[r]) * (Wu[e] rows[r])`` for the rows ``offsets[e] .. offsets[e + 1]`` of every expert
    ``e`` of ``w_gate_up`` [E, 2F, D] (gate rows, then up rows); ``rows`` [pairs, D] as ``expert_gather`` leaves them.
    An expert's weights are read once for up to eight of its rows.  Returns [pairs, F]; rows behind ``offsets[E]`` (pairs of
    outputs that are no experts) are left unwritten."""
    _gpu(rows, w_gate_up, offsets)
    _expert_rows(rows, w_gate_up, offsets, "expert_glu_rows")
    if w_gate_up.shape[1] % 2:
        raise KernelError("expert_glu_rows: gate rows and up rows of every expert")
    E, F, D = w_gate_up.shape[0], w_gate_up.shape[1] // 2, rows.shape[1]
    mid = torch.empty((rows.shape[0], F), dtype=rows.dtype, device=rows.device)
    check(core().tl_expert_glu_rows(rows.data_ptr(), w_gate_up.data_ptr(), offsets.data_ptr(), E, mid.data_ptr(), D, F,
                                    rows.shape[0], dtype_code(rows.dtype), _stream()))
    return mid


def expert_down_rows(mid: torch.Tensor, w_down: torch.Tensor, offsets: torch.Tensor) -> torch.Tensor:
    """``y[r] = Wd[e] mid[r]`` in 32-bit for the rows ``offsets[e] .. offsets[e + 1]`` of every expert of ``w_down``
    [E, D, F].  Returns float32 [pairs, D]."""
    _gpu(mid, w_down, offsets)
    _expert_rows(mid, w_down, offsets, "expert_down_rows")
    E, D, F = w_down.shape
    y = torch.empty((mid.shape[0], D), dtype=torch.float32, device=mid.device)
    check(core().tl_expert_down_rows(mid.data_ptr(), w_down.data_ptr(), offsets.data_ptr(), E, y.data_ptr(), D, F,
                                     mid.shape[0], dtype_code(mid.dtype), _stream()))
    return y


#: the most (token, choice) pairs of a bfloat16 step that ``expert_pair_products`` is meant for: every pair costs two
#: launches, and each launch reads its expert's weights whoever else reads them too
PAIR_PRODUCTS_MOST = 4


def expert_pair_products(x: torch.Tensor, w_gate_up: torch.Tensor, w_down: torch.Tensor, ids: torch.Tensor) -> torch.Tensor:
    """``y[t, j] = Wd[e] (silu(Wg[e] x[t]) * (Wu[e] x[t]))`` with ``e = ids[t, j]`` for the few pairs of a small decode
    step, each pair by the weight-streaming products that dense layers use (bfloat16; the gate and up products are
    rounded to bfloat16 before the activation, as theirs are), told on the device which expert's matrix to read.  A
    pair whose ``e`` is no expert of the weights gets some expert's result, which nobody reads.  Returns float32
    [n * top, D], the pairs in their own order."""
    _gpu(x, w_gate_up, w_down, ids)
    E = w_gate_up.shape[0] if w_gate_up.dim() == 3 else -1
    _pairs(x, ids, E)
    n, D = x.shape
    if x.dtype != torch.bfloat16 or w_gate_up.dtype != x.dtype or w_down.dtype != x.dtype:
        raise KernelError("expert_pair_products: bfloat16 rows and weights")
    if w_gate_up.dim() != 3 or w_gate_up.shape[2] != D or w_gate_up.shape[1] % 2 or not w_gate_up.is_contiguous():
        raise KernelError(f"expert_pair_products: gate and up weights must be contiguous [E, 2F, {D}]")
    F = w_gate_up.shape[1] // 2
    if tuple(w_down.shape) != (E, D, F) or not w_down.is_contiguous():
        raise KernelError(f"expert_pair_products: down weights must be contiguous [{E}, {D}, {F}]")
    if D % 8 or F % 8:
        raise KernelError("expert_pair_products: widths must be multiples of 8")
    top = ids.shape[1]
    pairs = n * top
    mid = torch.empty((pairs, F), dtype=x.dtype, device=x.device)
    y = torch.empty((pairs, D), dtype=torch.float32, device=x.device)
    lib, stream = core(), _stream()
    for p in range(pairs):
        which = ids.data_ptr() + 4 * p
        check(lib.tl_gemm_stream_glu_select(x.data_ptr() + 2 * D * (p // top), D, w_gate_up.data_ptr(), D, mid.data_ptr() + 2 * F * p, F,
                                            1, F, D, 0, 16, which, 2 * F * D, E, stream))
        check(lib.tl_gemm_stream_select(mid.data_ptr() + 2 * F * p, F, w_down.data_ptr(), F, y.data_ptr() + 4 * D * p, D, 1, D, F,
                                        F32, 0, which, D * F, E, stream))
    return y


def expert_gather(x: torch.Tensor, ids: torch.Tensor, n_out: int):
    """The (token, choice) pairs in the order of their experts.  Returns ``(rows, pos, offsets)``: ``rows`` [n * top, D]
    holds for every pair its token's row of ``x``, the pairs of output e in the rows ``offsets[e] .. offsets[e + 1]``
    (int32 [n_out + 1], on the device); ``pos`` int32 [n, top] says which row each pair got."""
    _gpu(x, ids)
    _pairs(x, ids, 0)
    n, D = x.shape
    top = ids.shape[1]
    work = torch.zeros(3 * n_out + 1, dtype=torch.int32, device=x.device)
    counts, offsets, cursor = work[:n_out], work[n_out : 2 * n_out + 1], work[2 * n_out + 1 :]
    pos = torch.empty((n, top), dtype=torch.int32, device=x.device)
    rows = torch.empty((n * top, D), dtype=x.dtype, device=x.device)
    check(core().tl_expert_gather(x.data_ptr(), ids.data_ptr(), n, top, n_out, counts.data_ptr(), offsets.data_ptr(), cursor.data_ptr(),
                                  pos.data_ptr(), rows.data_ptr(), D, dtype_code(x.dtype), _stream()))
    return rows, pos, offsets


def expert_combine(
    y: torch.Tensor,
    pos: torch.Tensor,
    ids: torch.Tensor,
    weights: torch.Tensor,
    n_experts: int,
    x: torch.Tensor,
    shared: Optional[torch.Tensor] = None,
    shared_gate: Optional[torch.Tensor] = None,
) -> torch.Tensor:
    """``out[t] = sum_j weights[t, j] * (y[pos[t, j]] if ids[t, j] < n_experts else x[t])``, plus
    ``sigmoid(shared_gate[t]) * shared[t]`` (``shared[t]`` as it is without a gate): the experts' results (rows in the order ``expert_gather`` gave them) back
    in the order of the tokens; ``y`` is 32-bit (``expert_down_rows``) or of x's dtype (matrix products over the
    gathered rows).  Returns [n, D] of x's dtype."""
    _gpu(y, pos, ids, weights, x, shared, shared_gate)
    _pairs(x, ids, n_experts)
    n, D = x.shape
    top = ids.shape[1]
    if y.dim() != 2 or y.shape[1] != D or y.dtype not in (x.dtype, torch.float32) or not y.is_contiguous():
        raise KernelError("expert_combine: y must be a contiguous [rows, D] matrix of x's dtype or of float32")
    if tuple(pos.shape) != (n, top) or pos.dtype != torch.int32 or not pos.is_contiguous():
        raise KernelError("expert_combine: pos must be contiguous int32 [n, top]")
    if tuple(weights.shape) != (n, top) or weights.dtype != torch.float32 or not weights.is_contiguous():
        raise KernelError("expert_combine: weights must be contiguous float32 [n, top]")
    sg_stride = 0
    if shared is not None:
        if tuple(shared.shape) != (n, D) or shared.dtype != x.dtype or not shared.is_contiguous():
            raise KernelError("expert_combine: the shared expert's result must be contiguous [n, D] of x's dtype")
        if shared_gate is not None and (shared_gate.dtype != torch.float32 or shared_gate.numel() != n or shared_gate.dim() > 2):
            raise KernelError("expert_combine: the shared expert's gate must be float32, one number a token")
        sg_stride = shared_gate.stride(0) if (n > 1 and shared_gate is not None) else 1
    out = torch.empty((n, D), dtype=x.dtype, device=x.device)
    check(core().tl_expert_combine(y.data_ptr(), 1 if y.dtype == torch.float32 else 0, pos.data_ptr(), ids.data_ptr(), weights.data_ptr(), top, n_experts, x.data_ptr(),
                                   _ptr(shared), _ptr(shared_gate), sg_stride, out.data_ptr(), n, D, dtype_code(x.dtype), _stream()))
    return out


def bias_gelu_(x: torch.Tensor, bias: torch.Tensor) -> torch.Tensor:
    """``x <- gelu(x + bias)`` in place, row by row, with the exact gelu ``z/2 (1 + erf(z / sqrt 2))`` in 32-bit."""
    _gpu(x, bias)
    if x.dim() != 2 or not x.is_contiguous():
        raise KernelError("bias_gelu_: x must be a contiguous matrix")
    if tuple(bias.shape) != (x.shape[1],) or bias.dtype != x.dtype or not bias.is_contiguous():
        raise KernelError(f"bias_gelu_: bias must be a contiguous vector of {x.shape[1]} entries of x's dtype")
    check(core().tl_bias_gelu(x.data_ptr(), bias.data_ptr(), x.shape[0], x.shape[1], dtype_code(x.dtype), _stream()))
    return x


def weighted_pair(a: torch.Tensor, a_scale: float, b: torch.Tensor, b_scale: float) -> torch.Tensor:
    """``a_scale * a + b_scale * b`` in 32-bit, rounded once to the tensors' dtype."""
    _gpu(a, b)
    if a.shape != b.shape or a.dtype != b.dtype or not a.is_contiguous() or not b.is_contiguous():
        raise KernelError("weighted_pair: two contiguous tensors of one shape and dtype")
    out = torch.empty_like(a)
    check(core().tl_weighted_pair(a.data_ptr(), float(a_scale), b.data_ptr(), float(b_scale), out.data_ptr(), a.numel(),
                                  dtype_code(a.dtype), _stream()))
    return out


def post_norm_add_norm(
    stream: torch.Tensor,
    branch: torch.Tensor,
    post_weight: torch.Tensor,
    eps: float,
    next_weight: Optional[torch.Tensor] = None,
    next_eps: float = 0.0,
) -> Optional[torch.Tensor]:
    """``stream += branch / rms(branch) * post_weight`` in place and in 32-bit, and, with ``next_weight``, the rows
    ``stream / rms(stream) * next_weight`` in the branch's dtype: the norm behind a branch and the norm before the next
    one, one pass over each row.  Both weights are 32-bit vectors (whatever factors a norm has, folded into one)."""
    _gpu(stream, branch, post_weight, next_weight)
    if stream.dim() != 2 or stream.dtype != torch.float32 or not stream.is_contiguous():
        raise KernelError("post_norm_add_norm: the stream must be a contiguous float32 matrix")
    n, hidden = stream.shape
    if tuple(branch.shape) != (n, hidden) or not branch.is_contiguous():
        raise KernelError("post_norm_add_norm: the branch must be contiguous and of the stream's shape")
    for w in (post_weight, next_weight):
        if w is not None and (tuple(w.shape) != (hidden,) or w.dtype != torch.float32 or not w.is_contiguous()):
            raise KernelError(f"post_norm_add_norm: weights must be float32 vectors of {hidden} entries")
    rows = torch.empty_like(branch) if next_weight is not None else None
    check(core().tl_post_norm_add_norm(stream.data_ptr(), branch.data_ptr(), post_weight.data_ptr(), float(eps), _ptr(next_weight),
                                       float(next_eps), _ptr(rows), n, hidden, dtype_code(branch.dtype), _stream()))
    return rows
