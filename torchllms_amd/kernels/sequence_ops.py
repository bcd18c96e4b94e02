"""Kernels of layers other than pre-norm attention: a scaled embedding into a 32-bit residual stream,
layer norm fused with a scaled sum of branches, gated activations, rotation with a unit norm of
queries and keys and the cache write, short causal convolutions with a history per request, the
selective scan of a diagonal state-space layer and the gated delta rule.

Recurrent state lives in rows of a 32-bit tensor ``[request slots, elements]`` (a ``StateView``); a
mixer keeps several things in one row and names each by its offset, ``state_region`` below."""

from __future__ import annotations

from typing import Optional, Sequence

import torch

from .base import F32, KernelError, Unfinished, _gpu, _i32, _ptr, _stream, check, core, dtype_code, resolved


class ScaledSum(Unfinished):
    """``mult * (sum of terms)`` that has not been added to the residual stream yet: a norm whose kernel
    takes it (``takes_scaled_sums``) adds it on the way, in 32-bit; anybody else gets the tensor."""

    def __init__(self, terms: Sequence[torch.Tensor], mult: float):
        self.terms = [resolved(t) for t in terms]
        self.mult = float(mult)

    @property
    def shape(self):
        return tuple(self.terms[0].shape)

    def resolve(self) -> torch.Tensor:
        total = self.terms[0].float()
        for t in self.terms[1:]:
            total = total + t.float()
        return (total * self.mult).to(self.terms[0].dtype)


def embed_scaled(tokens: torch.Tensor, table: torch.Tensor, scale: float) -> torch.Tensor:
    """``float(table[tokens]) * scale`` as a 32-bit tensor [n, hidden]."""
    _gpu(tokens, table)
    _i32(tokens, "tokens")
    if table.dim() != 2 or not table.is_contiguous():
        raise KernelError("embedding table must be a contiguous matrix")
    n, hidden = tokens.numel(), table.shape[1]
    out = torch.empty((n, hidden), dtype=torch.float32, device=table.device)
    check(core().tl_embed_scaled(tokens.data_ptr(), table.data_ptr(), out.data_ptr(), n, hidden, float(scale),
                                 dtype_code(table.dtype), _stream()))
    return out


def layernorm(
    x: torch.Tensor,
    weight: torch.Tensor,
    bias: torch.Tensor,
    eps: float,
    out_dtype: torch.dtype,
    delta: Optional[ScaledSum] = None,
    rows: Optional[torch.Tensor] = None,
    return_sum: bool = False,
):
    """Layer norm (mean and variance over the row, weight and bias, both 32-bit vectors) of
    ``x + delta.mult * sum(delta.terms)`` row by row, optionally of the rows ``rows`` only; ``x`` is the
    residual stream (32-bit, or ``out_dtype``), the result has ``out_dtype``.  With ``return_sum`` the
    sum replaces ``x`` in place and ``(x, y)`` is returned."""
    terms = [] if delta is None else list(delta.terms)
    if len(terms) > 2:
        extra = ScaledSum(terms[1:], 1.0).resolve()
        terms = [terms[0], extra]
    _gpu(x, weight, bias, rows, *terms)
    _i32(rows, "rows")
    if x.dim() != 2 or not x.is_contiguous():
        raise KernelError("layernorm input must be a contiguous [rows, hidden] tensor")
    hidden = x.shape[1]
    for v in (weight, bias):
        if v.shape != (hidden,) or v.dtype != torch.float32 or not v.is_contiguous():
            raise KernelError(f"layernorm weight and bias must be float32 vectors of {hidden} entries")
    for t in terms:
        if t.shape != x.shape or t.dtype != out_dtype or not t.is_contiguous():
            raise KernelError("layernorm: a term of the sum must have the input's shape and the result's dtype")
    if x.dtype not in (torch.float32, out_dtype):
        raise KernelError(f"layernorm: a residual stream of {x.dtype} with results of {out_dtype}")
    if rows is not None and return_sum:
        raise KernelError("layernorm cannot return the sum together with a row gather")
    n = x.shape[0] if rows is None else rows.numel()
    y = torch.empty((n, hidden), dtype=out_dtype, device=x.device)
    check(
        core().tl_layernorm(
            x.data_ptr(), _ptr(terms[0]) if terms else None, _ptr(terms[1]) if len(terms) > 1 else None,
            delta.mult if delta is not None else 0.0, _ptr(rows), weight.data_ptr(), bias.data_ptr(),
            x.data_ptr() if return_sum else None, y.data_ptr(), n, hidden, float(eps), dtype_code(x.dtype),
            dtype_code(out_dtype), _stream(),
        )
    )
    return (x, y) if return_sum else y


def gelu_mul(gate_up: torch.Tensor) -> torch.Tensor:
    """``gelu_tanh(gate) * up`` for ``gate_up`` [n, 2F] = gate | up, computed in 32-bit, rounded once."""
    _gpu(gate_up)
    if gate_up.dim() != 2 or gate_up.shape[1] % 2 or not gate_up.is_contiguous():
        raise KernelError("gelu_mul input must be contiguous [n, 2F]")
    n, inter = gate_up.shape[0], gate_up.shape[1] // 2
    out = torch.empty((n, inter), dtype=gate_up.dtype, device=gate_up.device)
    check(core().tl_gelu_mul(gate_up.data_ptr(), out.data_ptr(), n, inter, dtype_code(gate_up.dtype), _stream()))
    return out


def rope_norm_kv_write(
    qkv: torch.Tensor,
    n_q_heads: int,
    n_kv_heads: int,
    head_dim: int,
    v_head_dim: int,
    cos_sin: Optional[torch.Tensor],
    rotary_dim: int,
    pairing: int,
    norm_eps: float,
    k_pages: Optional[torch.Tensor] = None,
    v_pages: Optional[torch.Tensor] = None,
    slot_mapping: Optional[torch.Tensor] = None,
    page_size: int = 0,
) -> None:
    """Rotate the query and key heads of ``qkv`` [n, (Hq + Hkv) * dk + Hkv * dv] by the step's table of
    cosines and sines, divide each by its root mean square (``norm_eps`` > 0; 0: no norm), write the
    queries back and the keys and values into their pages ([pages, Hkv, page, dk] and [.., dv])."""
    _gpu(qkv, cos_sin, k_pages, v_pages, slot_mapping)
    _i32(slot_mapping, "slot_mapping")
    n = qkv.shape[0]
    width = (n_q_heads + n_kv_heads) * head_dim + n_kv_heads * v_head_dim
    if qkv.dim() != 2 or qkv.shape[1] != width or not qkv.is_contiguous():
        raise KernelError(f"qkv must be contiguous [n, {width}], got {tuple(qkv.shape)}")
    if rotary_dim > 0 and (cos_sin is None or cos_sin.dtype != torch.float32 or tuple(cos_sin.shape) != (n, rotary_dim // 2, 2)
                           or not cos_sin.is_contiguous()):
        raise KernelError(f"cos_sin must be contiguous float32 [{n}, {rotary_dim // 2}, 2]")
    if k_pages is not None:
        if v_pages is None or slot_mapping is None or slot_mapping.numel() != n:
            raise KernelError("pages need v_pages and one slot per token")
        for pg, d in ((k_pages, head_dim), (v_pages, v_head_dim)):
            if pg.dim() != 4 or pg.shape[1:] != (n_kv_heads, page_size, d) or pg.dtype != qkv.dtype or not pg.is_contiguous():
                raise KernelError(f"pages must be contiguous [pages, {n_kv_heads}, {page_size}, {d}] of {qkv.dtype}, got {tuple(pg.shape)} {pg.dtype}")
    check(
        core().tl_rope_norm_kv_write(
            qkv.data_ptr(), n, n_q_heads, n_kv_heads, head_dim, v_head_dim, _ptr(cos_sin), rotary_dim, pairing, float(norm_eps),
            _ptr(k_pages), _ptr(v_pages), _ptr(slot_mapping), page_size, dtype_code(qkv.dtype), _stream(),
        )
    )


# ----------------------------------------------------------------------------- recurrent state
def state_region(state: torch.Tensor, offset: int, size: int):
    """``(address, row stride)`` of the ``size`` elements from ``offset`` of every row of a 32-bit state
    tensor [slots, elements], as the kernels below take them."""
    if state.dim() != 2 or state.dtype != torch.float32 or not state.is_contiguous() or not state.is_cuda:
        raise KernelError("recurrent state must be a contiguous float32 GPU tensor [slots, elements]")
    if offset < 0 or size < 0 or offset + size > state.shape[1]:
        raise KernelError(f"a region of {size} elements at {offset} does not lie in rows of {state.shape[1]}")
    return state.data_ptr() + 4 * offset, state.shape[1]


def _step_rows(ctx_token_seq, qo_indptr, slot_ids, n_tokens: int, state: torch.Tensor):
    _gpu(ctx_token_seq, qo_indptr, slot_ids)
    _i32(ctx_token_seq, "token_seq")
    _i32(qo_indptr, "qo_indptr")
    _i32(slot_ids, "slot_ids")
    n_seqs = slot_ids.numel()
    if qo_indptr.numel() != n_seqs + 1 or (ctx_token_seq is not None and ctx_token_seq.numel() != n_tokens):
        raise KernelError("the step's row offsets, slots and tokens do not fit each other")
    return n_seqs


def causal_conv(
    x: torch.Tensor,
    taps: torch.Tensor,
    bias: Optional[torch.Tensor],
    state: torch.Tensor,
    state_offset: int,
    token_seq: torch.Tensor,
    qo_indptr: torch.Tensor,
    slot_ids: torch.Tensor,
    silu: bool = True,
) -> torch.Tensor:
    """Causal convolution over time, channel by channel, of ``x`` [n, C] (a view of some columns of a
    matrix will do) with ``taps`` float32 [K, C] (the last row multiplies the current token) and
    ``bias`` float32 [C] or None, then silu.  What lies before a request's first token of this step is
    its history: (K - 1) * C floats at ``state_offset`` of its state row, which is brought up to date."""
    _gpu(x, taps, bias)
    if x.dim() != 2 or x.stride(1) != 1:
        raise KernelError("causal_conv: x must be a matrix whose rows are contiguous")
    n, C = x.shape
    if taps.dim() != 2 or taps.shape[1] != C or taps.dtype != torch.float32 or not taps.is_contiguous():
        raise KernelError(f"causal_conv: taps must be contiguous float32 [K, {C}]")
    K = taps.shape[0]
    if bias is not None and (bias.shape != (C,) or bias.dtype != torch.float32 or not bias.is_contiguous()):
        raise KernelError(f"causal_conv: bias must be a float32 vector of {C} entries")
    n_seqs = _step_rows(token_seq, qo_indptr, slot_ids, n, state)
    region, stride = state_region(state, state_offset, (K - 1) * C)
    out = torch.empty((n, C), dtype=x.dtype, device=x.device)
    check(
        core().tl_causal_conv(
            x.data_ptr(), x.stride(0), taps.data_ptr(), _ptr(bias), region, stride, token_seq.data_ptr(), qo_indptr.data_ptr(),
            slot_ids.data_ptr(), out.data_ptr(), out.stride(0), n, n_seqs, C, K, 1 if silu else 0, dtype_code(x.dtype), _stream(),
        )
    )
    return out


#: tokens of a segment when a long row's recurrence is cut into segments that run side by side, and the
#: longest row of a step from which on that is done
SCAN_SEGMENT = 64
SCAN_SEGMENTS_FROM = 256


class ScanSegments:
    """The rows of a step cut into segments of at most ``SCAN_SEGMENT`` consecutive tokens: ``segs``
    int32 [n, 2] (first token, one past the last) with every row's segments in order, ``row_seg`` int32
    [rows + 1] (the first segment of every row), both on the device, made from the host's row offsets."""

    def __init__(self, qo_indptr_host, device, length: int = SCAN_SEGMENT):
        import numpy as np

        bounds = [int(v) for v in qo_indptr_host]
        segs, row_seg = [], [0]
        for lo, hi in zip(bounds[:-1], bounds[1:]):
            for t in range(lo, hi, length):
                segs.append((t, min(t + length, hi)))
            row_seg.append(len(segs))
        self.n = len(segs)
        packed = np.asarray([v for seg in segs for v in seg] + row_seg, dtype=np.int32)
        dev = torch.from_numpy(packed).to(device)
        self.segs = dev[: 2 * self.n]
        self.row_seg = dev[2 * self.n :]


def selective_scan(
    x: torch.Tensor,
    dt_pre: torch.Tensor,
    proj: torch.Tensor,
    b_offset: int,
    c_offset: int,
    z: torch.Tensor,
    dt_bias: torch.Tensor,
    A: torch.Tensor,
    D: torch.Tensor,
    state: torch.Tensor,
    state_offset: int,
    qo_indptr: torch.Tensor,
    slot_ids: torch.Tensor,
    segments: Optional[ScanSegments] = None,
) -> torch.Tensor:
    """The recurrence of a diagonal state-space layer over each request's tokens, in 32-bit:
    ``dt = softplus(dt_pre + dt_bias)``; ``S[c, n] = exp(dt[c] A[c, n]) S[c, n] + dt[c] x[c] B[n]``;
    ``y[c] = sum_n S[c, n] C[n] + D[c] x[c]``; result ``y * silu(z)``.  ``x`` [n, inner]; ``dt_pre``
    [n, inner] (32-bit or x's dtype); B and C are the ``N`` columns of ``proj`` from ``b_offset`` and
    ``c_offset``; ``z`` [n, inner] may be a view of columns; ``A`` float32 [inner, N] (negative);
    ``S`` lives at ``state_offset`` of the request's state row, inner * N floats.  With ``segments`` the
    rows' segments run side by side: each is walked from a zero state, a carry joins the segments of a
    row in order (a state's decay over a segment is exp(A * the sum of the segment's step sizes)), and
    each is walked again from the state that enters it.  The result then depends on the cut by rounding."""
    _gpu(x, dt_pre, proj, z, dt_bias, A, D)
    n, inner = x.shape
    N = A.shape[1]
    if not x.is_contiguous() or dt_pre.shape != x.shape or not dt_pre.is_contiguous():
        raise KernelError("selective_scan: x and dt_pre must be contiguous [n, inner]")
    if proj.dim() != 2 or proj.shape[0] != n or proj.stride(1) != 1 or proj.dtype != x.dtype or max(b_offset, c_offset) + N > proj.shape[1]:
        raise KernelError("selective_scan: B and C do not lie in the rows of proj")
    if z.shape != x.shape or z.stride(1) != 1 or z.dtype != x.dtype:
        raise KernelError("selective_scan: z must be [n, inner] of x's dtype with contiguous rows")
    for v, shape in ((dt_bias, (inner,)), (A, (inner, N)), (D, (inner,))):
        if tuple(v.shape) != shape or v.dtype != torch.float32 or not v.is_contiguous():
            raise KernelError(f"selective_scan: a float32 tensor of shape {shape} expected, got {tuple(v.shape)} {v.dtype}")
    n_seqs = _step_rows(None, qo_indptr, slot_ids, n, state)
    region, stride = state_region(state, state_offset, inner * N)
    out = torch.empty_like(x)
    ws = seg_dt = None
    if segments is not None:
        if segments.row_seg.numel() != n_seqs + 1:
            raise KernelError("selective_scan: the segments are not those of this step's rows")
        ws = torch.empty((segments.n, inner * N), dtype=torch.float32, device=x.device)
        seg_dt = torch.empty((segments.n, inner), dtype=torch.float32, device=x.device)
    check(
        core().tl_selective_scan(
            x.data_ptr(), dt_pre.data_ptr(), dtype_code(dt_pre.dtype), proj.data_ptr(), proj.stride(0), b_offset, c_offset,
            z.data_ptr(), z.stride(0), dt_bias.data_ptr(), A.data_ptr(), D.data_ptr(), region, stride, qo_indptr.data_ptr(),
            slot_ids.data_ptr(), out.data_ptr(), n_seqs, inner, N, dtype_code(x.dtype),
            _ptr(segments.segs) if segments is not None else None, _ptr(segments.row_seg) if segments is not None else None,
            segments.n if segments is not None else 0, _ptr(ws), _ptr(seg_dt), _stream(),
        )
    )
    return out


def gated_delta(
    qkv: torch.Tensor,
    proj: torch.Tensor,
    gate_offset: int,
    b_offset: int,
    a_offset: int,
    A_log: torch.Tensor,
    dt_bias: torch.Tensor,
    norm_weight: torch.Tensor,
    eps: float,
    state: torch.Tensor,
    state_offset: int,
    qo_indptr: torch.Tensor,
    slot_ids: torch.Tensor,
    n_heads: int,
    n_key_heads: int,
    head_dim: int,
    v_head_dim: int,
    gate: Optional[torch.Tensor] = None,
    gate_act: str = "silu",
    channel_decay: Optional[torch.Tensor] = None,
) -> torch.Tensor:
    """The gated delta rule over each request's tokens, in 32-bit.  ``qkv`` [n, 2 G dk + H dv]: query
    heads | key heads | value heads, already convolved and activated.  Of ``proj`` [n, ..] the output
    gate (H dv columns from ``gate_offset``) and the pre-activations of the write strength and of the
    decay (H columns each from ``b_offset`` and ``a_offset``) are read.  Per head, with unit q and k
    (q also times dk^-1/2): ``S <- decay S; u = beta (v - S^T k); S <- S + k u^T; o = S^T q``; then o
    over its root mean square, times ``norm_weight`` [dv], times silu(gate).  ``S`` lives at
    ``state_offset`` of the request's state row, H * dv * dk floats.  Returns [n, H * dv].

    ``gate``: a matrix of its own that holds the output gate's columns from ``gate_offset`` (None: ``proj``);
    ``gate_act`` "sigmoid": the gate is the logistic function of them, not silu.  ``channel_decay`` float32
    [n, H * dk]: every key channel of a head (row of S) has a decay of its own,
    ``exp(-exp(A_log[h]) softplus(channel_decay[t, h, i] + dt_bias[h, i]))`` with ``dt_bias`` of H * dk entries;
    the column ``a_offset`` of ``proj`` is then not read."""
    _gpu(qkv, proj, A_log, dt_bias, norm_weight, gate, channel_decay)
    H, G, dk, dv = n_heads, n_key_heads, head_dim, v_head_dim
    n = qkv.shape[0]
    if gate_act not in ("silu", "sigmoid"):
        raise KernelError(f"gated_delta: gate_act {gate_act!r} (silu, sigmoid)")
    gate_src = proj if gate is None else gate
    if gate_src.dim() != 2 or gate_src.shape[0] != n or gate_src.stride(1) != 1 or gate_src.dtype != qkv.dtype:
        raise KernelError("gated_delta: the gate must be a matrix of qkv's dtype with a row per token")
    if channel_decay is not None and (channel_decay.dim() != 2 or tuple(channel_decay.shape) != (n, H * dk)
                                      or channel_decay.dtype != torch.float32 or channel_decay.stride(1) != 1):
        raise KernelError(f"gated_delta: channel_decay must be float32 [n, {H * dk}] with contiguous rows")
    if qkv.dim() != 2 or qkv.shape[1] != 2 * G * dk + H * dv or qkv.stride(1) != 1:
        raise KernelError(f"gated_delta: qkv must be [n, {2 * G * dk + H * dv}] with contiguous rows")
    if proj.dim() != 2 or proj.shape[0] != n or proj.stride(1) != 1 or proj.dtype != qkv.dtype:
        raise KernelError("gated_delta: proj must be a matrix of qkv's dtype with a row per token")
    if gate_offset + H * dv > gate_src.shape[1] or (b_offset if channel_decay is not None else max(b_offset, a_offset)) + H > proj.shape[1]:
        raise KernelError("gated_delta: gate, b or a do not lie in the rows of proj")
    for v, size in ((A_log, H), (dt_bias, H if channel_decay is None else H * dk), (norm_weight, dv)):
        if tuple(v.shape) != (size,) or v.dtype != torch.float32 or not v.is_contiguous():
            raise KernelError(f"gated_delta: a float32 vector of {size} entries expected, got {tuple(v.shape)} {v.dtype}")
    n_seqs = _step_rows(None, qo_indptr, slot_ids, n, state)
    region, stride = state_region(state, state_offset, H * dv * dk)
    out = torch.empty((n, H * dv), dtype=qkv.dtype, device=qkv.device)
    o_raw = torch.empty((n, H * dv), dtype=torch.float32, device=qkv.device)
    check(
        core().tl_gated_delta(
            qkv.data_ptr(), qkv.stride(0), proj.data_ptr(), proj.stride(0), gate_offset, b_offset, a_offset, A_log.data_ptr(),
            dt_bias.data_ptr(), norm_weight.data_ptr(), float(eps), region, stride, qo_indptr.data_ptr(), slot_ids.data_ptr(),
            out.data_ptr(), n, n_seqs, H, G, dk, dv, o_raw.data_ptr(), dtype_code(qkv.dtype), gate_src.data_ptr(), gate_src.stride(0),
            1 if gate_act == "sigmoid" else 0, _ptr(channel_decay), channel_decay.stride(0) if channel_decay is not None else 0,
            0.0, _stream(),
        )
    )
    return out


def gated_linear(
    qkv: torch.Tensor,
    decay_pre: torch.Tensor,
    decay_bias: torch.Tensor,
    decay_power: float,
    gate: torch.Tensor,
    gate_offset: int,
    norm_weight: torch.Tensor,
    eps: float,
    state: torch.Tensor,
    state_offset: int,
    qo_indptr: torch.Tensor,
    slot_ids: torch.Tensor,
    n_heads: int,
    head_dim: int,
    v_head_dim: int,
) -> torch.Tensor:
    """Gated linear attention over each request's tokens, in 32-bit.  ``qkv`` [n, 2 H dk + H dv]: query heads | key
    heads | value heads as projected.  Per head, with q times dk^-1/2 and a decay for every key channel
    ``alpha = sigmoid(decay_pre[t, h, i] + decay_bias[h, i]) ** decay_power`` (``decay_pre`` float32 [n, H * dk]):
    ``S <- diag(alpha) S + k v^T; o = S^T q``; then o over its root mean square, times ``norm_weight`` [dv], times
    silu of the gate (H dv columns of ``gate`` from ``gate_offset``).  ``S`` lives at ``state_offset`` of the request's
    state row, H * dv * dk floats.  Returns [n, H * dv].  The recurrence is the delta rule's kernel with its plain rule."""
    _gpu(qkv, decay_pre, decay_bias, gate, norm_weight)
    H, dk, dv = n_heads, head_dim, v_head_dim
    n = qkv.shape[0]
    if qkv.dim() != 2 or qkv.shape[1] != 2 * H * dk + H * dv or qkv.stride(1) != 1:
        raise KernelError(f"gated_linear: qkv must be [n, {2 * H * dk + H * dv}] with contiguous rows")
    if gate.dim() != 2 or gate.shape[0] != n or gate.stride(1) != 1 or gate.dtype != qkv.dtype or gate_offset < 0 or gate_offset + H * dv > gate.shape[1]:
        raise KernelError("gated_linear: the gate must be a matrix of qkv's dtype with a row per token that holds H * dv columns from gate_offset")
    if decay_pre.dim() != 2 or tuple(decay_pre.shape) != (n, H * dk) or decay_pre.dtype != torch.float32 or decay_pre.stride(1) != 1:
        raise KernelError(f"gated_linear: decay_pre must be float32 [n, {H * dk}] with contiguous rows")
    for v, size in ((decay_bias, H * dk), (norm_weight, dv)):
        if tuple(v.shape) != (size,) or v.dtype != torch.float32 or not v.is_contiguous():
            raise KernelError(f"gated_linear: a float32 vector of {size} entries expected, got {tuple(v.shape)} {v.dtype}")
    if not decay_power > 0:
        raise KernelError("gated_linear: the decay's power must be positive")
    n_seqs = _step_rows(None, qo_indptr, slot_ids, n, state)
    region, stride = state_region(state, state_offset, H * dv * dk)
    out = torch.empty((n, H * dv), dtype=qkv.dtype, device=qkv.device)
    o_raw = torch.empty((n, H * dv), dtype=torch.float32, device=qkv.device)
    check(
        core().tl_gated_delta(
            qkv.data_ptr(), qkv.stride(0), None, 0, gate_offset, 0, 0, None, decay_bias.data_ptr(), norm_weight.data_ptr(), float(eps),
            region, stride, qo_indptr.data_ptr(), slot_ids.data_ptr(), out.data_ptr(), n, n_seqs, H, H, dk, dv, o_raw.data_ptr(),
            dtype_code(qkv.dtype), gate.data_ptr(), gate.stride(0), 0, decay_pre.data_ptr(), decay_pre.stride(0), float(decay_power),
            _stream(),
        )
    )
    return out


def matrix_memory_state_size(n_heads: int, head_dim: int, v_head_dim: int) -> int:
    """32-bit elements of a request's state row that ``matrix_memory`` keeps: per head the matrix and the normaliser
    as dv + 1 columns of dk, and the running maximum once for every column."""
    return n_heads * (v_head_dim + 1) * head_dim + n_heads * (v_head_dim + 1)


def matrix_memory(
    proj: torch.Tensor,
    q_offset: int,
    k_offset: int,
    v_offset: int,
    i_offset: int,
    f_offset: int,
    gate_offset: int,
    i_bias: torch.Tensor,
    f_bias: torch.Tensor,
    gate_cap: float,
    norm_weight: torch.Tensor,
    eps: float,
    state: torch.Tensor,
    state_offset: int,
    qo_indptr: torch.Tensor,
    slot_ids: torch.Tensor,
    n_heads: int,
    head_dim: int,
    v_head_dim: int,
) -> torch.Tensor:
    """The matrix memory of an mLSTM layer over each request's tokens, in 32-bit.  Of ``proj`` [n, ..] the columns of
    q and k (H heads of dk each), v and the output gate (H heads of dv) and the pre-activations of the input and the
    forget gate (H each) are read from their offsets.  Per head, with ``i = cap tanh((i~ + i_bias) / cap)`` and
    ``f = logsigmoid(cap tanh((f~ + f_bias) / cap))`` and a running maximum m (0 at the start):
    ``m' = max(f + m, i); C <- exp(f + m - m') C + exp(i - m') k v^T``, n likewise with k alone,
    ``o = C^T q dk^-1/2 / (max(|n . q dk^-1/2|, exp(-m')) + 1e-6)``; then o over its root mean square, times
    ``norm_weight`` [H * dv], times sigmoid(gate).  C, n and m live at ``state_offset`` of the request's state row
    (``matrix_memory_state_size`` floats).  Returns [n, H * dv]."""
    _gpu(proj, i_bias, f_bias, norm_weight)
    H, dk, dv = n_heads, head_dim, v_head_dim
    n = proj.shape[0]
    if proj.dim() != 2 or proj.stride(1) != 1:
        raise KernelError("matrix_memory: proj must be a matrix with contiguous rows")
    width = proj.shape[1]
    for off, size, what in ((q_offset, H * dk, "q"), (k_offset, H * dk, "k"), (v_offset, H * dv, "v"), (gate_offset, H * dv, "gate"),
                            (i_offset, H, "i"), (f_offset, H, "f")):
        if off < 0 or off + size > width:
            raise KernelError(f"matrix_memory: the columns of {what} do not lie in the rows of proj")
    for v, size in ((i_bias, H), (f_bias, H), (norm_weight, H * dv)):
        if tuple(v.shape) != (size,) or v.dtype != torch.float32 or not v.is_contiguous():
            raise KernelError(f"matrix_memory: a float32 vector of {size} entries expected, got {tuple(v.shape)} {v.dtype}")
    if not gate_cap > 0:
        raise KernelError("matrix_memory: the gates' cap must be positive")
    n_seqs = _step_rows(None, qo_indptr, slot_ids, n, state)
    region, stride = state_region(state, state_offset, matrix_memory_state_size(H, dk, dv))
    out = torch.empty((n, H * dv), dtype=proj.dtype, device=proj.device)
    o_raw = torch.empty((n, H * dv), dtype=torch.float32, device=proj.device)
    den = torch.empty((n, H), dtype=torch.float32, device=proj.device)
    check(
        core().tl_matrix_memory(
            proj.data_ptr(), proj.stride(0), q_offset, k_offset, v_offset, i_offset, f_offset, i_bias.data_ptr(), f_bias.data_ptr(),
            float(gate_cap), proj.data_ptr(), proj.stride(0), gate_offset, norm_weight.data_ptr(), float(eps), region, stride,
            qo_indptr.data_ptr(), slot_ids.data_ptr(), out.data_ptr(), n, n_seqs, H, dk, dv, o_raw.data_ptr(), den.data_ptr(),
            dtype_code(proj.dtype), _stream(),
        )
    )
    return out
