"""Mixers that carry a state of fixed size per request instead of keys and values: the selective scan
of a diagonal state-space layer and the gated delta rule, both behind a short causal convolution.

Everything such a mixer keeps for a request lies in one 32-bit row of its ``StateView`` (the
convolution's history first, then the recurrence's state); rows are zeroed when a request is admitted,
and a step reads and writes the rows of its requests' slots (``ctx.slot_ids``), so a sequence may be
cut into steps anywhere and batched with anything."""

from __future__ import annotations

from typing import Dict, Optional

import torch

from ..kernels import ops
from .base import MIXERS, Mixer, ParamSpec, StateNeed


@MIXERS.register("selective_scan")
class SelectiveScan(Mixer):
    """``[x | z] = W_in h``; x through a causal convolution over ``conv`` taps (with bias) and silu;
    ``[dt | B | C] = W_x x``; ``dt <- softplus(W_dt dt + b_dt)`` per channel; ``A = -exp(A_log)``;
    ``S[c, n] <- exp(dt_c A[c, n]) S[c, n] + dt_c x_c B_n``; ``y_c = sum_n S[c, n] C_n + D_c x_c``;
    the output is ``W_o (y * silu(z))``.  Step sizes, decays and the state are 32-bit."""

    graph_safe = True

    def __init__(self, hidden_size: int, inner_size: int, state_size: int, dt_rank: int, conv_taps: int):
        for name, v in (("inner_size", inner_size), ("state_size", state_size), ("dt_rank", dt_rank), ("conv_taps", conv_taps)):
            if not isinstance(v, int) or v <= 0:
                raise ValueError(f"selective_scan: {name} must be a positive integer, got {v!r}")
        self.hidden_size, self.inner, self.n_state, self.dt_rank, self.taps = hidden_size, inner_size, state_size, dt_rank, conv_taps
        self.w_in = self.w_x = self.w_dt = self.w_o = None
        self.conv_w = self.conv_b = self.dt_b = self.A = self.D = None

    def param_specs(self) -> Dict[str, ParamSpec]:
        d, c, n, r = self.hidden_size, self.inner, self.n_state, self.dt_rank
        return {
            "in": ParamSpec((2 * c, d)),
            "conv": ParamSpec((c, self.taps), init="conv"),
            "conv.b": ParamSpec((c,), init="zeros"),
            "x": ParamSpec((r + 2 * n, c)),
            "dt": ParamSpec((c, r), init="wide"),
            "dt.b": ParamSpec((c,), init="zeros"),
            "A_log": ParamSpec((c, n), init="zeros"),
            "D": ParamSpec((c,), init="ones"),
            "o": ParamSpec((d, c)),
        }

    def check_sizes(self, dtype: torch.dtype) -> None:
        if self.n_state > 256:
            raise ValueError(f"selective_scan: {self.n_state} states a channel; the kernel takes up to 256")
        if self.taps > 64:
            raise ValueError(f"selective_scan: a convolution over {self.taps} taps; the kernel takes up to 64")

    def cache_need(self):
        return StateNeed(shape=((self.taps - 1) * self.inner + self.inner * self.n_state,), dtype="float32")

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        self.w_in = tensors["in"].contiguous()
        self.w_x = tensors["x"].contiguous()
        self.w_dt = tensors["dt"].contiguous()
        self.w_o = tensors["o"].contiguous()
        self.conv_w = tensors["conv"].float().t().contiguous()  # [taps, channels]: a tap's weights lie side by side
        self.conv_b = tensors["conv.b"].float().contiguous()
        self.dt_b = tensors["dt.b"].float().contiguous()
        self.A = (-torch.exp(tensors["A_log"].float())).contiguous()
        self.D = tensors["D"].float().contiguous()

    def linear_weights(self):
        return [self.w_in, self.w_x, (self.w_dt, "plain", torch.float32), (self.w_o, "sum")]

    def forward(self, x, ctx, cache):
        c, n, r = self.inner, self.n_state, self.dt_rank
        state = cache.tensor
        x = ops.resolved(x)
        xz = ops.linear(x, self.w_in)
        xc = ops.causal_conv(xz[:, :c], self.conv_w, self.conv_b, state, 0, ctx.token_seq, ctx.qo_indptr, ctx.slot_ids)
        proj = ops.linear(xc, self.w_x)
        dt_pre = ops.linear(proj[:, :r], self.w_dt, out_dtype=torch.float32)
        # a long prompt's recurrence is cut into segments that run side by side; in 32-bit every row is
        # walked in one piece, so that no bit depends on how the prompt was cut into steps
        segments = None
        if x.dtype != torch.float32 and ctx.host.max_q_len >= ops.SCAN_SEGMENTS_FROM:
            segments = ctx.scratch.get("scan_segments")
            if segments is None:
                segments = ctx.scratch["scan_segments"] = ops.ScanSegments(ctx.host.qo_indptr, x.device)
        y = ops.selective_scan(xc, dt_pre, proj, r, r + n, xz[:, c:], self.dt_b, self.A, self.D, state, (self.taps - 1) * c,
                               ctx.qo_indptr, ctx.slot_ids, segments=segments)
        return ops.linear_to_sum(y, self.w_o)


@MIXERS.register("gated_delta")
class GatedDelta(Mixer):
    """The gated delta rule.  ``q, k`` (``num_key_heads`` heads of ``head_dim``) and ``v`` (``num_heads``
    heads of ``v_head_dim``) are projections of the input, each through a causal convolution over
    ``conv_taps`` taps (no bias) and silu; head h reads q/k head ``h // (num_heads / num_key_heads)``.
    q and k become unit vectors (q also times head_dim^-1/2); ``beta = sigmoid(W_b h)``;
    ``decay = exp(-exp(A_log) softplus(W_a h + dt_bias))`` per head.  Per head and token
    ``S <- decay S; u = beta (v - S^T k); S <- S + k u^T; o = S^T q``; o is divided by its root mean
    square over v_head_dim, multiplied by the weight ``norm`` and by ``silu(W_g h)``, then projected by
    W_o.  Gates, decays, unit norms and the state are 32-bit.

    ``decay`` "channel": every key channel of a head (row of S) has a decay of its own,
    ``exp(-exp(A_log_h) softplus(a_{h,i} + dt_bias_{h,i}))``, whose pre-activation comes through two matrices,
    ``a = W_a2 (W_a1 h)`` with ``decay_rank`` numbers in between (tensors ``a1``, ``a2``; 32-bit results).
    ``gate_rank`` r: the output gate comes through two matrices as well, ``W_g2 (W_g1 h)`` (tensors ``g1``, ``g2``).
    ``gate_act`` "sigmoid": the gate is the logistic function of its pre-activation instead of silu."""

    graph_safe = True

    def __init__(self, hidden_size: int, num_heads: int, num_key_heads: int, head_dim: int, v_head_dim: int, conv_taps: int,
                 norm_eps: float, decay: str = "head", decay_rank: Optional[int] = None, gate_rank: Optional[int] = None,
                 gate_act: str = "silu"):
        if num_heads % num_key_heads:
            raise ValueError(f"gated_delta: {num_heads} heads are not a multiple of {num_key_heads} key heads")
        if decay not in ("head", "channel") or gate_act not in ("silu", "sigmoid"):
            raise ValueError("gated_delta: decay is \"head\" or \"channel\", gate_act \"silu\" or \"sigmoid\"")
        if (decay == "channel") != (decay_rank is not None):
            raise ValueError("gated_delta: a decay per channel comes through two matrices (decay_rank), a decay per head through one")
        for name, v in (("decay_rank", decay_rank), ("gate_rank", gate_rank)):
            if v is not None and (not isinstance(v, int) or v <= 0):
                raise ValueError(f"gated_delta: {name} must be a positive integer, got {v!r}")
        self.hidden_size, self.H, self.G, self.dk, self.dv, self.taps = hidden_size, num_heads, num_key_heads, head_dim, v_head_dim, conv_taps
        self.norm_eps = float(norm_eps)
        self.decay, self.decay_rank, self.gate_rank, self.gate_act = decay, decay_rank, gate_rank, gate_act
        self.w_all = self.w_o = self.conv_w = self.A_log = self.dt_bias = self.norm_w = self.w_a2 = self.w_g2 = None

    @property
    def conv_channels(self) -> int:
        return 2 * self.G * self.dk + self.H * self.dv

    def param_specs(self) -> Dict[str, ParamSpec]:
        d, qk, v = self.hidden_size, self.G * self.dk, self.H * self.dv
        specs = {
            "q": ParamSpec((qk, d)), "q.conv": ParamSpec((qk, self.taps), init="conv"),
            "k": ParamSpec((qk, d)), "k.conv": ParamSpec((qk, self.taps), init="conv"),
            "v": ParamSpec((v, d)), "v.conv": ParamSpec((v, self.taps), init="conv"),
            "b": ParamSpec((self.H, d)),
            "A_log": ParamSpec((self.H,), init="zeros"),
            "norm": ParamSpec((self.dv,), init="ones"),
            "o": ParamSpec((d, v)),
        }
        if self.decay == "channel":
            specs["a1"] = ParamSpec((self.decay_rank, d))
            specs["a2"] = ParamSpec((self.H * self.dk, self.decay_rank), init="wide")
            specs["dt_bias"] = ParamSpec((self.H * self.dk,), init="zeros")
        else:
            specs["a"] = ParamSpec((self.H, d))
            specs["dt_bias"] = ParamSpec((self.H,), init="zeros")
        if self.gate_rank is not None:
            specs["g1"] = ParamSpec((self.gate_rank, d))
            specs["g2"] = ParamSpec((v, self.gate_rank), init="wide")
        else:
            specs["g"] = ParamSpec((v, d))
        return specs

    def check_sizes(self, dtype: torch.dtype) -> None:
        if self.dk > 256:
            raise ValueError(f"gated_delta: keys of {self.dk} channels; the kernel takes up to 256 (values: any number)")
        if self.taps > 64:
            raise ValueError(f"gated_delta: a convolution over {self.taps} taps; the kernel takes up to 64")

    def cache_need(self):
        return StateNeed(shape=((self.taps - 1) * self.conv_channels + self.H * self.dv * self.dk,), dtype="float32")

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        # one projection [q | k | v | output gate | write strength | decay]: a single product per step (of a gate or
        # a decay that comes through two matrices, the first)
        gate, decay = "g" if self.gate_rank is None else "g1", "a" if self.decay == "head" else "a1"
        self.w_all = torch.cat([tensors[n] for n in ("q", "k", "v", gate, "b", decay)], dim=0).contiguous()
        self.w_g2 = tensors["g2"].contiguous() if self.gate_rank is not None else None
        self.w_a2 = tensors["a2"].contiguous() if self.decay == "channel" else None
        self.conv_w = torch.cat([tensors[n + ".conv"] for n in ("q", "k", "v")], dim=0).float().t().contiguous()  # [taps, channels]
        self.w_o = tensors["o"].contiguous()
        self.A_log = tensors["A_log"].float().contiguous()
        self.dt_bias = tensors["dt_bias"].float().contiguous()
        self.norm_w = tensors["norm"].float().contiguous()

    def linear_weights(self):
        return [self.w_all, (self.w_o, "sum"), self.w_g2, (self.w_a2, "plain", torch.float32)]

    def forward(self, x, ctx, cache):
        c = self.conv_channels
        g_cols = self.H * self.dv if self.gate_rank is None else self.gate_rank
        b_at = c + g_cols
        a_at = b_at + self.H
        state = cache.tensor
        proj = ops.linear(ops.resolved(x), self.w_all)
        qkv = ops.causal_conv(proj[:, :c], self.conv_w, None, state, 0, ctx.token_seq, ctx.qo_indptr, ctx.slot_ids)
        gate, gate_at = None, c
        if self.gate_rank is not None:
            gate, gate_at = ops.linear(proj[:, c:b_at], self.w_g2), 0
        channel = None
        if self.decay == "channel":
            channel = ops.linear(proj[:, a_at : a_at + self.decay_rank], self.w_a2, out_dtype=torch.float32)
        y = ops.gated_delta(qkv, proj, gate_at, b_at, a_at, self.A_log, self.dt_bias, self.norm_w, self.norm_eps, state,
                            (self.taps - 1) * c, ctx.qo_indptr, ctx.slot_ids, self.H, self.G, self.dk, self.dv,
                            gate=gate, gate_act=self.gate_act, channel_decay=channel)
        return ops.linear_to_sum(y, self.w_o)


@MIXERS.register("matrix_memory")
class MatrixMemory(Mixer):
    """The matrix memory of an mLSTM layer.  ``q`` (times head_dim^-1/2) and ``k`` (``num_heads`` heads of
    ``head_dim``) and ``v`` (heads of ``v_head_dim``) are projections of the input, and so are, per head, the
    pre-activations of a log input gate ``i = cap tanh((W_i h + b_i) / cap)`` and of a log forget gate
    ``f = logsigmoid(cap tanh((W_f h + b_f) / cap))``.  Per head a matrix C, a vector n and a running maximum m
    start at zero; for every token ``m' = max(f + m, i)``, ``C <- exp(f + m - m') C + exp(i - m') k v^T``, n likewise
    with k alone, ``o = C^T q / (max(|n . q|, exp(-m')) + 1e-6)``.  Each head's o is divided by its root mean square,
    the heads side by side are multiplied by the weight ``norm`` and by ``sigmoid(W_g h)``, then projected by W_o.
    Gates, maxima, exponentials, the state and the norm are 32-bit."""

    graph_safe = True

    def __init__(self, hidden_size: int, num_heads: int, head_dim: int, v_head_dim: int, gate_cap: float, norm_eps: float):
        for name, v in (("num_heads", num_heads), ("head_dim", head_dim), ("v_head_dim", v_head_dim)):
            if not isinstance(v, int) or v <= 0:
                raise ValueError(f"matrix_memory: {name} must be a positive integer, got {v!r}")
        if not float(gate_cap) > 0:
            raise ValueError(f"matrix_memory: gate_cap must be positive, got {gate_cap!r}")
        self.hidden_size, self.H, self.dk, self.dv = hidden_size, num_heads, head_dim, v_head_dim
        self.gate_cap, self.norm_eps = float(gate_cap), float(norm_eps)
        self.w_all = self.w_o = self.i_b = self.f_b = self.norm_w = None

    def param_specs(self) -> Dict[str, ParamSpec]:
        d, qk, v = self.hidden_size, self.H * self.dk, self.H * self.dv
        return {
            "q": ParamSpec((qk, d)), "k": ParamSpec((qk, d)), "v": ParamSpec((v, d)), "g": ParamSpec((v, d)),
            "i": ParamSpec((self.H, d)), "i.b": ParamSpec((self.H,), init="zeros"),
            "f": ParamSpec((self.H, d)), "f.b": ParamSpec((self.H,), init="ones"),
            "norm": ParamSpec((v,), init="ones"), "o": ParamSpec((d, v)),
        }

    def check_sizes(self, dtype: torch.dtype) -> None:
        if self.dk > 256:
            raise ValueError(f"matrix_memory: keys of {self.dk} channels; the kernel takes up to 256 (values: any number)")

    def cache_need(self):
        return StateNeed(shape=(ops.matrix_memory_state_size(self.H, self.dk, self.dv),), dtype="float32")

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        # one projection [q | k | v | output gate | input gate | forget gate]: a single product per step
        self.w_all = torch.cat([tensors[n] for n in ("q", "k", "v", "g", "i", "f")], dim=0).contiguous()
        self.w_o = tensors["o"].contiguous()
        self.i_b = tensors["i.b"].float().contiguous()
        self.f_b = tensors["f.b"].float().contiguous()
        self.norm_w = tensors["norm"].float().contiguous()

    def linear_weights(self):
        return [self.w_all, (self.w_o, "sum")]

    def forward(self, x, ctx, cache):
        qk, v = self.H * self.dk, self.H * self.dv
        proj = ops.linear(ops.resolved(x), self.w_all)
        y = ops.matrix_memory(proj, 0, qk, 2 * qk, 2 * qk + 2 * v, 2 * qk + 2 * v + self.H, 2 * qk + v, self.i_b, self.f_b,
                              self.gate_cap, self.norm_w, self.norm_eps, cache.tensor, 0, ctx.qo_indptr, ctx.slot_ids,
                              self.H, self.dk, self.dv)
        return ops.linear_to_sum(y, self.w_o)


@MIXERS.register("gated_linear")
class GatedLinearAttention(Mixer):
    """Gated linear attention.  ``q`` (times head_dim^-1/2) and ``k`` (``num_heads`` heads of ``head_dim``) and ``v``
    (heads of ``v_head_dim``) are projections of the input.  Every key channel has a decay
    ``alpha = sigmoid(W_a2 (W_a1 h) + b_a2) ** (1 / tau)`` with ``decay_rank`` numbers between the two matrices.  Per head
    the state, zero at the start, goes ``S <- diag(alpha) S + k v^T`` (the decay acts on the rows that belong to key
    channels) and ``o = S^T q``; o is divided by its root mean square over v_head_dim, multiplied by the weight ``norm``
    (shared by the heads) and by ``silu(W_g h)``, then projected by W_o.  Decays, the state and the norm are 32-bit.
    The recurrence runs in the delta rule's kernels under their plain rule."""

    graph_safe = True

    def __init__(self, hidden_size: int, num_heads: int, head_dim: int, v_head_dim: int, tau: float, decay_rank: int, norm_eps: float):
        for name, v in (("num_heads", num_heads), ("head_dim", head_dim), ("v_head_dim", v_head_dim), ("decay_rank", decay_rank)):
            if not isinstance(v, int) or v <= 0:
                raise ValueError(f"gated_linear: {name} must be a positive integer, got {v!r}")
        if not float(tau) > 0:
            raise ValueError(f"gated_linear: tau must be positive, got {tau!r}")
        self.hidden_size, self.H, self.dk, self.dv, self.rank = hidden_size, num_heads, head_dim, v_head_dim, decay_rank
        self.tau, self.norm_eps = float(tau), float(norm_eps)
        self.w_all = self.w_a2 = self.w_o = self.a_bias = self.norm_w = None

    def param_specs(self) -> Dict[str, ParamSpec]:
        d, qk, v = self.hidden_size, self.H * self.dk, self.H * self.dv
        return {
            "q": ParamSpec((qk, d)), "k": ParamSpec((qk, d)), "v": ParamSpec((v, d)), "g": ParamSpec((v, d)),
            "a1": ParamSpec((self.rank, d)), "a2": ParamSpec((qk, self.rank), init="wide"), "a2.b": ParamSpec((qk,), init="zeros"),
            "norm": ParamSpec((self.dv,), init="ones"), "o": ParamSpec((d, v)),
        }

    def check_sizes(self, dtype: torch.dtype) -> None:
        if self.dk > 256:
            raise ValueError(f"gated_linear: keys of {self.dk} channels; the kernel takes up to 256 (values: any number)")

    def cache_need(self):
        return StateNeed(shape=(self.H * self.dv * self.dk,), dtype="float32")

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        # one projection [q | k | v | output gate | the decay's first matrix]: a single product per step
        self.w_all = torch.cat([tensors[n] for n in ("q", "k", "v", "g", "a1")], dim=0).contiguous()
        self.w_a2 = tensors["a2"].contiguous()
        self.a_bias = tensors["a2.b"].float().contiguous()
        self.norm_w = tensors["norm"].float().contiguous()
        self.w_o = tensors["o"].contiguous()

    def linear_weights(self):
        return [self.w_all, (self.w_a2, "plain", torch.float32), (self.w_o, "sum")]

    def forward(self, x, ctx, cache):
        qk, v = self.H * self.dk, self.H * self.dv
        c = 2 * qk + v
        proj = ops.linear(ops.resolved(x), self.w_all)
        pre = ops.linear(proj[:, c + v : c + v + self.rank], self.w_a2, out_dtype=torch.float32)
        y = ops.gated_linear(proj[:, :c], pre, self.a_bias, 1.0 / self.tau, proj, c, self.norm_w, self.norm_eps, cache.tensor, 0,
                             ctx.qo_indptr, ctx.slot_ids, self.H, self.dk, self.dv)
        return ops.linear_to_sum(y, self.w_o)
