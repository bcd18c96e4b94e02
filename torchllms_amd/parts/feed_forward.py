"""Feed-forward networks."""

from __future__ import annotations

from typing import Dict, Optional

import torch

from ..kernels import ops
from .base import FEED_FORWARDS, FeedForward, ParamSpec


@FEED_FORWARDS.register("swiglu")
class SwiGLU(FeedForward):
    """``w2( act(w1 x) * (w3 x) )`` without biases, act = silu
    (reference: torchllms/models/networks.py:592-605) or, with ``activation="gelu_tanh"``, the tanh form of gelu."""

    graph_safe = True
    takes_normed_rows = True

    def __init__(self, hidden_size: int, intermediate_size: int, activation: str = "silu"):
        if activation not in ("silu", "gelu_tanh"):
            raise ValueError(f"gated feed-forward: activation {activation!r} (silu, gelu_tanh)")
        self.activation = activation
        self.hidden_size = hidden_size
        self.intermediate_size = intermediate_size
        self.w13: Optional[torch.Tensor] = None
        self.w2: Optional[torch.Tensor] = None

    def param_specs(self) -> Dict[str, ParamSpec]:
        f, d = self.intermediate_size, self.hidden_size
        return {"w1.weight": ParamSpec((f, d)), "w3.weight": ParamSpec((f, d)), "w2.weight": ParamSpec((d, f))}

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        # gate and up projections fused into one [2F, D] matrix: one product, then silu(gate) * up
        self.w13 = torch.cat([tensors["w1.weight"], tensors["w3.weight"]], dim=0).contiguous()
        self.w2 = tensors["w2.weight"].contiguous()

    def linear_weights(self):
        return [(self.w13, "glu"), (self.w2, "sum")]

    def forward(self, x, ctx):
        return ops.linear_to_sum(ops.linear_glu(x, self.w13, self.activation), self.w2, may_wait=True)


@FEED_FORWARDS.register("dense_gelu")
class DenseGelu(FeedForward):
    """``W_down gelu(W_up x + b_up) + b_down`` with the exact gelu ``z/2 (1 + erf(z / sqrt 2))``."""

    graph_safe = True

    def __init__(self, hidden_size: int, intermediate_size: int):
        self.hidden_size, self.intermediate_size = hidden_size, intermediate_size
        self.w_up = self.b_up = self.w_down = self.b_down = None

    def param_specs(self) -> Dict[str, ParamSpec]:
        f, d = self.intermediate_size, self.hidden_size
        return {"up.weight": ParamSpec((f, d)), "up.bias": ParamSpec((f,), init="zeros"),
                "down.weight": ParamSpec((d, f)), "down.bias": ParamSpec((d,), init="zeros")}

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        self.w_up, self.w_down = tensors["up.weight"].contiguous(), tensors["down.weight"].contiguous()
        self.b_up, self.b_down = tensors["up.bias"].contiguous(), tensors["down.bias"].contiguous()

    def linear_weights(self):
        return [self.w_up, self.w_down]

    def forward(self, x, ctx):
        mid = ops.bias_gelu_(ops.linear(ops.resolved(x), self.w_up), self.b_up)
        return ops.add_bias_(ops.linear(mid, self.w_down), self.b_down)


@FEED_FORWARDS.register("routed")
class RoutedExperts(FeedForward):
    """A mixture of ``num_experts`` gated feed-forwards ``W_down (silu(W_gate x) * (W_up x))`` without biases, of which
    every token uses ``top``.  The router's outputs ``z = W_router x`` (32-bit) number ``num_experts + num_identity``;
    the last ``num_identity`` stand for experts that hand their input through.  Scores ``s = softmax(z)`` over all
    outputs; the ``top`` outputs with the largest ``s + correction`` are chosen, and the result is the sum of the
    chosen experts' outputs times their ``s`` (not renormalised).  ``shared_size`` f > 0: an expert of that width runs
    for every token and is added times ``sigmoid(W_sg x)``, one number a token (``shared_gate`` False: as it is).
    ``correction`` False: there is no correction, the largest scores are chosen.  ``groups`` g > 0 with ``keep_groups``:
    the experts form g equal groups of neighbours, a group's score is the largest score in it, and only experts of
    the best ``keep_groups`` groups can be chosen.  ``normalize``: the chosen scores are divided by their sum
    (+ 1e-20); ``route_scale`` then multiplies them.

    A token's result depends on nothing but the token.  The (token, choice) pairs of a step are put in the order of
    their experts on the device, and a kernel walks every expert's rows with the expert's weights read once for eight
    of them; each row's sums have an order of their own, so in 32-bit a token's result has the same bits in every
    step, and the launches are fixed by the step's shape (decode steps are replayed from graphs).  A bfloat16 step
    that brings prompts and has ``GROUPED_FROM`` pairs or more runs one matrix product per expert over its rows
    instead; for that the host reads how many rows each expert got, once a layer.  A bfloat16 step of at most
    ``ops.PAIR_PRODUCTS_MOST`` pairs (one or two requests decoding) gathers nothing: every pair runs through the dense
    layers' weight-streaming products, which read on the device which expert's matrix is meant."""

    graph_safe = True
    #: (token, choice) pairs of a bfloat16 step with prompts from which on the experts run as matrix products
    GROUPED_FROM = 512

    def __init__(self, hidden_size: int, expert_size: int, num_experts: int, top: int, num_identity: int = 0, shared_size: int = 0,
                 shared_gate: bool = True, correction: bool = True, groups: int = 0, keep_groups: int = 0, normalize: bool = False,
                 route_scale: float = 1.0):
        for name, v in (("expert_size", expert_size), ("num_experts", num_experts), ("top", top)):
            if not isinstance(v, int) or v <= 0:
                raise ValueError(f"routed: {name} must be a positive integer, got {v!r}")
        if num_identity < 0 or shared_size < 0 or top > num_experts + num_identity:
            raise ValueError(f"routed: {top} choices among {num_experts} + {num_identity} outputs; sizes must not be negative")
        self.hidden_size, self.F, self.E, self.I, self.top, self.shared = hidden_size, expert_size, num_experts, num_identity, top, shared_size
        self.shared_gate, self.has_correction = bool(shared_gate) and shared_size > 0, bool(correction)
        self.groups, self.keep_groups, self.normalize, self.route_scale = int(groups or 0), int(keep_groups or 0), bool(normalize), float(route_scale)
        n_out = num_experts + num_identity
        if self.groups and (self.groups < 0 or n_out % self.groups or not 0 < self.keep_groups <= self.groups
                            or self.keep_groups * (n_out // self.groups) < top):
            raise ValueError(f"routed: {self.groups} groups of which {self.keep_groups} stay do not fit {n_out} outputs and {top} choices")
        self.w_router = self.correction = self.w_gu = self.w_down = self.shared_w13 = self.shared_w2 = None
        self._rows_in_order: Dict[int, torch.Tensor] = {}

    def param_specs(self) -> Dict[str, ParamSpec]:
        d, f, n = self.hidden_size, self.F, self.E + self.I
        specs = {"router.weight": ParamSpec((n, d), init="wide")}
        if self.has_correction:
            specs["correction"] = ParamSpec((n,), init="zeros")
        for e in range(self.E):
            specs[f"experts.{e}.w1.weight"] = ParamSpec((f, d))
            specs[f"experts.{e}.w3.weight"] = ParamSpec((f, d))
            specs[f"experts.{e}.w2.weight"] = ParamSpec((d, f))
        if self.shared:
            specs["shared.w1.weight"] = ParamSpec((self.shared, d))
            specs["shared.w3.weight"] = ParamSpec((self.shared, d))
            specs["shared.w2.weight"] = ParamSpec((d, self.shared))
            if self.shared_gate:
                specs["shared.gate.weight"] = ParamSpec((1, d))
        return specs

    def check_sizes(self, dtype: torch.dtype) -> None:
        if self.groups > 64:
            raise ValueError(f"routed: {self.groups} groups of experts; the kernel takes up to 64")
        if self.E + self.I > ops.ROUTER_MAX_OUTPUTS:
            raise ValueError(f"routed: a router of {self.E + self.I} outputs; the kernel takes up to {ops.ROUTER_MAX_OUTPUTS}")
        lds = ops.device_facts()[1]
        if 4 * max(self.hidden_size, self.top * self.F) > lds:
            raise ValueError(f"routed: rows of {self.hidden_size} elements or {self.top} choices of {self.F} do not fit {lds} bytes of LDS")

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        # the router's matrix, and under it the shared expert's gate: one product with 32-bit results
        rows = [tensors["router.weight"]] + ([tensors["shared.gate.weight"]] if self.shared_gate else [])
        self.w_router = torch.cat(rows, dim=0).contiguous()
        self.correction = tensors["correction"].float().contiguous() if self.has_correction else None
        self.w_gu = torch.stack([torch.cat([tensors[f"experts.{e}.w1.weight"], tensors[f"experts.{e}.w3.weight"]], dim=0)
                                 for e in range(self.E)]).contiguous()
        self.w_down = torch.stack([tensors[f"experts.{e}.w2.weight"] for e in range(self.E)]).contiguous()
        if self.shared:
            self.shared_w13 = torch.cat([tensors["shared.w1.weight"], tensors["shared.w3.weight"]], dim=0).contiguous()
            self.shared_w2 = tensors["shared.w2.weight"].contiguous()

    def linear_weights(self):
        return [(self.w_router, "plain", torch.float32), (self.shared_w13, "glu"), self.shared_w2]

    def _own_rows(self, n: int, device) -> torch.Tensor:
        """int32 [n, top]: pair (t, j) lies in row t * top + j (results that were never put in the experts' order)."""
        kept = self._rows_in_order.get(n)
        if kept is None:
            kept = self._rows_in_order[n] = torch.arange(n * self.top, dtype=torch.int32, device=device).view(n, self.top).contiguous()
        return kept

    def forward(self, x, ctx):
        x = ops.resolved(x)
        n_out = self.E + self.I
        z = ops.linear(x, self.w_router, out_dtype=torch.float32)
        ids, weights = ops.router_topk(z, n_out, self.correction, self.top, groups=self.groups, keep_groups=self.keep_groups,
                                       normalize=self.normalize, scale=self.route_scale)
        shared = gate = None
        if self.shared:
            shared = ops.linear(ops.linear_glu(x, self.shared_w13), self.shared_w2)
            gate = z[:, n_out] if self.shared_gate else None
        pairs = x.shape[0] * self.top
        if x.dtype == torch.bfloat16 and pairs <= ops.PAIR_PRODUCTS_MOST and self.hidden_size % 8 == 0 and self.F % 8 == 0:
            # a decode step of one or two requests: every pair by the dense layers' weight-streaming products
            y = ops.expert_pair_products(x, self.w_gu, self.w_down, ids)
            return ops.expert_combine(y, self._own_rows(x.shape[0], x.device), ids, weights, self.E, x, shared, gate)
        rows, pos, offsets = ops.expert_gather(x, ids, n_out)
        if x.dtype == torch.float32 or ctx.host.max_q_len <= 1 or x.shape[0] * self.top < self.GROUPED_FROM:
            y = ops.expert_down_rows(ops.expert_glu_rows(rows, self.w_gu, offsets), self.w_down, offsets)
            return ops.expert_combine(y, pos, ids, weights, self.E, x, shared, gate)
        bounds = offsets.tolist()  # (the one place a step with prompts waits for the GPU)
        parts = []
        for e in range(self.E):
            lo, hi = bounds[e], bounds[e + 1]
            if hi > lo:
                parts.append(ops.linear(ops.linear_glu(rows[lo:hi], self.w_gu[e]), self.w_down[e], out_dtype=torch.float32))
        # (the rows of experts that hand their input through lie behind all others and are never read)
        y = torch.cat(parts) if parts else rows  # (32-bit results: the weighted sum rounds once)
        return ops.expert_combine(y, pos, ids, weights, self.E, x, shared, gate)
