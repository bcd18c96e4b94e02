"""Attention through a latent: keys and values of all heads are expanded from one compressed vector per token."""

from __future__ import annotations

from typing import Dict, Optional

import torch

from ..config.spec import PartSpec
from ..kernels import ops
from ..kernels.attention import paged_attention
from .base import MIXERS, POSITIONS, KVNeed, Mixer, ParamSpec
from .positions import step_table


@MIXERS.register("latent_attention")
class LatentAttention(Mixer):
    """Every token leaves one latent ``c`` of ``kv_rank`` channels (a projection of the layer's input, RMS-normed
    with a weight) and one rotated key part of ``rot_dim`` channels that all heads share.  Head h's key is
    ``[W_uk[h] c | rotated part]``, its value ``W_uv[h] c``; queries come through a normed latent of their own
    (``q_rank`` channels) as ``[dim unrotated | rot_dim rotated]`` per head.  Causal softmax attention, an optional
    gate per head (the sigmoid of a projection of the layer's input), the output projection.

    Only ``c`` and the rotated part are cached, as one key row ``[c | rotated part]`` of a single kv head; the
    expansions never happen per cached token.  With ``q' = W_uk[h]^T q_unrotated`` the score of head h is
    ``q' . c + q_rotated . k_rotated``, and the head's output is ``W_uv[h] (sum_j p_j c_j)``: attention of H query
    heads of ``kv_rank + rot_dim`` channels over one kv head whose values are the first ``kv_rank`` channels of
    its keys (``KVNeed.values_in_keys``), with one small product per head before and after it.
    """

    graph_safe = True

    def __init__(
        self,
        hidden_size: int,
        num_heads: int,
        head_dim: int,
        rot_dim: int,
        v_head_dim: int,
        q_rank: Optional[int],
        kv_rank: int,
        softmax_scale: float,
        norm_eps: float,
        position: PartSpec,
        head_gate: bool = False,
        kv_page_size: Optional[int] = None,
        window: int = 0,
    ):
        if rot_dim < 0 or rot_dim % 2:
            raise ValueError(f"latent attention: {rot_dim} rotated channels (even, not negative)")
        self.hidden_size = hidden_size
        self.num_heads = num_heads
        self.head_dim = head_dim
        self.rot_dim = rot_dim
        self.v_head_dim = v_head_dim
        self.q_rank = int(q_rank) if q_rank else 0  # 0: the queries are projected from the layer's input directly (tensor ``q``)
        self.window = int(window)
        if self.window < 0:
            raise ValueError("latent attention: window must not be negative")
        self.kv_rank = kv_rank
        self.softmax_scale = float(softmax_scale)
        self.norm_eps = float(norm_eps)
        self.head_gate = bool(head_gate)
        self.kv_page_size = kv_page_size
        self.position = POSITIONS.build(position)
        self.w_down: Optional[torch.Tensor] = None   # [q_rank + kv_rank + rot_dim + gates, hidden]
        self.w_uq: Optional[torch.Tensor] = None     # [H * (dim + rot_dim), q_rank]
        self.w_uk_t: Optional[torch.Tensor] = None   # [H, kv_rank, dim]: q' = W_uk[h]^T q
        self.w_uv: Optional[torch.Tensor] = None     # [H, vdim, kv_rank]
        self.wo: Optional[torch.Tensor] = None
        self.q_norm: Optional[torch.Tensor] = None
        self.kv_norm: Optional[torch.Tensor] = None

    @property
    def key_dim(self) -> int:
        """Channels of a cached row, and of a query against it."""
        return self.kv_rank + self.rot_dim

    def param_specs(self) -> Dict[str, ParamSpec]:
        H, d, r, dv = self.num_heads, self.head_dim, self.rot_dim, self.v_head_dim
        specs = {
            "dkv.weight": ParamSpec((self.kv_rank + r, self.hidden_size)),
            "dkv_norm.weight": ParamSpec((self.kv_rank,), kind="vector", init="ones"),
            "uk.weight": ParamSpec((H * d, self.kv_rank)),
            "uv.weight": ParamSpec((H * dv, self.kv_rank)),
            "wo.weight": ParamSpec((self.hidden_size, H * dv)),
        }
        if self.q_rank:
            specs.update({"dq.weight": ParamSpec((self.q_rank, self.hidden_size)), "dq_norm.weight": ParamSpec((self.q_rank,), kind="vector", init="ones"),
                          "uq.weight": ParamSpec((H * (d + r), self.q_rank))})
        else:
            specs["q.weight"] = ParamSpec((H * (d + r), self.hidden_size))
        if self.head_gate:
            specs["wg.weight"] = ParamSpec((H, self.hidden_size))
        return specs

    def check_sizes(self, dtype: torch.dtype) -> None:
        if self.key_dim > min(ops.ATTENTION_MAX_KEY_DIM, ops.HEAD_PREPARE_MAX_DIM):
            raise ValueError(f"latent attention: rows of {self.key_dim} channels (latent and rotated part); the kernels take "
                             f"{min(ops.ATTENTION_MAX_KEY_DIM, ops.HEAD_PREPARE_MAX_DIM)}")
        if self.head_dim + self.rot_dim > ops.HEAD_PREPARE_MAX_DIM:
            raise ValueError(f"latent attention: query heads of {self.head_dim + self.rot_dim} channels, at most {ops.HEAD_PREPARE_MAX_DIM}")
        if self.rot_dim and getattr(self.position, "rotary_dim", 0) != self.rot_dim:
            raise ValueError("latent attention: the position encoding must rotate exactly the rotated part")

    def cache_need(self):
        return KVNeed(num_kv_heads=1, head_dim=self.key_dim, window=self.window, page_size=self.kv_page_size, v_head_dim=self.kv_rank,
                      values_in_keys=True)

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        H, d, dv = self.num_heads, self.head_dim, self.v_head_dim
        # one product for [query latent, or the queries themselves | latent | shared rotated key part | gates]
        first = tensors["dq.weight"] if self.q_rank else tensors["q.weight"]
        down = [first, tensors["dkv.weight"]] + ([tensors["wg.weight"]] if self.head_gate else [])
        self.w_down = torch.cat(down, dim=0).contiguous()
        self.w_uq = tensors["uq.weight"].contiguous() if self.q_rank else None
        self.w_uk_t = tensors["uk.weight"].reshape(H, d, self.kv_rank).transpose(1, 2).contiguous()
        self.w_uv = tensors["uv.weight"].reshape(H, dv, self.kv_rank).contiguous()
        self.wo = tensors["wo.weight"].contiguous()
        self.q_norm = tensors["dq_norm.weight"].float().contiguous() if self.q_rank else None
        self.kv_norm = tensors["dkv_norm.weight"].float().contiguous()
        self.position.to(self.wo.device)

    def linear_weights(self):
        return [self.w_down, self.w_uq, (self.wo, "sum")]  # (a None is skipped)

    def _per_head(self, x: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
        """``out[h] = x[:, h, :] @ w[h].T`` as [H, n, rows of w[h]]: x a view [n, H, k] whose rows may lie apart."""
        H, n = w.shape[0], x.shape[0]
        if x.dtype == torch.float32:
            # the 32-bit product kernel, head by head: every sum in an order that the batch does not change
            out = torch.empty((H, n, w.shape[1]), dtype=torch.float32, device=x.device)
            for h in range(H):
                ops.gemm_f32(x[:, h, :], w[h], out=out[h])
            return out
        return torch.bmm(x.transpose(0, 1), w.transpose(1, 2))

    def _mixed_latents(self, queries, n, ctx, cache):
        """Attention of the packed queries over the cached rows: every head's softmax-weighted sum of the latents,
        [n, H, kv_rank]."""
        H, r, R = self.num_heads, self.rot_dim, self.kv_rank
        g, kd = cache.group, self.key_dim
        per_call = 8 if kd == 256 else 16  # query heads per kv head that the matrix-core kernels take
        if (ops.decode_attention_supported(queries.dtype, per_call, 1, kd)
                and ops.prefill_attention_supported(queries.dtype, per_call, 1, kd, cache.page_size)):
            # rows of a size that the matrix-core kernels take: they mix whole rows (the rotated part rides along
            # and is dropped), one kv head for up to per_call query heads at a time
            outs = []
            for h0 in range(0, H, per_call):
                hg = min(per_call, H - h0)
                outs.append(paged_attention(queries[:, h0 * kd : (h0 + hg) * kd], hg, 1, kd, cache.k_pages, cache.v_pages, ctx, g, self.window,
                                            self.softmax_scale).view(n, hg, kd)[:, :, :R])
            return outs[0] if len(outs) == 1 else torch.cat(outs, dim=1)
        # the plain kernel reads the values out of the key rows; a latent wider than its values is mixed in pieces
        piece = ops.ATTENTION_MAX_HEAD_DIM
        parts = [
            paged_attention(queries, H, 1, kd, cache.k_pages, cache.v_pages, ctx, g, self.window, self.softmax_scale,
                            v_head_dim=min(piece, R - at), values_in_keys=True, value_offset=at).view(n, H, -1)
            for at in range(0, R, piece)
        ]
        return parts[0] if len(parts) == 1 else torch.cat(parts, dim=2)

    def forward(self, x, ctx, cache):
        H, d, r, R = self.num_heads, self.head_dim, self.rot_dim, self.kv_rank
        g = cache.group
        rot = self.position.rotary_args()
        table = None
        if r > 0:
            table = step_table(rot, ctx)
        pairing = rot.pairing if rot else 0
        x = ops.resolved(x)
        n = x.shape[0]
        down = ops.linear(x, self.w_down)  # query latent (or queries) | latent | shared rotated key part | gates
        q_cols = self.q_rank or H * (d + r)
        # the latent is normed, the shared part rotated, and the row goes to its page as one key
        ops.head_prepare(
            down[:, q_cols:], 0, 1, R + r, 0, k_norm=self.kv_norm, norm_dims=R, eps=self.norm_eps, cos_sin=table,
            rot_offset=R, rot_dims=r, pairing=pairing, k_pages=cache.k_pages if cache.writes else None,
            slot_mapping=ctx.slot_mappings[g] if cache.writes else None, page_size=cache.page_size if cache.writes else 0,
        )
        if self.q_rank:
            cq = ops.rmsnorm_columns(down[:, : self.q_rank], self.q_norm, self.norm_eps, x.dtype)
            q = ops.linear(cq, self.w_uq)  # [n, H * (d + r)]
        else:
            q = down[:, :q_cols]
        if r > 0:
            ops.head_prepare(q, H, 0, d + r, 0, cos_sin=table, rot_offset=d, rot_dims=r, pairing=pairing)
        q_lat = self._per_head(q.view(n, H, d + r)[:, :, :d], self.w_uk_t)       # [H, n, R]
        queries = ops.pack_heads(q_lat, q, d + r, d, r)                           # [n, H * (R + r)]
        mixed = self._mixed_latents(queries, n, ctx, cache)                       # [n, H, R]
        heads = self._per_head(mixed, self.w_uv)                                  # [H, n, dv]
        gates = down[:, q_cols + R + r :] if self.head_gate else None
        out = ops.unpack_heads_gate(heads.contiguous(), gates)
        return ops.linear_to_sum(out, self.wo, may_wait=True)
