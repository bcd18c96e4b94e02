"""Chooses the attention kernel for a step.

float32 always takes the plain kernel, whose result for a token depends only on that token's
position and the cache contents.  bfloat16 takes the MFMA kernels where they support the sizes and
the plain kernel otherwise.
"""

from __future__ import annotations

import torch

from . import ops

#: contexts beyond this many keys give every block of 64 keys a wave of its own in the plain kernel
GENERIC_SPLIT_FROM = 128


def paged_attention(
    qkv: torch.Tensor,
    n_q_heads: int,
    n_kv_heads: int,
    head_dim: int,
    k_pages: torch.Tensor,
    v_pages: torch.Tensor,
    ctx,
    group: int,
    window: int,
    scale: float,
    softcap: float = 0.0,
    chunk: int = 0,
    sinks=None,
    v_head_dim=None,
    values_in_keys: bool = False,
    value_offset: int = 0,
    keep_first: int = 0,
    value_heads=None,
) -> torch.Tensor:
    """Attention of this step's queries (first Hq * dh columns of ``qkv``) over their requests'
    cached keys and values; returns [n_tokens, Hq * dv].  Capped scores (``softcap``), chunks
    (``chunk``) and sinks are every kernel's; values of another head size than the keys, or values that are
    channels of the key rows (``values_in_keys``, from ``value_offset`` on), are the plain kernel's alone.  First keys
    that stay visible behind a window (``keep_first``), values with fewer heads than the keys (``value_heads``) and
    values whose head size is a whole multiple of the keys' are every kernel's: the MFMA kernels then take the value
    channels in calls of one key head size each."""
    n = qkv.shape[0]
    n_dec = ctx.host.n_decode
    v_dim = head_dim if v_head_dim is None else int(v_head_dim)
    kept = keep_first if window > 0 or chunk > 0 else 0  # (without a window every key is seen anyway)
    fewer_values = value_heads is not None and value_heads != n_kv_heads
    # (the MFMA kernels take a cap, chunks, sinks, kept first keys and fewer value heads, and values of the keys' head size a call)
    plain_only = values_in_keys or v_dim % head_dim != 0
    extended = softcap > 0 or chunk > 0 or sinks is not None or plain_only or kept > 0 or fewer_values or v_dim != head_dim
    extras = dict(softcap=softcap, chunk=chunk, sinks=sinks, v_head_dim=v_dim, values_in_keys=values_in_keys, value_offset=value_offset,
                  keep_first=kept, value_heads=value_heads) if extended else {}
    fast_extras = dict(softcap=softcap, chunk=chunk, sinks=sinks, keep_first=kept, value_heads=value_heads) if extended else {}
    fast_decode = not plain_only and n_dec > 0 and ops.decode_attention_supported(qkv.dtype, n_q_heads, n_kv_heads, head_dim)
    # the MFMA prefill kernel takes positive softmax scales only; anything else runs the plain kernel
    fast_prefill = (not plain_only and n_dec < n and scale > 0 and not (kept > 0 and softcap > 0)
                    and ops.prefill_attention_supported(qkv.dtype, n_q_heads, n_kv_heads, head_dim, k_pages.shape[2]))
    out = torch.empty((n, n_q_heads * v_dim), dtype=qkv.dtype, device=qkv.device)
    # rows with a single new token come first in the batch
    if n_dec > 0:
        if ctx.decode_longest is not None:
            longest = ctx.decode_longest
        else:
            longest = int(ctx.host.positions[:n_dec].max()) + 1
        if fast_decode:
            # the split-KV MFMA kernel
            if window > 0:
                longest = min(longest, window + 15)
            if chunk > 0:
                longest = min(longest, chunk + 15)
            uneven = ctx.decode_uneven if ctx.decode_uneven is not None else ctx.host.decode_uneven
            for at in range(0, v_dim, head_dim):  # (values wider than the keys: a call for every head_dim channels of them)
                ops.attention_decode(
                    qkv[:n_dec], n_q_heads, n_kv_heads, head_dim, k_pages, v_pages, ctx.token_seq[:n_dec],
                    ctx.positions[:n_dec], ctx.block_tables[group], window, scale, longest, out=out[:n_dec],
                    uneven=uneven, **fast_extras, **(dict(v_offset=at) if at or v_dim != head_dim else {}),
                )
        else:
            # the plain kernel: one wave a (token, head) would walk the whole context alone, so the
            # blocks of 64 keys get waves of their own (the same bits either way)
            if window > 0:
                longest = min(longest, window)
            if chunk > 0:
                longest = min(longest, chunk)
            # (kept first keys come as blocks of their own, which the split form counts by itself)
            plain = ops.attention_generic_split if longest > GENERIC_SPLIT_FROM else ops.attention_generic
            extra = dict(longest=longest) if longest > GENERIC_SPLIT_FROM else {}
            plain(
                qkv[:n_dec], n_q_heads, n_kv_heads, head_dim, k_pages, v_pages, ctx.token_seq[:n_dec],
                ctx.positions[:n_dec], ctx.block_tables[group], window, scale, out=out[:n_dec], **extra, **extras,
            )
    # rows that bring a portion of a prompt take the tiled MFMA kernel
    if n_dec < n:
        if fast_prefill:
            qpt = ops.prefill_queries_per_tile(n_q_heads, n_kv_heads, head_dim)
            key = ("prefill_tiles", qpt, window, chunk, n_kv_heads, kept)
            tiles = ctx.scratch.get(key)
            if tiles is None:
                host = ctx.host
                longest = int(max(host.kv_lens[n_dec : host.n_seqs]))
                if window > 0:
                    longest = min(longest, window + qpt)
                if chunk > 0:
                    longest = min(longest, chunk + qpt)
                longest += kept
                key_groups = ops.prefill_key_groups(ops.prefill_tile_count(host.qo_indptr, n_dec, host.n_seqs, qpt), n_kv_heads, longest)
                rows, q0s = ops.prefill_tiles(host.qo_indptr, n_dec, host.n_seqs, qpt, host.kv_lens, window)
                both = torch.tensor([rows, q0s], dtype=torch.int32).to(qkv.device)
                tiles = (both[0], both[1], key_groups)
                ctx.scratch[key] = tiles
            for at in range(0, v_dim, head_dim):
                ops.attention_prefill(
                    qkv, n_q_heads, n_kv_heads, head_dim, k_pages, v_pages, ctx.qo_indptr, ctx.kv_lens,
                    ctx.block_tables[group], tiles[0], tiles[1], window, scale, out, key_groups=tiles[2], **fast_extras,
                    **(dict(v_offset=at) if at or v_dim != head_dim else {}),
                )
        else:
            ops.attention_generic(
                qkv[n_dec:], n_q_heads, n_kv_heads, head_dim, k_pages, v_pages, ctx.token_seq[n_dec:],
                ctx.positions[n_dec:], ctx.block_tables[group], window, scale, out=out[n_dec:], **extras,
            )
    return out
