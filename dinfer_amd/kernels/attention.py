"""Chooses the attention kernel for a step.

float32 storage: always the plain kernel (fixed key order, any sizes).
bfloat16 storage: MFMA kernels where the sizes fit them, the plain kernel otherwise.
"""
from __future__ import annotations

import torch

from . import ops


class Workspace:
    """Scratch of the split-K decode kernel, sized once for the largest step."""

    def __init__(self, ctx, heads: int, kv_heads: int, head_dim: int):
        self.ctx = ctx


def paged_attention(qkv: torch.Tensor, out: torch.Tensor, k_cache, v_cache, batch, group: int, ws: Workspace, *,
                    scale: float, window: int, heads: int, kv_heads: int, head_dim: int, page_size: int):
    """q is read from the first heads*head_dim columns of qkv; out [T, heads*head_dim]."""
    return ops.attn_paged_ref(qkv, out, k_cache, v_cache, batch.block_table[group], batch.cu_seqlens,
                              batch.seq_lens, batch.num_reqs, batch.num_tokens, scale=scale, window=window,
                              heads=heads, kv_heads=kv_heads, head_dim=head_dim, page_size=page_size)
