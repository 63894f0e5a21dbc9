"""Chooses the attention kernels for a step.

float32 storage: always the plain kernel (fixed key order, any sizes).
bfloat16 storage: MFMA kernels where the geometry fits them (head size from the
instantiated list, page size a multiple of 8): split-K decode for the requests that
bring one row, flash for the others; the plain kernel otherwise.
"""
from __future__ import annotations

import torch

from . import ops

TARGET_WAVES = 1024   # split-K aims at about this many waves (measured: more, shorter waves cost more than they hide)
MAX_SPLITS = 128      # the kernels take up to 256
MIN_KEYS_PER_SPLIT = 512   # of the longest request the engine admits, beyond 32 parts
SHORTEST_PART = 64         # keys of the longest request in one part, at least


class Workspace:
    """Geometry checks and the split-K scratch of one attention shape, sized once."""

    def __init__(self, ctx, heads: int, kv_heads: int, head_dim: int):
        self.max_reqs = ctx.max_reqs
        # measured on MI355X (head 128, 8 kv heads): one request of 2k-4k keys is fastest with 32 parts,
        # of 32k with 64, of 128k with 128; the count may not depend on the lengths of a step (a captured
        # graph must stay valid), so it is bounded by the longest request the engine admits
        longest = ctx.max_seq_len or 4096
        self.max_splits = min(MAX_SPLITS, max(32, longest // MIN_KEYS_PER_SPLIT))
        # an engine for short requests: no part shorter than 64 keys of the longest, so up to 256 keys there are at
        # most four parts, which meet inside the workgroup and need no merge kernel (28 layers of 1,024 wide, 256
        # keys: 1.17 -> 1.0x ms a step at one request)
        self.max_splits = max(1, min(self.max_splits, -(-longest // SHORTEST_PART)))
        self.mfma = (ctx.dtype == torch.bfloat16 and ops.attn_mfma_supports(head_dim, ctx.page_size, heads, kv_heads))
        self.split_k = self.mfma and heads // kv_heads <= 16
        self.part = None
        self.kv_heads = kv_heads
        # a step of single rows: the split-K kernel can take the per-head norms, the rotation and the cache write along
        self.decode_takes_post = self.split_k and ops.attn_decode_post_supports(head_dim)
        if self.split_k:
            max_units = max(self.splits(n) * n for n in range(1, ctx.max_reqs + 1)) * kv_heads
            elems = max_units * (heads // kv_heads) * (head_dim + 4)
            self.part = ctx.workspace.buffer("attn_partials", elems, dtype=torch.float32, rows=1)

    def splits(self, num_reqs: int) -> int:
        """Parts per request: a function of the batch size only, so a captured graph stays valid."""
        return max(1, min(self.max_splits, TARGET_WAVES // (num_reqs * self.kv_heads)))


def decode_with_post(qkv, out, k_cache, v_cache, batch, group: int, ws: Workspace, *, write: bool, **kw):
    """A step in which every request brings one row (ws.decode_takes_post): norms, rotation, cache write and attention
    in one kernel (and the merge of its parts). kw: geometry, norm and rotation as ops.attn_decode_post takes them."""
    B = batch.num_reqs
    return ops.attn_decode_post(qkv, out, ws.part, k_cache, v_cache, batch.block_table[group], batch.seq_lens, B,
                                ws.splits(B), slot_mapping=batch.slot_mapping[group] if write else None, **kw)


def paged_attention(qkv: torch.Tensor, out: torch.Tensor, k_cache, v_cache, batch, group: int, ws: Workspace, *,
                    scale: float, window: int, heads: int, kv_heads: int, head_dim: int, page_size: int):
    """q is read from the first heads*head_dim columns of qkv; out [T, heads*head_dim]."""
    geo = dict(scale=scale, window=window, heads=heads, kv_heads=kv_heads, head_dim=head_dim, page_size=page_size)
    bt = batch.block_table[group]
    B, T = batch.num_reqs, batch.num_tokens
    if not ws.mfma:
        return ops.attn_paged_ref(qkv, out, k_cache, v_cache, bt, batch.cu_seqlens, batch.seq_lens, B, T, **geo)
    singles = batch.num_singles if ws.split_k else 0
    # a few single rows beside long portions are not worth two more launches
    use_decode = singles == B or singles >= 4
    if use_decode:
        ops.attn_decode(qkv, out, ws.part, k_cache, v_cache, bt, None if singles == B else batch.cu_seqlens,
                        batch.seq_lens, B, ws.splits(B), **geo)
        if singles == B:
            return out
    return ops.attn_flash(qkv, out, k_cache, v_cache, bt, batch.cu_seqlens, batch.seq_lens, B, T, batch.max_q_len,
                          skip_single=use_decode, **geo)
