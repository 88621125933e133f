"""Chooses the latent-attention kernels for a step.

float32 storage: always the plain kernel (fixed key order, any sizes). bfloat16 storage: the MFMA kernel where the
sizes fit it (latent a multiple of 16 up to 512, rotated part a multiple of 8 up to 128, pages of a multiple of 8), with the keys of single rows cut into parts on the
device; the plain kernel otherwise.
"""
from __future__ import annotations

import torch

from . import ops

TARGET_WORKGROUPS = 256   # measured at 16 heads of 512 + 64, 2,048 keys: 64 requests are fastest with 4 parts, 8 with 16 to 32
MAX_SPLITS = 64
SHORTEST_PART = 128    # keys of the longest request in one part (its four waves take a quarter each), at least


class Workspace:
    """Geometry checks and the split-K scratch of one latent shape, sized once."""

    def __init__(self, ctx, heads: int, rank: int, rot_dim: int):
        self.heads, self.rank, self.rot_dim = heads, rank, rot_dim
        self.mfma = ctx.dtype == torch.bfloat16 and ops.latent_mfma_supports(rank, rot_dim, ctx.page_size)
        longest = ctx.max_seq_len or 4096
        self.max_splits = max(1, min(MAX_SPLITS, -(-longest // SHORTEST_PART)))
        self.part = None
        if self.mfma:
            units = max(self.splits(n) * n for n in range(1, ctx.max_reqs + 1)) * heads
            self.part = ctx.workspace.buffer("latent_partials", units * (rank + 4), dtype=torch.float32, rows=1)

    def splits(self, num_reqs: int) -> int:
        """Parts per request in a step of single rows: a function of the batch size only, so a captured graph stays valid."""
        tiles = -(-self.heads // 16)
        return max(1, min(self.max_splits, TARGET_WORKGROUPS // max(1, num_reqs * tiles)))


def paged_attention(qa: torch.Tensor, out: torch.Tensor, cache: torch.Tensor, cache_t, batch, group: int, ws: Workspace, *,
                    scale: float, window: int, heads: int, rank: int, rot_dim: int, page_size: int):
    """qa [T, heads * (rank + rot_dim)] -> out [T, heads * rank] (the attention's output in latent space)."""
    geo = dict(scale=scale, window=window, heads=heads, rank=rank, rot_dim=rot_dim, page_size=page_size)
    bt = batch.block_table[group]
    B, T = batch.num_reqs, batch.num_tokens
    if not ws.mfma:
        return ops.latent_attn_ref(qa, out, cache, bt, batch.cu_seqlens, batch.seq_lens, B, T, **geo)
    splits = ws.splits(B) if batch.all_decode else 1
    return ops.latent_attn_mfma(qa, out, cache, cache_t, bt, batch.cu_seqlens, batch.seq_lens, B, T, splits, ws.part, **geo)
