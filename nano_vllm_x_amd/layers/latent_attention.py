"""Latent attention: keys and values of every head are linear maps of one cached vector per token."""
from __future__ import annotations

import torch
import torch.nn.functional as F
from torch import nn

from .. import ops


class LatentAttention(nn.Module):
    """q = W_uq RMSnorm(W_dq h), c = RMSnorm(W_dkv h) (both norms with a plain weight); per head k = W_uk c, v = W_uv c,
    softmax(scale * q . k) over the causal prefix, the head's output times sigmoid(W_g h)_head, then W_o.  No positions.

    The cache holds c alone (kv_rank values per token).  The kernel attends over the cached latents directly: the key map is
    folded into the query (q~ = W_uk^T q, per head) and the value map is applied to the weighted sum of latents, which is
    the same function and reads kv_rank instead of heads * (dim + vdim) values per key.  The three projections of h (query
    latent, key/value latent, gates) are one matrix product."""

    def __init__(self, width: int, heads: int, dim: int, vdim: int, q_rank: int, kv_rank: int, scale: float, eps: float, layer_id: int):
        super().__init__()
        self.heads, self.dim, self.vdim, self.q_rank, self.kv_rank = heads, dim, vdim, q_rank, kv_rank
        self.scale, self.eps, self.layer_id = scale, eps, layer_id
        self.down_proj = nn.Linear(width, q_rank + kv_rank + heads, bias=False)     # rows: dq | dkv | g
        self.q_norm = nn.Parameter(torch.ones(q_rank, dtype=torch.float32))
        self.kv_norm = nn.Parameter(torch.ones(kv_rank, dtype=torch.float32))
        self.uq_proj = nn.Linear(q_rank, heads * dim, bias=False)
        self.uk = nn.Parameter(torch.empty(heads, dim, kv_rank))       # W_uk, head by head
        self.uv = nn.Parameter(torch.empty(heads, vdim, kv_rank))      # W_uv, head by head
        self.o_proj = nn.Linear(heads * vdim, width, bias=False)

    def forward(self, h: torch.Tensor, md) -> torch.Tensor:
        t = h.shape[0]
        cache = md.cache.latent(self.layer_id)
        cq, gate = ops.latent_prep(self.down_proj(h), self.q_norm, self.kv_norm, self.eps, md.out_slots, cache, self.heads)
        q = self.uq_proj(cq).view(t, self.heads, self.dim).transpose(0, 1)              # (heads, T, dim)
        q_folded = torch.bmm(q, self.uk)                                                 # (heads, T, kv_rank)
        o = ops.latent_attn(q_folded, cache, md.kv_indices, md.kv_start, md.kv_len, md.layout, self.scale, gate=gate)
        v = torch.bmm(o, self.uv.transpose(1, 2))                                        # (heads, T, vdim)
        return self.o_proj(v.transpose(0, 1).reshape(t, self.heads * self.vdim))
