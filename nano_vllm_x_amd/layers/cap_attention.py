"""Causal attention with grouped key/value heads, separate key and value sizes, rotary positions on a leading part of each
head, unit-mean-square values and capped scores, over per-token key and value rows in the token cache."""
from __future__ import annotations

import torch
from torch import nn

from .. import ops
from .rotary_embedding import rotary_frequencies


class SoftcapAttention(nn.Module):
    """q = W_q h, k = W_k h (rotated by position), v = W_v h (each head divided by its root mean square, cached so);
    score = scale * q . k, then cap * tanh(score / cap) (cap None or 0: none), softmax over the causal prefix, W_o on the
    concatenated heads.  Query head j reads key/value head j // (heads / kv_heads).  `rot` = {dims, base, scaling | None}.
    The three projections are one matrix product; the cache holds two rows per token under `cache_names`."""

    def __init__(self, width: int, heads: int, kv_heads: int, dim: int, vdim: int, rot: dict, scale: float, softcap, eps: float, cache_names):
        super().__init__()
        if heads % kv_heads:
            raise ValueError("query heads must be a multiple of key/value heads")
        self.heads, self.kv_heads, self.dim, self.vdim = heads, kv_heads, dim, vdim
        self.scale, self.softcap, self.eps = float(scale), float(softcap or 0.0), eps
        self.k_name, self.v_name = cache_names
        self.rot_dims = int(rot["dims"]) if rot else 0
        if self.rot_dims % 2 or self.rot_dims > dim:
            raise ValueError("the rotated part of a head must be even and within the head")
        if self.rot_dims:
            freq, self.mag = rotary_frequencies(self.rot_dims, rot["base"], rot.get("scaling"))
            self.register_buffer("freq", freq.to(torch.float64), persistent=False)
        else:
            self.freq, self.mag = None, 1.0
        self.qkv_proj = nn.Linear(width, heads * dim + kv_heads * (dim + vdim), bias=False)     # rows: q | k | v
        self.o_proj = nn.Linear(heads * vdim, width, bias=False)

    def cache_rows(self) -> dict:
        return {self.k_name: self.kv_heads * self.dim, self.v_name: self.kv_heads * self.vdim}

    def forward(self, h: torch.Tensor, positions: torch.Tensor, md) -> torch.Tensor:
        k_cache, v_cache = md.cache.latent(self.k_name), md.cache.latent(self.v_name)
        q = ops.rope_vnorm_store(self.qkv_proj(h), positions, self.freq, self.mag, self.rot_dims, self.eps, md.out_slots, k_cache, v_cache,
                                 self.heads, self.kv_heads, self.dim, self.vdim)
        o = ops.softcap_attn(q, k_cache, v_cache, md.kv_indices, md.kv_start, md.kv_len, md.layout, self.scale, self.softcap, self.heads,
                             self.kv_heads, self.dim, self.vdim)
        return self.o_proj(o)
