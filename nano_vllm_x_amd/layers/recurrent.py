"""Recurrent token mixers backed by the HIP scan kernels."""
from __future__ import annotations

import torch
import torch.nn.functional as F
from torch import nn

from .. import ops


class MinGRU(nn.Module):
    """Gated recurrence with gates that are functions of the current token alone (no dependence on the state): with z = sigmoid(W_z h + b_z), u = W_x h + b_x and
    cand = u + 1/2 (u >= 0) or sigmoid(u) (u < 0), the state moves as S <- (1 - z) S + z cand and the layer returns
    W_o (S * silu(W_g h)).  The three input projections are one matrix product; gates, candidate and state are float32
    inside the scan kernel, and the state (`inner` floats per sequence) lives in the state pool under `state_name`."""

    def __init__(self, width: int, inner: int, state_name):
        super().__init__()
        self.width, self.inner, self.state_name = width, inner, state_name
        self.zxg_proj = nn.Linear(width, 3 * inner, bias=True)     # rows: z | x | g (the gate g has no bias: zeros)
        self.o_proj = nn.Linear(inner, width, bias=False)

    def state_shapes(self) -> dict:
        return {self.state_name: (self.inner,)}

    def forward(self, h: torch.Tensor, md) -> torch.Tensor:
        zxg = self.zxg_proj(h)
        y = ops.mingru_scan(zxg, md.cache.state(self.state_name), md.layout)
        return self.o_proj(y)
