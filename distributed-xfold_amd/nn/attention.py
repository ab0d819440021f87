"""Triangle (grid) self-attention around the starting / ending node."""

from __future__ import annotations

import torch
import torch.nn as nn

from .. import check, ops
from .base import HipModule, bf16, drop_mesh, f32, in_check_mode, pad_rows


class GridSelfAttention(HipModule):
    """Same constructor keywords, parameters and call signature as the reference's
    DistributeGridSelfAttention (nn/d_attention.py:23-34,88)."""

    def __init__(self, *args, c_pair: int = 128, num_head: int = 4, transpose: bool = False) -> None:
        super().__init__()
        args = drop_mesh(args)
        vals = list(args) + [c_pair, num_head, transpose][len(args):]
        c_pair, num_head, transpose = vals
        if c_pair != 128 or c_pair // num_head != 32:
            raise ValueError("the HIP triangle attention is built for c_pair = 128 and head dim 32")
        self.c_pair, self.num_head, self.transpose = c_pair, num_head, transpose
        self.qkv_dim = c_pair // num_head
        self.act_norm = nn.LayerNorm(c_pair)
        self.pair_bias_projection = nn.Linear(c_pair, num_head, bias=False)
        self.q_projection = nn.Linear(c_pair, c_pair, bias=False)
        self.k_projection = nn.Linear(c_pair, c_pair, bias=False)
        self.v_projection = nn.Linear(c_pair, c_pair, bias=False)
        self.gating_query = nn.Linear(c_pair, c_pair, bias=False)
        self.output_projection = nn.Linear(c_pair, c_pair, bias=False)

    def _pack(self):
        return dict(
            w_qkvg=bf16(torch.stack([self.q_projection.weight, self.k_projection.weight,
                                     self.v_projection.weight, self.gating_query.weight])),
            w_out=bf16(self.output_projection.weight),
            w_bias=pad_rows(bf16(self.pair_bias_projection.weight), 32),
            ln_w=f32(self.act_norm.weight), ln_b=f32(self.act_norm.bias),
        )

    def run(self, pair, mask, residual: bool):
        p = self.packed()
        return ops.grid_self_attn(pair, mask, self.transpose, p["ln_w"], p["ln_b"], p["w_bias"], None,
                                  p["w_qkvg"], p["w_out"], self.num_head, residual=residual)

    def forward(self, pair, mask, full_pair=None):
        """pair [N, N, c_pair], mask [N, N] -> update [N, N, c_pair].

        `full_pair` is the un-sharded tensor the reference's data-parallel path
        takes the pair bias from (nn/d_attention.py:58-62); on one GPU it is
        `pair` itself, anything else is rejected."""
        if full_pair is not None and full_pair is not pair:
            if full_pair.shape != pair.shape or full_pair.data_ptr() != pair.data_ptr():
                raise ValueError("single-GPU build: full_pair must be the same tensor as pair")
        if in_check_mode():
            return check.grid_self_attention(self, pair, mask)
        return self.run(pair.contiguous(), mask, residual=False)
