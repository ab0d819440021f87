"""Triangle (grid) self-attention around the starting / ending node."""

from __future__ import annotations

import torch
import torch.nn as nn

from .. import check, ops
from .base import HipModule, bf16, drop_mesh, f32, in_check_mode, pad_channels, pad_rows, pad_to


class GridSelfAttention(HipModule):
    """Same constructor keywords, parameters and call signature as the reference's
    DistributeGridSelfAttention (nn/d_attention.py:23-34,88)."""

    def __init__(self, *args, c_pair: int = 128, num_head: int = 4, transpose: bool = False) -> None:
        super().__init__()
        args = drop_mesh(args)
        vals = list(args) + [c_pair, num_head, transpose][len(args):]
        c_pair, num_head, transpose = vals
        if c_pair % num_head or c_pair // num_head not in (16, 24, 32, 48):
            raise ValueError("head dim must be 16, 24, 32 or 48")
        self.fused = c_pair == 128 and c_pair // num_head == 32
        # fewer channels, four heads of at most 32: the 128-channel kernels on zero-padded operands
        self.padded = c_pair < 128 and c_pair % 8 == 0 and num_head == 4 and c_pair // num_head <= 32
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
        if self.padded:
            c, h, d = self.c_pair, self.num_head, self.qkv_dim

            def heads_out(w):        # [h * d, c] -> [h * 32, 128]: each head's rows at the front of a 32-row slot
                return pad_to(w.detach().reshape(h, d, c), h, 32, 128).reshape(128, 128)

            w_out = pad_to(self.output_projection.weight.detach().reshape(c, h, d), 128, h, 32).reshape(128, 128)
            vec = lambda t: f32(pad_to(t, 128))
            return dict(
                w_qkvg=bf16(torch.stack([heads_out(m.weight) for m in (self.q_projection, self.k_projection,
                                                                       self.v_projection, self.gating_query)])),
                w_out=bf16(w_out), w_bias=bf16(pad_to(self.pair_bias_projection.weight, 32, 128)),
                ln_w=vec(self.act_norm.weight), ln_b=vec(self.act_norm.bias))
        if not self.fused:
            return dict(
                w_qkvg=bf16(torch.cat([self.q_projection.weight, self.k_projection.weight,
                                       self.v_projection.weight, self.gating_query.weight], dim=0)),
                w_out=bf16(self.output_projection.weight), w_bias=bf16(self.pair_bias_projection.weight),
                ln_w=f32(self.act_norm.weight), ln_b=f32(self.act_norm.bias))
        return dict(
            w_qkvg=bf16(torch.stack([self.q_projection.weight, self.k_projection.weight,
                                     self.v_projection.weight, self.gating_query.weight])),
            w_out=bf16(self.output_projection.weight),
            w_bias=pad_rows(bf16(self.pair_bias_projection.weight), 32),
            ln_w=f32(self.act_norm.weight), ln_b=f32(self.act_norm.bias),
        )

    def _run_other_width(self, pair, mask, residual: bool):
        """Pair widths other than 128 (the 64-channel blocks of the template
        embedding): LayerNorm, the pair-bias projection, the pair-biased gated
        attention over the rows (or columns) with one key mask per row, and the
        output projection as separate launches of the general kernels."""
        p = self.packed()
        n, c, h = pair.shape[0], self.c_pair, self.num_head
        x = ops.layer_norm(pair, p["ln_w"], p["ln_b"])                                       # [q, k, c]
        bias = ops.linear(x, p["w_bias"], out_dtype=torch.float32).permute(2, 0, 1).contiguous()   # [h, q, k]
        if self.transpose:
            # bias and key mask are taken before the activations are transposed (nn/d_attention.py:60-65)
            x = x.transpose(0, 1).contiguous()
        o = ops.batch_diffusion_self_attention(x, mask.to(torch.float32).contiguous(), bias, p["w_qkvg"], None,
                                               h)                                              # [b, s, h, d]
        if not self.transpose:
            return ops.linear(o.view(n, n, c), p["w_out"], out_dtype=pair.dtype, mode=ops._L.LINEAR_GATE_RES,
                              residual=pair if residual else None, out=pair if residual else None)
        upd = ops.linear(o.view(n, n, c), p["w_out"], out_dtype=pair.dtype).transpose(0, 1)
        if residual:
            pair += upd
            return pair
        return upd.contiguous()

    def run_padded(self, pair128, mask, residual: bool):
        """`pair128`: the [N, N, c_pair] tensor zero-padded to 128 channels; so is the result."""
        p = self.packed()
        return ops.grid_self_attn(pair128, mask, self.transpose, p["ln_w"], p["ln_b"], p["w_bias"], None,
                                  p["w_qkvg"], p["w_out"], self.num_head, residual=residual,
                                  valid_channels=self.c_pair)

    def run(self, pair, mask, residual: bool):
        if self.padded:
            res = self.run_padded(pad_channels(pair), mask, residual)[..., :self.c_pair]
            if residual:
                pair.copy_(res)
                return pair
            return res.contiguous()
        if not self.fused:
            return self._run_other_width(pair, mask, residual)
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
