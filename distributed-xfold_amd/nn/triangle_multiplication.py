"""Triangle multiplication (AF3 Algorithms 12/13) on the HIP kernels."""

from __future__ import annotations

import torch
import torch.nn as nn

from .. import check, ops
from .base import HipModule, bf16, drop_mesh, f32, in_check_mode


class TriangleMultiplication(HipModule):
    """Same constructor keywords, parameters and call signature as the reference's
    XSMMTriangleMultiplication / DistributeTriangleMultiplication
    (nn/d_triangle_multiplication.py:22-40,103-124)."""

    def __init__(self, *args, c_pair: int = 128, _outgoing: bool = True) -> None:
        super().__init__()
        args = drop_mesh(args)
        if len(args) > 0:
            c_pair = args[0]
        if len(args) > 1:
            _outgoing = args[1]
        if c_pair != 128:
            raise ValueError("the HIP triangle multiplication is built for c_pair = 128")
        self.c_pair = c_pair
        self.left_norm_input = nn.LayerNorm(c_pair)
        self.projection = nn.Linear(c_pair, 2 * c_pair, bias=False)
        self.gate = nn.Linear(c_pair, 2 * c_pair, bias=False)
        self.center_norm = nn.LayerNorm(c_pair)
        self.output_projection = nn.Linear(c_pair, c_pair, bias=False)
        self.gating_linear = nn.Linear(c_pair, c_pair, bias=False)
        self._outgoing = _outgoing
        # equation strings as in d_triangle_multiplication.py:116-124
        self.c_equation = "ikc,jkc->ijc" if _outgoing else "kjc,kic->ijc"
        self.equation = "cik,cjk->cij" if _outgoing else "ckj,cki->cij"

    def _pack(self):
        # operand a of channel c is output row 2c of projection/gate, operand b row
        # 2c+1 (d_triangle_multiplication.py:162-165; de-interleave as :128-129),
        # regrouped into four [64 projection rows | 64 gate rows] chunks.
        wp, wg = self.projection.weight, self.gate.weight
        chunks = []
        for half in (0, 1):              # a, b
            p, g = wp[half::2], wg[half::2]
            for lo in (0, 64):
                chunks.append(torch.cat([p[lo:lo + 64], g[lo:lo + 64]], dim=0))
        return dict(
            w_proj_gate=bf16(torch.stack(chunks)),
            w_out=bf16(self.output_projection.weight),
            w_gl=bf16(self.gating_linear.weight),
            ln_in_w=f32(self.left_norm_input.weight), ln_in_b=f32(self.left_norm_input.bias),
            ln_c_w=f32(self.center_norm.weight), ln_c_b=f32(self.center_norm.bias),
        )

    def run(self, pair: torch.Tensor, mask, residual: bool):
        p = self.packed()
        return ops.triangle_multiplication(
            pair, mask, 0 if self._outgoing else 1, p["ln_in_w"], p["ln_in_b"], p["w_proj_gate"],
            p["ln_c_w"], p["ln_c_b"], p["w_out"], p["w_gl"], residual=residual)

    def forward(self, pair: torch.Tensor, mask: torch.Tensor, head: int = 0) -> torch.Tensor:
        """pair [N, N, c_pair], mask [N, N] -> update [N, N, c_pair] (same dtype)."""
        if in_check_mode():
            return check.triangle_multiplication(self, pair, mask)
        return self.run(pair.contiguous(), mask, residual=False)
