"""Triangle multiplication (AF3 Algorithms 12/13) on the HIP kernels."""

from __future__ import annotations

import torch
import torch.nn as nn

from .. import check, ops
from .base import HipModule, bf16, drop_mesh, f32, in_check_mode, pad_channels, pad_to


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
        if c_pair % 8:
            raise ValueError("c_pair must be a multiple of 8")
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

    @property
    def padded(self) -> bool:
        """Fewer than 128 channels: run on the 128-channel kernels with zero-padded operands."""
        return self.c_pair < 128 and self.c_pair % 8 == 0

    def _pack(self):
        if self.padded:
            c = self.c_pair
            chunks = []
            for half in (0, 1):              # a, b (d_triangle_multiplication.py:162-165)
                p = pad_to(self.projection.weight[half::2], 128, 128)
                g = pad_to(self.gate.weight[half::2], 128, 128)
                for lo in (0, 64):
                    chunks.append(torch.cat([p[lo:lo + 64], g[lo:lo + 64]], dim=0))
            vec = lambda t: f32(pad_to(t, 128))
            return dict(
                w_proj_gate=bf16(torch.stack(chunks)),
                w_out=bf16(pad_to(self.output_projection.weight, 128, 128)),
                w_gl=bf16(pad_to(self.gating_linear.weight, 128, 128)),
                ln_in_w=vec(self.left_norm_input.weight), ln_in_b=vec(self.left_norm_input.bias),
                ln_c_w=vec(self.center_norm.weight), ln_c_b=vec(self.center_norm.bias))
        if self.c_pair != 128:
            return dict(
                w_proj=bf16(self.projection.weight), w_gate=bf16(self.gate.weight),
                w_out=bf16(self.output_projection.weight), w_gl=bf16(self.gating_linear.weight),
                ln_in_w=f32(self.left_norm_input.weight), ln_in_b=f32(self.left_norm_input.bias),
                ln_c_w=f32(self.center_norm.weight), ln_c_b=f32(self.center_norm.bias))
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

    def _run_other_width(self, pair: torch.Tensor, mask, residual: bool):
        """Pair widths other than 128 (the 64-channel blocks of the template
        embedding, nn/d_template.py:198-201): the same steps as separate
        launches — LayerNorm, projections and the per-channel contraction on the
        MFMA kernels, the gating products and layout changes as elementwise passes."""
        p = self.packed()
        n, c = pair.shape[0], self.c_pair
        x = ops.layer_norm(pair, p["ln_in_w"], p["ln_in_b"])
        proj = ops.linear(x, p["w_proj"], out_dtype=torch.float32)
        gate = ops.linear(x, p["w_gate"], out_dtype=torch.float32, sigmoid=True)
        pg = proj * gate * mask.to(torch.float32)[..., None]                      # [i, k, 2c]
        # operand a of channel ch is row 2 ch, operand b row 2 ch + 1 (:162-165); channel-major, k last
        if self._outgoing:       # out[i, j] = sum_k a[i, k] b[j, k]
            lhs, rhs = pg[..., 0::2].permute(2, 0, 1), pg[..., 1::2].permute(2, 0, 1)
        else:                    # out[i, j] = sum_k b[k, i] a[k, j]
            lhs, rhs = pg[..., 1::2].permute(2, 1, 0), pg[..., 0::2].permute(2, 1, 0)
        pad = (0, (-n) % 8)
        lhs = torch.nn.functional.pad(lhs.to(torch.bfloat16), pad).contiguous()
        rhs = torch.nn.functional.pad(rhs.to(torch.bfloat16), pad).contiguous()
        t = ops.batched_nt_product(lhs, rhs).permute(1, 2, 0).contiguous()        # [i, j, c]
        y = ops.layer_norm(t, p["ln_c_w"], p["ln_c_b"])
        out_gate = ops.linear(x, p["w_gl"], out_dtype=torch.float32, sigmoid=True)
        return ops.linear(y, p["w_out"], out_dtype=pair.dtype, mode=ops._L.LINEAR_GATE_RES,
                          gate=out_gate.view(n * n, c), residual=pair if residual else None,
                          out=pair if residual else None)

    def run_padded(self, pair128: torch.Tensor, mask, residual: bool):
        """`pair128`: the [N, N, c_pair] tensor zero-padded to 128 channels; so is the result."""
        p = self.packed()
        return ops.triangle_multiplication(
            pair128, mask, 0 if self._outgoing else 1, p["ln_in_w"], p["ln_in_b"], p["w_proj_gate"],
            p["ln_c_w"], p["ln_c_b"], p["w_out"], p["w_gl"], residual=residual, valid_channels=self.c_pair)

    def run(self, pair: torch.Tensor, mask, residual: bool):
        if self.padded:
            res = self.run_padded(pad_channels(pair), mask, residual)[..., :self.c_pair]
            if residual:
                pair.copy_(res)
                return pair
            return res.contiguous()
        if self.c_pair != 128:
            return self._run_other_width(pair, mask, residual)
        p = self.packed()
        return ops.triangle_multiplication(
            pair, mask, 0 if self._outgoing else 1, p["ln_in_w"], p["ln_in_b"], p["w_proj_gate"],
            p["ln_c_w"], p["ln_c_b"], p["w_out"], p["w_gl"], residual=residual)

    def forward(self, pair: torch.Tensor, mask: torch.Tensor, head: int = 0) -> torch.Tensor:
        """pair [N, N, c_pair], mask [N, N] -> update [N, N, c_pair] (same dtype)."""
        if in_check_mode():
            return check.triangle_multiplication(self, pair, mask)
        return self.run(pair.contiguous(), mask, residual=False)
