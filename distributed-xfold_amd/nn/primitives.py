"""SwiGLU transition."""

from __future__ import annotations

import torch
import torch.nn as nn

from .. import check
from .. import lib as L
from .. import ops
from .base import HipModule, bf16, drop_mesh, f32, in_check_mode, pack_swiglu, pad_channels, pad_to


class Transition(HipModule):
    """Same constructor keywords, parameters and call signature as the reference's
    DistributeTransition (nn/d_primitives.py:21-31): LN -> GLU(transition1) ->
    transition2, no biases.  128-channel inputs (the pair tensor) run as one
    fused kernel; other widths as LayerNorm + two MFMA projections."""

    def __init__(self, *args, c_x: int = None, num_intermediate_factor: int = 4) -> None:
        super().__init__()
        args = drop_mesh(args)
        if len(args) > 0:
            c_x = args[0]
        if len(args) > 1:
            num_intermediate_factor = args[1]
        if c_x is None or c_x % 8:
            raise ValueError("c_x must be given and be a multiple of 8")
        self.c_x = c_x
        self.num_intermediate_factor = num_intermediate_factor
        self.input_layer_norm = nn.LayerNorm(c_x)
        self.transition1 = nn.Linear(c_x, num_intermediate_factor * c_x * 2, bias=False)
        self.transition2 = nn.Linear(num_intermediate_factor * c_x, c_x, bias=False)

    @property
    def padded(self) -> bool:
        """Fewer than 128 channels: run on the fused 128-channel kernel with zero-padded operands."""
        return self.c_x < 128

    def _pack(self):
        if self.padded:
            hidden = self.num_intermediate_factor * self.c_x
            hp = (hidden + 63) // 64 * 64            # zero hidden units give silu(0) * 0 = 0
            w1 = self.transition1.weight.detach()
            w1p = torch.cat([pad_to(w1[:hidden], hp, 128), pad_to(w1[hidden:], hp, 128)], dim=0)
            return dict(ln_w=f32(pad_to(self.input_layer_norm.weight, 128)),
                        ln_b=f32(pad_to(self.input_layer_norm.bias, 128)),
                        w1=bf16(pack_swiglu(w1p, 64)).reshape(hp // 64, 128, 128),
                        w2=bf16(pad_to(self.transition2.weight, 128, hp)))
        d = dict(ln_w=f32(self.input_layer_norm.weight), ln_b=f32(self.input_layer_norm.bias),
                 w2=bf16(self.transition2.weight))
        if self.c_x == 128:
            hidden = self.num_intermediate_factor * 128
            d["w1"] = bf16(pack_swiglu(self.transition1.weight, 64)).reshape(hidden // 64, 128, 128)
        else:
            d["w1"] = bf16(pack_swiglu(self.transition1.weight, 32))
        return d

    def run_padded(self, x128, residual: bool):
        """`x128`: the rows zero-padded to 128 channels; so is the result."""
        p = self.packed()
        return ops.transition128(x128, p["ln_w"], p["ln_b"], p["w1"], p["w2"], residual=residual,
                                 valid_channels=self.c_x)

    def run(self, x, residual: bool):
        if self.padded:
            res = self.run_padded(pad_channels(x), residual)[..., :self.c_x]
            if residual:
                x.copy_(res)
                return x
            return res.contiguous()
        p = self.packed()
        if self.c_x == 128:
            return ops.transition128(x, p["ln_w"], p["ln_b"], p["w1"], p["w2"], residual=residual)
        xn = ops.layer_norm(x, p["ln_w"], p["ln_b"])
        h = ops.linear(xn, p["w1"], mode=L.LINEAR_SWIGLU)
        return ops.linear(h, p["w2"], out_dtype=x.dtype, mode=L.LINEAR_GATE_RES,
                          residual=x if residual else None, out=x if residual else None)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        if in_check_mode():
            return check.transition(self, x)
        return self.run(x.contiguous(), residual=False)
