"""Evoformer (MSA) block: outer-product mean, MSA pair-weighted averaging, MSA
transition and the five pair operators (nn/d_pairformer.py:174-252,
nn/d_primitives.py:42-70, nn/d_attention.py:113-156).  Same constructor
keywords, parameter names and `forward` signatures as the reference's
Distribute* classes; msa and pair are updated in place as the reference's `+=`.

Both MSA operators are products over long axes and run on the bf16 MFMA
kernels:
  * outer-product mean: out[b, d, :] = W^T vec(sum_a L[a, b, :] (x) R[a, d, :]).
    The sum over the MSA rows is one product [(b, c), a] x [(d, e), a]^T per
    block of 128 tokens b, whose epilogue stores element ((b, c), (d, e)) at
    [(b, d)][(c, e)], the layout the second product with W [(c, e), f] reads
    (a 200 MB bf16 slab at 768 tokens, inside the 256 MB last-level cache); the
    [N, N, 32, 32] tensor the reference's einsum materialises (1.2 GB) never
    exists as a whole and nothing is permuted.
  * pair-weighted averaging: per head, softmax(pair logits) [q, k] times the
    head's values of all MSA rows [(row, channel), k]^T.
Both sum over an index (MSA rows, tokens) that the activations [rows, N, c]
carry as an outer one, while the dense kernels want it innermost: the operands
are produced transposed (projection weights as the left operand) or run through
the bf16 transpose kernel, not through strided copies.
"""

from __future__ import annotations

from typing import Optional

import torch
import torch.nn as nn
import torch.nn.functional as F

from .. import check, ops
from .attention import GridSelfAttention
from .base import HipModule, bf16, drop_mesh, f32, in_check_mode, pad_rows
from .primitives import Transition
from .triangle_multiplication import TriangleMultiplication


def _pad_last(x: torch.Tensor, multiple: int = 8) -> torch.Tensor:
    k = x.shape[-1]
    return x if k % multiple == 0 else F.pad(x, (0, (-k) % multiple))


class OuterProductMean(HipModule):
    """nn/d_primitives.py:42-70."""

    def __init__(self, *args, c_msa: int = 64, num_output_channel: int = 128, num_outer_channel: int = 32,
                 epsilon: float = 1e-3) -> None:
        super().__init__()
        args = drop_mesh(args)
        vals = list(args) + [c_msa, num_output_channel, num_outer_channel][len(args):]
        c_msa, num_output_channel, num_outer_channel = vals[:3]
        self.c_msa, self.num_output_channel, self.num_outer_channel = c_msa, num_output_channel, num_outer_channel
        self.epsilon = epsilon
        self.layer_norm_input = nn.LayerNorm(c_msa)
        self.left_projection = nn.Linear(c_msa, num_outer_channel, bias=False)
        self.right_projection = nn.Linear(c_msa, num_outer_channel, bias=False)
        self.output_w = nn.Parameter(torch.zeros(num_outer_channel, num_outer_channel, num_output_channel))
        self.output_b = nn.Parameter(torch.zeros(num_output_channel))

    def _pack(self):
        co = self.num_outer_channel
        return dict(ln_w=f32(self.layer_norm_input.weight), ln_b=f32(self.layer_norm_input.bias),
                    w_l=bf16(self.left_projection.weight), w_r=bf16(self.right_projection.weight),
                    w_out=bf16(self.output_w.detach().reshape(co * co, -1).t()), b_out=f32(self.output_b))

    @torch.no_grad()
    def run(self, msa, mask, residual: Optional[torch.Tensor] = None, block: int = 128):
        """-> [N, N, c_pair] fp32, or `residual` (the pair tensor) updated in place."""
        p = self.packed()
        a, n, _ = msa.shape
        co, cf = self.num_outer_channel, self.num_output_channel
        m = mask.float()
        x = ops.layer_norm(msa.contiguous(), p["ln_w"], p["ln_b"])
        mb = m[..., None].to(torch.bfloat16)

        def projected(w):        # [(token, channel), MSA row]: the summation index innermost
            y = ops.linear(x, w) * mb                                                       # [a, N, co]
            if a % 8 == 0 and (n * co) % 8 == 0:
                return ops.transpose2d(y.view(a, n * co))
            return _pad_last(y.permute(1, 2, 0).reshape(n * co, a)).contiguous()
        lt, rt = projected(p["w_l"]), projected(p["w_r"])
        inv_norm = (1.0 / (self.epsilon + m.t() @ m)).contiguous()                         # [b, d]
        out = residual if residual is not None else torch.zeros((n, n, cf), dtype=torch.float32, device=msa.device)
        for b0 in range(0, n, block):
            b1 = min(n, b0 + block)
            if co == 32:
                outer = ops.linear(lt[b0 * co:b1 * co], rt, mode=ops._L.LINEAR_REGROUP32)  # [(b, d), (c, e)]
            else:
                outer = ops.linear(lt[b0 * co:b1 * co], rt)                                # [(b, c), (d, e)]
                outer = outer.view(b1 - b0, co, n, co).permute(0, 2, 1, 3).reshape((b1 - b0) * n, co * co)
            # (outer W + b) / (eps + coverage), added to the pair rows, in the product's epilogue
            rows = out[b0:b1].view(-1, cf)
            ops.linear(outer, p["w_out"], bias=p["b_out"], out_dtype=out.dtype, mode=ops._L.LINEAR_ROWGATE_RES,
                       gate=inv_norm[b0:b1], residual=rows, out=rows)
        return out

    def forward(self, msa: torch.Tensor, mask: torch.Tensor) -> torch.Tensor:
        if in_check_mode():
            return _check_outer_product_mean(self, msa, mask)
        return self.run(msa, mask)


class MSAAttention(HipModule):
    """nn/d_attention.py:113-156."""

    def __init__(self, *args, c_msa: int = 64, c_pair: int = 128, num_head: int = 8) -> None:
        super().__init__()
        args = drop_mesh(args)
        vals = list(args) + [c_msa, c_pair, num_head][len(args):]
        c_msa, c_pair, num_head = vals[:3]
        if c_pair != 128:
            raise ValueError("the HIP pair-logit projection is built for c_pair = 128")
        self.c_msa, self.c_pair, self.num_head = c_msa, c_pair, num_head
        self.value_dim = c_msa // num_head
        self.act_norm = nn.LayerNorm(c_msa)
        self.pair_norm = nn.LayerNorm(c_pair)
        self.pair_logits = nn.Linear(c_pair, num_head, bias=False)
        self.v_projection = nn.Linear(c_msa, c_msa, bias=False)
        self.gating_query = nn.Linear(c_msa, c_msa, bias=False)
        self.output_projection = nn.Linear(c_msa, c_msa, bias=False)

    def _pack(self):
        return dict(ln_w=f32(self.act_norm.weight), ln_b=f32(self.act_norm.bias),
                    pn_w=f32(self.pair_norm.weight), pn_b=f32(self.pair_norm.bias),
                    w_logits=pad_rows(bf16(self.pair_logits.weight), 32), w_v=bf16(self.v_projection.weight),
                    w_g=bf16(self.gating_query.weight), w_o=bf16(self.output_projection.weight))

    @torch.no_grad()
    def run(self, msa, msa_mask, pair, residual: bool):
        p = self.packed()
        a, n, c = msa.shape
        h, d = self.num_head, self.value_dim
        x = ops.layer_norm(msa.contiguous(), p["ln_w"], p["ln_b"])
        logits = ops.pair_logits(pair.contiguous(), p["pn_w"], p["pn_b"], p["w_logits"], h)     # [h, q, k] fp32
        # softmax over the keys of logits + 1e9 (key mask - 1), bf16, rows padded to a multiple of 8
        w = ops.masked_softmax_rows(logits, msa_mask.float().max(dim=0).values.contiguous())        # [h, q, k]
        if n % 8 == 0 and (a * n) % 8 == 0 and c % 8 == 0:
            # Everything with the tokens innermost: the value and gate projections are taken
            # transposed (weights as the left operand), [(h, d), (row, k)], which is per head the
            # k-contiguous right operand of the averaging product; its result [(h, d), (row, q)]
            # has the same layout, takes the gate there and is transposed once for the output projection.
            x2 = x.view(a * n, c)
            v_t = ops.linear(p["w_v"], x2)                                                        # [(h d), (row, k)]
            gate_t = ops.linear(p["w_g"], x2, sigmoid=True)
            avg_t = ops.batched_nt_product(v_t.view(h, d * a, n), w)                              # [h, (d, row), q]
            avg = ops.transpose2d(avg_t.view(c, a * n) * gate_t).view(a, n, c)
        else:
            v = ops.linear(x, p["w_v"])                                                           # [a, k, (h d)]
            gate = ops.linear(x, p["w_g"], sigmoid=True)
            vt = _pad_last(v.view(a, n, h, d).permute(2, 0, 3, 1).reshape(h, a * d, n)).contiguous()
            avg = ops.batched_nt_product(w, vt)                                                   # [h, q, (row, d)]
            avg = avg.view(h, n, a, d).permute(2, 1, 0, 3).reshape(a, n, c) * gate
        if residual:
            return ops.linear(avg, p["w_o"], out_dtype=msa.dtype, mode=ops._L.LINEAR_GATE_RES, residual=msa, out=msa)
        return ops.linear(avg, p["w_o"], out_dtype=msa.dtype)

    def forward(self, msa: torch.Tensor, msa_mask: torch.Tensor, pair: torch.Tensor) -> torch.Tensor:
        if in_check_mode():
            return _check_msa_attention(self, msa, msa_mask, pair)
        return self.run(msa, msa_mask, pair, residual=False)


class EvoformerBlock(HipModule):
    """nn/d_pairformer.py:174-252."""

    def __init__(self, *args, c_msa: int = 64, c_pair: int = 128, n_heads_pair: int = 4) -> None:
        super().__init__()
        args = drop_mesh(args)
        vals = list(args) + [c_msa, c_pair, n_heads_pair][len(args):]
        c_msa, c_pair, n_heads_pair = vals[:3]
        self.c_msa, self.c_pair = c_msa, c_pair
        self.outer_product_mean = OuterProductMean(c_msa=c_msa, num_output_channel=c_pair)
        self.msa_attention1 = MSAAttention(c_msa=c_msa, c_pair=c_pair)
        self.msa_transition = Transition(c_x=c_msa)
        self.triangle_multiplication_outgoing = TriangleMultiplication(c_pair=c_pair, _outgoing=True)
        self.triangle_multiplication_incoming = TriangleMultiplication(c_pair=c_pair, _outgoing=False)
        self.pair_attention1 = GridSelfAttention(c_pair=c_pair, num_head=n_heads_pair, transpose=False)
        self.pair_attention2 = GridSelfAttention(c_pair=c_pair, num_head=n_heads_pair, transpose=True)
        self.pair_transition = Transition(c_x=c_pair)

    def _pack(self):
        return {}

    @torch.no_grad()
    def forward(self, msa: torch.Tensor, pair: torch.Tensor, msa_mask: torch.Tensor, pair_mask: torch.Tensor):
        """msa [rows, N, c_msa], pair [N, N, c_pair], msa_mask [rows, N],
        pair_mask [N, N] -> (msa, pair), both updated in place."""
        if in_check_mode():
            pair = pair + self.outer_product_mean(msa, msa_mask)
            msa = msa + self.msa_attention1(msa, msa_mask, pair)
            msa = msa + self.msa_transition(msa)
            pair = pair + self.triangle_multiplication_outgoing(pair, pair_mask)
            pair = pair + self.triangle_multiplication_incoming(pair, pair_mask.t().contiguous())
            pair = pair + self.pair_attention1(pair, pair_mask)
            pair = pair + self.pair_attention2(pair, pair_mask)
            pair = pair + self.pair_transition(pair)
            return msa, pair
        if not (pair.is_contiguous() and msa.is_contiguous()):
            raise ValueError("msa and pair must be contiguous (they are updated in place)")
        self.outer_product_mean.run(msa, msa_mask, residual=pair)
        self.msa_attention1.run(msa, msa_mask, pair, residual=True)
        self.msa_transition.run(msa, residual=True)
        self.triangle_multiplication_outgoing.run(pair, pair_mask, residual=True)
        self.triangle_multiplication_incoming.run(pair, pair_mask.t().contiguous(), residual=True)   # :217
        self.pair_attention1.run(pair, pair_mask, residual=True)
        self.pair_attention2.run(pair, pair_mask, residual=True)
        self.pair_transition.run(pair, residual=True)
        return msa, pair


# ------------------------------------------------------------ fp32 check mode

def _check_outer_product_mean(mod: OuterProductMean, msa, mask):
    m = mask.float()[..., None]
    x = check._ln(msa.float().contiguous(), mod.layer_norm_input)
    left = m * check._lin(x, mod.left_projection)
    right = m * check._lin(x, mod.right_projection)
    a, n, co = left.shape
    lt = left.permute(1, 2, 0).reshape(n * co, a).contiguous()
    rt = right.permute(1, 2, 0).reshape(n * co, a).contiguous()
    outer = ops.ck_linear(lt, rt).view(n, co, n, co).permute(0, 2, 1, 3).reshape(n * n, co * co).contiguous()
    w = mod.output_w.detach().float().reshape(co * co, -1).t().contiguous()
    act = ops.ck_linear(outer, w, bias=mod.output_b.detach().float().contiguous()).view(n, n, -1)
    norm = (mask.float().t() @ mask.float())[..., None]
    return act / (mod.epsilon + norm)


def _check_msa_attention(mod: MSAAttention, msa, msa_mask, pair):
    a, n, c = msa.shape
    h, d = mod.num_head, mod.value_dim
    x = check._ln(msa.float().contiguous(), mod.act_norm)
    z = check._ln(pair.float().contiguous(), mod.pair_norm)
    logits = check._lin(z, mod.pair_logits).permute(2, 0, 1)
    logits = logits + 1e9 * (msa_mask.float().max(dim=0).values - 1.0)
    w = torch.softmax(logits, dim=-1).contiguous()
    v = check._lin(x, mod.v_projection)
    vt = v.view(a, n, h, d).permute(2, 0, 3, 1).reshape(h, a * d, n).contiguous()
    avg = torch.stack([ops.ck_linear(w[i], vt[i]) for i in range(h)])
    avg = avg.view(h, n, a, d).permute(2, 1, 0, 3).reshape(a, n, c)
    avg = (avg * torch.sigmoid(check._lin(x, mod.gating_query))).contiguous()
    return check._lin(avg, mod.output_projection)
