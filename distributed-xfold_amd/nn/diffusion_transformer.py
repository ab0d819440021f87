"""Diffusion-transformer modules: adaptive LayerNorm, AdaLN-Zero, pair-biased
self-attention, conditioned SwiGLU transition, the 24-block transformer and the
windowed atom cross-attention transformer."""

from __future__ import annotations

from typing import Optional

import torch
import torch.nn as nn

from .. import check
from .. import lib as L
from .. import ops
from .base import HipModule, bf16, drop_mesh, f32, in_check_mode, pack_swiglu, pad_rows


class AdaptiveLayerNorm(HipModule):
    """nn/d_diffusion_transformer.py:37-74.  Output is bf16 (it always feeds a
    projection)."""

    def __init__(self, c_x: int, c_single_cond: int, use_single_cond: bool = False) -> None:
        super().__init__()
        self.c_x, self.c_single_cond, self.use_single_cond = c_x, c_single_cond, use_single_cond
        if use_single_cond:
            self.layer_norm = nn.LayerNorm(c_x, elementwise_affine=False)
            self.single_cond_layer_norm = nn.LayerNorm(c_single_cond, bias=False)
            self.single_cond_scale = nn.Linear(c_single_cond, c_x, bias=True)
            self.single_cond_bias = nn.Linear(c_single_cond, c_x, bias=False)
        else:
            self.layer_norm = nn.LayerNorm(c_x)

    def _pack(self):
        if not self.use_single_cond:
            return dict(ln_w=f32(self.layer_norm.weight), ln_b=f32(self.layer_norm.bias))
        w = torch.cat([self.single_cond_scale.weight, self.single_cond_bias.weight], dim=0)
        b = torch.cat([self.single_cond_scale.bias, torch.zeros_like(self.single_cond_scale.bias)])
        return dict(cond_ln_w=f32(self.single_cond_layer_norm.weight), w_ss=bf16(w), b_ss=f32(b))

    def forward(self, x: torch.Tensor, single_cond: Optional[torch.Tensor] = None,
                scale_shift: Optional[torch.Tensor] = None) -> torch.Tensor:
        """`scale_shift`: fp32 [cond_rows, 2 c_x] view (unit column stride) holding
        what the two conditioning projections of this module give for
        `single_cond`, computed by the caller for many modules at once."""
        assert (single_cond is None) == (self.use_single_cond is False)
        if in_check_mode():
            return check.adaptive_layer_norm(self, x, single_cond)
        x = x.contiguous()
        if scale_shift is not None:
            return ops.layer_norm(x, scale=scale_shift[:, :self.c_x], shift=scale_shift[:, self.c_x:])
        p = self.packed()
        if not self.use_single_cond:
            return ops.layer_norm(x, p["ln_w"], p["ln_b"])
        s = ops.layer_norm(single_cond.contiguous(), p["cond_ln_w"])
        ss = ops.linear(s, p["w_ss"], bias=p["b_ss"], out_dtype=torch.float32)      # [.., 2 c_x]
        ss = ss.reshape(-1, 2 * self.c_x)
        return ops.layer_norm(x, scale=ss[:, :self.c_x], shift=ss[:, self.c_x:])


class AdaLNZero(HipModule):
    """nn/d_diffusion_transformer.py:80-118: transition2(x), gated by
    sigmoid(adaptive_zero_cond(single_cond)) when conditioned."""

    def __init__(self, *args, c_in: int = None, c_out: int = None, c_single_cond: int = None,
                 use_single_cond: bool = False, shard_out: bool = False) -> None:
        super().__init__()
        args = drop_mesh(args)
        vals = list(args) + [c_in, c_out, c_single_cond, use_single_cond][len(args):]
        c_in, c_out, c_single_cond, use_single_cond = vals[:4]
        self.c_in, self.c_out, self.c_single_cond = c_in, c_out, c_single_cond
        self.use_single_cond = use_single_cond
        self.transition2 = nn.Linear(c_in, c_out, bias=False)
        if use_single_cond:
            self.adaptive_zero_cond = nn.Linear(c_single_cond, c_out, bias=True)

    def _pack(self):
        d = dict(w=bf16(self.transition2.weight))
        if self.use_single_cond:
            d["w_cond"] = bf16(self.adaptive_zero_cond.weight)
            d["b_cond"] = f32(self.adaptive_zero_cond.bias)
        return d

    def run(self, x, single_cond, out_dtype, residual=None, gate=None):
        """x bf16 [..., c_in] -> [..., c_out]; `residual` (same shape as the
        result) is added and overwritten in place when given.  `gate`: the
        sigmoid of this module's conditioning projection, fp32 [cond_rows,
        c_out] contiguous, when the caller has computed it already."""
        p = self.packed()
        if self.use_single_cond and gate is None:
            gate = ops.linear(single_cond.to(torch.bfloat16).contiguous(), p["w_cond"], bias=p["b_cond"],
                              out_dtype=torch.float32, sigmoid=True)
        return ops.linear(x, p["w"], out_dtype=out_dtype, mode=L.LINEAR_GATE_RES, gate=gate,
                          residual=residual, out=residual)

    def forward(self, x: torch.Tensor, single_cond: Optional[torch.Tensor] = None) -> torch.Tensor:
        assert (single_cond is None) == (self.use_single_cond is False)
        if in_check_mode():
            return check.adaln_zero(self, x, single_cond)
        return self.run(x.to(torch.bfloat16).contiguous(), single_cond, x.dtype)


class DiffusionTransition(HipModule):
    """nn/d_diffusion_transformer.py:120-145."""

    def __init__(self, *args, c_x: int = None, c_single_cond: int = None,
                 num_intermediate_factor: int = 2, use_single_cond: bool = False) -> None:
        super().__init__()
        args = drop_mesh(args)
        vals = list(args) + [c_x, c_single_cond, num_intermediate_factor, use_single_cond][len(args):]
        c_x, c_single_cond, num_intermediate_factor, use_single_cond = vals[:4]
        self.c_x, self.c_single_cond = c_x, c_single_cond
        self.num_intermediate_factor, self.use_single_cond = num_intermediate_factor, use_single_cond
        self.adaptive_layernorm = AdaptiveLayerNorm(c_x, c_single_cond, use_single_cond)
        self.transition1 = nn.Linear(c_x, 2 * c_x * num_intermediate_factor, bias=False)
        self.adaptive_zero_init = AdaLNZero(c_in=num_intermediate_factor * c_x, c_out=c_x,
                                            c_single_cond=c_single_cond, use_single_cond=use_single_cond)

    def _pack(self):
        return dict(w1=bf16(pack_swiglu(self.transition1.weight, 32)))

    def run(self, x, single_cond, residual: bool, cond=None):
        """`cond` = (scale_shift, gate) computed by the caller, see AdaptiveLayerNorm / AdaLNZero."""
        ss, gate = cond if cond is not None else (None, None)
        xa = self.adaptive_layernorm(x, single_cond, scale_shift=ss)
        h = ops.linear(xa, self.packed()["w1"], mode=L.LINEAR_SWIGLU)
        return self.adaptive_zero_init.run(h, single_cond, x.dtype, residual=x if residual else None, gate=gate)

    def forward(self, x: torch.Tensor, single_cond: Optional[torch.Tensor] = None) -> torch.Tensor:
        if in_check_mode():
            return check.diffusion_transition(self, x, single_cond)
        return self.run(x.contiguous(), single_cond, residual=False)


class SelfAttention(HipModule):
    """nn/d_diffusion_transformer.py:148-265 (pair-biased attention of the
    Pairformer single track and of the diffusion transformer)."""

    def __init__(self, *args, c_x: int = 768, c_single_cond: int = 384, num_head: int = 16,
                 use_single_cond: bool = False, use_batch_infer: bool = False) -> None:
        super().__init__()
        args = drop_mesh(args)
        vals = list(args) + [c_x, c_single_cond, num_head, use_single_cond, use_batch_infer][len(args):]
        c_x, c_single_cond, num_head, use_single_cond, use_batch_infer = vals[:5]
        self.c_x, self.c_single_cond, self.num_head = c_x, c_single_cond, num_head
        self.qkv_dim = c_x // num_head
        if self.qkv_dim not in (24, 32, 48):
            raise ValueError("head dimension must be 24, 32 or 48")
        self.use_single_cond, self.use_batch_infer = use_single_cond, use_batch_infer
        self.adaptive_layernorm = AdaptiveLayerNorm(c_x, c_single_cond, use_single_cond)
        self.q_projection = nn.Linear(c_x, c_x, bias=True)
        self.k_projection = nn.Linear(c_x, c_x, bias=False)
        self.v_projection = nn.Linear(c_x, c_x, bias=False)
        self.gating_query = nn.Linear(c_x, c_x, bias=False)
        self.adaptive_zero_init = AdaLNZero(c_in=c_x, c_out=c_x, c_single_cond=c_single_cond,
                                            use_single_cond=use_single_cond)

    def _pack(self):
        w = torch.cat([self.q_projection.weight, self.k_projection.weight, self.v_projection.weight,
                       self.gating_query.weight], dim=0)
        return dict(w_qkvg=bf16(w), q_b=f32(self.q_projection.bias))

    def run(self, x, mask, pair_logits, single_cond, residual: bool, cond=None):
        """`cond` = (scale_shift, gate) computed by the caller, see AdaptiveLayerNorm / AdaLNZero."""
        p = self.packed()
        ss, gate = cond if cond is not None else (None, None)
        xa = self.adaptive_layernorm(x, single_cond, scale_shift=ss)
        batched = xa.dim() == 3
        xb = xa if batched else xa.unsqueeze(0)
        if pair_logits is not None:
            pair_logits = pair_logits.to(torch.float32).contiguous()
        avg = ops.batch_diffusion_self_attention(xb, mask, pair_logits, p["w_qkvg"], p["q_b"], self.num_head)
        avg = avg.reshape(xb.shape)
        if not batched:
            avg = avg.squeeze(0)
        return self.adaptive_zero_init.run(avg, single_cond, x.dtype, residual=x if residual else None, gate=gate)

    def forward(self, x: torch.Tensor, mask: torch.Tensor, pair_logits: Optional[torch.Tensor] = None,
                single_cond: Optional[torch.Tensor] = None) -> torch.Tensor:
        """x [N, c] or [B, N, c]; mask [N]; pair_logits [H, N, N]."""
        assert (single_cond is None) == (self.use_single_cond is False)
        if in_check_mode():
            pl = None if pair_logits is None else pair_logits.to(torch.float32).contiguous()
            return check.self_attention(self, x, mask, pl, single_cond)
        return self.run(x.contiguous(), mask, pair_logits, single_cond, residual=False)


class DiffusionTransformer(HipModule):
    """nn/d_diffusion_transformer.py:267-310: 24 blocks in 6 super-blocks that
    share one pair-logit projection each."""

    def __init__(self, *args, c_act: int = 768, c_single_cond: int = 384, c_pair_cond: int = 128,
                 num_head: int = 16, num_blocks: int = 24, super_block_size: int = 4,
                 use_batch_infer: bool = False) -> None:
        super().__init__()
        args = drop_mesh(args)
        vals = list(args) + [c_act, c_single_cond, c_pair_cond, num_head, num_blocks, super_block_size,
                             use_batch_infer][len(args):]
        c_act, c_single_cond, c_pair_cond, num_head, num_blocks, super_block_size, use_batch_infer = vals[:7]
        if c_pair_cond != 128:
            raise ValueError("the HIP pair-logit projection is built for c_pair_cond = 128")
        self.c_act, self.c_single_cond, self.c_pair_cond = c_act, c_single_cond, c_pair_cond
        self.num_head, self.num_blocks, self.super_block_size = num_head, num_blocks, super_block_size
        self.num_super_blocks = num_blocks // super_block_size
        self.pair_input_layer_norm = nn.LayerNorm(c_pair_cond, bias=False)
        self.pair_logits_projection = nn.ModuleList(
            [nn.Linear(c_pair_cond, super_block_size * num_head, bias=False) for _ in range(self.num_super_blocks)])
        self.self_attention = nn.ModuleList(
            [SelfAttention(c_x=c_act, c_single_cond=c_single_cond, num_head=num_head, use_single_cond=True,
                           use_batch_infer=use_batch_infer) for _ in range(num_blocks)])
        self.transition_block = nn.ModuleList(
            [DiffusionTransition(c_x=c_act, c_single_cond=c_single_cond, use_single_cond=True)
             for _ in range(num_blocks)])

    def _pack(self):
        # Every block conditions on the same single_cond, so the 4 conditioning
        # projections of each block (adaptive LayerNorm scale | shift and the
        # AdaLN-Zero gate, for the attention and for the transition) are taken
        # out of the blocks: two products for all blocks before the first one.
        # Each adaptive LayerNorm normalises single_cond with its own weight and
        # no bias, LN_w(s) W^T = LN_1(s) (W diag(w))^T, so the weight goes into
        # the projection and one plain normalisation serves them all.
        w_ss, b_ss, w_gate, b_gate = [], [], [], []
        for att, tr in zip(self.self_attention, self.transition_block):
            for m in (att, tr):
                aln, az = m.adaptive_layernorm, m.adaptive_zero_init
                lnw = aln.single_cond_layer_norm.weight.detach().float()
                w = torch.cat([aln.single_cond_scale.weight, aln.single_cond_bias.weight], dim=0).detach().float()
                w_ss.append(w * lnw[None, :])
                b_ss.append(torch.cat([aln.single_cond_scale.bias, torch.zeros_like(aln.single_cond_scale.bias)]))
                w_gate.append(az.adaptive_zero_cond.weight)
                b_gate.append(az.adaptive_zero_cond.bias)
        return dict(ln_w=f32(self.pair_input_layer_norm.weight),
                    w_logits=[pad_rows(bf16(m.weight), 32) for m in self.pair_logits_projection],
                    w_ss=bf16(torch.cat(w_ss, dim=0)), b_ss=f32(torch.cat(b_ss)),
                    w_gate=bf16(torch.cat(w_gate, dim=0)), b_gate=f32(torch.cat(b_gate)))

    def pair_logits(self, pair_cond: torch.Tensor):
        """The pair logits of every super-block, [num_super_blocks] x [b, h, N, N]
        (stored as [b, h, N/4, N, 4], the order the attention kernel reads best,
        when N is a multiple of 4).
        They depend on pair_cond only: a caller that evaluates the transformer
        many times on one pair_cond (the diffusion sampler) computes them once
        and hands them to `forward(..., pair_logits=...)`."""
        p = self.packed()
        pair_cond = pair_cond.contiguous()
        n_out = self.super_block_size * self.num_head
        out = []
        for sb in range(self.num_super_blocks):
            logits = ops.pair_logits(pair_cond, p["ln_w"], None, p["w_logits"][sb], n_out)
            logits = logits.view(self.super_block_size, self.num_head, *logits.shape[1:])     # (b h) n s -> b h n s
            if logits.shape[-1] % 4 == 0:
                logits = ops.quad_major_bias(logits)     # computed once, read by every evaluation
            out.append(logits)
        return out

    def forward(self, act: torch.Tensor, mask: torch.Tensor, single_cond: torch.Tensor,
                pair_cond: torch.Tensor, pair_logits=None) -> torch.Tensor:
        """act [B, N, c_act] (updated in place, as the reference's `act +=`),
        mask [N], single_cond [N, c_single_cond], pair_cond [N, N, c_pair_cond]."""
        if in_check_mode():
            return check.diffusion_transformer(self, act, mask, single_cond, pair_cond)
        p = self.packed()
        if not act.is_contiguous():
            raise ValueError("act must be contiguous (it is updated in place)")
        n_out = self.super_block_size * self.num_head
        c, n_mod = self.c_act, 2 * self.num_blocks
        sc = single_cond.contiguous()
        rows = sc.numel() // sc.shape[-1]
        ss_all = ops.linear(ops.layer_norm(sc), p["w_ss"], bias=p["b_ss"], out_dtype=torch.float32)
        ss_all = ss_all.view(rows, n_mod, 2 * c)                       # column slices, read in place
        gate_all = ops.linear(sc.to(torch.bfloat16), p["w_gate"], bias=p["b_gate"], out_dtype=torch.float32,
                              sigmoid=True)
        gate_all = gate_all.view(rows, n_mod, c).permute(1, 0, 2)      # [module][row][c]: column slices, read in place
        for sb in range(self.num_super_blocks):
            if pair_logits is not None:
                logits = pair_logits[sb]
            else:
                logits = ops.pair_logits(pair_cond.contiguous(), p["ln_w"], None, p["w_logits"][sb], n_out)
                logits = logits.view(self.super_block_size, self.num_head, *logits.shape[1:])  # (b h) n s -> b h n s
            for j in range(self.super_block_size):
                i = sb * self.super_block_size + j
                self.self_attention[i].run(act, mask, logits[j], single_cond, residual=True,
                                           cond=(ss_all[:, 2 * i], gate_all[2 * i]))
                self.transition_block[i].run(act, single_cond, residual=True,
                                             cond=(ss_all[:, 2 * i + 1], gate_all[2 * i + 1]))
        return act


class CrossAttention(HipModule):
    """nn/d_diffusion_transformer.py:313-464: windowed atom cross-attention."""

    def __init__(self, *args, key_dim: int = 128, value_dim: int = 128, c_single_cond: int = 128,
                 num_head: int = 4, use_batch_infer: bool = False) -> None:
        super().__init__()
        args = drop_mesh(args)
        vals = list(args) + [key_dim, value_dim, c_single_cond, num_head, use_batch_infer][len(args):]
        key_dim, value_dim, c_single_cond, num_head, use_batch_infer = vals[:5]
        if key_dim != value_dim:
            raise ValueError("key_dim and value_dim must match")
        self.key_dim, self.value_dim, self.c_single_cond, self.num_head = key_dim, value_dim, c_single_cond, num_head
        self.key_dim_per_head = key_dim // num_head
        self.value_dim_per_head = value_dim // num_head
        self.q_scale = self.key_dim_per_head ** -0.5
        self.use_batch_infer = use_batch_infer
        self.q_adaptive_layernorm = AdaptiveLayerNorm(key_dim, c_single_cond, use_single_cond=True)
        self.k_adaptive_layernorm = AdaptiveLayerNorm(key_dim, c_single_cond, use_single_cond=True)
        self.q_projection = nn.Linear(key_dim, key_dim, bias=True)
        self.k_projection = nn.Linear(key_dim, key_dim, bias=False)
        self.v_projection = nn.Linear(value_dim, value_dim, bias=False)
        self.gating_query = nn.Linear(key_dim, value_dim, bias=False)
        self.adaptive_zero_init = AdaLNZero(c_in=value_dim, c_out=value_dim, c_single_cond=key_dim,
                                            use_single_cond=True)

    def _pack(self):
        return dict(
            w_qg=bf16(torch.cat([self.q_projection.weight, self.gating_query.weight], dim=0)),
            w_kv=bf16(torch.cat([self.k_projection.weight, self.v_projection.weight], dim=0)),
            q_b=f32(self.q_projection.bias))

    def run(self, x_q, x_k, mask_q, mask_k, pair_logits, single_cond_q, single_cond_k, residual: bool, cond=None):
        """`cond` = (scale_shift_q, scale_shift_k, gate) computed by the caller, see AdaptiveLayerNorm / AdaLNZero."""
        p = self.packed()
        n_sub, n_q, c = x_q.shape[-3:]
        n_k = x_k.shape[-2]
        ss_q, ss_k, gate = cond if cond is not None else (None, None, None)
        xq = self.q_adaptive_layernorm(x_q, single_cond_q, scale_shift=ss_q)
        xk = self.k_adaptive_layernorm(x_k, single_cond_k, scale_shift=ss_k)
        mq = mask_q.reshape(-1, n_q)
        mk = mask_k.reshape(-1, n_k)
        pl = None
        if pair_logits is not None:
            pl = pair_logits.reshape(-1, self.num_head, n_q, n_k).to(torch.float32).contiguous()
        avg = ops.batch_diffusion_cross_attention(
            xq.reshape(-1, n_q, c), xk.reshape(-1, n_k, c), pl, mq, mk, p["w_qg"], p["w_kv"], p["q_b"],
            self.num_head)
        avg = avg.reshape(x_q.shape)
        return self.adaptive_zero_init.run(avg, single_cond_q, x_q.dtype, residual=x_q if residual else None,
                                           gate=gate)

    def run_gathered(self, x_q, key_rows, mask_q, mask_k, pair_logits, single_cond_q, cond):
        """`run(..., residual=True)` for keys that are query atoms: key k of
        subset s is atom key_rows[s, k] of the flattened (subset, query) axis of
        x_q (negative: a masked slot, whose gathered activation and conditioning
        are zero, hence K = V = 0).  The keys' adaptive LayerNorm and K / V
        projection then run once per atom, not once per (subset, key), and no
        key tensor is gathered: cond = (scale_shift_q, scale_shift_k of the
        ATOMS [S * Q, 2c], gate)."""
        p = self.packed()
        n_sub, n_q, c = x_q.shape[-3:]
        ss_q, ss_k_atoms, gate = cond
        xq = self.q_adaptive_layernorm(x_q, single_cond_q, scale_shift=ss_q)
        xk = self.k_adaptive_layernorm(x_q, single_cond_q, scale_shift=ss_k_atoms)
        pl = None
        if pair_logits is not None:
            pl = pair_logits.reshape(-1, self.num_head, n_q, key_rows.shape[-1]).to(torch.float32).contiguous()
        avg = ops.gathered_cross_attention(
            xq.reshape(-1, n_q, c), xk.reshape(-1, n_sub * n_q, c), key_rows, pl, mask_q.reshape(-1, n_q),
            mask_k.reshape(-1, key_rows.shape[-1]), p["w_qg"], p["w_kv"], p["q_b"], self.num_head)
        return self.adaptive_zero_init.run(avg.reshape(x_q.shape), single_cond_q, x_q.dtype, residual=x_q, gate=gate)

    def forward(self, x_q, x_k, mask_q, mask_k, pair_logits=None, single_cond_q=None, single_cond_k=None):
        """x_q [(B,) S, Q, c], x_k [(B,) S, K, c], masks [(1,) S, Q] / [(1,) S, K],
        pair_logits [(1,) S, H, Q, K], conditioning [(1,) S, Q|K, c]."""
        if in_check_mode():
            return check.cross_attention(self, x_q.contiguous(), x_k.contiguous(), mask_q, mask_k, pair_logits,
                                         single_cond_q, single_cond_k)
        return self.run(x_q.contiguous(), x_k.contiguous(), mask_q, mask_k, pair_logits, single_cond_q,
                        single_cond_k, residual=False)


class DiffusionCrossAttTransformer(HipModule):
    """nn/d_diffusion_transformer.py:466-543.

    `queries_to_keys` is the gather that builds each subset's key window from
    the query layout; it may be an object with `gather_idxs` / `gather_mask`
    attributes (as xfold's atom_layout.GatherInfo has) or a `(gather_idxs,
    gather_mask)` pair, with indices into the flattened (subset, query) axis."""

    def __init__(self, *args, c_query: int = 128, c_single_cond: int = 128, c_pair_cond: int = 16,
                 num_blocks: int = 3, num_head: int = 4, use_batch_infer: bool = True) -> None:
        super().__init__()
        args = drop_mesh(args)
        vals = list(args) + [c_query, c_single_cond, c_pair_cond, num_blocks, num_head, use_batch_infer][len(args):]
        c_query, c_single_cond, c_pair_cond, num_blocks, num_head, use_batch_infer = vals[:6]
        self.c_query, self.c_single_cond, self.c_pair_cond = c_query, c_single_cond, c_pair_cond
        self.num_blocks, self.num_head, self.use_batch_infer = num_blocks, num_head, use_batch_infer
        self.pair_input_layer_norm = nn.LayerNorm(c_pair_cond, bias=False)
        self.pair_logits_projection = nn.Linear(c_pair_cond, num_blocks * num_head, bias=False)
        self.cross_attention = nn.ModuleList(
            [CrossAttention(num_head=num_head, use_batch_infer=use_batch_infer) for _ in range(num_blocks)])
        self.transition_block = nn.ModuleList(
            [DiffusionTransition(c_x=c_query, c_single_cond=c_single_cond, use_single_cond=True)
             for _ in range(num_blocks)])

    def _pack(self):
        # The conditioning inputs are the same for every block: all adaptive
        # LayerNorm scale | shift projections and AdaLN-Zero gates are computed
        # before the first block, one product per input (see DiffusionTransformer._pack).
        def ss(aln):
            w = torch.cat([aln.single_cond_scale.weight, aln.single_cond_bias.weight], dim=0).detach().float()
            b = torch.cat([aln.single_cond_scale.bias, torch.zeros_like(aln.single_cond_scale.bias)])
            return w * aln.single_cond_layer_norm.weight.detach().float()[None, :], b
        wq, bq, wk, bk, wg, bg = [], [], [], [], [], []
        for ca, tr in zip(self.cross_attention, self.transition_block):
            for aln in (ca.q_adaptive_layernorm, tr.adaptive_layernorm):
                w, b = ss(aln)
                wq.append(w)
                bq.append(b)
            w, b = ss(ca.k_adaptive_layernorm)
            wk.append(w)
            bk.append(b)
            for az in (ca.adaptive_zero_init, tr.adaptive_zero_init):
                wg.append(az.adaptive_zero_cond.weight)
                bg.append(az.adaptive_zero_cond.bias)
        return dict(ln_w=f32(self.pair_input_layer_norm.weight), w=bf16(self.pair_logits_projection.weight),
                    w_f32=f32(self.pair_logits_projection.weight),
                    w_ss_q=bf16(torch.cat(wq, dim=0)), b_ss_q=f32(torch.cat(bq)),
                    w_ss_k=bf16(torch.cat(wk, dim=0)), b_ss_k=f32(torch.cat(bk)),
                    w_gate=bf16(torch.cat(wg, dim=0)), b_gate=f32(torch.cat(bg)))

    @staticmethod
    def _gather_info(queries_to_keys):
        if hasattr(queries_to_keys, "gather_idxs"):
            return queries_to_keys.gather_idxs, queries_to_keys.gather_mask
        return queries_to_keys

    @staticmethod
    def _gather(queries_to_keys, queries_act):
        idx, gmask = DiffusionCrossAttTransformer._gather_info(queries_to_keys)
        lead = queries_act.shape[:-3]
        s, q, c = queries_act.shape[-3:]
        flat = queries_act.reshape(lead + (s * q, c))
        keys = flat[..., idx.reshape(-1), :].reshape(lead + tuple(idx.shape) + (c,))
        return (keys * gmask.to(keys.dtype)[..., None]).contiguous()

    def conditioning(self, queries_single_cond, keys_single_cond, pair_cond, keys_are_query_atoms=None):
        """Everything the blocks take from the conditioning inputs: the pair
        logits of every block, the adaptive LayerNorm scale | shift of queries
        and keys and the AdaLN-Zero gates.  None of it depends on queries_act,
        so a caller that runs the transformer many times on one conditioning
        (the diffusion sampler) computes it once and passes it as
        `forward(..., cond=...)`.

        `keys_are_query_atoms`: the `queries_to_keys` gather, given by a caller
        whose keys_single_cond IS that gather of queries_single_cond (the atom
        cross-attention encoder and decoder build it so,
        nn/d_atom_cross_attention.py:205-209).  The key side is then computed per
        atom (see CrossAttention.run_gathered) instead of per (subset, key)."""
        p = self.packed()
        key_rows = None
        if keys_are_query_atoms is not None:
            idx, gmask = self._gather_info(keys_are_query_atoms)
            n_atoms = queries_single_cond.shape[-3] * queries_single_cond.shape[-2]
            if int(idx.min()) < 0 or int(idx.max()) >= n_atoms:
                raise ValueError("queries_to_keys indexes beyond the query atoms")
            key_rows = torch.where(gmask.bool(), idx, torch.full_like(idx, -1)).to(torch.int32).contiguous()
            key_rows._af3_checked_rows = n_atoms
            keys_single_cond = queries_single_cond          # per atom
        if pair_cond.dtype == torch.float32 and pair_cond.dim() == 4 and pair_cond.shape[-1] == 16 \
                and self.num_blocks * self.num_head <= 32:
            # LayerNorm, projection and the split into [block][S][head][Q][K] planes in one fp32 pass
            logits = ops.atom_pair_logits(pair_cond.contiguous(), p["ln_w"], p["w_f32"], self.num_blocks, self.num_head)
        else:
            pair_act = ops.layer_norm(pair_cond.contiguous(), p["ln_w"])
            logits = ops.linear(pair_act, p["w"], out_dtype=torch.float32)           # [S, Q, K, (b h)]
            s, q, k, _ = logits.shape
            logits = logits.reshape(s, q, k, self.num_blocks, self.num_head).permute(3, 0, 4, 1, 2).contiguous()
        c = self.c_query
        cq = queries_single_cond.contiguous()
        ck = keys_single_cond.contiguous()
        rq, rk = cq.numel() // cq.shape[-1], ck.numel() // ck.shape[-1]
        ss_q = ops.linear(ops.layer_norm(cq), p["w_ss_q"], bias=p["b_ss_q"], out_dtype=torch.float32)
        ss_q = ss_q.view(rq, 2 * self.num_blocks, 2 * c)                # column slices, read in place
        ss_k = ops.linear(ops.layer_norm(ck), p["w_ss_k"], bias=p["b_ss_k"], out_dtype=torch.float32)
        ss_k = ss_k.view(rk, self.num_blocks, 2 * c)
        gate = ops.linear(cq.to(torch.bfloat16), p["w_gate"], bias=p["b_gate"], out_dtype=torch.float32, sigmoid=True)
        gate = gate.view(rq, 2 * self.num_blocks, c).permute(1, 0, 2).contiguous()   # [module][row][c]
        return logits, ss_q, ss_k, gate, key_rows

    def forward(self, queries_act, queries_mask, queries_to_keys, keys_mask, queries_single_cond,
                keys_single_cond, pair_cond, cond=None):
        if in_check_mode():
            return check.cross_att_transformer(self, queries_act, queries_mask, queries_to_keys, keys_mask,
                                               queries_single_cond, keys_single_cond, pair_cond)
        if not queries_act.is_contiguous():
            raise ValueError("queries_act must be contiguous (it is updated in place)")
        if cond is None:
            cond = self.conditioning(queries_single_cond, keys_single_cond, pair_cond)
        logits, ss_q, ss_k, gate, key_rows = cond
        for blk in range(self.num_blocks):
            if key_rows is not None:
                self.cross_attention[blk].run_gathered(queries_act, key_rows, queries_mask, keys_mask, logits[blk],
                                                       queries_single_cond,
                                                       cond=(ss_q[:, 2 * blk], ss_k[:, blk], gate[2 * blk]))
            else:
                keys_act = self._gather(queries_to_keys, queries_act)
                self.cross_attention[blk].run(queries_act, keys_act, queries_mask, keys_mask, logits[blk],
                                              queries_single_cond, keys_single_cond, residual=True,
                                              cond=(ss_q[:, 2 * blk], ss_k[:, blk], gate[2 * blk]))
            self.transition_block[blk].run(queries_act, queries_single_cond, residual=True,
                                           cond=(ss_q[:, 2 * blk + 1], gate[2 * blk + 1]))
        return queries_act
