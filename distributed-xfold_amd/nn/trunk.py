"""Evoformer trunk driver (d_alphafold3.py:32-254) and the recycling loop
around it (:410-440): input embeddings, the MSA stack of Evoformer blocks and
the 48 Pairformer blocks, with the reference's parameter names.

Not included: the template embedding (:219-223, nn/d_template.py; its
Pairformer blocks run on 64 pair channels, for which the pair kernels are not
built) — a caller that has one passes it as `template_embedding`; and the MSA
featurisation (shuffle / truncate / create_msa_feat, :173-178), which is data
pipeline: the batch carries `msa_feat [rows, N, 34]` and `msa_mask [rows, N]`.
"""

from __future__ import annotations

from typing import Callable, Optional

import torch
import torch.nn as nn
import torch.nn.functional as F

from .. import check, ops
from .base import HipModule, bf16, drop_mesh, f32, in_check_mode
from .diffusion_head import create_relative_encoding
from .evoformer import EvoformerBlock
from .pairformer import PairformerBlock, pairformer_loop


def _pad_k(w: torch.Tensor) -> torch.Tensor:
    return bf16(F.pad(w.detach().float(), (0, (-w.shape[1]) % 8)))


class Evoformer(HipModule):
    def __init__(self, *args, msa_channel: int = 64, msa_stack_num_layer: int = 4, pairformer_num_layer: int = 48,
                 template_embedding: Optional[Callable] = None, act_dtype: torch.dtype = torch.bfloat16) -> None:
        super().__init__()
        args = drop_mesh(args)
        if args:
            msa_channel = args[0]
        self.msa_channel, self.pair_channel, self.seq_channel = msa_channel, 128, 384
        self.target_feat_dim, self.msa_feat_dim, self.rel_dim = 447, 34, 139
        self.act_dtype = act_dtype
        cp, cs, ct = self.pair_channel, self.seq_channel, self.target_feat_dim

        def lin(cin, cout):
            return nn.Linear(cin, cout, bias=False)
        self.left_single, self.right_single = lin(ct, cp), lin(ct, cp)
        self.prev_embedding_layer_norm = nn.LayerNorm(cp)
        self.prev_embedding = lin(cp, cp)
        self.position_activations = lin(self.rel_dim, cp)
        self.bond_embedding = lin(1, cp)
        self.template_embedding = template_embedding
        self.msa_activations = lin(self.msa_feat_dim, msa_channel)
        self.extra_msa_target_feat = lin(ct, msa_channel)
        self.msa_stack = nn.ModuleList([EvoformerBlock(c_msa=msa_channel) for _ in range(msa_stack_num_layer)])
        self.single_activations = lin(ct, cs)
        self.prev_single_embedding_layer_norm = nn.LayerNorm(cs)
        self.prev_single_embedding = lin(cs, cs)
        self.trunk_pairformer = nn.ModuleList([PairformerBlock(with_single=True) for _ in range(pairformer_num_layer)])

    def _pack(self):
        return dict(
            w_lr=_pad_k(torch.cat([self.left_single.weight, self.right_single.weight], dim=0)),
            w_tf_msa=_pad_k(self.extra_msa_target_feat.weight), w_tf_single=_pad_k(self.single_activations.weight),
            w_msa=_pad_k(self.msa_activations.weight),
            prev_ln_w=f32(self.prev_embedding_layer_norm.weight), prev_ln_b=f32(self.prev_embedding_layer_norm.bias),
            w_prev=bf16(self.prev_embedding.weight),
            prevs_ln_w=f32(self.prev_single_embedding_layer_norm.weight),
            prevs_ln_b=f32(self.prev_single_embedding_layer_norm.bias), w_prevs=bf16(self.prev_single_embedding.weight))

    @staticmethod
    def _lin(x, layer, w_padded):
        """layer(x) -> fp32 for an input width that may not be a multiple of 8."""
        if in_check_mode():
            return check._lin(x.float().contiguous(), layer)
        x = F.pad(x.float(), (0, (-x.shape[-1]) % 8)).to(torch.bfloat16).contiguous()
        return ops.linear(x, w_padded, out_dtype=torch.float32)

    @staticmethod
    def contact_matrix(batch, n, device):
        """:103-137."""
        rows = []
        for info in (batch.polymer_ligand_bond_info.tokens_to_polymer_ligand_bonds,
                     batch.ligand_ligand_bond_info.tokens_to_ligand_ligand_bonds):
            ok = info.gather_mask.to(torch.long).prod(dim=1)[:, None]
            rows.append(info.gather_idxs.long() * ok)
        idx = torch.cat(rows)
        cm = torch.zeros(n, n, dtype=torch.float32, device=device)
        cm[idx[:, 0], idx[:, 1]] = 1.0
        cm[0, 0] = 0.0
        return cm

    @torch.no_grad()
    def forward(self, batch, prev, target_feat):
        """:193-254 -> {'single' [N, 384], 'pair' [N, N, 128], 'target_feat'}."""
        p = self.packed()
        chk = in_check_mode()
        dt = torch.float32 if chk else self.act_dtype
        mask = batch.token_features.mask.float()
        n = mask.shape[0]
        if chk:
            lr = torch.cat([check._lin(target_feat.float().contiguous(), self.left_single),
                            check._lin(target_feat.float().contiguous(), self.right_single)], dim=-1)
        else:
            lr = self._lin(target_feat, None, p["w_lr"])
        cp = self.pair_channel
        pair = lr[:, None, :cp] + lr[None, :, cp:]
        pair_mask = (mask[:, None] * mask[None, :]).contiguous()
        if chk:
            pair = pair + check._lin(check._ln(prev["pair"].float().contiguous(), self.prev_embedding_layer_norm),
                                     self.prev_embedding)
        else:
            pair = pair + ops.linear(ops.layer_norm(prev["pair"].contiguous(), p["prev_ln_w"], p["prev_ln_b"]),
                                     p["w_prev"], out_dtype=torch.float32)
        # one-hot relative encoding and the 0/1 contact matrix: look-ups / a scaled weight column
        rel = create_relative_encoding(batch.token_features, 32, 2)
        wpos = self.position_activations.weight.float().t()                      # [139, 128]
        off = (0, 66, 132, 133)
        pair = pair + wpos[off[0] + rel[..., :66].argmax(-1)] + wpos[off[1] + rel[..., 66:132].argmax(-1)]
        pair = pair + rel[..., 132:133].float() * wpos[132] + wpos[off[3] + rel[..., 133:].argmax(-1)]
        pair = pair + self.contact_matrix(batch, n, pair.device)[:, :, None] * self.bond_embedding.weight.float()[:, 0]
        pair = pair.to(dt).contiguous()
        if self.template_embedding is not None:
            asym = batch.token_features.asym_id
            pair = pair + self.template_embedding(query_embedding=pair, templates=batch.templates,
                                                  multichain_mask_2d=(asym[:, None] == asym[None, :]).to(pair.dtype),
                                                  padding_mask_2d=pair_mask)
        msa = self._lin(batch.msa_feat, self.msa_activations, p["w_msa"])
        msa = (msa + self._lin(target_feat, self.extra_msa_target_feat, p["w_tf_msa"])[None]).to(dt).contiguous()
        msa_mask = batch.msa_mask.float().contiguous()
        for blk in self.msa_stack:
            msa, pair = blk(msa=msa, pair=pair, msa_mask=msa_mask, pair_mask=pair_mask)
        single = self._lin(target_feat, self.single_activations, p["w_tf_single"])
        if chk:
            single = single + check._lin(check._ln(prev["single"].float().contiguous(),
                                                   self.prev_single_embedding_layer_norm), self.prev_single_embedding)
        else:
            single = single + ops.linear(ops.layer_norm(prev["single"].contiguous(), p["prevs_ln_w"], p["prevs_ln_b"]),
                                         p["w_prevs"], out_dtype=torch.float32)
        single = single.to(dt).contiguous()
        pair, single = pairformer_loop(self.trunk_pairformer, pair, pair_mask, single, mask)
        return {"single": single, "pair": pair, "target_feat": target_feat}

    @torch.no_grad()
    def recycle(self, batch, target_feat, num_recycles: int = 10):
        """:410-440: zero embeddings, then `num_recycles` passes, each fed the previous one's output."""
        n, dev = target_feat.shape[0], target_feat.device
        emb = {"pair": torch.zeros(n, n, self.pair_channel, device=dev),
               "single": torch.zeros(n, self.seq_channel, device=dev), "target_feat": target_feat}
        for _ in range(num_recycles):
            emb = self.forward(batch, emb, target_feat)
        return emb
