"""Atom cross-attention encoder / decoder of the diffusion head
(nn/d_atom_cross_attention.py:39-414): per-atom conditioning from the reference
conformers, the windowed atom transformer (32 queries x 128 keys per subset),
aggregation of atoms to tokens and the broadcast back.

Everything that does not depend on the atom positions — the per-atom single
conditioning, the [subsets, 32, 128, 16] pair conditioning with its three-layer
MLP, the masks and the transformer's conditioning projections — is computed by
`conditioning()` once per batch; `forward` takes it back through its
`conditioning=` argument, so the 200 evaluations of a diffusion sampling run
pay for it once.  Without the argument `forward` computes it on the spot, which
is what the reference does on every call.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Optional

import torch
import torch.nn as nn

from .. import check, ops
from .atom_layout import GatherInfo, convert
from .base import HipModule, bf16, drop_mesh, f32, in_check_mode
from .diffusion_transformer import DiffusionCrossAttTransformer


def _lin(x: torch.Tensor, layer: nn.Linear, relu_input: bool = False, residual=None) -> torch.Tensor:
    """fp32 product with a narrow weight: K of 1 or 3 as explicit FMAs, the 128 -> 16 / 16 -> 16 /
    128 -> 3 layers on the narrow fp32 kernel (optionally relu on the way in, a residual on the way out)."""
    w = layer.weight.float()
    x = x.float()
    if w.shape[1] <= 4:
        if relu_input:
            x = torch.relu(x)
        out = x[..., 0:1] * w[:, 0]
        for j in range(1, w.shape[1]):
            out = out + x[..., j:j + 1] * w[:, j]
        return out if residual is None else out + residual
    return ops.narrow_linear_f32(x.contiguous(), w.contiguous(), relu_input, residual)


def _ln_lin(x: torch.Tensor, norm: nn.LayerNorm, layer: nn.Linear, ln_w, w_bf16) -> torch.Tensor:
    """layer(norm(x)) -> fp32, LayerNorm and bf16 MFMA product on the HIP kernels."""
    if in_check_mode():
        return check._lin(check._ln(x.float().contiguous(), norm), layer)
    return ops.linear(ops.layer_norm(x.contiguous(), ln_w), w_bf16, out_dtype=torch.float32)


@dataclass
class AtomCrossAttEncoderOutput:
    token_act: torch.Tensor             # [(samples), N, per_token_channels]
    skip_connection: torch.Tensor       # [(samples), S, 32, 128]
    queries_mask: torch.Tensor          # [S, 32]
    queries_single_cond: torch.Tensor   # [S, 32, 128]
    keys_mask: torch.Tensor             # [S, 128]
    keys_single_cond: torch.Tensor      # [S, 128, 128]
    pair_cond: torch.Tensor             # [S, 32, 128, 16]
    transformer_cond: Any = None        # conditioning of the atom transformers (shared by encoder and decoder)


@dataclass
class EncoderConditioning:
    queries_mask: torch.Tensor
    queries_single_cond: torch.Tensor
    keys_mask: torch.Tensor
    keys_single_cond: torch.Tensor
    pair_cond: torch.Tensor
    transformer_cond: Any


class AtomCrossAttEncoder(HipModule):
    """nn/d_atom_cross_attention.py:39-343."""

    def __init__(self, *args, per_token_channels: int = 384, per_atom_channels: int = 128,
                 per_atom_pair_channels: int = 16, with_token_atoms_act: bool = False,
                 with_trunk_single_cond: bool = False, with_trunk_pair_cond: bool = False,
                 use_batch_infer: bool = False, c_trunk_single: int = 384, c_trunk_pair: int = 128) -> None:
        super().__init__()
        args = drop_mesh(args)
        vals = list(args) + [per_token_channels, per_atom_channels, per_atom_pair_channels, with_token_atoms_act,
                             with_trunk_single_cond, with_trunk_pair_cond, use_batch_infer][len(args):]
        (per_token_channels, per_atom_channels, per_atom_pair_channels, with_token_atoms_act,
         with_trunk_single_cond, with_trunk_pair_cond, use_batch_infer) = vals[:7]
        self.per_token_channels, self.per_atom_channels = per_token_channels, per_atom_channels
        self.per_atom_pair_channels = per_atom_pair_channels
        self.c_query = per_atom_channels
        self.with_token_atoms_act, self.with_trunk_single_cond = with_token_atoms_act, with_trunk_single_cond
        self.with_trunk_pair_cond, self.use_batch_infer = with_trunk_pair_cond, use_batch_infer
        ca, cp = per_atom_channels, per_atom_pair_channels

        def lin(cin, cout):
            return nn.Linear(cin, cout, bias=False)
        self.embed_ref_pos, self.embed_ref_mask = lin(3, ca), lin(1, ca)
        self.embed_ref_element, self.embed_ref_charge = lin(128, ca), lin(1, ca)
        self.embed_ref_atom_name = lin(64 * 4, ca)
        self.single_to_pair_cond_row, self.single_to_pair_cond_col = lin(ca, cp), lin(ca, cp)
        self.embed_pair_offsets, self.embed_pair_distances = lin(3, cp), lin(1, cp)
        self.single_to_pair_cond_row_1, self.single_to_pair_cond_col_1 = lin(ca, cp), lin(ca, cp)
        self.embed_pair_offsets_1, self.embed_pair_distances_1 = lin(3, cp), lin(1, cp)
        self.embed_pair_offsets_valid = lin(1, cp)
        self.pair_mlp_1, self.pair_mlp_2, self.pair_mlp_3 = lin(cp, cp), lin(cp, cp), lin(cp, cp)
        if with_trunk_single_cond:
            self.lnorm_trunk_single_cond = nn.LayerNorm(c_trunk_single, bias=False)
            self.embed_trunk_single_cond = lin(c_trunk_single, ca)
        if with_trunk_pair_cond:
            self.lnorm_trunk_pair_cond = nn.LayerNorm(c_trunk_pair, bias=False)
            self.embed_trunk_pair_cond = lin(c_trunk_pair, cp)
        if with_token_atoms_act:
            self.atom_positions_to_features = lin(3, ca)
        self.atom_transformer_encoder = DiffusionCrossAttTransformer(c_query=ca, use_batch_infer=use_batch_infer)
        self.project_atom_features_for_aggr = lin(ca, per_token_channels)

    def _pack(self):
        d = dict(w_aggr=bf16(self.project_atom_features_for_aggr.weight))
        if self.with_trunk_single_cond:
            d["ts_ln"] = f32(self.lnorm_trunk_single_cond.weight)
            d["ts_w"] = bf16(self.embed_trunk_single_cond.weight)
        if self.with_trunk_pair_cond:
            d["tp_ln"] = f32(self.lnorm_trunk_pair_cond.weight)
            d["tp_w"] = bf16(self.embed_trunk_pair_cond.weight)
        if hasattr(self, "atom_positions_to_features"):
            d["w_pos"] = f32(self.atom_positions_to_features.weight)
        return d

    def _per_atom_conditioning(self, batch):
        """:87-156 -> (act [N, A, 128], pair_act [N, A, A, 16]), fp32.  The
        one-hot inputs of :98-110 are table look-ups into the weight columns."""
        rs = batch.ref_structure
        m = rs.mask.float()
        act = _lin(rs.positions, self.embed_ref_pos) + _lin(m[:, :, None], self.embed_ref_mask)
        act = act + self.embed_ref_element.weight.float().t()[rs.element.long()]
        act = act + _lin(torch.arcsinh(rs.charge.float())[:, :, None], self.embed_ref_charge)
        wn = self.embed_ref_atom_name.weight.float().t().reshape(4, 64, -1)
        chars = rs.atom_name_chars.long()
        for j in range(4):
            act = act + wn[j][chars[..., j]]
        act = act * m[:, :, None]
        pair_act = (_lin(act, self.single_to_pair_cond_row, relu_input=True)[:, :, None, :]
                    + _lin(act, self.single_to_pair_cond_col, relu_input=True)[:, None, :, :])
        pos = rs.positions.float()
        d = pos[:, :, None, :] - pos[:, None, :, :]
        pair_act = pair_act + _lin(d, self.embed_pair_offsets)
        pair_act = pair_act + _lin(1.0 / (1 + (d * d).sum(-1, keepdim=True)), self.embed_pair_distances)
        return act, pair_act

    @torch.no_grad()
    def conditioning(self, batch, trunk_single_cond, trunk_pair_cond) -> EncoderConditioning:
        """The position-independent part of `forward` (:168-179, 205-311)."""
        p = self.packed()
        aca = batch.atom_cross_att
        tok_single, _ = self._per_atom_conditioning(batch)
        q_cond = convert(aca.token_atoms_to_queries, tok_single, (-3, -2))
        q_mask = convert(aca.token_atoms_to_queries, batch.predicted_structure_info.atom_mask, (-2, -1))
        if trunk_single_cond is not None:
            ts = _ln_lin(trunk_single_cond, self.lnorm_trunk_single_cond, self.embed_trunk_single_cond,
                         p.get("ts_ln"), p.get("ts_w"))
            q_cond = q_cond + convert(aca.tokens_to_queries, ts, (-2,))
        k_cond = convert(aca.queries_to_keys, q_cond, (-3, -2))
        k_mask = convert(aca.queries_to_keys, q_mask, (-2, -1))
        rs = batch.ref_structure
        q_pos = convert(aca.token_atoms_to_queries, rs.positions.float(), (-3, -2))
        q_uid = convert(aca.token_atoms_to_queries, rs.ref_space_uid, (-2, -1))
        k_pos = convert(aca.queries_to_keys, q_pos, (-3, -2))
        # :279-283: the keys' uid is gathered from the token-atom layout with the query-layout gather
        k_uid = convert(aca.queries_to_keys, rs.ref_space_uid, (-2, -1))
        row = _lin(q_cond, self.single_to_pair_cond_row_1, relu_input=True)
        col = _lin(k_cond, self.single_to_pair_cond_col_1, relu_input=True)
        tp = None
        if trunk_pair_cond is not None:
            tp = _ln_lin(trunk_pair_cond, self.lnorm_trunk_pair_cond, self.embed_trunk_pair_cond,
                         p.get("tp_ln"), p.get("tp_w"))
        t2q, t2k = aca.tokens_to_queries, aca.tokens_to_keys
        if in_check_mode():
            pair_act = row[:, :, None, :] + col[:, None, :, :]
            if tp is not None:
                n_tok = tp.shape[0]
                idx = n_tok * t2q.gather_idxs[:, :, None] + t2k.gather_idxs[:, None, :]
                msk = t2q.gather_mask[:, :, None] & t2k.gather_mask[:, None, :]
                pair_act = pair_act + tp.reshape(n_tok * n_tok, -1)[idx] * msk[..., None].float()
            valid = (q_uid[:, :, None] == k_uid[:, None, :]).float()[..., None]
            off = q_pos[:, :, None, :] - k_pos[:, None, :, :]
            pair_act = pair_act + _lin(off, self.embed_pair_offsets_1) * valid
            pair_act = pair_act + _lin(1.0 / (1 + (off * off).sum(-1, keepdim=True)), self.embed_pair_distances_1) * valid
            pair_act = pair_act + _lin(valid, self.embed_pair_offsets_valid)
            pair_act = pair_act.contiguous()
            h = _lin(pair_act, self.pair_mlp_1, relu_input=True)
            h = _lin(h, self.pair_mlp_2, relu_input=True)
            pair_act = _lin(h, self.pair_mlp_3, relu_input=True, residual=pair_act)
        else:
            # every term above and the three-layer MLP in one pass over the [S, 32, 128, 16] tensor
            i32 = lambda t: t.to(torch.int32).contiguous()
            tq = tk = None
            if tp is not None:
                tq = i32(torch.where(t2q.gather_mask, t2q.gather_idxs, -1))
                tk = i32(torch.where(t2k.gather_mask, t2k.gather_idxs, -1))
                tp = tp.float().contiguous()
            w = lambda layer: layer.weight.detach().float().contiguous()
            pair_act = ops.atom_pair_cond(row.contiguous(), col.contiguous(), tp, tq, tk, q_pos.float().contiguous(),
                                          k_pos.float().contiguous(), i32(q_uid), i32(k_uid), w(self.embed_pair_offsets_1),
                                          w(self.embed_pair_distances_1), w(self.embed_pair_offsets_valid),
                                          w(self.pair_mlp_1), w(self.pair_mlp_2), w(self.pair_mlp_3))
        q_cond, k_cond = q_cond.contiguous(), k_cond.contiguous()
        tcond = None
        if not in_check_mode():
            tcond = self.atom_transformer_encoder.conditioning(q_cond, k_cond, pair_act,
                                                               keys_are_query_atoms=aca.queries_to_keys)
        return EncoderConditioning(q_mask, q_cond, k_mask, k_cond, pair_act, tcond)

    @torch.no_grad()
    def forward(self, batch, token_atoms_act: Optional[torch.Tensor], trunk_single_cond: Optional[torch.Tensor],
                trunk_pair_cond: Optional[torch.Tensor], conditioning: Optional[EncoderConditioning] = None,
                act_dtype: torch.dtype = torch.bfloat16) -> AtomCrossAttEncoderOutput:
        """:159-343.  `act_dtype` is the dtype of the atom activations that run
        through the transformer (fp32 in the check mode)."""
        c = conditioning if conditioning is not None else self.conditioning(batch, trunk_single_cond,
                                                                            trunk_pair_cond)
        aca = batch.atom_cross_att
        batched = self.use_batch_infer
        if in_check_mode():
            act_dtype = torch.float32
        qm = c.queries_mask.float()
        qm = qm[None, ..., None] if batched else qm[..., None]
        if token_atoms_act is None:
            q_act = c.queries_single_cond.clone()
        elif in_check_mode():
            q_act = convert(aca.token_atoms_to_queries, token_atoms_act.float(), (-3, -2))
            q_act = _lin(q_act, self.atom_positions_to_features) * qm
            q_act = q_act + (c.queries_single_cond[None] if batched else c.queries_single_cond)
        else:
            # conversion to the query layout, 3 -> channels projection, query mask and conditioning in one pass
            gi = aca.token_atoms_to_queries
            rows = getattr(gi, "_af3_rows32", None)
            if rows is None or rows.device != token_atoms_act.device:
                live = gi.gather_mask & (c.queries_mask != 0)
                rows = torch.where(live, gi.gather_idxs, -1).to(torch.int32).reshape(-1).contiguous()
                try:
                    gi._af3_rows32 = rows
                except AttributeError:
                    pass
            cond = c.queries_single_cond
            n_slots = token_atoms_act.shape[-3] * token_atoms_act.shape[-2]
            q_act = ops.atom_position_features(token_atoms_act.float().reshape(-1, n_slots, 3).contiguous(), rows,
                                               self.packed()["w_pos"],
                                               cond.float().reshape(-1, cond.shape[-1]).contiguous(), out_dtype=act_dtype)
            q_act = q_act.view(*token_atoms_act.shape[:-3], *cond.shape)
        q_act = q_act.to(act_dtype).contiguous()
        q_act = self.atom_transformer_encoder(
            queries_act=q_act, queries_mask=c.queries_mask, queries_to_keys=aca.queries_to_keys,
            keys_mask=c.keys_mask, queries_single_cond=c.queries_single_cond,
            keys_single_cond=c.keys_single_cond, pair_cond=c.pair_cond, cond=c.transformer_cond)
        q_act = q_act * qm.to(q_act.dtype)
        skip = q_act
        if in_check_mode():
            agg = check._lin(q_act.contiguous(), self.project_atom_features_for_aggr)
        else:
            agg = ops.linear(q_act.to(torch.bfloat16).contiguous(), self.packed()["w_aggr"])
        tm = batch.predicted_structure_info.atom_mask.float()
        # mask_mean over the atoms of a token (:328-331); the gather zeroes the absent atoms
        count = torch.clamp(tm.sum(-1), min=1e-10)
        if in_check_mode():
            tok_atoms = convert(aca.queries_to_token_atoms, agg, (-3, -2))
            tok_act = torch.relu(tok_atoms).float().sum(-2) / count[..., None]
        else:
            # conversion to the token-atom layout, ReLU and the mean in one pass over the atoms that exist
            gi = aca.queries_to_token_atoms
            rows = getattr(gi, "_af3_rows32", None)
            if rows is None or rows.device != agg.device:
                rows = torch.where(gi.gather_mask, gi.gather_idxs, -1).to(torch.int32).contiguous()
                try:
                    gi._af3_rows32 = rows          # the layout of a batch does not change between evaluations
                except AttributeError:
                    pass
            n_src = agg.shape[-3] * agg.shape[-2]
            tok_act = ops.gathered_relu_mean(agg.reshape(-1, n_src, agg.shape[-1]), rows, count.contiguous())
            if not batched:
                tok_act = tok_act[0]
        return AtomCrossAttEncoderOutput(tok_act, skip, c.queries_mask, c.queries_single_cond, c.keys_mask,
                                         c.keys_single_cond, c.pair_cond, c.transformer_cond)


class AtomCrossAttDecoder(HipModule):
    """nn/d_atom_cross_attention.py:346-414."""

    def __init__(self, *args, use_batch_infer: bool = False, per_token_channels: int = 768,
                 per_atom_channels: int = 128) -> None:
        super().__init__()
        args = drop_mesh(args)
        if args:
            use_batch_infer = args[0]
        self.use_batch_infer = use_batch_infer
        self.per_atom_channels = per_atom_channels
        self.project_token_features_for_broadcast = nn.Linear(per_token_channels, per_atom_channels, bias=False)
        self.atom_transformer_decoder = DiffusionCrossAttTransformer(c_query=per_atom_channels,
                                                                     use_batch_infer=use_batch_infer)
        self.atom_features_layer_norm = nn.LayerNorm(per_atom_channels, bias=False)
        self.atom_features_to_position_update = nn.Linear(per_atom_channels, 3, bias=False)

    def _pack(self):
        return dict(w_bcast=bf16(self.project_token_features_for_broadcast.weight),
                    ln_w=f32(self.atom_features_layer_norm.weight),
                    w_upd=f32(self.atom_features_to_position_update.weight))

    @torch.no_grad()
    def conditioning(self, enc, queries_to_keys=None):
        """The decoder transformer's conditioning projections for the
        encoder's (position-independent) conditioning tensors; `queries_to_keys`
        (batch.atom_cross_att.queries_to_keys) selects the per-atom key path."""
        if in_check_mode():
            return None
        return self.atom_transformer_decoder.conditioning(enc.queries_single_cond, enc.keys_single_cond,
                                                          enc.pair_cond, keys_are_query_atoms=queries_to_keys)

    @torch.no_grad()
    def forward(self, batch, token_act: torch.Tensor, enc: AtomCrossAttEncoderOutput,
                transformer_cond=None) -> torch.Tensor:
        """:355-414 -> position update [(samples), N, A, 3], fp32."""
        aca = batch.atom_cross_att
        batched = self.use_batch_infer
        p = self.packed()
        if in_check_mode():
            t = check._lin(token_act.float().contiguous(), self.project_token_features_for_broadcast)
        else:
            t = ops.linear(token_act.to(torch.bfloat16).contiguous(), p["w_bcast"])
        # every atom slot of a token carries the token's row (:371-384), so the
        # conversion to the query layout is the gather of token rows
        ta2q = aca.token_atoms_to_queries
        n_dense = aca.queries_to_token_atoms.gather_idxs.shape[1]
        qm = enc.queries_mask.to(t.dtype)
        qm = qm[None, ..., None] if batched else qm[..., None]
        fused = not in_check_mode() and enc.skip_connection.dtype == torch.bfloat16
        if fused:
            # gather, + skip connection and query mask in one pass (the skip connection is zero where the mask is)
            rows = getattr(ta2q, "_af3_token_rows32", None)
            if rows is None or rows.device != t.device:
                live = ta2q.gather_mask & (enc.queries_mask != 0)
                rows = torch.where(live, ta2q.gather_idxs // n_dense, -1).to(torch.int32).reshape(-1).contiguous()
                try:
                    ta2q._af3_token_rows32 = rows
                except AttributeError:
                    pass
            skip = enc.skip_connection
            q_act = ops.gather_rows_add(t.reshape(-1, t.shape[-2], t.shape[-1]), rows,
                                        skip.reshape(-1, rows.shape[0], skip.shape[-1]).contiguous()).view(skip.shape)
        else:
            q_act = convert(GatherInfo(ta2q.gather_idxs // n_dense, ta2q.gather_mask, (t.shape[-2],)), t, (-2,))
            q_act = q_act + enc.skip_connection.to(q_act.dtype)
            q_act = (q_act * qm.to(q_act.dtype)).to(enc.skip_connection.dtype).contiguous()
        q_act = self.atom_transformer_decoder(
            queries_act=q_act, queries_mask=enc.queries_mask, queries_to_keys=aca.queries_to_keys,
            keys_mask=enc.keys_mask, queries_single_cond=enc.queries_single_cond,
            keys_single_cond=enc.keys_single_cond, pair_cond=enc.pair_cond, cond=transformer_cond)
        if fused:
            # LayerNorm, projection to the position update and conversion to the token-atom layout in one
            # pass over the atoms that exist (their query mask is one)
            gi = aca.queries_to_token_atoms
            rows = getattr(gi, "_af3_rows32_flat", None)
            if rows is None or rows.device != q_act.device:
                rows = torch.where(gi.gather_mask, gi.gather_idxs, -1).to(torch.int32).reshape(-1).contiguous()
                try:
                    gi._af3_rows32_flat = rows
                except AttributeError:
                    pass
            n_src = q_act.shape[-3] * q_act.shape[-2]
            upd = ops.position_update(q_act.reshape(-1, n_src, q_act.shape[-1]), rows, p["ln_w"], p["w_upd"])
            return upd.view(*q_act.shape[:-3], *gi.gather_idxs.shape, 3)
        q_act = q_act * qm.to(q_act.dtype)
        if in_check_mode():
            q_act = check._ln(q_act.contiguous(), self.atom_features_layer_norm)
        else:
            q_act = ops.layer_norm(q_act.contiguous(), p["ln_w"])
        upd = _lin(q_act, self.atom_features_to_position_update)
        return convert(aca.queries_to_token_atoms, upd, (-3, -2))
