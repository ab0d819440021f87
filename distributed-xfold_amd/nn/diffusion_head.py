"""Diffusion head (nn/d_diffusion_head.py:65-227) and the sampling loop that
drives it (d_alphafold3.py:316-404): the direct caller of the diffusion
transformer and of the atom cross-attention.

One denoising evaluation is: scale the noisy positions, atom cross-attention
encoder (atoms -> tokens), 24-block diffusion transformer over the tokens,
atom cross-attention decoder (tokens -> position update), blend with the
input.  The sampler evaluates it `diffusion_steps` times on one batch, and most
of what the reference recomputes on every evaluation does not depend on the
positions or the noise level: the atoms' single and pair conditioning with its
MLP, the conditioning projections of both atom transformers, and the 6 x 64
pair-logit planes [N, N] of the token transformer.  `DiffusionHead.prepare`
computes those once (they stay resident in HBM: 0.9 GB at 768 tokens) and
`forward(..., state=...)` reuses them; without `state` forward computes them on
the spot, as the reference does.
"""

from __future__ import annotations

import math
from dataclasses import dataclass
from typing import Any, Optional

import torch
import torch.nn as nn
import torch.nn.functional as F

from .. import check, ops
from .atom_cross_attention import AtomCrossAttDecoder, AtomCrossAttEncoder, EncoderConditioning
from .base import HipModule, bf16, drop_mesh, f32, in_check_mode
from .diffusion_transformer import DiffusionTransformer, DiffusionTransition

SIGMA_DATA = 16.0   # nn/d_diffusion_head.py:47


def create_relative_encoding(token_features, max_relative_idx: int = 32, max_relative_chain: int = 2):
    """Relative position features of a token pair (AlphaFold 3 supplement,
    Algorithm 3; the reference takes it from xfold's featurization module, call
    site nn/d_diffusion_head.py:106-108): one-hot clipped residue offset within
    a chain (66), one-hot clipped token offset within a residue (66), same
    entity (1), one-hot clipped chain-copy offset within an entity (6)."""
    tf = token_features

    def lr(x):
        x = x.long()
        return x[:, None], x[None, :]
    la, ra = lr(tf.asym_id)
    lres, rres = lr(tf.residue_index)
    ltok, rtok = lr(tf.token_index)
    lent, rent = lr(tf.entity_id)
    lsym, rsym = lr(tf.sym_id)
    r, c = max_relative_idx, max_relative_chain
    same_chain = la == ra
    off = torch.where(same_chain, torch.clamp(lres - rres + r, 0, 2 * r), 2 * r + 1)
    same_res = same_chain & (lres == rres)
    toff = torch.where(same_res, torch.clamp(ltok - rtok + r, 0, 2 * r), 2 * r + 1)
    same_ent = lent == rent
    coff = torch.where(same_ent, torch.clamp(lsym - rsym + c, 0, 2 * c), 2 * c + 1)
    return torch.cat([F.one_hot(off, 2 * r + 2), F.one_hot(toff, 2 * r + 2), same_ent[..., None].long(),
                      F.one_hot(coff, 2 * c + 2)], dim=-1)


def noise_schedule(t: torch.Tensor, smin: float = 0.0004, smax: float = 160.0, p: float = 7.0) -> torch.Tensor:
    """Noise level at time t in [0, 1] (call site d_alphafold3.py:361-362)."""
    return SIGMA_DATA * (smax ** (1 / p) + t * (smin ** (1 / p) - smax ** (1 / p))) ** p


def random_rotation(gen: Optional[torch.Generator], device, dtype=torch.float32) -> torch.Tensor:
    """A rotation matrix drawn uniformly (Gram-Schmidt on two normal vectors)."""
    v = torch.randn(2, 3, generator=gen, device=device, dtype=dtype)
    e0 = v[0] / torch.clamp(v[0].norm(), min=1e-10)
    v1 = v[1] - e0 * (e0 @ v[1])
    e1 = v1 / torch.clamp(v1.norm(), min=1e-10)
    return torch.stack([e0, e1, torch.linalg.cross(e0, e1)])


def random_augmentation(positions: torch.Tensor, mask: torch.Tensor, rot: torch.Tensor,
                        trans: torch.Tensor) -> torch.Tensor:
    """Centre on the masked mean over all atoms, rotate by `rot` [3, 3], shift
    by `trans` [3], zero the padding atoms (call site d_alphafold3.py:337-339)."""
    m = mask.to(positions.dtype)[..., None]
    count = torch.clamp(m.expand_as(positions[..., :1]).sum(dim=(-2, -3), keepdim=True), min=1e-6)
    center = (m * positions).sum(dim=(-2, -3), keepdim=True) / count
    return (torch.einsum("...i,ij->...j", positions - center, rot) + trans) * m


class FourierEmbeddings(nn.Module):
    """nn/d_diffusion_head.py:49-62."""

    def __init__(self, *args, dim: int = 256) -> None:
        super().__init__()
        args = drop_mesh(args)
        if args:
            dim = args[0]
        self.dim = dim
        self.weight = nn.Parameter(torch.ones(dim))
        self.bias = nn.Parameter(torch.ones(dim))

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return torch.cos(2 * math.pi * (x.float()[..., None] * self.weight.float() + self.bias.float()))


@dataclass
class HeadState:
    """What `DiffusionHead.prepare` keeps for the evaluations of one batch."""
    encoder: EncoderConditioning
    decoder_cond: Any
    pair_logits: Any


class DiffusionHead(HipModule):
    """nn/d_diffusion_head.py:65-227.  `num_blocks` (24 in the model) is a
    constructor argument here so that tests can build a shallow head."""

    def __init__(self, *args, use_batch_infer: bool = True, num_blocks: int = 24, c_target_feat: int = 447,
                 c_relative: int = 139) -> None:
        super().__init__()
        args = drop_mesh(args)
        if args:
            use_batch_infer = args[0]
        self.pair_channel, self.seq_channel, self.c_act = 128, 384, 768
        self.use_batch_infer = use_batch_infer
        cp, cs, ca = self.pair_channel, self.seq_channel, self.c_act
        self.pair_cond_initial_norm = nn.LayerNorm(cp + c_relative, bias=False)
        self.pair_cond_initial_projection = nn.Linear(cp + c_relative, cp, bias=False)
        self.pair_transition_0 = DiffusionTransition(c_x=cp, c_single_cond=None)
        self.pair_transition_1 = DiffusionTransition(c_x=cp, c_single_cond=None)
        self.single_cond_initial_norm = nn.LayerNorm(cs + c_target_feat, bias=False)
        self.single_cond_initial_projection = nn.Linear(cs + c_target_feat, cs, bias=False)
        self.fourier_embeddings = FourierEmbeddings(dim=256)
        self.noise_embedding_initial_norm = nn.LayerNorm(256, bias=False)
        self.noise_embedding_initial_projection = nn.Linear(256, cs, bias=False)
        self.single_transition_0 = DiffusionTransition(c_x=cs, c_single_cond=None)
        self.single_transition_1 = DiffusionTransition(c_x=cs, c_single_cond=None)
        self.atom_cross_att_encoder = AtomCrossAttEncoder(
            per_token_channels=ca, with_token_atoms_act=True, with_trunk_pair_cond=True,
            with_trunk_single_cond=True, use_batch_infer=use_batch_infer)
        self.single_cond_embedding_norm = nn.LayerNorm(cs, bias=False)
        self.single_cond_embedding_projection = nn.Linear(cs, ca, bias=False)
        self.transformer = DiffusionTransformer(num_blocks=num_blocks, use_batch_infer=use_batch_infer)
        self.output_norm = nn.LayerNorm(ca, bias=False)
        self.atom_cross_att_decoder = AtomCrossAttDecoder(use_batch_infer=use_batch_infer)

    @staticmethod
    def _pad_k(w: torch.Tensor) -> torch.Tensor:
        """bf16 weight with its input width padded with zero columns to a multiple of 8."""
        k = w.shape[1]
        return bf16(F.pad(w.detach().float(), (0, (-k) % 8)))

    def _pack(self):
        # first layer of the pair conditioning (ops.pair_cond_init): the pair channels' LayerNorm weights and
        # projection columns, and the one-hot channels' columns folded with their LayerNorm weights
        cp = self.pair_channel
        wp, gp = self.pair_cond_initial_projection.weight.detach().float(), self.pair_cond_initial_norm.weight.detach().float()
        g_hot = (wp[:, cp:] * gp[cp:]).t().contiguous()
        return dict(w_pair0=self._pad_k(self.pair_cond_initial_projection.weight),
                    pair_ln=f32(gp[:cp]), w_pair=bf16(wp[:, :cp]), g_hot=f32(g_hot), g_sum=f32(g_hot.sum(0)),
                    w_single0=self._pad_k(self.single_cond_initial_projection.weight),
                    noise_ln=f32(self.noise_embedding_initial_norm.weight),
                    w_noise=bf16(self.noise_embedding_initial_projection.weight),
                    emb_ln=f32(self.single_cond_embedding_norm.weight),
                    w_emb=bf16(self.single_cond_embedding_projection.weight),
                    out_ln=f32(self.output_norm.weight))

    def _norm_project(self, x, norm, layer, w_padded):
        """layer(norm(x)) for an input width that is not a multiple of 8 (the
        concatenated features of :109-113): fp32 normalisation, then the bf16
        MFMA product on the zero-padded width."""
        if in_check_mode():
            return check._lin(check._ln(x.float().contiguous(), norm), layer)
        y = F.layer_norm(x.float(), (x.shape[-1],), norm.weight.float(), None, 1e-5)
        y = F.pad(y, (0, (-x.shape[-1]) % 8)).to(torch.bfloat16)
        return ops.linear(y, w_padded, out_dtype=torch.float32)

    @torch.no_grad()
    def pre_conditioning(self, batch, embeddings, noise_level: torch.Tensor, use_conditioning):
        """:96-169 -> (single_cond [T, N, 384] fp32, pair_cond [N, N, 128] fp32)
        for the noise levels [T] of all steps."""
        p = self.packed()
        single = use_conditioning * embeddings["single"].float()
        f1d = torch.cat([single, embeddings["target_feat"].float()], dim=-1)
        if in_check_mode() or p["g_hot"].shape[0] != 139:
            pair = use_conditioning * embeddings["pair"].float()
            rel = create_relative_encoding(batch.token_features, 32, 2).to(pair.dtype)
            f2d = torch.cat([pair, rel], dim=-1)
            pair_cond = self._norm_project(f2d, self.pair_cond_initial_norm, self.pair_cond_initial_projection,
                                           p["w_pair0"])
            del f2d, rel
        else:
            # one kernel: the relative encoding is one-hot, so its LayerNorm statistics and its share of the
            # projection follow from the token indices; the [N, N, 267] tensor is never made
            tf = batch.token_features
            ids = tuple(getattr(tf, k).to(torch.int32).contiguous()
                        for k in ("asym_id", "residue_index", "token_index", "entity_id", "sym_id"))
            pair_in = embeddings["pair"]
            if pair_in.dtype not in (torch.float32, torch.bfloat16):
                pair_in = pair_in.float()
            pair_cond = ops.pair_cond_init(pair_in.contiguous(), ids, p["pair_ln"], p["w_pair"], p["g_hot"], p["g_sum"],
                                           in_scale=float(use_conditioning), max_relative_idx=32, max_relative_chain=2)
        pair_cond = self._transition(self.pair_transition_0, pair_cond)
        pair_cond = self._transition(self.pair_transition_1, pair_cond)
        noise = self.fourier_embeddings(0.25 * torch.log(noise_level.float() / SIGMA_DATA))
        if in_check_mode():
            noise = check._lin(check._ln(noise.contiguous(), self.noise_embedding_initial_norm),
                               self.noise_embedding_initial_projection)
        else:
            noise = ops.linear(ops.layer_norm(noise.contiguous(), p["noise_ln"]), p["w_noise"],
                               out_dtype=torch.float32)
        single_cond = self._norm_project(f1d, self.single_cond_initial_norm, self.single_cond_initial_projection,
                                         p["w_single0"])
        single_cond = (single_cond[None] + noise[:, None, :]).contiguous()
        single_cond = self._transition(self.single_transition_0, single_cond)
        single_cond = self._transition(self.single_transition_1, single_cond)
        return single_cond, pair_cond

    @staticmethod
    def _transition(mod: DiffusionTransition, x: torch.Tensor) -> torch.Tensor:
        """x + mod(x) (the reference's `x += mod(x)`), in place on x."""
        if in_check_mode():
            return x + mod(x)
        return mod.run(x, None, residual=True)

    @torch.no_grad()
    def prepare(self, batch, embeddings, trunk_pair_cond: torch.Tensor) -> HeadState:
        """Everything `forward` needs that depends neither on the positions nor
        on the noise level."""
        enc = self.atom_cross_att_encoder.conditioning(batch, embeddings["single"], trunk_pair_cond)
        dec = self.atom_cross_att_decoder.conditioning(enc, batch.atom_cross_att.queries_to_keys)
        logits = None if in_check_mode() else self.transformer.pair_logits(trunk_pair_cond)
        return HeadState(enc, dec, logits)

    @torch.no_grad()
    def forward(self, positions_noisy: torch.Tensor, noise_level: torch.Tensor, batch, embeddings,
                trunk_single_cond: torch.Tensor, trunk_pair_cond: torch.Tensor,
                state: Optional[HeadState] = None, act_dtype: torch.dtype = torch.bfloat16) -> torch.Tensor:
        """:171-227.  positions_noisy [(samples), N, A, 3]; noise_level a scalar
        tensor; trunk_single_cond [N, 384] (the row of pre_conditioning's result
        for this noise level), trunk_pair_cond [N, N, 128].  Returns the
        denoised positions, fp32."""
        if state is None:
            state = self.prepare(batch, embeddings, trunk_pair_cond)
        if in_check_mode():
            act_dtype = torch.float32
        p = self.packed()
        batched = self.use_batch_infer
        positions_noisy = positions_noisy.float()
        am = batch.predicted_structure_info.atom_mask.float()
        am = am[None, ..., None] if batched else am[..., None]
        act = positions_noisy * am / torch.sqrt(noise_level ** 2 + SIGMA_DATA ** 2)
        enc = self.atom_cross_att_encoder(batch=batch, token_atoms_act=act, trunk_single_cond=embeddings["single"],
                                          trunk_pair_cond=trunk_pair_cond, conditioning=state.encoder,
                                          act_dtype=act_dtype)
        if in_check_mode():
            emb = check._lin(check._ln(trunk_single_cond.float().contiguous(), self.single_cond_embedding_norm),
                             self.single_cond_embedding_projection)
        else:
            emb = ops.linear(ops.layer_norm(trunk_single_cond.contiguous(), p["emb_ln"]), p["w_emb"],
                             out_dtype=torch.float32)
        act = (enc.token_act + (emb[None] if batched else emb)).to(act_dtype).contiguous()
        act = self.transformer(act=act, mask=batch.token_features.mask, single_cond=trunk_single_cond,
                               pair_cond=trunk_pair_cond, pair_logits=state.pair_logits)
        if in_check_mode():
            act = check._ln(act.contiguous(), self.output_norm)
        else:
            act = ops.layer_norm(act, p["out_ln"])
        upd = self.atom_cross_att_decoder(batch=batch, token_act=act, enc=enc, transformer_cond=state.decoder_cond)
        skip = SIGMA_DATA ** 2 / (noise_level ** 2 + SIGMA_DATA ** 2)
        out = noise_level * SIGMA_DATA / torch.sqrt(noise_level ** 2 + SIGMA_DATA ** 2)
        return (skip * positions_noisy + out * upd) * am


class DiffusionSampler:
    """The sampling loop of d_alphafold3.py:316-404 around a DiffusionHead.

    As in the reference (:340-342, where the normal draw is commented out) the
    noise term added in a step is the scalar `noise_scale` of that step;
    `gaussian_noise=True` adds `noise_scale * N(0, 1)` per coordinate instead,
    which is what the published algorithm does."""

    def __init__(self, head: DiffusionHead, num_samples: int = 5, diffusion_steps: int = 200,
                 gamma_0: float = 0.8, gamma_min: float = 1.0, noise_scale: float = 1.003,
                 step_scale: float = 1.5, gaussian_noise: bool = False) -> None:
        self.head, self.num_samples, self.diffusion_steps = head, num_samples, diffusion_steps
        self.gamma_0, self.gamma_min, self.noise_scale, self.step_scale = gamma_0, gamma_min, noise_scale, step_scale
        self.gaussian_noise = gaussian_noise

    def schedule(self, device):
        """(noise_levels [steps + 1], t_hat [steps], noise_scale [steps]), :361-371."""
        levels = noise_schedule(torch.linspace(0, 1, self.diffusion_steps + 1, device=device))
        prev, cur = levels[:-1], levels[1:]
        gamma = self.gamma_0 * (cur > self.gamma_min).to(levels.dtype)
        t_hat = prev * (1 + gamma)
        return levels, t_hat, self.noise_scale * torch.sqrt(t_hat ** 2 - prev ** 2)

    @torch.no_grad()
    def __call__(self, batch, embeddings, generator: Optional[torch.Generator] = None, positions=None,
                 rotations=None, translations=None, noises=None):
        """Returns {'atom_positions': [samples, N, A, 3], 'mask': [N, A]}.  The
        random draws (start positions [samples, N, A, 3] ~ N(0, 1), per-step
        rotations [steps, 3, 3] and translations [steps, 3], and with
        gaussian_noise per-step noise [steps, samples, N, A, 3]) may be handed
        in; otherwise they come from `generator`."""
        head = self.head
        mask = batch.predicted_structure_info.atom_mask
        dev = mask.device
        levels, t_hat, nscale = self.schedule(dev)
        single_cond, pair_cond = head.pre_conditioning(batch, embeddings, t_hat, True)
        state = head.prepare(batch, embeddings, pair_cond)
        if positions is None:
            positions = torch.randn((self.num_samples,) + tuple(mask.shape) + (3,), generator=generator, device=dev)
        positions = positions.float() * levels[0]
        for i in range(self.diffusion_steps):
            rot = rotations[i] if rotations is not None else random_rotation(generator, dev)
            trans = translations[i] if translations is not None else torch.randn(3, generator=generator, device=dev)
            positions = random_augmentation(positions, mask[None], rot.float(), trans.float())
            if noises is not None:
                noisy = positions + nscale[i] * noises[i]
            elif self.gaussian_noise:
                noisy = positions + nscale[i] * torch.randn(positions.shape, generator=generator, device=dev)
            else:
                noisy = positions + nscale[i]
            denoised = head(noisy, t_hat[i], batch, embeddings, single_cond[i], pair_cond, state=state)
            grad = (noisy - denoised) / t_hat[i]
            positions = noisy + self.step_scale * (levels[i + 1] - t_hat[i]) * grad
        return {"atom_positions": positions, "mask": mask}
