"""CPU oracle for the diffusion head that drives the diffusion transformer and
the atom cross-attention (the direct caller of the hot path).

TEST INFRASTRUCTURE ONLY, like af3_oracle.py: plain eager PyTorch on the CPU,
in the dtype of its inputs; nothing in the product package imports it.

Reference files restated (paths relative to src/distributed_xfold/):

  per_atom_conditioning      nn/d_atom_cross_attention.py:87-156
  atom_cross_att_encoder     nn/d_atom_cross_attention.py:159-343
  atom_cross_att_decoder     nn/d_atom_cross_attention.py:355-414
  pre_conditioning           nn/d_diffusion_head.py:96-169
  diffusion_head             nn/d_diffusion_head.py:171-227
  fourier_embeddings         nn/d_diffusion_head.py:57-62
  sample_diffusion           d_alphafold3.py:316-404

The reference calls into the `xfold` package for the pieces below; its sources
are not in the reference tree, so they are restated from the published
AlphaFold 3 algorithm that xfold ports (alphafold3/model/atom_layout,
model/network/featurization.py, model/network/diffusion_head.py,
model/network/utils.py), anchored on the reference's call sites:

  convert / GatherInfo       atom_layout.convert as called at
                             nn/d_atom_cross_attention.py:169-179,238-242
  mask_mean                  utils.mask_mean, call site :328-331
  create_relative_encoding   featurization.create_relative_encoding, call site
                             nn/d_diffusion_head.py:106-108
  noise_schedule             diffusion_head.noise_schedule, call site
                             d_alphafold3.py:361-362
  random_augmentation        diffusion_head.random_augmentation, call site
                             d_alphafold3.py:337-339

Pinning status (tests/test_head_oracle_pins.py):

  convert, mask_mean, create_relative_encoding, fourier_embeddings,
  noise_schedule, random_augmentation: pinned by brute-force loops on tiny
  inputs, closed forms and invariants (end points of the schedule, a rigid
  motion keeps pairwise distances, one-hot rows sum to the number of groups).
  per_atom_conditioning, atom_cross_att_encoder, atom_cross_att_decoder,
  pre_conditioning, diffusion_head, sample_diffusion: wiring of pinned
  operations; pinned by an independently written per-atom loop formulation on
  a tiny batch (encoder pair conditioning, aggregation to tokens, decoder
  broadcast) and by closed forms (zero output weights return
  skip_scaling * positions_noisy).
  PARITY UNPINNED at the boundary of the absent `xfold` package: the
  constructor details of AtomCrossAttEncoder / AtomCrossAttDecoder /
  DiffusionHead (every Linear without bias, every LayerNorm with a weight and
  no bias, channel counts 128 / 16 / 768 / 384, 139 relative-encoding
  channels, 447 target-feature channels), the epsilon of mask_mean (1e-10)
  and the constants of noise_schedule and of the sampler.  The forms used here
  are those of the published algorithm.
"""

from __future__ import annotations

import math
from dataclasses import dataclass
from typing import Mapping

import torch
import torch.nn.functional as F

from . import af3_oracle as O

Params = Mapping[str, torch.Tensor]
SIGMA_DATA = 16.0      # nn/d_diffusion_head.py:47


# --------------------------------------------------------------------------
# pieces of xfold restated from the published algorithm
# --------------------------------------------------------------------------

def convert(gather_info, arr, layout_axes=(0,)):
    """atom_layout.convert: flatten the layout axes of `arr`, take
    `gather_idxs` along the flattened axis, zero where `gather_mask` is false.
    The layout axes must be consecutive and their sizes must multiply to the
    product of `input_shape`."""
    axes = tuple(a if a >= 0 else a + arr.dim() for a in layout_axes)
    begin, end = axes[0], axes[-1] + 1
    if axes != tuple(range(begin, end)):
        raise ValueError("layout_axes must be consecutive")
    idx, msk = gather_info.gather_idxs, gather_info.gather_mask
    lead, feat = tuple(arr.shape[:begin]), tuple(arr.shape[end:])
    n_in = 1
    for s in arr.shape[begin:end]:
        n_in *= int(s)
    n_expect = 1
    for s in tuple(gather_info.input_shape):
        n_expect *= int(s)
    if n_in != n_expect:
        raise ValueError(f"layout of {n_in} slots given to a gather built for {n_expect}")
    flat = arr.reshape(lead + (n_in,) + feat)
    out = flat.index_select(begin, idx.reshape(-1).long()).reshape(lead + tuple(idx.shape) + feat)
    m = msk.reshape((1,) * len(lead) + tuple(msk.shape) + (1,) * len(feat))
    if out.dtype == torch.bool:
        return out & m
    return out * m.to(out.dtype)


def mask_mean(mask, value, dim, eps=1e-10):
    """utils.mask_mean over one axis on which mask and value have the same
    size (mask may be 1 on other axes)."""
    mask = mask.to(value.dtype)
    return (mask * value).sum(dim) / torch.clamp(mask.expand_as(value).sum(dim), min=eps)


def create_relative_encoding(tf, max_relative_idx=32, max_relative_chain=2):
    """featurization.create_relative_encoding (AlphaFold 3 supplement,
    Algorithm 3): one-hot relative residue position (66), one-hot relative token
    position inside a residue (66), same entity (1), one-hot relative chain
    copy (6): 139 channels."""
    def lr(x):
        return x[:, None], x[None, :]
    la, ra = lr(tf.asym_id.long())
    lres, rres = lr(tf.residue_index.long())
    ltok, rtok = lr(tf.token_index.long())
    lent, rent = lr(tf.entity_id.long())
    lsym, rsym = lr(tf.sym_id.long())
    same_chain = la == ra
    off = torch.clamp(lres - rres + max_relative_idx, 0, 2 * max_relative_idx)
    off = torch.where(same_chain, off, torch.full_like(off, 2 * max_relative_idx + 1))
    rel_pos = F.one_hot(off, 2 * max_relative_idx + 2)
    same_res = same_chain & (lres == rres)
    toff = torch.clamp(ltok - rtok + max_relative_idx, 0, 2 * max_relative_idx)
    toff = torch.where(same_res, toff, torch.full_like(toff, 2 * max_relative_idx + 1))
    rel_tok = F.one_hot(toff, 2 * max_relative_idx + 2)
    same_ent = lent == rent
    coff = torch.clamp(lsym - rsym + max_relative_chain, 0, 2 * max_relative_chain)
    coff = torch.where(same_ent, coff, torch.full_like(coff, 2 * max_relative_chain + 1))
    rel_chain = F.one_hot(coff, 2 * max_relative_chain + 2)
    return torch.cat([rel_pos, rel_tok, same_ent[..., None].long(), rel_chain], dim=-1)


def fourier_embeddings(x, weight, bias):
    """nn/d_diffusion_head.py:57-62."""
    return torch.cos(2 * math.pi * (x[..., None] * weight + bias))


def noise_schedule(t, smin=0.0004, smax=160.0, p=7.0):
    """diffusion_head.noise_schedule: sigma_data * (smax^(1/p) + t (smin^(1/p) - smax^(1/p)))^p."""
    return SIGMA_DATA * (smax ** (1 / p) + t * (smin ** (1 / p) - smax ** (1 / p))) ** p


def random_augmentation(positions, mask, rot, trans):
    """diffusion_head.random_augmentation with the random rotation matrix
    `rot` [3,3] and translation `trans` [3] handed in: centre on the masked
    mean over all atoms, rotate, translate, zero the padding atoms."""
    m = mask.to(positions.dtype)[..., None]
    center = (m * positions).sum(dim=(-2, -3), keepdim=True) / torch.clamp(
        m.expand_as(positions[..., :1]).sum(dim=(-2, -3), keepdim=True), min=1e-6)
    return (torch.einsum("...i,ij->...j", positions - center, rot) + trans) * m


# --------------------------------------------------------------------------
# atom cross-attention encoder / decoder
# --------------------------------------------------------------------------

def per_atom_conditioning(batch, p: Params):
    """nn/d_atom_cross_attention.py:87-156 -> (act [N,A,128], pair_act [N,A,A,16])."""
    rs = batch.ref_structure
    dt = p["embed_ref_pos.weight"].dtype
    pos = rs.positions.to(dt)
    m = rs.mask.to(dt)
    act = O.linear(pos, p["embed_ref_pos.weight"])
    act = act + O.linear(m[:, :, None], p["embed_ref_mask.weight"])
    act = act + O.linear(F.one_hot(rs.element.long(), 128).to(dt), p["embed_ref_element.weight"])
    act = act + O.linear(torch.arcsinh(rs.charge.to(dt))[:, :, None], p["embed_ref_charge.weight"])
    name = F.one_hot(rs.atom_name_chars.long(), 64).to(dt)
    n_tok, n_dense = act.shape[:2]
    act = act + O.linear(name.reshape(n_tok, n_dense, -1), p["embed_ref_atom_name.weight"])
    act = act * m[:, :, None]
    row = O.linear(torch.relu(act), p["single_to_pair_cond_row.weight"])
    col = O.linear(torch.relu(act), p["single_to_pair_cond_col.weight"])
    pair_act = row[:, :, None, :] + col[:, None, :, :]
    d = pos[:, :, None, :] - pos[:, None, :, :]
    pair_act = pair_act + O.linear(d, p["embed_pair_offsets.weight"])
    sq = (d * d).sum(-1)
    pair_act = pair_act + O.linear(1.0 / (1 + sq[..., None]), p["embed_pair_distances.weight"])
    return act, pair_act


@dataclass
class EncoderOutput:
    token_act: torch.Tensor
    skip_connection: torch.Tensor
    queries_mask: torch.Tensor
    queries_single_cond: torch.Tensor
    keys_mask: torch.Tensor
    keys_single_cond: torch.Tensor
    pair_cond: torch.Tensor


def atom_cross_att_encoder(batch, token_atoms_act, trunk_single_cond, trunk_pair_cond, p: Params,
                           batched: bool = True):
    """nn/d_atom_cross_attention.py:159-343.  `batched` is the reference's
    use_batch_infer: token_atoms_act carries a leading sample axis."""
    aca = batch.atom_cross_att
    dt = p["embed_ref_pos.weight"].dtype
    tok_single, _ = per_atom_conditioning(batch, p)
    tok_mask = batch.predicted_structure_info.atom_mask
    q_cond = convert(aca.token_atoms_to_queries, tok_single, (-3, -2))
    q_mask = convert(aca.token_atoms_to_queries, tok_mask, (-2, -1))
    if trunk_single_cond is not None:
        ts = O.linear(O.layer_norm(trunk_single_cond.to(dt), p["lnorm_trunk_single_cond.weight"]),
                      p["embed_trunk_single_cond.weight"])
        q_cond = q_cond + convert(aca.tokens_to_queries, ts, (-2,))
    qm = q_mask.to(dt)
    if token_atoms_act is None:
        q_act = q_cond.clone()
    else:
        q_act = convert(aca.token_atoms_to_queries, token_atoms_act.to(dt), (-3, -2))
        q_act = O.linear(q_act, p["atom_positions_to_features.weight"])
        q_act = q_act * (qm[None, ..., None] if batched else qm[..., None])
        q_act = q_act + (q_cond[None] if batched else q_cond)
    k_cond = convert(aca.queries_to_keys, q_cond, (-3, -2))
    k_mask = convert(aca.queries_to_keys, q_mask, (-2, -1))

    row = O.linear(torch.relu(q_cond), p["single_to_pair_cond_row_1.weight"])
    col = O.linear(torch.relu(k_cond), p["single_to_pair_cond_col_1.weight"])
    pair_act = row[:, :, None, :] + col[:, None, :, :]
    if trunk_pair_cond is not None:
        tp = O.linear(O.layer_norm(trunk_pair_cond.to(dt), p["lnorm_trunk_pair_cond.weight"]),
                      p["embed_trunk_pair_cond.weight"])
        n_tok = tp.shape[0]
        t2q, t2k = aca.tokens_to_queries, aca.tokens_to_keys
        idx = n_tok * t2q.gather_idxs.long()[:, :, None] + t2k.gather_idxs.long()[:, None, :]
        msk = t2q.gather_mask[:, :, None] & t2k.gather_mask[:, None, :]
        pair_act = pair_act + tp.reshape(n_tok * n_tok, -1)[idx] * msk[..., None].to(dt)
    rs = batch.ref_structure
    q_pos = convert(aca.token_atoms_to_queries, rs.positions.to(dt), (-3, -2))
    q_uid = convert(aca.token_atoms_to_queries, rs.ref_space_uid, (-2, -1))
    k_pos = convert(aca.queries_to_keys, q_pos, (-3, -2))
    # :279-283 gathers the keys' uid from the token-atom layout with the
    # query-layout gather (not from queries_ref_space_uid); restated as written
    k_uid = convert(aca.queries_to_keys, rs.ref_space_uid, (-2, -1))
    valid = (q_uid[:, :, None] == k_uid[:, None, :]).to(dt)[..., None]
    off = q_pos[:, :, None, :] - k_pos[:, None, :, :]
    pair_act = pair_act + O.linear(off, p["embed_pair_offsets_1.weight"]) * valid
    sq = (off * off).sum(-1)
    pair_act = pair_act + O.linear(1.0 / (1 + sq[..., None]), p["embed_pair_distances_1.weight"]) * valid
    pair_act = pair_act + O.linear(valid, p["embed_pair_offsets_valid.weight"])
    h = O.linear(torch.relu(pair_act), p["pair_mlp_1.weight"])
    h = O.linear(torch.relu(h), p["pair_mlp_2.weight"])
    pair_act = pair_act + O.linear(torch.relu(h), p["pair_mlp_3.weight"])

    q2k = aca.queries_to_keys
    q_act = O.cross_att_transformer(q_act, q_mask, q2k.gather_idxs, q2k.gather_mask, k_mask, q_cond, k_cond,
                                    pair_act, O._sub(p, "atom_transformer_encoder"))
    q_act = q_act * (qm[None, ..., None] if batched else qm[..., None])
    skip = q_act
    agg = O.linear(q_act, p["project_atom_features_for_aggr.weight"])
    tok_atoms = convert(aca.queries_to_token_atoms, agg, (-3, -2))
    tm = tok_mask.to(dt)
    tok_act = mask_mean(tm[None, ..., None] if batched else tm[..., None], torch.relu(tok_atoms), dim=-2)
    return EncoderOutput(tok_act, skip, q_mask, q_cond, k_mask, k_cond, pair_act)


def atom_cross_att_decoder(batch, token_act, enc: EncoderOutput, p: Params, batched: bool = True):
    """nn/d_atom_cross_attention.py:355-414."""
    aca = batch.atom_cross_att
    dt = token_act.dtype
    t = O.linear(token_act, p["project_token_features_for_broadcast.weight"])
    n_tok, n_dense = aca.queries_to_token_atoms.gather_idxs.shape
    if batched:
        ta = t[:, :, None, :].expand(t.shape[0], n_tok, n_dense, t.shape[-1])
    else:
        ta = t[:, None, :].expand(n_tok, n_dense, t.shape[-1])
    q_act = convert(aca.token_atoms_to_queries, ta, (-3, -2))
    q_act = q_act + enc.skip_connection
    qm = enc.queries_mask.to(dt)
    qm = qm[None, ..., None] if batched else qm[..., None]
    q_act = q_act * qm
    q2k = aca.queries_to_keys
    q_act = O.cross_att_transformer(q_act, enc.queries_mask, q2k.gather_idxs, q2k.gather_mask, enc.keys_mask,
                                    enc.queries_single_cond, enc.keys_single_cond, enc.pair_cond,
                                    O._sub(p, "atom_transformer_decoder"))
    q_act = q_act * qm
    q_act = O.layer_norm(q_act, p["atom_features_layer_norm.weight"])
    upd = O.linear(q_act, p["atom_features_to_position_update.weight"])
    return convert(aca.queries_to_token_atoms, upd, (-3, -2))


# --------------------------------------------------------------------------
# diffusion head
# --------------------------------------------------------------------------

def pre_conditioning(batch, embeddings, noise_level, use_conditioning, p: Params):
    """nn/d_diffusion_head.py:96-169 -> (single_cond [T,N,384], pair_cond [N,N,128])."""
    dt = p["pair_cond_initial_projection.weight"].dtype
    single = use_conditioning * embeddings["single"].to(dt)
    pair = use_conditioning * embeddings["pair"].to(dt)
    rel = create_relative_encoding(batch.token_features, 32, 2).to(dt)
    f2d = torch.cat([pair, rel], dim=-1)
    f1d = torch.cat([single, embeddings["target_feat"].to(dt)], dim=-1)
    pair_cond = O.linear(O.layer_norm(f2d, p["pair_cond_initial_norm.weight"]),
                         p["pair_cond_initial_projection.weight"])
    pair_cond = pair_cond + O.diffusion_transition(pair_cond, None, O._sub(p, "pair_transition_0"))
    pair_cond = pair_cond + O.diffusion_transition(pair_cond, None, O._sub(p, "pair_transition_1"))
    noise = fourier_embeddings(0.25 * torch.log(noise_level.to(dt) / SIGMA_DATA),
                               p["fourier_embeddings.weight"], p["fourier_embeddings.bias"])
    noise = O.linear(O.layer_norm(noise, p["noise_embedding_initial_norm.weight"]),
                     p["noise_embedding_initial_projection.weight"])
    single_cond = O.linear(O.layer_norm(f1d, p["single_cond_initial_norm.weight"]),
                           p["single_cond_initial_projection.weight"])
    single_cond = single_cond[None] + noise[:, None, :]
    single_cond = single_cond + O.diffusion_transition(single_cond, None, O._sub(p, "single_transition_0"))
    single_cond = single_cond + O.diffusion_transition(single_cond, None, O._sub(p, "single_transition_1"))
    return single_cond, pair_cond


def diffusion_head(positions_noisy, noise_level, batch, embeddings, trunk_single_cond, trunk_pair_cond,
                   p: Params, batched: bool = True, num_blocks: int = 24):
    """nn/d_diffusion_head.py:171-227: one denoising evaluation."""
    dt = positions_noisy.dtype
    seq_mask = batch.token_features.mask
    am = batch.predicted_structure_info.atom_mask.to(dt)
    am = am[None, ..., None] if batched else am[..., None]
    act = positions_noisy * am
    act = act / torch.sqrt(noise_level ** 2 + SIGMA_DATA ** 2)
    enc = atom_cross_att_encoder(batch, act, embeddings["single"], trunk_pair_cond,
                                 O._sub(p, "atom_cross_att_encoder"), batched)
    act = enc.token_act
    emb = O.linear(O.layer_norm(trunk_single_cond.to(dt), p["single_cond_embedding_norm.weight"]),
                   p["single_cond_embedding_projection.weight"])
    act = act + (emb[None] if batched else emb)
    act = O.diffusion_transformer(act, seq_mask, trunk_single_cond.to(dt), trunk_pair_cond.to(dt),
                                  O._sub(p, "transformer"), num_blocks=num_blocks)
    act = O.layer_norm(act, p["output_norm.weight"])
    upd = atom_cross_att_decoder(batch, act, enc, O._sub(p, "atom_cross_att_decoder"), batched)
    skip = SIGMA_DATA ** 2 / (noise_level ** 2 + SIGMA_DATA ** 2)
    out = noise_level * SIGMA_DATA / torch.sqrt(noise_level ** 2 + SIGMA_DATA ** 2)
    return (skip * positions_noisy + out * upd) * am


def sampler_schedule(steps, dtype=torch.float64, gamma_0=0.8, gamma_min=1.0, noise_scale=1.003):
    """d_alphafold3.py:359-371 -> (noise_levels [steps+1], t_hat [steps], noise_scale [steps])."""
    levels = noise_schedule(torch.linspace(0, 1, steps + 1, dtype=dtype))
    prev, cur = levels[:-1], levels[1:]
    gamma = gamma_0 * (cur > gamma_min).to(dtype)
    t_hat = prev * (1 + gamma)
    return levels, t_hat, noise_scale * torch.sqrt(t_hat ** 2 - prev ** 2)


def sample_diffusion(batch, embeddings, p: Params, positions, rots, transs, steps, step_scale=1.5,
                     num_blocks: int = 24, noises=None):
    """d_alphafold3.py:316-404 with the random draws handed in: `positions`
    [S,N,A,3] is the standard-normal start (scaled here by the first noise
    level), rots [steps,3,3] / transs [steps,3] the augmentation of each step.
    As in the reference (:340-342, where the normal draw is commented out) the
    step's noise term is the scalar noise_scale itself unless `noises`
    [steps,S,N,A,3] is given, in which case it is noise_scale * noises[step]."""
    dt = positions.dtype
    mask = batch.predicted_structure_info.atom_mask
    levels, t_hat, nscale = sampler_schedule(steps, dt)
    single_cond, pair_cond = pre_conditioning(batch, embeddings, t_hat, True, p)
    positions = positions * levels[0]
    for i in range(steps):
        positions = random_augmentation(positions, mask[None], rots[i], transs[i])
        noisy = positions + (nscale[i] if noises is None else nscale[i] * noises[i])
        den = diffusion_head(noisy, t_hat[i], batch, embeddings, single_cond[i], pair_cond, p, True, num_blocks)
        grad = (noisy - den) / t_hat[i]
        positions = noisy + step_scale * (levels[i + 1] - t_hat[i]) * grad
    return positions


# --------------------------------------------------------------------------
# parameter generators (reference parameter names)
# --------------------------------------------------------------------------

def _lin(gen, c_out, c_in, std, dtype):
    return O._randn(gen, c_out, c_in, std=std, dtype=dtype)


def make_encoder_params(gen, per_token_channels=768, with_token_atoms_act=True, with_trunk_single_cond=True,
                        with_trunk_pair_cond=True, c_atom=128, c_pair=16, c_trunk_single=384,
                        c_trunk_pair=128, std=0.02, dtype=torch.float32):
    p = {}
    for name, cin in (("embed_ref_pos", 3), ("embed_ref_mask", 1), ("embed_ref_element", 128),
                      ("embed_ref_charge", 1), ("embed_ref_atom_name", 256)):
        p[f"{name}.weight"] = _lin(gen, c_atom, cin, std, dtype)
    for name, cin in (("single_to_pair_cond_row", c_atom), ("single_to_pair_cond_col", c_atom),
                      ("embed_pair_offsets", 3), ("embed_pair_distances", 1),
                      ("single_to_pair_cond_row_1", c_atom), ("single_to_pair_cond_col_1", c_atom),
                      ("embed_pair_offsets_1", 3), ("embed_pair_distances_1", 1),
                      ("embed_pair_offsets_valid", 1), ("pair_mlp_1", c_pair), ("pair_mlp_2", c_pair),
                      ("pair_mlp_3", c_pair)):
        p[f"{name}.weight"] = _lin(gen, c_pair, cin, std if cin > 3 else 0.3, dtype)
    if with_trunk_single_cond:
        O._put(p, "lnorm_trunk_single_cond", O.make_ln(gen, c_trunk_single, bias=False, dtype=dtype))
        p["embed_trunk_single_cond.weight"] = _lin(gen, c_atom, c_trunk_single, std, dtype)
    if with_trunk_pair_cond:
        O._put(p, "lnorm_trunk_pair_cond", O.make_ln(gen, c_trunk_pair, bias=False, dtype=dtype))
        p["embed_trunk_pair_cond.weight"] = _lin(gen, c_pair, c_trunk_pair, std, dtype)
    if with_token_atoms_act:
        p["atom_positions_to_features.weight"] = _lin(gen, c_atom, 3, 0.3, dtype)
    O._put(p, "atom_transformer_encoder",
           O.make_cross_att_transformer_params(gen, c_atom, c_atom, c_pair, std=std, dtype=dtype))
    p["project_atom_features_for_aggr.weight"] = _lin(gen, per_token_channels, c_atom, std, dtype)
    return p


def make_decoder_params(gen, c_token=768, c_atom=128, c_pair=16, std=0.02, dtype=torch.float32):
    p = {"project_token_features_for_broadcast.weight": _lin(gen, c_atom, c_token, std, dtype)}
    O._put(p, "atom_transformer_decoder",
           O.make_cross_att_transformer_params(gen, c_atom, c_atom, c_pair, std=std, dtype=dtype))
    O._put(p, "atom_features_layer_norm", O.make_ln(gen, c_atom, bias=False, dtype=dtype))
    p["atom_features_to_position_update.weight"] = _lin(gen, 3, c_atom, std, dtype)
    return p


def make_diffusion_head_params(gen, num_blocks=24, c_pair=128, c_single=384, c_act=768, c_target=447,
                               c_rel=139, c_fourier=256, std=0.02, dtype=torch.float32):
    p = {}
    O._put(p, "pair_cond_initial_norm", O.make_ln(gen, c_pair + c_rel, bias=False, dtype=dtype))
    p["pair_cond_initial_projection.weight"] = _lin(gen, c_pair, c_pair + c_rel, std, dtype)
    for i in (0, 1):
        O._put(p, f"pair_transition_{i}", O.make_diffusion_transition_params(gen, c_pair, None, 2, False, std, dtype))
        O._put(p, f"single_transition_{i}",
               O.make_diffusion_transition_params(gen, c_single, None, 2, False, std, dtype))
    O._put(p, "single_cond_initial_norm", O.make_ln(gen, c_single + c_target, bias=False, dtype=dtype))
    p["single_cond_initial_projection.weight"] = _lin(gen, c_single, c_single + c_target, std, dtype)
    p["fourier_embeddings.weight"] = O._randn(gen, c_fourier, dtype=dtype)
    p["fourier_embeddings.bias"] = torch.rand(c_fourier, generator=gen).to(dtype)
    O._put(p, "noise_embedding_initial_norm", O.make_ln(gen, c_fourier, bias=False, dtype=dtype))
    p["noise_embedding_initial_projection.weight"] = _lin(gen, c_single, c_fourier, std, dtype)
    O._put(p, "atom_cross_att_encoder", make_encoder_params(gen, c_act, std=std, dtype=dtype))
    O._put(p, "single_cond_embedding_norm", O.make_ln(gen, c_single, bias=False, dtype=dtype))
    p["single_cond_embedding_projection.weight"] = _lin(gen, c_act, c_single, std, dtype)
    O._put(p, "transformer", O.make_diffusion_transformer_params(gen, c_act, c_single, c_pair,
                                                                  num_blocks=num_blocks, std=std, dtype=dtype))
    O._put(p, "output_norm", O.make_ln(gen, c_act, bias=False, dtype=dtype))
    O._put(p, "atom_cross_att_decoder", make_decoder_params(gen, c_act, std=std, dtype=dtype))
    return p
