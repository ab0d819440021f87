"""Layout conversions between the token-atom layout [N_token, atoms_per_token],
the flat query layout [subsets, 32] and the key windows [subsets, 128] of the
atom cross-attention, and the feature batch the diffusion head reads.

The reference takes these from the `xfold` package (`atom_layout.GatherInfo`,
`atom_layout.convert`, `feat_batch.Batch`; call sites
nn/d_atom_cross_attention.py:169-179, 238-242 and nn/d_diffusion_head.py:180-182);
the classes here carry the same attribute names, so a batch built by the
reference's data pipeline can be passed as it is (any object with these
attributes works).  `synthetic_batch` builds a batch of the same structure from
a per-token atom count, for tests and benchmarks: the featurisation pipeline
itself is not part of this package.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Optional, Sequence, Tuple

import torch

QUERIES_PER_SUBSET = 32
KEYS_PER_SUBSET = 128


@dataclass
class GatherInfo:
    """out[i...] = flat(in)[gather_idxs[i...]] where gather_mask, else 0."""
    gather_idxs: torch.Tensor       # integer, output layout shape
    gather_mask: torch.Tensor       # bool, same shape
    input_shape: Tuple[int, ...]    # layout shape of the input

    @property
    def shape(self):
        return tuple(self.gather_idxs.shape)

    def to(self, device):
        return GatherInfo(self.gather_idxs.to(device), self.gather_mask.to(device), tuple(self.input_shape))


def convert(gather_info, arr: torch.Tensor, layout_axes: Sequence[int] = (0,)) -> torch.Tensor:
    """Gather `arr` from one layout into another.  `layout_axes` are the
    consecutive axes of `arr` that hold the input layout; they are flattened,
    indexed with `gather_idxs`, and entries whose `gather_mask` is false are
    zeroed."""
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
        raise ValueError(f"layout axes hold {n_in} slots, the gather was built for {n_expect}")
    flat = arr.reshape(lead + (n_in,) + feat)
    out = flat.index_select(begin, idx.reshape(-1)).reshape(lead + tuple(idx.shape) + feat)
    m = msk.reshape((1,) * len(lead) + tuple(msk.shape) + (1,) * len(feat))
    if out.dtype == torch.bool:
        return out & m
    return out * m.to(out.dtype)


@dataclass
class TokenFeatures:
    mask: torch.Tensor            # [N]
    token_index: torch.Tensor     # [N]
    residue_index: torch.Tensor   # [N]
    asym_id: torch.Tensor         # [N]
    entity_id: torch.Tensor       # [N]
    sym_id: torch.Tensor          # [N]


@dataclass
class RefStructure:
    positions: torch.Tensor        # [N, A, 3]
    mask: torch.Tensor             # [N, A]
    element: torch.Tensor          # [N, A] atomic number (< 128)
    charge: torch.Tensor           # [N, A]
    atom_name_chars: torch.Tensor  # [N, A, 4] ASCII code - 32 (< 64)
    ref_space_uid: torch.Tensor    # [N, A]


@dataclass
class PredictedStructureInfo:
    atom_mask: torch.Tensor        # [N, A]


@dataclass
class AtomCrossAtt:
    token_atoms_to_queries: GatherInfo   # [S, 32]  <- [N, A]
    tokens_to_queries: GatherInfo        # [S, 32]  <- [N]
    tokens_to_keys: GatherInfo           # [S, 128] <- [N]
    queries_to_keys: GatherInfo          # [S, 128] <- [S, 32]
    queries_to_token_atoms: GatherInfo   # [N, A]   <- [S, 32]


@dataclass
class Batch:
    token_features: TokenFeatures
    ref_structure: RefStructure
    predicted_structure_info: PredictedStructureInfo
    atom_cross_att: AtomCrossAtt

    def to(self, device):
        def mv(obj):
            kw = {}
            for k, v in vars(obj).items():
                kw[k] = v.to(device) if isinstance(v, (torch.Tensor, GatherInfo)) else mv(v)
            return type(obj)(**kw)
        return mv(self)


def atom_cross_att_layout(atom_mask: torch.Tensor) -> AtomCrossAtt:
    """The gathers of the atom cross-attention for a token-atom mask [N, A]:
    the atoms that are present are laid out flat in token order and padded to
    N * A slots, cut into subsets of 32 queries; each subset attends to the
    window of 128 flat atoms centred on it (shifted inwards at both ends)."""
    n_tok, n_dense = atom_mask.shape
    total = n_tok * n_dense
    if total % QUERIES_PER_SUBSET or total < KEYS_PER_SUBSET:
        raise ValueError("N * atoms_per_token must be a multiple of 32 and at least 128")
    am = atom_mask.bool().cpu()
    tok = torch.arange(n_tok)[:, None].expand(n_tok, n_dense)[am]        # token of each flat atom
    slot = torch.arange(total).reshape(n_tok, n_dense)[am]               # its [N, A] slot
    n_real = int(tok.numel())
    n_sub = total // QUERIES_PER_SUBSET
    q_tok = torch.zeros(total, dtype=torch.long)
    q_slot = torch.zeros(total, dtype=torch.long)
    q_mask = torch.zeros(total, dtype=torch.bool)
    q_tok[:n_real], q_slot[:n_real], q_mask[:n_real] = tok, slot, True
    shape_q = (n_sub, QUERIES_PER_SUBSET)
    centre = torch.arange(n_sub) * QUERIES_PER_SUBSET + QUERIES_PER_SUBSET // 2
    start = torch.clamp(centre - KEYS_PER_SUBSET // 2, 0, total - KEYS_PER_SUBSET)
    k_idx = start[:, None] + torch.arange(KEYS_PER_SUBSET)[None, :]     # [S, 128] into flat queries
    back = torch.zeros(total, dtype=torch.long)                          # [N, A] slot -> flat query
    back[slot] = torch.arange(n_real)
    return AtomCrossAtt(
        token_atoms_to_queries=GatherInfo(q_slot.reshape(shape_q), q_mask.reshape(shape_q), (n_tok, n_dense)),
        tokens_to_queries=GatherInfo(q_tok.reshape(shape_q), q_mask.reshape(shape_q), (n_tok,)),
        tokens_to_keys=GatherInfo(q_tok[k_idx], q_mask[k_idx], (n_tok,)),
        queries_to_keys=GatherInfo(k_idx, q_mask[k_idx], shape_q),
        queries_to_token_atoms=GatherInfo(back.reshape(n_tok, n_dense), am.clone(), shape_q),
    )


def synthetic_batch(n_token: int, gen: Optional[torch.Generator] = None, atoms_per_token: int = 24,
                    n_padding_tokens: int = 0, chain_len: int = 97) -> Batch:
    """A random batch with the structure the diffusion head reads: chains of
    `chain_len` tokens (every third chain a copy of the first entity), 1 to
    `atoms_per_token` atoms per token, reference conformers N(0, 2 A), the last
    `n_padding_tokens` tokens padding (no atoms, token mask 0)."""
    g = gen
    live = n_token - n_padding_tokens
    n_atoms = torch.randint(1, atoms_per_token + 1, (n_token,), generator=g)
    n_atoms[live:] = 0
    atom_mask = torch.arange(atoms_per_token)[None, :] < n_atoms[:, None]
    idx = torch.arange(n_token)
    chain = idx // chain_len
    tf = TokenFeatures(mask=(idx < live).float(), token_index=idx.clone(), residue_index=idx % chain_len,
                       asym_id=chain + 1, entity_id=chain % 3 + 1, sym_id=chain // 3 + 1)
    shp = (n_token, atoms_per_token)
    rs = RefStructure(
        positions=torch.randn(shp + (3,), generator=g) * 2.0 * atom_mask[..., None],
        mask=atom_mask.float(),
        element=torch.randint(1, 35, shp, generator=g) * atom_mask,
        charge=torch.randint(-1, 2, shp, generator=g).float() * atom_mask,
        atom_name_chars=torch.randint(0, 64, shp + (4,), generator=g) * atom_mask[..., None],
        ref_space_uid=idx[:, None].expand(shp).contiguous(),
    )
    return Batch(tf, rs, PredictedStructureInfo(atom_mask.float()), atom_cross_att_layout(atom_mask))


@dataclass
class PolymerLigandBondInfo:
    tokens_to_polymer_ligand_bonds: GatherInfo     # gather_idxs / gather_mask [bonds, 2]


@dataclass
class LigandLigandBondInfo:
    tokens_to_ligand_ligand_bonds: GatherInfo      # gather_idxs / gather_mask [bonds, 2]


@dataclass
class TrunkBatch:
    """What the Evoformer trunk reads (d_alphafold3.py:67-191), with the MSA
    already featurised: msa_feat [rows, N, 34], msa_mask [rows, N]."""
    token_features: TokenFeatures
    polymer_ligand_bond_info: PolymerLigandBondInfo
    ligand_ligand_bond_info: LigandLigandBondInfo
    msa_feat: torch.Tensor
    msa_mask: torch.Tensor

    to = Batch.to


def synthetic_trunk_batch(n_token: int, msa_rows: int, gen: Optional[torch.Generator] = None,
                          n_padding_tokens: int = 0, chain_len: int = 97, n_bonds: int = 6) -> TrunkBatch:
    """A random trunk batch: the token features of `synthetic_batch`, a few
    bonds between random live tokens (one of each kind with a masked end) and
    random MSA features with a 0/1 mask whose first row covers every live token."""
    g = gen
    live = n_token - n_padding_tokens
    idx = torch.arange(n_token)
    chain = idx // chain_len
    tf = TokenFeatures(mask=(idx < live).float(), token_index=idx.clone(), residue_index=idx % chain_len,
                       asym_id=chain + 1, entity_id=chain % 3 + 1, sym_id=chain // 3 + 1)

    def bonds():
        gi = torch.randint(0, live, (n_bonds, 2), generator=g)
        gm = torch.ones(n_bonds, 2, dtype=torch.bool)
        gm[-1, 1] = False
        return GatherInfo(gi, gm, (n_token,))
    seq = tf.mask
    mm = (torch.rand(msa_rows, n_token, generator=g) > 0.2).float() * seq[None, :]
    mm[0] = seq
    feat = torch.randn(msa_rows, n_token, 34, generator=g) * mm[..., None]
    return TrunkBatch(tf, PolymerLigandBondInfo(bonds()), LigandLigandBondInfo(bonds()), feat, mm)
