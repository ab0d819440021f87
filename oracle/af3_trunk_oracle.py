"""CPU oracle for the Evoformer trunk driver: input embeddings, MSA stack,
Pairformer stack and the recycling loop around them.

TEST INFRASTRUCTURE ONLY, like af3_oracle.py; nothing in the product package
imports it.

Reference restated (src/distributed_xfold/d_alphafold3.py): _seq_pair_embedding
:67-80, _relative_encoding :82-96, _embed_bonds :98-143, _embed_process_msa
:165-191 (from the embedded MSA features on: shuffling, truncation and
create_msa_feat belong to the data pipeline and are inputs here), forward
:193-254 without the template embedding (:219-223; its 64-channel Pairformer
blocks are not built), and the recycling loop :433-440.

Pinning: wiring of operations pinned elsewhere (af3_oracle, af3_msa_oracle,
af3_head_oracle.create_relative_encoding); tests/test_trunk_oracle_pins.py
re-derives the embedding sums with loops over token pairs and checks the
recycling recurrence.  PARITY UNPINNED at the boundary of the absent `xfold`
package (base class xfold.alphafold3.Evoformer): every embedding Linear without
bias, 447 target-feature and 34 MSA-feature channels, LayerNorms with weight
and bias on the recycled pair / single representation.
"""

from __future__ import annotations

from typing import Mapping

import torch

from . import af3_head_oracle as H
from . import af3_msa_oracle as M
from . import af3_oracle as O

Params = Mapping[str, torch.Tensor]


def contact_matrix(batch, n, dtype):
    """_embed_bonds :103-137: 1 where a polymer-ligand or ligand-ligand bond
    joins two tokens; bonds with a masked end collapse onto (0, 0), which is
    cleared."""
    rows = []
    for info in (batch.polymer_ligand_bond_info.tokens_to_polymer_ligand_bonds,
                 batch.ligand_ligand_bond_info.tokens_to_ligand_ligand_bonds):
        ok = info.gather_mask.to(torch.long).prod(dim=1)[:, None]
        rows.append(info.gather_idxs.long() * ok)
    idx = torch.cat(rows)
    cm = torch.zeros(n, n, dtype=dtype)
    cm[idx[:, 0], idx[:, 1]] = 1.0
    cm[0, 0] = 0.0
    return cm


def evoformer(batch, prev, target_feat, p: Params, num_msa_blocks: int, num_pairformer_blocks: int):
    """d_alphafold3.py:193-254 -> {'single', 'pair', 'target_feat'}."""
    dt = p["left_single.weight"].dtype
    tf = target_feat.to(dt)
    mask = batch.token_features.mask.to(dt)
    n = mask.shape[0]
    pair = O.linear(tf, p["left_single.weight"])[:, None] + O.linear(tf, p["right_single.weight"])[None]
    pair_mask = mask[:, None] * mask[None, :]
    pair = pair + O.linear(O.layer_norm(prev["pair"].to(dt), p["prev_embedding_layer_norm.weight"],
                                        p["prev_embedding_layer_norm.bias"]), p["prev_embedding.weight"])
    rel = H.create_relative_encoding(batch.token_features, 32, 2).to(dt)
    pair = pair + O.linear(rel, p["position_activations.weight"])
    pair = pair + O.linear(contact_matrix(batch, n, dt)[:, :, None], p["bond_embedding.weight"])
    msa = O.linear(batch.msa_feat.to(dt), p["msa_activations.weight"])
    msa = msa + O.linear(tf, p["extra_msa_target_feat.weight"])[None]
    msa_mask = batch.msa_mask.to(dt)
    for i in range(num_msa_blocks):
        msa, pair = M.evoformer_block(msa, pair, msa_mask, pair_mask, O._sub(p, f"msa_stack.{i}"))
    single = O.linear(tf, p["single_activations.weight"])
    single = single + O.linear(O.layer_norm(prev["single"].to(dt), p["prev_single_embedding_layer_norm.weight"],
                                            p["prev_single_embedding_layer_norm.bias"]),
                               p["prev_single_embedding.weight"])
    for i in range(num_pairformer_blocks):
        pair, single = O.pairformer_block(pair, pair_mask, single, mask, O._sub(p, f"trunk_pairformer.{i}"))
    return {"single": single, "pair": pair, "target_feat": target_feat}


def recycle(batch, target_feat, p: Params, num_recycles: int, num_msa_blocks: int, num_pairformer_blocks: int):
    """d_alphafold3.py:410-440: zero embeddings, then num_recycles passes."""
    dt = p["left_single.weight"].dtype
    n = target_feat.shape[0]
    emb = {"pair": torch.zeros(n, n, p["prev_embedding.weight"].shape[1], dtype=dt),
           "single": torch.zeros(n, p["prev_single_embedding.weight"].shape[1], dtype=dt),
           "target_feat": target_feat}
    for _ in range(num_recycles):
        emb = evoformer(batch, emb, target_feat, p, num_msa_blocks, num_pairformer_blocks)
    return emb


def make_evoformer_params(gen, num_msa_blocks=4, num_pairformer_blocks=48, c_pair=128, c_single=384, c_msa=64,
                          c_target=447, c_msa_feat=34, c_rel=139, std=0.02, dtype=torch.float32):
    p = {}
    for name, cout, cin in (("left_single", c_pair, c_target), ("right_single", c_pair, c_target),
                            ("prev_embedding", c_pair, c_pair), ("position_activations", c_pair, c_rel),
                            ("bond_embedding", c_pair, 1), ("msa_activations", c_msa, c_msa_feat),
                            ("extra_msa_target_feat", c_msa, c_target), ("single_activations", c_single, c_target),
                            ("prev_single_embedding", c_single, c_single)):
        p[f"{name}.weight"] = O._randn(gen, cout, cin, std=max(std, 0.05), dtype=dtype)
    O._put(p, "prev_embedding_layer_norm", O.make_ln(gen, c_pair, dtype=dtype))
    O._put(p, "prev_single_embedding_layer_norm", O.make_ln(gen, c_single, dtype=dtype))
    for i in range(num_msa_blocks):
        O._put(p, f"msa_stack.{i}", M.make_evoformer_block_params(gen, c_msa, c_pair, std=std, dtype=dtype))
    for i in range(num_pairformer_blocks):
        O._put(p, f"trunk_pairformer.{i}", O.make_pairformer_block_params(gen, c_pair, c_single, std=std, dtype=dtype))
    return p
