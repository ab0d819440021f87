"""Pins of the Evoformer trunk oracle (oracle/af3_trunk_oracle.py) on the CPU:
the input embeddings re-derived pair by pair with loops, the contact matrix by
hand, and the recycling recurrence."""

import torch

from oracle import af3_head_oracle as H
from oracle import af3_oracle as O
from oracle import af3_trunk_oracle as T

D = torch.float64


def gen(seed):
    return torch.Generator().manual_seed(seed)


def case(pkg, n=10, rows=4, msa_blocks=0, pf_blocks=0, seed=1):
    g = gen(seed)
    batch = pkg.nn.atom_layout.synthetic_trunk_batch(n, rows, g, n_padding_tokens=2, chain_len=4)
    p = T.make_evoformer_params(g, msa_blocks, pf_blocks, dtype=D)
    tf = torch.randn(n, 447, generator=g, dtype=D)
    return g, batch, p, tf


def test_contact_matrix_by_hand(pkg):
    g, batch, p, tf = case(pkg)
    cm = T.contact_matrix(batch, 10, D)
    want = torch.zeros(10, 10, dtype=D)
    for info in (batch.polymer_ligand_bond_info.tokens_to_polymer_ligand_bonds,
                 batch.ligand_ligand_bond_info.tokens_to_ligand_ligand_bonds):
        for b in range(info.gather_idxs.shape[0]):
            if bool(info.gather_mask[b].all()):
                want[int(info.gather_idxs[b, 0]), int(info.gather_idxs[b, 1])] = 1
    want[0, 0] = 0
    assert torch.equal(cm, want) and cm.sum() > 0
    assert torch.equal(pkg.nn.Evoformer.contact_matrix(batch, 10, "cpu").double(), want)


def test_embeddings_pair_by_pair(pkg):
    g, batch, p, tf = case(pkg)
    n = 10
    prev = {"pair": torch.randn(n, n, 128, generator=g, dtype=D), "single": torch.randn(n, 384, generator=g, dtype=D)}
    out = T.evoformer(batch, prev, tf, p, 0, 0)
    rel = H.create_relative_encoding(batch.token_features).to(D)
    cm = T.contact_matrix(batch, n, D)

    def ln(x, w, b):
        mu = x.mean()
        return (x - mu) / torch.sqrt(((x - mu) ** 2).mean() + 1e-5) * w + b
    for (i, j) in [(0, 0), (1, 5), (7, 2), (9, 9), (3, 8)]:
        want = p["left_single.weight"] @ tf[i] + p["right_single.weight"] @ tf[j]
        want = want + p["prev_embedding.weight"] @ ln(prev["pair"][i, j], p["prev_embedding_layer_norm.weight"],
                                                      p["prev_embedding_layer_norm.bias"])
        want = want + p["position_activations.weight"] @ rel[i, j] + p["bond_embedding.weight"][:, 0] * cm[i, j]
        assert torch.allclose(out["pair"][i, j], want, atol=1e-10), (i, j)
    for i in (0, 4, 9):
        want = p["single_activations.weight"] @ tf[i] + p["prev_single_embedding.weight"] @ ln(
            prev["single"][i], p["prev_single_embedding_layer_norm.weight"], p["prev_single_embedding_layer_norm.bias"])
        assert torch.allclose(out["single"][i], want, atol=1e-10)


def test_recycling_recurrence_and_stack_order(pkg):
    g, batch, p, tf = case(pkg, n=8, rows=3, msa_blocks=1, pf_blocks=1, seed=2)
    n = 8
    zero = {"pair": torch.zeros(n, n, 128, dtype=D), "single": torch.zeros(n, 384, dtype=D)}
    one = T.evoformer(batch, zero, tf, p, 1, 1)
    two = T.evoformer(batch, one, tf, p, 1, 1)
    got = T.recycle(batch, tf, p, 2, 1, 1)
    assert torch.allclose(got["pair"], two["pair"], atol=1e-12) and torch.allclose(got["single"], two["single"], atol=1e-12)
    assert not torch.allclose(one["pair"], two["pair"], atol=1e-3)
    # the MSA block comes before the Pairformer block and both see the embedded pair tensor
    emb = T.evoformer(batch, zero, tf, p, 0, 0)
    from oracle import af3_msa_oracle as M
    mask = batch.token_features.mask.double()
    pm = mask[:, None] * mask[None, :]
    msa = O.linear(batch.msa_feat.double(), p["msa_activations.weight"]) + O.linear(tf, p["extra_msa_target_feat.weight"])[None]
    _, z = M.evoformer_block(msa, emb["pair"], batch.msa_mask.double(), pm, O._sub(p, "msa_stack.0"))
    z, s = O.pairformer_block(z, pm, emb["single"], mask, O._sub(p, "trunk_pairformer.0"))
    assert torch.allclose(one["pair"], z, atol=1e-12) and torch.allclose(one["single"], s, atol=1e-12)
