#!/usr/bin/env python3
"""Writes tests/golden/*.npz: seeded inputs are regenerated from their seeds, the
file holds the float64-oracle outputs (stored as float32) for small problems.

The reference ships no golden vectors (its tests compare two live computations
under torch.manual_seed(11), e.g. xsmm_kernels/kernel_test/triangle_multiplication.py:139-189)
and its Python cannot be imported here (the xfold / tpp submodules are empty),
so these vectors come from this repository's own pinned oracle.  They freeze the
oracle against accidental edits and give the GPU tests a reference that does not
depend on the oracle code being present.

Run from the repository root:  python tests/golden/make_golden.py
"""

import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
from oracle import af3_oracle as O  # noqa: E402

D = torch.float64
SIZES = (5, 17)


def case_inputs(n, seed):
    """Inputs and bf16-representable parameters of case (n, seed); shared with the tests."""
    g = torch.Generator().manual_seed(seed)
    rb = O.round_bf16
    params = {k: rb(v) for k, v in O.make_pairformer_block_params(g).items()}
    pair = rb(torch.randn(n, n, 128, generator=g))
    single = rb(torch.randn(n, 384, generator=g))
    live = max(1, n - max(1, n // 8))
    seq_mask = (torch.arange(n) < live).float()
    pair_mask = (torch.rand(n, n, generator=g) > 0.15).float() * seq_mask[None, :]
    pair_mask[:, 0] = 1.0
    return params, pair, single, seq_mask, pair_mask


def diffusion_inputs(n, seed):
    g = torch.Generator().manual_seed(seed)
    rb = O.round_bf16
    params = {k: rb(v) for k, v in O.make_diffusion_transformer_params(g, num_blocks=4, std=0.05).items()}
    act = rb(torch.randn(2, n, 768, generator=g))
    single_cond = rb(torch.randn(n, 384, generator=g))
    pair_cond = rb(torch.randn(n, n, 128, generator=g))
    mask = (torch.arange(n) < max(1, n - 2)).float()
    return params, act, mask, single_cond, pair_cond


def expected(n, seed):
    params, pair, single, seq_mask, pair_mask = case_inputs(n, seed)
    p = O.cast_params(params, D)
    x, s, sm, pm = pair.double(), single.double(), seq_mask.double(), pair_mask.double()
    out = {
        "trimul_out": O.triangle_multiplication(x, pm, O._sub(p, "triangle_multiplication_outgoing"), True),
        "trimul_in": O.triangle_multiplication(x, pm, O._sub(p, "triangle_multiplication_incoming"), False),
        "triattn_start": O.grid_self_attention(x, pm, O._sub(p, "pair_attention1"), 4, False),
        "triattn_end": O.grid_self_attention(x, pm, O._sub(p, "pair_attention2"), 4, True),
        "pair_transition": O.transition(x, O._sub(p, "pair_transition")),
    }
    bp, bs = O.pairformer_block(x, sm[:, None] * sm[None, :], s, sm, p)
    out["block_pair"], out["block_single"] = bp, bs
    dp, act, mask, sc, pc = diffusion_inputs(n, seed + 1000)
    out["diffusion_transformer"] = O.diffusion_transformer(act.double(), mask.double(), sc.double(), pc.double(),
                                                           O.cast_params(dp, D), 16, 4, 4)
    return {k: v.float().numpy() for k, v in out.items()}


def head_inputs(n=8, seed=300, blocks=1, samples=2):
    """Inputs of the diffusion-head case; the feature batch comes from the
    product package's synthetic layout builder (pure PyTorch, no kernels)."""
    from oracle import af3_head_oracle as H
    import __graft_entry__ as ge
    al = ge.load_package().nn.atom_layout
    g = torch.Generator().manual_seed(seed)
    rb = O.round_bf16
    batch = al.synthetic_batch(n, g, n_padding_tokens=1, chain_len=3)
    params = {k: rb(v) for k, v in H.make_diffusion_head_params(g, num_blocks=blocks, std=0.05).items()}
    emb = {"single": rb(torch.randn(n, 384, generator=g)), "pair": rb(torch.randn(n, n, 128, generator=g)),
           "target_feat": rb(torch.randn(n, 447, generator=g))}
    pos = torch.randn(samples, n, 24, 3, generator=g)
    return batch, params, emb, pos


def head_expected(n=8, seed=300, blocks=1):
    from oracle import af3_head_oracle as H
    batch, params, emb, pos = head_inputs(n, seed, blocks)
    p = O.cast_params(params, D)
    embd = {k: v.double() for k, v in emb.items()}
    _, t_hat, _ = H.sampler_schedule(6)
    sc, pc = H.pre_conditioning(batch, embd, t_hat, True, p)
    out = {"single_cond": sc, "pair_cond": pc}
    for step in (1, 4):
        out[f"denoised_step{step}"] = H.diffusion_head(pos.double() * float(t_hat[step]), t_hat[step], batch, embd,
                                                       sc[step], pc, p, True, blocks)
    return {k: v.float().numpy() for k, v in out.items()}


def evoformer_inputs(rows=7, n=12, seed=400):
    from oracle import af3_msa_oracle as M
    g = torch.Generator().manual_seed(seed)
    rb = O.round_bf16
    params = {k: rb(v) for k, v in M.make_evoformer_block_params(g, std=0.05).items()}
    msa = rb(torch.randn(rows, n, 64, generator=g))
    pair = rb(torch.randn(n, n, 128, generator=g))
    mm = (torch.rand(rows, n, generator=g) > 0.2).float()
    mm[0] = 1
    mm[:, n - 1] = 0
    seq = mm.max(dim=0).values
    pm = seq[:, None] * seq[None, :]
    return params, msa, pair, mm, pm


def evoformer_expected(rows=7, n=12, seed=400):
    from oracle import af3_msa_oracle as M
    params, msa, pair, mm, pm = evoformer_inputs(rows, n, seed)
    m, z = M.evoformer_block(msa.double(), pair.double(), mm.double(), pm.double(), O.cast_params(params, D))
    return {"msa": m.float().numpy(), "pair": z.float().numpy()}


def main():
    path = os.path.join(HERE, "diffusion_head_n8.npz")
    np.savez_compressed(path, **head_expected())
    print(path, os.path.getsize(path) // 1024, "KiB")
    path = os.path.join(HERE, "evoformer_n12.npz")
    np.savez_compressed(path, **evoformer_expected())
    print(path, os.path.getsize(path) // 1024, "KiB")
    for n in SIZES:
        path = os.path.join(HERE, f"pairformer_n{n}.npz")
        np.savez_compressed(path, **expected(n, seed=100 + n))
        print(path, os.path.getsize(path) // 1024, "KiB")


if __name__ == "__main__":
    main()
