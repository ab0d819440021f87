"""Golden vectors (tests/golden/*.npz, written by tests/golden/make_golden.py).

CPU: the oracle still reproduces them (freezes the oracle).
GPU: the HIP path matches them, without calling the oracle's formulas."""

import importlib.util
import os

import numpy as np
import pytest
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
_spec = importlib.util.spec_from_file_location("make_golden", os.path.join(HERE, "golden", "make_golden.py"))
G = importlib.util.module_from_spec(_spec)
_spec.loader.exec_module(G)

SIZES = G.SIZES


def load(n):
    return dict(np.load(os.path.join(HERE, "golden", f"pairformer_n{n}.npz")))


def rms_err(got, want):
    got, want = torch.as_tensor(got).double(), torch.as_tensor(want).double()
    return float(torch.sqrt(((got - want) ** 2).mean()) / torch.sqrt((want ** 2).mean()))


@pytest.mark.parametrize("n", SIZES)
def test_oracle_reproduces_golden(n):
    want = load(n)
    got = G.expected(n, seed=100 + n)
    assert sorted(got) == sorted(want)
    for k in want:
        assert np.allclose(got[k], want[k], rtol=1e-5, atol=1e-6), k


@pytest.mark.gpu
@pytest.mark.parametrize("n", SIZES)
def test_hip_matches_golden(gpu_pkg, n):
    want = load(n)
    dev = torch.device("cuda:0")
    params, pair, single, seq_mask, pair_mask = G.case_inputs(n, 100 + n)
    blk = gpu_pkg.nn.PairformerBlock()
    blk.load_state_dict(params)
    blk.to(dev)
    x, pm = pair.to(dev), pair_mask.to(dev)
    got = {
        "trimul_out": blk.triangle_multiplication_outgoing(x, pm),
        "trimul_in": blk.triangle_multiplication_incoming(x, pm),
        "triattn_start": blk.pair_attention1(x, pm),
        "triattn_end": blk.pair_attention2(x, pm),
        "pair_transition": blk.pair_transition(x),
    }
    sm = seq_mask.to(dev)
    bp, bs = blk(pair.to(dev).clone(), (sm[:, None] * sm[None, :]).contiguous(), single.to(dev).clone(), sm)
    got["block_pair"], got["block_single"] = bp, bs
    dp, act, mask, sc, pc = G.diffusion_inputs(n, 100 + n + 1000)
    dt = gpu_pkg.nn.DiffusionTransformer(num_blocks=4, use_batch_infer=True)
    dt.load_state_dict(dp)
    dt.to(dev)
    got["diffusion_transformer"] = dt(act.to(dev).clone(), mask.to(dev), sc.to(dev), pc.to(dev))
    for k, w in want.items():
        e = rms_err(got[k].float().cpu(), w)
        print(f"golden n={n} {k}: rms err {e:.3e}", flush=True)
        assert e < 1e-2, (k, e)        # bf16 operands vs the float64 golden output


def load_file(name):
    return dict(np.load(os.path.join(HERE, "golden", name)))


def test_oracle_reproduces_golden_head_and_evoformer():
    for name, fn in (("diffusion_head_n8.npz", G.head_expected), ("evoformer_n12.npz", G.evoformer_expected)):
        want, got = load_file(name), fn()
        assert sorted(got) == sorted(want)
        for k in want:
            assert np.allclose(got[k], want[k], rtol=1e-5, atol=1e-5), (name, k)


@pytest.mark.gpu
def test_hip_head_matches_golden(gpu_pkg):
    want = load_file("diffusion_head_n8.npz")
    dev = torch.device("cuda:0")
    batch, params, emb, pos = G.head_inputs()
    head = gpu_pkg.nn.DiffusionHead(num_blocks=1)
    head.load_state_dict(params)
    head.to(dev)
    gb, ge = batch.to(dev), {k: v.to(dev) for k, v in emb.items()}
    sampler = gpu_pkg.nn.DiffusionSampler(head, diffusion_steps=6)
    _, t_hat, _ = sampler.schedule(dev)
    sc, pc = head.pre_conditioning(gb, ge, t_hat, True)
    got = {"single_cond": sc, "pair_cond": pc}
    am = batch.predicted_structure_info.atom_mask[None, ..., None]
    for step in (1, 4):
        t = t_hat[step]
        noisy = (pos * float(t)).to(dev)
        den = head(noisy, t, gb, ge, torch.as_tensor(want["single_cond"][step]).to(dev),
                   torch.as_tensor(want["pair_cond"]).to(dev))
        # compare the update: the skip term of the blend is the input itself
        skip = (256.0 / (float(t) ** 2 + 256.0)) * noisy.cpu() * am
        got[f"denoised_step{step}"] = den.cpu() - skip
        want[f"denoised_step{step}"] = want[f"denoised_step{step}"] - skip.numpy()
    for k, w in want.items():
        e = rms_err(got[k].float().cpu(), w)
        print(f"golden head {k}: rms err {e:.3e}", flush=True)
        assert e < 1e-2, (k, e)


@pytest.mark.gpu
def test_hip_evoformer_matches_golden(gpu_pkg):
    want = load_file("evoformer_n12.npz")
    dev = torch.device("cuda:0")
    params, msa, pair, mm, pm = G.evoformer_inputs()
    blk = gpu_pkg.nn.EvoformerBlock()
    blk.load_state_dict(params)
    blk.to(dev)
    m, z = blk(msa.to(dev).clone(), pair.to(dev).clone(), mm.to(dev), pm.to(dev))
    live = pm[..., None]
    for name, got, w, base, msk in (("msa", m, want["msa"], msa, 1.0), ("pair", z, want["pair"], pair, live)):
        e = rms_err((got.cpu() - base) * msk, (torch.as_tensor(w) - base) * msk)
        print(f"golden evoformer {name} update: rms err {e:.3e}", flush=True)
        assert e < 1e-2, (name, e)
