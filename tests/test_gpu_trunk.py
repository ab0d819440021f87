"""Evoformer trunk driver with recycling on the GPU against the float64 CPU
oracle (oracle/af3_trunk_oracle.py): 1 MSA block + 2 Pairformer blocks, two
recycles.  Tolerances on the live part of the outputs: fp32 check mode 2e-4 rms,
bf16 2e-2 rms (two passes through three blocks on bf16 residual streams)."""

import pytest
import torch

from oracle import af3_oracle as O
from oracle import af3_trunk_oracle as T

pytestmark = pytest.mark.gpu
D = torch.float64


def compare(name, got, ref, rms_tol, max_tol):
    got, ref = got.double().cpu(), ref.double().cpu()
    scale = float((ref ** 2).mean().sqrt())
    rms = float(((got - ref) ** 2).mean().sqrt()) / scale
    mx = float((got - ref).abs().max()) / scale
    print(f"trunk {name}: rms {rms:.3e} max {mx:.3e} (rms of reference {scale:.3e})", flush=True)
    assert torch.isfinite(got).all() and scale > 0
    assert rms <= rms_tol and mx <= max_tol, (name, rms, mx)


@pytest.mark.parametrize("n,rows", [(16, 6)])
def test_trunk_with_recycling_against_oracle(gpu_pkg, n, rows):
    dev = torch.device("cuda:0")
    g = torch.Generator().manual_seed(5)
    batch = gpu_pkg.nn.atom_layout.synthetic_trunk_batch(n, rows, g, n_padding_tokens=2, chain_len=5)
    p = {k: O.round_bf16(v) for k, v in T.make_evoformer_params(g, 1, 2, std=0.05).items()}
    tf = O.round_bf16(torch.randn(n, 447, generator=g))
    want = T.recycle(batch, tf.double(), O.cast_params(p, D), 2, 1, 2)
    mod = gpu_pkg.nn.Evoformer(msa_stack_num_layer=1, pairformer_num_layer=2)
    mod.load_state_dict(p)
    mod.to(dev)
    gb = batch.to(dev)
    mask = batch.token_features.mask
    live_p = (mask[:, None] * mask[None, :])[..., None]
    for mode, rms_tol, max_tol in (("check", 2e-4, 2e-3), ("bf16", 2e-2, 2e-1)):
        with gpu_pkg.nn.check_mode(mode == "check"):
            got = mod.recycle(gb, tf.to(dev), num_recycles=2)
        compare(f"pair after 2 recycles, {mode}", got["pair"].float().cpu() * live_p, want["pair"] * live_p, rms_tol, max_tol)
        compare(f"single after 2 recycles, {mode}", got["single"].float().cpu() * mask[:, None],
                want["single"] * mask[:, None], rms_tol, max_tol)
