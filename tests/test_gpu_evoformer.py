"""Evoformer (MSA) block on the GPU against the float64 CPU oracle
(oracle/af3_msa_oracle.py) at small sizes, and the bf16 path against the fp32
check mode at 768 tokens x 512 MSA rows.

Tolerances: fp32 check mode 2e-4 rms / 2e-3 max of the update; bf16 path
1e-2 rms / 8e-2 max."""

import pytest
import torch

from oracle import af3_msa_oracle as M
from oracle import af3_oracle as O

pytestmark = pytest.mark.gpu
D = torch.float64


def dev():
    return torch.device("cuda:0")


def gen(seed):
    return torch.Generator().manual_seed(seed)


def compare(name, got, ref, rms_tol, max_tol):
    got, ref = got.double().cpu(), ref.double().cpu()
    scale = float((ref ** 2).mean().sqrt())
    rms = float(((got - ref) ** 2).mean().sqrt()) / scale
    mx = float((got - ref).abs().max()) / scale
    print(f"evoformer {name}: rms {rms:.3e} max {mx:.3e} (rms of reference {scale:.3e})", flush=True)
    assert torch.isfinite(got).all() and scale > 0
    assert rms <= rms_tol and mx <= max_tol, (name, rms, mx)


def inputs(a, n, seed, std=0.05):
    g = gen(seed)
    rb = O.round_bf16
    p = {k: rb(v) for k, v in M.make_evoformer_block_params(g, std=std).items()}
    msa = rb(torch.randn(a, n, 64, generator=g))
    pair = rb(torch.randn(n, n, 128, generator=g))
    mm = (torch.rand(a, n, generator=g) > 0.15).float()
    mm[0] = 1
    mm[:, n - 2:] = 0                      # trailing padding tokens
    seq = mm.max(dim=0).values
    pm = seq[:, None] * seq[None, :] * (torch.rand(n, n, generator=g) > 0.1).float()
    pm[:, 0] = 1
    return g, p, msa, pair, mm, pm


MODES = (("check", 2e-4, 2e-3), ("bf16", 1e-2, 8e-2))


@pytest.mark.parametrize("a,n", [(5, 12), (37, 45), (16, 24)])   # the last one takes the transposed-operand paths
def test_msa_operators_against_oracle(gpu_pkg, a, n):
    g, p, msa, pair, mm, pm = inputs(a, n, 70 + n)
    pd = O.cast_params(p, D)
    want_opm = M.outer_product_mean(msa.double(), mm.double(), O._sub(pd, "outer_product_mean"))
    want_att = M.msa_attention(msa.double(), mm.double(), pair.double(), O._sub(pd, "msa_attention1"))
    opm = gpu_pkg.nn.OuterProductMean()
    opm.load_state_dict(O._sub(p, "outer_product_mean"))
    att = gpu_pkg.nn.MSAAttention()
    att.load_state_dict(O._sub(p, "msa_attention1"))
    opm.to(dev())
    att.to(dev())
    t = lambda x: x.to(dev())
    for mode, rms_tol, max_tol in MODES:
        with gpu_pkg.nn.check_mode(mode == "check"):
            # pairs that no MSA row covers hold bias / epsilon, a thousand times the rest: compare the covered ones
            cover = ((mm.t() @ mm) > 0)[..., None]
            compare(f"outer product mean {mode}", opm(t(msa), t(mm)).cpu() * cover, want_opm * cover, rms_tol, max_tol)
            compare(f"outer product mean, uncovered pairs, {mode}", opm(t(msa), t(mm)).cpu() * ~cover,
                    want_opm * ~cover, 1e-6 if mode == "check" else 4e-3, 1e-5 if mode == "check" else 8e-3)
            compare(f"msa attention {mode}", att(t(msa), t(mm), t(pair)), want_att, rms_tol, max_tol)


@pytest.mark.parametrize("a,n", [(6, 17), (20, 40), (8, 16)])
def test_evoformer_block_against_oracle(gpu_pkg, a, n):
    g, p, msa, pair, mm, pm = inputs(a, n, 80 + n)
    pd = O.cast_params(p, D)
    want_msa, want_pair = M.evoformer_block(msa.double(), pair.double(), mm.double(), pm.double(), pd)
    blk = gpu_pkg.nn.EvoformerBlock()
    blk.load_state_dict(p)
    blk.to(dev())
    t = lambda x: x.to(dev())
    live_m = mm[..., None]
    live_p = (pm.max(dim=1).values[:, None] * pm.max(dim=0).values[None, :])[..., None]
    for mode, rms_tol, max_tol in MODES:
        with gpu_pkg.nn.check_mode(mode == "check"):
            got_msa, got_pair = blk(t(msa).clone(), t(pair).clone(), t(mm), t(pm))
        # the MSA update of every entry is defined (a masked key never contributes); padded pair rows carry no information
        compare(f"msa update {mode}", got_msa.cpu() - msa, want_msa - msa.double(), rms_tol, max_tol)
        compare(f"pair update {mode}", (got_pair.cpu() - pair) * live_p, (want_pair - pair.double()) * live_p,
                rms_tol, max_tol)
    # bf16 residual streams
    got_msa, got_pair = blk(t(msa).bfloat16(), t(pair).bfloat16(), t(mm), t(pm))
    assert got_msa.dtype == torch.bfloat16 and got_pair.dtype == torch.bfloat16
    compare("pair update, bf16 stream", (got_pair.float().cpu() - pair) * live_p, (want_pair - pair.double()) * live_p,
            2e-2, 2e-1)


def test_full_size_block_against_check_mode(gpu_pkg):
    a, n = 512, 768
    g, p, msa, pair, mm, pm = inputs(a, n, 90, std=0.02)
    blk = gpu_pkg.nn.EvoformerBlock()
    blk.load_state_dict(p)
    blk.to(dev())
    t = lambda x: x.to(dev())
    with gpu_pkg.nn.check_mode():
        want_opm = blk.outer_product_mean(t(msa), t(mm))
        want_att = blk.msa_attention1(t(msa), t(mm), t(pair))
    compare("outer product mean, bf16 vs fp32 check", blk.outer_product_mean(t(msa), t(mm)), want_opm, 1e-2, 8e-2)
    compare("msa attention, bf16 vs fp32 check", blk.msa_attention1(t(msa), t(mm), t(pair)), want_att, 1e-2, 8e-2)
    got_msa, got_pair = blk(t(msa).clone(), t(pair).clone(), t(mm), t(pm))
    assert torch.isfinite(got_msa).all() and torch.isfinite(got_pair).all()


@pytest.mark.parametrize("rows,cols", [(8, 8), (72, 200), (64, 4096), (1000, 24)])
def test_transpose_is_exact(gpu_pkg, rows, cols):
    x = torch.randn(rows, cols, generator=gen(rows + cols)).bfloat16().to(dev())
    y = gpu_pkg.ops.transpose2d(x)
    assert y.shape == (cols, rows) and torch.equal(y, x.t().contiguous())
    with pytest.raises(ValueError):
        gpu_pkg.ops.transpose2d(x[:, :cols - 1].contiguous() if cols > 8 else x[:7].contiguous())
