"""Pairformer block on 64 pair channels (factor 2, no single track), the
configuration of the template embedding's blocks (nn/d_template.py:198-201),
and its operators, against the float64 CPU oracle.  These widths run as
separate launches of the general kernels (LayerNorm, dense product, batched
contraction, pair-biased attention with head dim 16).

Tolerances on the update: fp32 check mode 2e-4 rms / 2e-3 max, bf16 1e-2 / 8e-2."""

import pytest
import torch

from oracle import af3_oracle as O

pytestmark = pytest.mark.gpu
D = torch.float64
MODES = (("check", 2e-4, 2e-3), ("bf16", 1e-2, 8e-2))


def dev():
    return torch.device("cuda:0")


def compare(name, got, ref, rms_tol, max_tol):
    got, ref = got.double().cpu(), ref.double().cpu()
    scale = float((ref ** 2).mean().sqrt())
    rms = float(((got - ref) ** 2).mean().sqrt()) / scale
    mx = float((got - ref).abs().max()) / scale
    print(f"c=64 {name}: rms {rms:.3e} max {mx:.3e} (rms of reference {scale:.3e})", flush=True)
    assert torch.isfinite(got).all() and scale > 0
    assert rms <= rms_tol and mx <= max_tol, (name, rms, mx)


def masks(n, g):
    seq = torch.ones(n)
    seq[n - 3:] = 0
    pm = seq[:, None] * seq[None, :] * (torch.rand(n, n, generator=g) > 0.15).float()
    pm[:, 0] = 1
    return seq, pm


@pytest.mark.parametrize("n", [19, 70])
def test_operators_on_64_channels(gpu_pkg, n):
    g = torch.Generator().manual_seed(100 + n)
    rb = O.round_bf16
    pair = rb(torch.randn(n, n, 64, generator=g))
    seq, pm = masks(n, g)
    t = lambda x: x.to(dev())
    for outgoing in (True, False):
        p = {k: rb(v) for k, v in O.make_triangle_multiplication_params(g, 64, std=0.1).items()}
        mod = gpu_pkg.nn.TriangleMultiplication(c_pair=64, _outgoing=outgoing)
        mod.load_state_dict(p)
        mod.to(dev())
        want = O.triangle_multiplication(pair.double(), pm.double(), O.cast_params(p, D), outgoing)
        for mode, rms_tol, max_tol in MODES:
            with gpu_pkg.nn.check_mode(mode == "check"):
                compare(f"trimul[{'out' if outgoing else 'in'}] n={n} {mode}", mod(t(pair), t(pm)), want, rms_tol, max_tol)
    for transpose in (False, True):
        p = {k: rb(v) for k, v in O.make_grid_self_attention_params(g, 64, 4, std=0.1).items()}
        mod = gpu_pkg.nn.GridSelfAttention(c_pair=64, num_head=4, transpose=transpose)
        mod.load_state_dict(p)
        mod.to(dev())
        want = O.grid_self_attention(pair.double(), pm.double(), O.cast_params(p, D), 4, transpose)
        for mode, rms_tol, max_tol in MODES:
            with gpu_pkg.nn.check_mode(mode == "check"):
                compare(f"triattn[{'end' if transpose else 'start'}] n={n} {mode}", mod(t(pair), t(pm)), want,
                        rms_tol, max_tol)


@pytest.mark.parametrize("n", [24, 130])
def test_block_on_64_channels(gpu_pkg, n):
    g = torch.Generator().manual_seed(200 + n)
    rb = O.round_bf16
    p = {k: rb(v) for k, v in O.make_pairformer_block_params(g, c_pair=64, factor=2, with_single=False,
                                                             std=0.05).items()}
    pair = rb(torch.randn(n, n, 64, generator=g))
    seq, _ = masks(n, g)
    pm = seq[:, None] * seq[None, :]
    blk = gpu_pkg.nn.PairformerBlock(c_pair=64, num_intermediate_factor=2, with_single=False)
    blk.load_state_dict(p)
    blk.to(dev())
    want = O.pairformer_block(pair.double(), pm.double(), None, None, O.cast_params(p, D), with_single=False)
    want = want[0] if isinstance(want, tuple) else want
    live = pm[..., None]
    for mode, rms_tol, max_tol in MODES:
        with gpu_pkg.nn.check_mode(mode == "check"):
            got = blk(pair.to(dev()).clone(), pm.to(dev()))
        got = got[0] if isinstance(got, tuple) else got
        compare(f"block update n={n} {mode}", (got.cpu() - pair) * live, (want - pair.double()) * live, rms_tol, max_tol)
    got = blk(pair.to(dev()).bfloat16(), pm.to(dev()))
    assert got.dtype == torch.bfloat16
    compare(f"block update n={n}, bf16 stream", (got.float().cpu() - pair) * live, (want - pair.double()) * live,
            3e-2, 3e-1)
