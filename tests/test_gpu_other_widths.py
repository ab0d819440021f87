"""Pairformer block on 64 pair channels (factor 2, no single track), the
configuration of the template embedding's blocks (nn/d_template.py:198-201),
and its operators, against the float64 CPU oracle.  Widths below 128 (a
multiple of 8; four attention heads of at most 32) run on the fused 128-channel
kernels over zero-padded operands (`af3_*_forward_padded`); anything else
(more than 128 channels, other head counts) runs as separate launches of the
general kernels, which the last test keeps exercised.

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


def test_transition_on_64_channels(gpu_pkg):
    g = torch.Generator().manual_seed(300)
    rb = O.round_bf16
    for factor in (2, 3, 4):                           # hidden 128, 192 (padded to 256 inside), 256
        p = {k: rb(v) for k, v in O.make_transition_params(g, 64, factor, std=0.1).items()}
        x = rb(torch.randn(70, 70, 64, generator=g))
        mod = gpu_pkg.nn.Transition(c_x=64, num_intermediate_factor=factor)
        mod.load_state_dict(p)
        mod.to(dev())
        assert mod.padded
        want = O.transition(x.double(), O.cast_params(p, D))
        compare(f"transition factor {factor}", mod(x.to(dev())), want, 1e-2, 8e-2)
        res = x.to(dev()).bfloat16()
        mod.run(res, residual=True)                    # in place on the caller's 64-channel tensor
        compare(f"transition factor {factor}, residual", res.float().cpu() - x, want, 2e-2, 2e-1)


def test_padded_operators_with_all_128_channels_real_change_no_bit(gpu_pkg):
    """`valid_channels = 128` through the padded entry points is the un-suffixed entry point."""
    g = torch.Generator().manual_seed(301)
    n = 70
    mod = gpu_pkg.nn.TriangleMultiplication(c_pair=128)
    att = gpu_pkg.nn.GridSelfAttention(c_pair=128, num_head=4, transpose=True)
    for m in (mod, att):
        for prm in m.parameters():
            prm.data.normal_(0.0, 0.1, generator=g)
        m.to(dev())
    pair = torch.randn(n, n, 128, generator=g).bfloat16().to(dev())
    _, pm = masks(n, g)
    pm = pm.to(dev())
    lib, ops = gpu_pkg.lib.load(), gpu_pkg.ops
    p = mod.packed()
    a = ops.triangle_multiplication(pair, pm, 0, p["ln_in_w"], p["ln_in_b"], p["w_proj_gate"], p["ln_c_w"], p["ln_c_b"],
                                    p["w_out"], p["w_gl"])
    out = torch.empty_like(pair)
    ws = torch.empty(lib.af3_triangle_multiplication_workspace_bytes(n), dtype=torch.uint8, device=dev())
    ptr = lambda t_: t_.data_ptr()
    rc = lib.af3_triangle_multiplication_forward_padded(
        ptr(pair), 0, ptr(pm), 0, ptr(p["ln_in_w"]), ptr(p["ln_in_b"]), ptr(p["w_proj_gate"]), ptr(p["ln_c_w"]),
        ptr(p["ln_c_b"]), ptr(p["w_out"]), ptr(p["w_gl"]), ptr(out), 0, n, 128, ptr(ws), ws.numel(),
        torch.cuda.current_stream().cuda_stream)
    assert rc == 0
    assert torch.equal(a, out), int((a != out).sum())
    q = att.packed()
    b = ops.grid_self_attn(pair, pm, True, q["ln_w"], q["ln_b"], q["w_bias"], None, q["w_qkvg"], q["w_out"], 4)
    ws = torch.empty(lib.af3_grid_self_attn_workspace_bytes(n, 4), dtype=torch.uint8, device=dev())
    rc = lib.af3_grid_self_attn_forward_padded(
        ptr(pair), 0, ptr(pm), 1, ptr(q["ln_w"]), ptr(q["ln_b"]), ptr(q["w_bias"]), None, ptr(q["w_qkvg"]),
        ptr(q["w_out"]), 4, ptr(out), 0, n, 128, ptr(ws), ws.numel(), torch.cuda.current_stream().cuda_stream)
    assert rc == 0
    # (n = 70, transposed: the last block of 32 queries is partly filled; what the padding lanes compute
    # must not decide anything for the real ones)
    assert torch.equal(b, out), int((b != out).sum())


def test_general_kernels_for_other_shapes(gpu_pkg):
    """What the padded route does not take: triangle attention with two heads of 48 on 96 channels."""
    g = torch.Generator().manual_seed(302)
    rb = O.round_bf16
    n = 40
    pair = rb(torch.randn(n, n, 96, generator=g))
    _, pm = masks(n, g)
    for transpose in (False, True):
        p = {k: rb(v) for k, v in O.make_grid_self_attention_params(g, 96, 2, std=0.1).items()}
        mod = gpu_pkg.nn.GridSelfAttention(c_pair=96, num_head=2, transpose=transpose)
        mod.load_state_dict(p)
        mod.to(dev())
        assert not mod.padded and not mod.fused
        want = O.grid_self_attention(pair.double(), pm.double(), O.cast_params(p, D), 2, transpose)
        compare(f"triattn 96 channels, 2 heads, transpose={transpose}", mod(pair.to(dev()), pm.to(dev())), want,
                1e-2, 8e-2)
