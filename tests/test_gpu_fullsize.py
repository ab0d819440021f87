"""The headline size (768 tokens, 128 pair channels, 384 single channels), which
the float64 CPU oracle does not reach in seconds: properties that hold at any
size and that a dropped tile, a wrapped index or a wrong tile-to-workgroup map
would break.

  * relabelling the tokens relabels the outputs (every op on the path is
    equivariant under a token permutation applied to pair rows and columns,
    single rows and both masks);
  * on a symmetric pair tensor, triangle attention around the ending node is
    the transpose of triangle attention around the starting node (bias and mask
    are taken before the activations are transposed);
  * the bf16 MFMA block against the plain fp32 check kernels on the same GPU:
    rms error of the update <= 1e-2, the bf16 tolerance;
  * diffusion samples that start equal stay equal, and a permutation of the
    tokens permutes the diffusion transformer's output.

Sums are taken in a different order after a permutation, so equality is up to
bf16 operand rounding of intermediates: the tolerance is the same 1e-2 (rms of
the update) and 8e-2 (max over rms) as for the comparison with the check mode.
"""

import pytest
import torch

from oracle import af3_oracle as O

pytestmark = pytest.mark.gpu
N = 768
RMS_TOL, MAX_TOL = 1e-2, 8e-2


def dev():
    return torch.device("cuda:0")


def gen(seed):
    return torch.Generator().manual_seed(seed)


def rparams(p):
    return {k: O.round_bf16(v) for k, v in p.items()}


def compare(name, got, ref, rms_tol=RMS_TOL, max_tol=MAX_TOL):
    got, ref = got.double(), ref.double()
    scale = float((ref ** 2).mean().sqrt())
    rms = float(((got - ref) ** 2).mean().sqrt()) / scale
    mx = float((got - ref).abs().max()) / scale
    print(f"full size {name}: rms {rms:.3e} max {mx:.3e} (rms of reference {scale:.3e})", flush=True)
    assert torch.isfinite(got).all()
    assert scale > 0
    assert rms <= rms_tol and mx <= max_tol, (name, rms, mx)


def block_inputs(seed, live, trailing=False):
    g = gen(seed)
    p = rparams(O.make_pairformer_block_params(g))
    pair = O.round_bf16(torch.randn(N, N, 128, generator=g))
    single = O.round_bf16(torch.randn(N, 384, generator=g))
    seq = torch.ones(N)
    if trailing:
        # padding at the end: whole key tiles are masked (the attention core leaves them out)
        seq[live:] = 0
    else:
        # padding scattered over the sequence
        seq[torch.randperm(N, generator=g)[: N - live]] = 0
    pm = seq[:, None] * seq[None, :]
    return g, p, pair, single, seq, pm


def test_block_commutes_with_a_token_permutation(gpu_pkg):
    g, p, pair, single, seq, pm = block_inputs(11, 700)
    perm = torch.randperm(N, generator=g).to(dev())
    blk = gpu_pkg.nn.PairformerBlock()
    blk.load_state_dict(p)
    blk.to(dev())
    pair, single, seq, pm = (t.to(dev()) for t in (pair, single, seq, pm))
    op, os_ = blk(pair.clone(), pm, single.clone(), seq)
    pp = pair[perm][:, perm].contiguous()
    qp, qs = blk(pp.clone(), pm[perm][:, perm].contiguous(), single[perm].contiguous(), seq[perm].contiguous())
    live2 = pm[perm][:, perm].bool()[..., None]
    # padded rows and columns carry no information the reference defines
    compare("pair update under permutation", ((qp - pp) * live2).cpu(),
            ((op - pair)[perm][:, perm] * live2).cpu())
    live1 = seq[perm].bool()[:, None]
    compare("single update under permutation", ((qs - single[perm]) * live1).cpu(),
            ((os_ - single)[perm] * live1).cpu())


def test_ending_node_attention_is_starting_node_attention_of_the_transpose(gpu_pkg):
    """The reference takes the pair bias and the key mask before it transposes
    the activations (src/distributed_xfold/nn/d_attention.py:63 and :88-111),
    so for a SYMMETRIC pair tensor and any mask the ending-node update is the
    transpose of the starting-node update."""
    g = gen(12)
    p = rparams(O.make_grid_self_attention_params(g, std=0.05))
    half = torch.randn(N, N, 128, generator=g)
    pair = O.round_bf16((half + half.transpose(0, 1)) * 0.7071).to(dev())
    assert torch.equal(pair, pair.transpose(0, 1))
    mask = (torch.rand(N, N, generator=g) > 0.1).float()
    mask[:, 0] = 1
    mask = mask.to(dev())
    end = gpu_pkg.nn.GridSelfAttention(transpose=True)
    start = gpu_pkg.nn.GridSelfAttention(transpose=False)
    for m in (end, start):
        m.load_state_dict(p)
        m.to(dev())
    a = end(pair, mask)                       # the module returns the update; the block adds it
    b = start(pair, mask).transpose(0, 1)
    compare("ending node vs transposed starting node", a.cpu(), b.cpu())


@pytest.mark.parametrize("live,trailing", [(700, False), (600, True)])
def test_bf16_block_against_fp32_check_mode(gpu_pkg, live, trailing):
    g, p, pair, single, seq, pm = block_inputs(13, live, trailing)
    blk = gpu_pkg.nn.PairformerBlock()
    blk.load_state_dict(p)
    blk.to(dev())
    with gpu_pkg.nn.check_mode():
        cp, cs = blk(pair.to(dev()), pm.to(dev()), single.to(dev()), seq.to(dev()))
    bp, bs = blk(pair.to(dev()).clone(), pm.to(dev()), single.to(dev()).clone(), seq.to(dev()))
    compare("pair update, bf16 vs fp32 check", bp.cpu() - pair, cp.cpu() - pair)
    compare("single update, bf16 vs fp32 check", bs.cpu() - single, cs.cpu() - single)


def test_diffusion_transformer_samples_and_permutation(gpu_pkg):
    g = gen(14)
    nb, B = 4, 5
    p = rparams(O.make_diffusion_transformer_params(g, num_blocks=nb, std=0.05))
    one = O.round_bf16(torch.randn(1, N, 768, generator=g))
    act = one.expand(B, N, 768).contiguous().to(dev())
    s = O.round_bf16(torch.randn(N, 384, generator=g)).to(dev())
    pc = O.round_bf16(torch.randn(N, N, 128, generator=g)).to(dev())
    mask = torch.ones(N)
    mask[torch.randperm(N, generator=g)[:60]] = 0
    mask = mask.to(dev())
    perm = torch.randperm(N, generator=g).to(dev())
    mod = gpu_pkg.nn.DiffusionTransformer(num_blocks=nb, use_batch_infer=True)
    mod.load_state_dict(p)
    mod.to(dev())
    out = mod(act.clone(), mask, s, pc)
    for b in range(1, B):
        assert torch.equal(out[b], out[0]), f"sample {b} differs from sample 0 on equal inputs"
    out_p = mod(act[:, perm].contiguous(), mask[perm].contiguous(), s[perm].contiguous(),
                pc[perm][:, perm].contiguous())
    live = mask[perm].bool()[None, :, None]
    compare("diffusion transformer update under permutation", ((out_p - act[:, perm]) * live).cpu(),
            ((out - act)[:, perm] * live).cpu())


def test_attention_core_more_than_64_key_tiles(gpu_pkg):
    """N = 4160 = 65 key tiles of 64: the attention core keeps its live key
    tiles in a 64-bit mask and must fall back to plain order beyond that.  A few
    rows are checked against an fp32 softmax computed by torch on the GPU."""
    n = 4160
    d = dev()
    g = torch.Generator(device=d).manual_seed(5)
    rnd = lambda *shape: (torch.randn(*shape, generator=g, device=d) * 0.7).bfloat16()
    q, k = rnd(n, 4, n, 32), rnd(n, 4, n, 32)
    vt = rnd(n, 4, 32, n)
    bias = rnd(4, n, n)
    mask = (torch.rand(n, n, generator=g, device=d) > 0.2).float()
    mask[:, 0] = 1
    mask[11, :] = 0                                   # a fully masked row
    mask[:, n - 100:] = 0                             # trailing padding: the last key tile is masked as a whole
    og = gpu_pkg.ops.grid_attention_core(q, k, gpu_pkg.ops.pack_vt(vt), gpu_pkg.ops.pack_pair_bias(bias), mask)
    og = og.view(n, n, 4, 32)
    log2e = 1.4426950408889634
    for b in (0, 11, 2077, n - 1):
        logits = (torch.einsum("hqd,hkd->hqk", q[b].float(), k[b].float()) + bias.float()) / log2e
        logits = logits.masked_fill(mask[b][None, None, :] == 0, -1e9)
        want = torch.einsum("hqk,hdk->hqd", torch.softmax(logits, -1), vt[b].float())
        # (a missing key tile would show as an error of the order of the output itself)
        compare(f"attention core N={n}, row {b}", og[b].permute(1, 0, 2).float().cpu(), want.cpu(),
                rms_tol=5e-3, max_tol=MAX_TOL)
