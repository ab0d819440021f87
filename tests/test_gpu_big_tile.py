"""GPU parity of the dense projections at sizes that take the 256x256-tile
kernel (at least 120 such tiles, in one round of the 256 CUs or more): plain / bias / scale / sigmoid, SwiGLU, the
regrouped store and the segmented q-k-v-gate projection of the diffusion
self-attention, against float64 products of the same bf16 operands.  Ragged
M (not a multiple of 256), N (a partial last tile) and K (not a multiple of
the 32-deep slab) are part of every case; the cases of more than 256 tiles make
some of the kernel's persistent workgroups walk on to a second tile."""

import pytest
import torch

from oracle import af3_oracle as O

pytestmark = pytest.mark.gpu


def dev():
    return torch.device("cuda:0")


def gen(seed):
    return torch.Generator().manual_seed(seed)


def within_bf16_ulp(name, got, want, ulps=1.01, atol=1e-4):
    got, want = got.detach().double().cpu(), want.double()
    bad = (got - want).abs() > ulps * 2.0 ** -8 * want.abs() + atol
    assert not bad.any(), f"{name}: {int(bad.sum())} elements beyond {ulps} bf16 ulp"


# (the launcher takes blocks of 192 rows where they need no more rounds of workgroups than blocks of 256; the
# last case is one round of 240 blocks of 256 rows against two rounds of 192-row ones, so it keeps the 256-row
# instance of the column epilogue covered)
@pytest.mark.parametrize("m,n,k", [(3850, 2824, 200), (4096, 2560, 768), (5000, 3400, 72), (4096, 3840, 136)])
def test_linear_bias_scale_sigmoid(gpu_pkg, m, n, k):
    print(f"test_linear_bias_scale_sigmoid m={m} n={n} k={k}", flush=True)
    g = gen(m + n + k)
    x, w = O.round_bf16(torch.randn(m, k, generator=g)), O.round_bf16(torch.randn(n, k, generator=g) * 0.1)
    b = torch.randn(n, generator=g)
    xd, wd = x.to(dev()).bfloat16(), w.to(dev()).bfloat16()
    y = x.double() @ w.double().T
    got = gpu_pkg.ops.linear(xd, wd)
    within_bf16_ulp("plain", got, y)
    got = gpu_pkg.ops.linear(xd, wd, bias=b.to(dev()), alpha=0.5)
    within_bf16_ulp("bias, scale", got, (y + b.double()) * 0.5)
    got = gpu_pkg.ops.linear(xd, wd, sigmoid=True)
    within_bf16_ulp("sigmoid", got, torch.sigmoid(y))
    # the same products from the 128x128-tile kernel (fp32 output is not a large-tile case)
    ref = gpu_pkg.ops.linear(xd, wd, bias=b.to(dev()), alpha=0.5, out_dtype=torch.float32)
    got = gpu_pkg.ops.linear(xd, wd, bias=b.to(dev()), alpha=0.5)
    assert torch.equal(got, ref.bfloat16()) or float((got.float() - ref).abs().max()) <= 2.0 ** -7 * float(ref.abs().max())


# N = 2 hidden: 11.25 / 13.5 / 15 tiles (the last on blocks of 256 rows, the others on blocks of 192)
@pytest.mark.parametrize("m,k,hidden", [(3850, 264, 1440), (5000, 104, 1728), (4096, 104, 1920)])
def test_linear_swiglu(gpu_pkg, m, k, hidden):
    print(f"test_linear_swiglu (large tile) m={m} k={k} hidden={hidden}", flush=True)
    from distributed_xfold_amd.nn.base import pack_swiglu
    g = gen(11)
    x = O.round_bf16(torch.randn(m, k, generator=g))
    w1 = O.round_bf16(torch.randn(2 * hidden, k, generator=g) * 0.1)
    h = gpu_pkg.ops.linear(x.to(dev()).bfloat16(), pack_swiglu(w1, 32).to(dev()).bfloat16(),
                           mode=gpu_pkg.lib.LINEAR_SWIGLU)
    y = x.double() @ w1.double().T
    within_bf16_ulp("swiglu", h, torch.nn.functional.silu(y[:, :hidden]) * y[:, hidden:])


@pytest.mark.parametrize("m,n,k", [(3872, 2720, 136), (6400, 3072, 40)])   # 176 tiles; 300: some workgroups take two
def test_linear_regrouped_store(gpu_pkg, m, n, k):
    print(f"test_linear_regrouped_store (large tile) m={m} n={n} k={k}", flush=True)
    g = gen(12)
    x, w = O.round_bf16(torch.randn(m, k, generator=g)), O.round_bf16(torch.randn(n, k, generator=g) * 0.1)
    got = gpu_pkg.ops.linear(x.to(dev()).bfloat16(), w.to(dev()).bfloat16(), mode=gpu_pkg.lib.LINEAR_REGROUP32)
    y = x.double() @ w.double().T
    want = y.reshape(m // 32, 32, n // 32, 32).permute(0, 2, 1, 3).reshape(-1, 1024)
    assert got.shape == want.shape
    within_bf16_ulp("regroup32", got, want)


def test_self_attention_projection_segments(gpu_pkg):
    """Five samples of 768 tokens send the q-k-v-gate projection (scaled and
    biased queries, plain keys and values, sigmoid gates) to the large tile; one
    sample alone goes through the 128x128-tile kernel.  Attention treats the
    samples independently, so the two must agree to the rounding of the bf16
    intermediates."""
    print("test_self_attention_projection_segments", flush=True)
    g = gen(13)
    b, s, c, h = 5, 768, 768, 16
    x = torch.randn(b, s, c, generator=g).to(dev()).bfloat16()
    w = (torch.randn(4 * c, c, generator=g) * 0.05).to(dev()).bfloat16()
    qb = torch.randn(c, generator=g).to(dev())
    mask = (torch.arange(s) < 700).float().to(dev())
    logits = torch.randn(h, s, s, generator=g).to(dev())
    full = gpu_pkg.ops.batch_diffusion_self_attention(x, mask, logits, w, qb, h, out_dtype=torch.float32)
    for i in (0, 4):
        one = gpu_pkg.ops.batch_diffusion_self_attention(x[i:i + 1].contiguous(), mask, logits, w, qb, h,
                                                         out_dtype=torch.float32)
        d = (full[i] - one[0]).double()
        rms = float(one.double().pow(2).mean().sqrt())
        e_max, e_rms = float(d.abs().max()) / rms, float(d.pow(2).mean().sqrt()) / rms
        print(f"  sample {i}: large tile vs 128 tile max {e_max:.3e} rms {e_rms:.3e}", flush=True)
        assert e_rms < 3e-3 and e_max < 5e-2
    # and against the float64 formula on the first sample, with the projections
    # rounded to bf16 where the kernel stores them
    xd, wd = x[0].double().cpu(), w.double().cpu()

    def r(t):
        return O.round_bf16(t.float()).double()
    q = r((xd @ wd[:c].T + qb.double().cpu()) / (c // h) ** 0.5).reshape(s, h, -1)
    k = r(xd @ wd[c:2 * c].T).reshape(s, h, -1)
    v = r(xd @ wd[2 * c:3 * c].T).reshape(s, h, -1)
    gate = r(torch.sigmoid(xd @ wd[3 * c:].T)).reshape(s, h, -1)
    lg = torch.einsum("qhd,khd->hqk", q, k) + logits.double().cpu() + (mask.double().cpu() - 1.0) * 1e9
    want = torch.einsum("hqk,khd->qhd", torch.softmax(lg, -1), v) * gate
    e = O.rel_err(full[0].cpu(), want)
    print(f"  vs float64: rel err {e:.3e}", flush=True)
    assert e < 2e-2


@pytest.mark.parametrize("b,s,c,h", [(5, 768, 768, 16), (2, 100, 128, 4), (1, 36, 64, 4)])
def test_quad_major_bias_is_bit_identical(gpu_pkg, b, s, c, h):
    """The pair bias given with quads of four keys as the outer index changes
    which addresses the attention kernel loads, not what it computes."""
    print(f"test_quad_major_bias_is_bit_identical b={b} s={s} c={c} h={h}", flush=True)
    g = gen(s)
    x = torch.randn(b, s, c, generator=g).to(dev()).bfloat16()
    w = (torch.randn(4 * c, c, generator=g) * 0.05).to(dev()).bfloat16()
    mask = (torch.arange(s) < s - 3).float().to(dev())
    logits = torch.randn(h, s, s, generator=g).to(dev())
    want = gpu_pkg.ops.batch_diffusion_self_attention(x, mask, logits, w, None, h, out_dtype=torch.float32)
    got = gpu_pkg.ops.batch_diffusion_self_attention(x, mask, gpu_pkg.ops.quad_major_bias(logits), w, None, h,
                                                     out_dtype=torch.float32)
    assert torch.equal(got, want)
