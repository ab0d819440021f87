"""The reference's operators under their own names (`torch.ops._alpha_attention.*`,
Alpha_Attention.cpp:181-211) with GPU kernels from this library.

CPU part: the five schemas are defined with the reference's strings, the shape
functions answer FakeTensor calls.  GPU part: every operator is called the way the
reference's call sites call it (operands as `load_xsmm_params()` leaves them) and
checked against the float64 oracle in the same operand layout
(`oracle.gating_attention` restates the eager `Net1` of
kernel_test/grid_self_attenion.py:61-95 and batch_diffusion_cross_attention.py:62-84).
Tolerances: bf16 operands, rms <= 1e-2 and max <= 6e-2 of the reference's rms."""

import pytest
import torch

from oracle import af3_oracle as O

D = torch.float64


def dev():
    return torch.device("cuda:0")


def compare(name, got, ref, rms_tol=1e-2, max_tol=6e-2):
    got, ref = got.double().cpu(), ref.double().cpu()
    scale = float((ref ** 2).mean().sqrt())
    rms = float(((got - ref) ** 2).mean().sqrt()) / scale
    mx = float((got - ref).abs().max()) / scale
    print(f"torch.ops {name}: rms {rms:.3e} max {mx:.3e}", flush=True)
    assert got.shape == ref.shape and torch.isfinite(got).all() and scale > 0
    assert rms <= rms_tol and mx <= max_tol, (name, rms, mx)


# ------------------------------------------------------------------ CPU: schemas and shape functions
def test_operators_are_defined_with_the_reference_schemas(pkg):
    from distributed_xfold_amd import torch_ops
    torch_ops.register()
    torch_ops.register()                                   # idempotent
    ns = torch.ops._alpha_attention
    for name, schema in torch_ops.SCHEMAS.items():
        op = getattr(ns, name).default
        text = str(op._schema)
        assert text.startswith(f"_alpha_attention::{name}(")
        # argument names and order as in Alpha_Attention.cpp
        want = [a.strip().split(" ")[-1] for a in schema[schema.index("(") + 1:schema.index(")")].split(",")]
        assert [a.name for a in op._schema.arguments] == want
    assert sorted(torch_ops.SCHEMAS) == sorted([
        "grid_self_attn_forward", "transition_forward", "batch_diffusion_self_attention_forward",
        "batch_diffusion_cross_attention_forward", "traingle_multiplication_forward"])


def test_shape_functions_under_fake_tensors(pkg):
    from torch._subclasses.fake_tensor import FakeTensorMode
    from distributed_xfold_amd import torch_ops
    torch_ops.register()
    ns = torch.ops._alpha_attention
    with FakeTensorMode():
        bf = lambda *s: torch.empty(*s, dtype=torch.bfloat16)
        f = lambda *s: torch.empty(*s)
        out = ns.grid_self_attn_forward(bf(70, 70, 128), f(70, 1, 1, 70), f(4, 70, 70), bf(128, 4, 32), bf(128, 4, 32),
                                        bf(128, 4, 32), bf(128, 4, 32), bf(4, 32, 128), 32, 32)
        assert out.shape == (70, 70, 128) and out.dtype == torch.bfloat16
        out = ns.traingle_multiplication_forward(bf(70, 70, 128), f(70, 70, 1), 0, bf(128), bf(128), bf(256, 128),
                                                 bf(256, 128), bf(128), bf(128), bf(128, 128), bf(128, 128))
        assert out.shape == (70, 70, 128)
        out = ns.batch_diffusion_self_attention_forward(bf(5, 70, 768), f(5, 1, 1, 70), f(16, 70, 70),
                                                        bf(768, 16, 48), f(16, 48), bf(768, 16, 48), bf(768, 16, 48),
                                                        bf(768, 16, 48), 48, 48)
        assert out.shape == (5, 70, 16, 48)
        out = ns.batch_diffusion_cross_attention_forward(f(9, 32, 128), f(9, 128, 128), f(9, 4, 32, 128),
                                                         f(128, 4, 32), f(4, 32), f(128, 4, 32), f(128, 4, 32),
                                                         f(128, 4, 32), 32, 32)
        assert out.shape == (9, 32, 4, 32) and out.dtype == torch.float32
        out = ns.transition_forward(bf(70, 70, 128), bf(128, 1024), f(512, 128), bf(128), bf(128))
        assert out.shape == (70, 70, 128)


def test_repacked_weights_follow_their_source_tensor(pkg):
    """The repacked form of a weight is reused only for the same, unmodified tensor object: another
    tensor that happens to get a freed one's address, or an in-place update, must be repacked."""
    from distributed_xfold_amd import torch_ops
    a = torch.ones(8, dtype=torch.bfloat16)
    first = torch_ops._f32(a)
    assert torch_ops._f32(a) is first
    a.add_(1)
    second = torch_ops._f32(a)
    assert second is not first and float(second[0]) == 2.0
    seen = set()
    for i in range(50):                       # fresh tensors, some of them at recycled addresses
        t = torch.full((8,), float(i), dtype=torch.bfloat16)
        seen.add(t.data_ptr())
        assert float(torch_ops._f32(t)[0]) == float(i)
        del t
    assert len(seen) < 50


def test_cache_entries_are_per_role_and_survive_inference_mode(pkg):
    """One tensor that reaches two builders gets one entry per builder (an fp32 copy is not a bf16 copy),
    and tensors made under torch.inference_mode(), which have no version counter, are simply not cached."""
    from distributed_xfold_amd import torch_ops
    torch_ops.clear_cache()
    a = torch.arange(8, dtype=torch.float64)
    f, b = torch_ops._f32(a), torch_ops._bf16(a)
    assert f.dtype == torch.float32 and b.dtype == torch.bfloat16
    assert torch_ops._f32(a) is f and torch_ops._bf16(a) is b
    with torch.inference_mode():
        t = torch.ones(8, dtype=torch.bfloat16)
        got = torch_ops._f32(t)
        assert got.dtype == torch.float32 and float(got.sum()) == 8.0
        assert torch_ops._key_mask(torch.zeros(1, 1, 1, 4), 2, 4).shape == (2, 4)


def test_operator_bias_must_be_a_key_mask(pkg):
    """The operators' `bias` argument is the additive key mask 1e9 * (mask - 1) (Alpha_Attention.cpp:182-185,
    built at d_attention.py:63 and d_diffusion_transformer.py:206).  The kernels take it as a 0/1 mask; any
    other additive value would be dropped, so it is refused instead."""
    from distributed_xfold_amd import torch_ops
    mask = torch.tensor([[1., 1., 0., 1.], [0., 1., 1., 1.]])
    bias = (1e9 * (mask - 1))[:, None, None, :]
    assert torch.equal(torch_ops._key_mask(bias, 2, 4), mask)
    assert torch.equal(torch_ops._key_mask(bias.bfloat16(), 2, 4), mask)          # -1e9 as bf16 rounds it
    assert torch.equal(torch_ops._key_mask(bias[:1], 3, 4), mask[:1].expand(3, 4))
    for bad in (bias + 0.5, bias * 0.5, torch.full((2, 1, 1, 4), -3.0)):
        with pytest.raises(ValueError, match="key-mask form"):
            torch_ops._key_mask(bad, 2, 4)
    with pytest.raises(ValueError, match="expected"):
        torch_ops._key_mask(bias, 3, 4)


# ------------------------------------------------------------------ GPU: the operators as the reference calls them
gpu = pytest.mark.gpu


def _chd(weight, heads):
    """nn.Linear weight [heads * d, c] -> the operator's [c, heads, d] (d_attention.py:42-43)."""
    return weight.t().reshape(weight.shape[1], heads, -1).contiguous()


@gpu
@pytest.mark.parametrize("n,outgoing", [(70, True), (70, False), (200, True)])
def test_traingle_multiplication_forward(gpu_pkg, n, outgoing):
    from distributed_xfold_amd import torch_ops
    torch_ops.register()
    g = torch.Generator().manual_seed(500 + n)
    rb = O.round_bf16
    p = {k: rb(v) for k, v in O.make_triangle_multiplication_params(g, 128, std=0.1).items()}
    pair = rb(torch.randn(n, n, 128, generator=g))
    mask = (torch.rand(n, n, generator=g) > 0.15).float()
    want = O.triangle_multiplication(pair.double(), mask.double(), O.cast_params(p, D), outgoing)
    t = lambda x, dt=torch.bfloat16: x.to(dev()).to(dt)
    # d_triangle_multiplication.py:125-139: de-interleaved projection / gate rows, everything bf16
    deint = lambda w: torch.cat((w[::2], w[1::2]), 0)
    got = torch.ops._alpha_attention.traingle_multiplication_forward(
        t(pair), t(mask[..., None], torch.float32), 0 if outgoing else 1, t(p["left_norm_input.weight"]),
        t(p["left_norm_input.bias"]), t(deint(p["projection.weight"])), t(deint(p["gate.weight"])),
        t(p["center_norm.weight"]), t(p["center_norm.bias"]), t(p["output_projection.weight"]),
        t(p["gating_linear.weight"]))
    assert got.dtype == torch.bfloat16
    compare(f"traingle_multiplication_forward n={n} outgoing={outgoing}", got, want)


@gpu
@pytest.mark.parametrize("n,transpose", [(70, False), (70, True), (200, False)])
def test_grid_self_attn_forward(gpu_pkg, n, transpose):
    """As DistributeGridSelfAttention.xsmm_forward (d_attention.py:58-85) calls it: LayerNorm and
    pair-bias projection outside, the tensor permuted for the ending node."""
    from distributed_xfold_amd import torch_ops
    torch_ops.register()
    g = torch.Generator().manual_seed(600 + n + int(transpose))
    rb = O.round_bf16
    p = {k: rb(v) for k, v in O.make_grid_self_attention_params(g, 128, 4, std=0.1).items()}
    pair = rb(torch.randn(n, n, 128, generator=g))
    mask = (torch.rand(n, n, generator=g) > 0.15).float()
    mask[:, 0] = 1
    x = rb(O.layer_norm(pair, p["act_norm.weight"], p["act_norm.bias"]))
    nb = O.linear(x, p["pair_bias_projection.weight"]).permute(2, 0, 1).contiguous()
    bias = 1e9 * (mask[:, None, None, :] - 1)
    q_data = x.permute(1, 0, 2).contiguous() if transpose else x
    w = [_chd(p[f"{k}.weight"], 4) for k in ("q_projection", "k_projection", "v_projection", "gating_query")]
    w_out = p["output_projection.weight"].t().reshape(4, 32, 128).contiguous()
    want = O.gating_attention(q_data.double(), q_data.double(), bias.double(), nb.double(),
                              *[t.double() for t in w], output_w=w_out.double())
    t = lambda x_, dt=torch.bfloat16: x_.to(dev()).to(dt)
    got = torch.ops._alpha_attention.grid_self_attn_forward(
        t(q_data), t(bias, torch.float32), t(nb, torch.float32), *[t(x_) for x_ in w], t(w_out), 32, 32)
    compare(f"grid_self_attn_forward n={n} transpose={transpose}", got, want)


@gpu
@pytest.mark.parametrize("b,s,c,h", [(3, 130, 768, 16), (1, 200, 384, 16)])
def test_batch_diffusion_self_attention_forward(gpu_pkg, b, s, c, h):
    from distributed_xfold_amd import torch_ops
    torch_ops.register()
    g = torch.Generator().manual_seed(700 + s)
    rb = O.round_bf16
    d = c // h
    x = rb(torch.randn(b, s, c, generator=g))
    w = [rb(torch.randn(c, h, d, generator=g) * 0.05) for _ in range(4)]
    q_b = torch.randn(h, d, generator=g) * 0.1
    mask = (torch.rand(s, generator=g) > 0.15).float()
    mask[0] = 1
    bias = (1e9 * (mask[None, None, None, :] - 1)).tile(b, 1, 1, 1)
    nb = torch.randn(h, s, s, generator=g)
    want = O.gating_attention(x.double(), x.double(), bias.double(), nb.double(), *[t.double() for t in w],
                              query_b=q_b.double())
    t = lambda x_, dt=torch.bfloat16: x_.to(dev()).to(dt)
    got = torch.ops._alpha_attention.batch_diffusion_self_attention_forward(
        t(x), t(bias, torch.float32), t(nb, torch.float32), t(w[0]), t(q_b, torch.float32), t(w[1]), t(w[2]), t(w[3]),
        d, d)
    assert got.shape == (b, s, h, d)
    compare(f"batch_diffusion_self_attention_forward {b}x{s}x{c}", got, want, max_tol=8e-2)


@gpu
def test_batch_diffusion_cross_attention_forward(gpu_pkg):
    """fp32 operands as CrossAttention.load_xsmm_params leaves them (d_diffusion_transformer.py:338-358);
    the bias carries +1e9 where query and key are both padding, plus the pair logits (:397-406)."""
    from distributed_xfold_amd import torch_ops
    torch_ops.register()
    g = torch.Generator().manual_seed(800)
    rb = O.round_bf16
    bsz, q, k, c, h = 12, 32, 128, 128, 4
    xq, xk = rb(torch.randn(bsz, q, c, generator=g)), rb(torch.randn(bsz, k, c, generator=g))
    w = [rb(torch.randn(c, h, 32, generator=g) * 0.1) for _ in range(4)]
    q_b = torch.randn(h, 32, generator=g) * 0.1
    mq = (torch.rand(bsz, q, generator=g) > 0.2)
    mk = (torch.rand(bsz, k, generator=g) > 0.2)
    mq[:, 0] = mk[:, 0] = True
    bias = 1e9 * (~mq)[:, None, :, None].float() * (~mk)[:, None, None, :].float() \
        + torch.randn(bsz, h, q, k, generator=g)
    want = O.gating_attention(xq.double(), xk.double(), bias.double(), None, *[t.double() for t in w],
                              query_b=q_b.double())
    t = lambda x_: x_.to(dev()).float()
    got = torch.ops._alpha_attention.batch_diffusion_cross_attention_forward(
        t(xq), t(xk), t(bias), t(w[0]), t(q_b), t(w[1]), t(w[2]), t(w[3]), 32, 32)
    assert got.shape == (bsz, q, h, 32) and got.dtype == torch.float32
    live = mq[:, :, None, None].expand_as(want)          # padded queries see a constant shift of every key
    compare("batch_diffusion_cross_attention_forward", got.cpu() * live, want * live)


@gpu
def test_transition_forward(gpu_pkg):
    from distributed_xfold_amd import torch_ops
    torch_ops.register()
    g = torch.Generator().manual_seed(900)
    rb = O.round_bf16
    p = {k: rb(v) for k, v in O.make_transition_params(g, 128, 4, std=0.1).items()}
    x = rb(torch.randn(70, 70, 128, generator=g))
    want = O.transition(x.double(), O.cast_params(p, D))
    t = lambda x_, dt=torch.bfloat16: x_.to(dev()).to(dt)
    got = torch.ops._alpha_attention.transition_forward(
        t(x), t(p["transition1.weight"].t().contiguous()), t(p["transition2.weight"].t().contiguous(), torch.float32),
        t(p["input_layer_norm.weight"]), t(p["input_layer_norm.bias"]))
    compare("transition_forward", got, want)
