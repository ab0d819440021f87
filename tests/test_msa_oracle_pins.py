"""Pins of the Evoformer-block oracle (oracle/af3_msa_oracle.py) on the CPU:
brute-force loops on tiny inputs, closed forms and an independently written
residual chain."""

import torch

from oracle import af3_msa_oracle as M
from oracle import af3_oracle as O

D = torch.float64


def gen(seed):
    return torch.Generator().manual_seed(seed)


def ln(x, w, b):
    mu = x.mean()
    return (x - mu) / torch.sqrt(((x - mu) ** 2).mean() + 1e-5) * w + b


def test_outer_product_mean_brute_force():
    g = gen(1)
    a, n, cm, co, cp = 3, 4, 8, 2, 5
    p = M.make_outer_product_mean_params(g, cm, cp, co, std=0.5, dtype=D)
    msa = torch.randn(a, n, cm, generator=g, dtype=D)
    mask = (torch.rand(a, n, generator=g) > 0.3).to(D)
    mask[:, 1] = 0                                                    # a token no row covers
    got = M.outer_product_mean(msa, mask, p)
    assert got.shape == (n, n, cp)
    for b in range(n):
        for d in range(n):
            acc = torch.zeros(co, co, dtype=D)
            cnt = 0.0
            for r in range(a):
                x_b = ln(msa[r, b], p["layer_norm_input.weight"], p["layer_norm_input.bias"])
                x_d = ln(msa[r, d], p["layer_norm_input.weight"], p["layer_norm_input.bias"])
                left = mask[r, b] * (p["left_projection.weight"] @ x_b)
                right = mask[r, d] * (p["right_projection.weight"] @ x_d)
                acc += left[:, None] * right[None, :]
                cnt += float(mask[r, b] * mask[r, d])
            want = (torch.einsum("ce,cef->f", acc, p["output_w"]) + p["output_b"]) / (1e-3 + cnt)
            assert torch.allclose(got[b, d], want, atol=1e-10), (b, d)
    # a pair no MSA row covers gets bias / epsilon
    assert torch.allclose(got[1, 2], p["output_b"] / 1e-3, atol=1e-9)


def test_outer_product_mean_is_not_symmetric_in_left_and_right():
    """out[b, d] uses the LEFT projection of token b and the RIGHT projection of
    token d; swapping the two projections transposes the (c, e) roles."""
    g = gen(2)
    p = M.make_outer_product_mean_params(g, 8, 5, 2, std=0.5, dtype=D)
    msa = torch.randn(3, 4, 8, generator=g, dtype=D)
    mask = torch.ones(3, 4, dtype=D)
    q = dict(p)
    q["left_projection.weight"], q["right_projection.weight"] = p["right_projection.weight"], p["left_projection.weight"]
    q["output_w"] = p["output_w"].transpose(0, 1)
    a = M.outer_product_mean(msa, mask, p)
    b = M.outer_product_mean(msa, mask, q)
    assert torch.allclose(a - p["output_b"] / (1e-3 + 3), (b - p["output_b"] / (1e-3 + 3)).transpose(0, 1), atol=1e-10)
    assert not torch.allclose(a, a.transpose(0, 1), atol=1e-3)


def test_msa_attention_brute_force():
    g = gen(3)
    a, n, cm, cp, h = 3, 5, 8, 6, 2
    p = M.make_msa_attention_params(g, cm, cp, h, std=0.5, dtype=D)
    msa = torch.randn(a, n, cm, generator=g, dtype=D)
    pair = torch.randn(n, n, cp, generator=g, dtype=D)
    mask = torch.ones(a, n, dtype=D)
    mask[:, 3] = 0                                                     # key 3 masked in every row
    mask[0, 1] = 0                                                     # key 1 only in one row: still a live key
    got = M.msa_attention(msa, mask, pair, p, h)
    d = cm // h
    for r in range(a):
        for q in range(n):
            x_q = ln(msa[r, q], p["act_norm.weight"], p["act_norm.bias"])
            out = torch.zeros(cm, dtype=D)
            for hh in range(h):
                logit = torch.stack([p["pair_logits.weight"][hh] @ ln(pair[q, k], p["pair_norm.weight"], p["pair_norm.bias"])
                                     for k in range(n)])
                logit[3] -= 1e9
                w = torch.softmax(logit, 0)
                assert float(w[3]) == 0.0
                for k in range(n):
                    v = p["v_projection.weight"] @ ln(msa[r, k], p["act_norm.weight"], p["act_norm.bias"])
                    out[hh * d:(hh + 1) * d] += w[k] * v[hh * d:(hh + 1) * d]
            out = out * torch.sigmoid(p["gating_query.weight"] @ x_q)
            assert torch.allclose(got[r, q], p["output_projection.weight"] @ out, atol=1e-10), (r, q)


def test_msa_attention_zero_logit_weights_give_the_masked_mean():
    g = gen(4)
    a, n, cm, cp, h = 2, 6, 8, 6, 2
    p = dict(M.make_msa_attention_params(g, cm, cp, h, std=0.5, dtype=D))
    p["pair_logits.weight"] = torch.zeros(h, cp, dtype=D)
    p["gating_query.weight"] = torch.zeros(cm, cm, dtype=D)          # gate = 1/2
    p["output_projection.weight"] = torch.eye(cm, dtype=D)
    msa = torch.randn(a, n, cm, generator=g, dtype=D)
    mask = torch.ones(a, n, dtype=D)
    mask[:, 4:] = 0
    got = M.msa_attention(msa, mask, torch.randn(n, n, cp, generator=g, dtype=D), p, h)
    v = O.linear(O.layer_norm(msa, p["act_norm.weight"], p["act_norm.bias"]), p["v_projection.weight"])
    want = 0.5 * v[:, :4].mean(dim=1, keepdim=True).expand(a, n, cm)
    assert torch.allclose(got, want, atol=1e-10)


def test_evoformer_block_wiring():
    g = gen(5)
    a, n = 3, 6
    p = M.make_evoformer_block_params(g, std=0.05, dtype=D)
    msa = torch.randn(a, n, 64, generator=g, dtype=D)
    pair = torch.randn(n, n, 128, generator=g, dtype=D)
    mm = (torch.rand(a, n, generator=g) > 0.2).to(D)
    mm[0] = 1
    pm = (torch.rand(n, n, generator=g) > 0.2).to(D)
    pm[:, 0] = 1
    got_msa, got_pair = M.evoformer_block(msa, pair, mm, pm, p)
    sub = lambda k: {kk[len(k) + 1:]: v for kk, v in p.items() if kk.startswith(k + ".")}
    z = pair + M.outer_product_mean(msa, mm, sub("outer_product_mean"))
    m1 = msa + M.msa_attention(msa, mm, z, sub("msa_attention1"))        # sees the UPDATED pair
    m1 = m1 + O.transition(m1, sub("msa_transition"))
    z = z + O.triangle_multiplication(z, pm, sub("triangle_multiplication_outgoing"), True)
    z = z + O.triangle_multiplication(z, pm.T, sub("triangle_multiplication_incoming"), False)   # transposed mask
    z = z + O.grid_self_attention(z, pm, sub("pair_attention1"), 4, False)
    z = z + O.grid_self_attention(z, pm, sub("pair_attention2"), 4, True)
    z = z + O.transition(z, sub("pair_transition"))
    assert torch.allclose(got_msa, m1, atol=1e-12) and torch.allclose(got_pair, z, atol=1e-12)
    # the transposed mask matters: with the plain mask the result differs
    z2 = pair + M.outer_product_mean(msa, mm, sub("outer_product_mean"))
    z2 = z2 + O.triangle_multiplication(z2, pm, sub("triangle_multiplication_outgoing"), True)
    z3 = z2 + O.triangle_multiplication(z2, pm, sub("triangle_multiplication_incoming"), False)
    z4 = z2 + O.triangle_multiplication(z2, pm.T, sub("triangle_multiplication_incoming"), False)
    assert not torch.allclose(z3, z4, atol=1e-6)
