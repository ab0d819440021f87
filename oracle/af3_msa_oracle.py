"""CPU oracle for the Evoformer (MSA) block that feeds the pair tensor of the
Pairformer trunk.

TEST INFRASTRUCTURE ONLY, like af3_oracle.py: plain eager PyTorch on the CPU,
in the dtype of its inputs; nothing in the product package imports it.

Reference files restated (paths relative to src/distributed_xfold/):

  outer_product_mean   nn/d_primitives.py:51-70
  msa_attention        nn/d_attention.py:123-156
  evoformer_block      nn/d_pairformer.py:202-252 (note pair_mask.T for the
                       incoming triangle multiplication, :217)

Pinning status (tests/test_msa_oracle_pins.py): outer_product_mean and
msa_attention by brute-force loops on tiny inputs and closed forms (one MSA row
gives the outer product of its two projections; zero logit weights give the
masked mean of the values); evoformer_block by re-deriving the residual chain
from the pinned operations with independently written code.
PARITY UNPINNED at the boundary of the absent `xfold` package (base-class
constructors of OuterProductMean and MSAAttention): projections without bias,
32 outer channels, output_w [32, 32, c_pair] with output_b [c_pair], epsilon
1e-3, 8 heads of c_msa / 8 value channels, LayerNorms with weight and bias.
The forms used are those of the published AlphaFold 3 algorithm.
"""

from __future__ import annotations

from typing import Mapping

import torch

from . import af3_oracle as O

Params = Mapping[str, torch.Tensor]


def outer_product_mean(msa, mask, p: Params, eps: float = 1e-3):
    """msa [a, N, c_msa], mask [a, N] -> [N, N, c_pair]:
    out[b, d, f] = (sum_{c,e} (sum_a L[a,b,c] R[a,d,e]) W[c,e,f] + bias[f])
                   / (eps + sum_a mask[a,b] mask[a,d])."""
    dt = msa.dtype
    m = mask.to(dt)[..., None]
    x = O.layer_norm(msa, p["layer_norm_input.weight"], p["layer_norm_input.bias"])
    left = m * O.linear(x, p["left_projection.weight"])
    right = m * O.linear(x, p["right_projection.weight"])
    outer = torch.einsum("abc,ade->bdce", left, right)
    act = torch.einsum("bdce,cef->bdf", outer, p["output_w"]) + p["output_b"]
    norm = torch.einsum("abc,adc->bdc", m, m)
    return act / (eps + norm)


def msa_attention(msa, msa_mask, pair, p: Params, num_head: int = 8):
    """msa [a, N, c_msa], msa_mask [a, N], pair [N, N, c_pair] -> [a, N, c_msa]:
    every MSA row is averaged over the tokens with weights
    softmax_k(pair_logits[h, q, k] + 1e9 (max_a mask[a, k] - 1))."""
    dt = msa.dtype
    x = O.layer_norm(msa, p["act_norm.weight"], p["act_norm.bias"])
    z = O.layer_norm(pair.to(dt), p["pair_norm.weight"], p["pair_norm.bias"])
    logits = O.linear(z, p["pair_logits.weight"]).permute(2, 0, 1)
    logits = logits + 1e9 * (msa_mask.to(dt).max(dim=0).values - 1.0)
    w = torch.softmax(logits, dim=-1)
    v = O.linear(x, p["v_projection.weight"])
    a, n, c = v.shape
    v = v.reshape(a, n, num_head, c // num_head)
    avg = torch.einsum("hqk,bkhc->bqhc", w, v).reshape(a, n, c)
    avg = avg * torch.sigmoid(O.linear(x, p["gating_query.weight"]))
    return O.linear(avg, p["output_projection.weight"])


def evoformer_block(msa, pair, msa_mask, pair_mask, p: Params, n_heads_pair: int = 4):
    """nn/d_pairformer.py:202-252 -> (msa, pair), out of place."""
    pair = pair + outer_product_mean(msa, msa_mask, O._sub(p, "outer_product_mean"))
    msa = msa + msa_attention(msa, msa_mask, pair, O._sub(p, "msa_attention1"))
    msa = msa + O.transition(msa, O._sub(p, "msa_transition"))
    pair = pair + O.triangle_multiplication(pair, pair_mask, O._sub(p, "triangle_multiplication_outgoing"), True)
    pair = pair + O.triangle_multiplication(pair, pair_mask.transpose(0, 1),
                                            O._sub(p, "triangle_multiplication_incoming"), False)
    pair = pair + O.grid_self_attention(pair, pair_mask, O._sub(p, "pair_attention1"), n_heads_pair, False)
    pair = pair + O.grid_self_attention(pair, pair_mask, O._sub(p, "pair_attention2"), n_heads_pair, True)
    pair = pair + O.transition(pair, O._sub(p, "pair_transition"))
    return msa, pair


# --------------------------------------------------------------------------
# parameter generators (reference parameter names)
# --------------------------------------------------------------------------

def make_outer_product_mean_params(gen, c_msa=64, c_pair=128, c_outer=32, std=0.05, dtype=torch.float32):
    p = {}
    O._put(p, "layer_norm_input", O.make_ln(gen, c_msa, dtype=dtype))
    p["left_projection.weight"] = O._randn(gen, c_outer, c_msa, std=std, dtype=dtype)
    p["right_projection.weight"] = O._randn(gen, c_outer, c_msa, std=std, dtype=dtype)
    p["output_w"] = O._randn(gen, c_outer, c_outer, c_pair, std=std, dtype=dtype)
    p["output_b"] = O._randn(gen, c_pair, std=std, dtype=dtype)
    return p


def make_msa_attention_params(gen, c_msa=64, c_pair=128, num_head=8, std=0.05, dtype=torch.float32):
    p = {}
    O._put(p, "act_norm", O.make_ln(gen, c_msa, dtype=dtype))
    O._put(p, "pair_norm", O.make_ln(gen, c_pair, dtype=dtype))
    p["pair_logits.weight"] = O._randn(gen, num_head, c_pair, std=std, dtype=dtype)
    for n in ("v_projection", "gating_query", "output_projection"):
        p[f"{n}.weight"] = O._randn(gen, c_msa, c_msa, std=std, dtype=dtype)
    return p


def make_evoformer_block_params(gen, c_msa=64, c_pair=128, n_heads_pair=4, std=0.02, dtype=torch.float32):
    p = {}
    O._put(p, "outer_product_mean", make_outer_product_mean_params(gen, c_msa, c_pair, std=max(std, 0.05), dtype=dtype))
    O._put(p, "msa_attention1", make_msa_attention_params(gen, c_msa, c_pair, std=max(std, 0.05), dtype=dtype))
    O._put(p, "msa_transition", O.make_transition_params(gen, c_msa, 4, std, dtype))
    O._put(p, "triangle_multiplication_outgoing", O.make_triangle_multiplication_params(gen, c_pair, std, dtype))
    O._put(p, "triangle_multiplication_incoming", O.make_triangle_multiplication_params(gen, c_pair, std, dtype))
    O._put(p, "pair_attention1", O.make_grid_self_attention_params(gen, c_pair, n_heads_pair, std, dtype))
    O._put(p, "pair_attention2", O.make_grid_self_attention_params(gen, c_pair, n_heads_pair, std, dtype))
    O._put(p, "pair_transition", O.make_transition_params(gen, c_pair, 4, std, dtype))
    return p
