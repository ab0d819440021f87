"""CPU oracle for the AlphaFold3 Pairformer / diffusion-transformer hot path.

TEST INFRASTRUCTURE ONLY.  This file restates, in plain eager PyTorch on the
CPU, the arithmetic the reference performs on this path.  It is the checker the
HIP kernels are compared against; nothing in the product package imports it.
Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may call it.

Every function works in the dtype of its inputs (pass float64 tensors and
float64 parameters for a tight check) and takes parameters as a flat
``state_dict``-style mapping whose keys are the reference's parameter names.

Reference files restated (paths relative to the reference tree,
src/distributed_xfold/...):

  layer_norm                 csrc/triangle_multiplication.h:51-52 (eps 1e-5),
                             xsmm_kernels/kernel_test/transition.py:30
  triangle_multiplication    nn/d_triangle_multiplication.py:141-178,
                             xsmm_kernels/kernel_test/triangle_multiplication.py:25-81
  dot_product_attention      test_utils/test_grid_attn.py:262-279,
                             xsmm_kernels/kernel_test/batch_diffusion_self_attention_bf16.py:129-141
  gating_attention           xsmm_kernels/kernel_test/grid_self_attenion.py:61-95
  grid_self_attention        nn/d_attention.py:58-111
  transition                 nn/d_primitives.py:31-38,
                             xsmm_kernels/kernel_test/transition.py:38-43
  adaptive_layer_norm        nn/d_diffusion_transformer.py:37-74
  adaln_zero                 nn/d_diffusion_transformer.py:99-118
  self_attention             nn/d_diffusion_transformer.py:221-265
  diffusion_transition       nn/d_diffusion_transformer.py:142-145
  diffusion_transformer      nn/d_diffusion_transformer.py:294-310
  cross_attention            nn/d_diffusion_transformer.py:364-383,433-464
  cross_att_transformer      nn/d_diffusion_transformer.py:495-543
  pairformer_block           nn/d_pairformer.py:99-171

Pinning status (what checks each function besides this file itself; see
tests/test_oracle_pins.py):

  layer_norm, transition, triangle_multiplication, dot_product_attention,
  gating_attention, grid_self_attention, self_attention, cross_attention:
      pinned by brute-force loops on tiny inputs, closed forms, and library
      routines (torch.nn.functional.layer_norm / silu /
      scaled_dot_product_attention).
  pairformer_block, diffusion_transformer, cross_att_transformer:
      wiring only; pinned by re-deriving the residual chain from the pinned
      sub-operations with independently written code.
  PARITY UNPINNED at the boundary of the absent third-party `xfold` package
  (its sources are not in the reference tree and it cannot be imported):
      constructor details of AdaLNZero (transition2 has no bias,
      adaptive_zero_cond has a bias), DiffusionTransformer /
      DiffusionCrossAttTransformer.pair_input_layer_norm (weight, no bias),
      AdaptiveLayerNorm.single_cond_layer_norm (weight, no bias) and
      CrossAttention.q_scale (= key_dim_per_head ** -0.5).  The forms used here
      follow the in-tree evidence cited in each function.
"""

from __future__ import annotations

import math
from typing import Mapping, Optional

import torch

Params = Mapping[str, torch.Tensor]

LN_EPS = 1e-5
MASK_FILL = -1e9


# bf16 emulation: inside `with bf16_emulation():` every point where the HIP
# kernels hand a value to the matrix cores or to HBM as bf16 is rounded here
# too (the reference's own bf16 kernels round at the same kind of points,
# csrc/triangle_multiplication_bf16.h:160-162,230,273,503 and
# csrc/grid_self_attention_bf16.h:250).  Outside the context `_r` is the
# identity and the functions are the exact formulas.
_EMULATE = False


class bf16_emulation:
    def __enter__(self):
        global _EMULATE
        self._old, _EMULATE = _EMULATE, True

    def __exit__(self, *exc):
        global _EMULATE
        _EMULATE = self._old


def _r(t: torch.Tensor) -> torch.Tensor:
    return t.to(torch.bfloat16).to(t.dtype) if _EMULATE else t


def _sub(p: Params, prefix: str) -> dict:
    """Entries of `p` below `prefix.` with the prefix removed."""
    pre = prefix + "."
    return {k[len(pre):]: v for k, v in p.items() if k.startswith(pre)}


def _w(p: Params, name: str, like: torch.Tensor) -> Optional[torch.Tensor]:
    t = p.get(name)
    return None if t is None else t.to(like.dtype)


def layer_norm(x, weight=None, bias=None, eps: float = LN_EPS):
    """Affine LayerNorm over the last axis with biased variance.

    csrc/triangle_multiplication.h:51-52 builds LayerNormFwdTPP(..., 0.00001);
    kernel_test/transition.py:30 uses torch.nn.LayerNorm as its equal.
    """
    mean = x.mean(dim=-1, keepdim=True)
    xc = x - mean
    var = (xc * xc).mean(dim=-1, keepdim=True)
    y = xc / torch.sqrt(var + eps)
    if weight is not None:
        y = y * weight.to(x.dtype)
    if bias is not None:
        y = y + bias.to(x.dtype)
    return y


def linear(x, weight, bias=None):
    """x @ weight.T + bias, weight stored [out, in] as in torch.nn.Linear."""
    y = x @ weight.to(x.dtype).transpose(-1, -2)
    if bias is not None:
        y = y + bias.to(x.dtype)
    return y


# --------------------------------------------------------------------------
# a1  triangle multiplication
# --------------------------------------------------------------------------

def triangle_multiplication(pair, mask, p: Params, outgoing: bool):
    """nn/d_triangle_multiplication.py:141-178.

    pair [N, N, c], mask [N, N] (0/1 float or None).  Parameters:
    left_norm_input.{weight,bias}, projection.weight [2c, c], gate.weight
    [2c, c], center_norm.{weight,bias}, output_projection.weight [c, c],
    gating_linear.weight [c, c].  Even output channels of `projection`/`gate`
    form operand a, odd ones operand b (the reshape(c, 2, ...) at :162-165).
    """
    c = pair.shape[-1]
    x = _r(layer_norm(pair, p["left_norm_input.weight"], p["left_norm_input.bias"]))
    proj = linear(x, p["projection.weight"]).permute(2, 0, 1)       # [2c, N, N]
    if mask is not None:
        proj = proj * mask.to(x.dtype)[None]
    gate = linear(x, p["gate.weight"]).permute(2, 0, 1)
    proj = _r(proj * torch.sigmoid(gate))
    proj = proj.reshape(c, 2, *proj.shape[1:])
    a, b = proj[:, 0], proj[:, 1]                                    # [c, N, N]
    if outgoing:
        out = torch.einsum("cik,cjk->cij", a, b)
    else:
        out = torch.einsum("ckj,cki->cij", a, b)
    out = _r(out).permute(1, 2, 0)
    out = _r(layer_norm(out, p["center_norm.weight"], p["center_norm.bias"]))
    out = linear(out, p["output_projection.weight"])
    out = out * torch.sigmoid(linear(x, p["gating_linear.weight"]))
    return out


# --------------------------------------------------------------------------
# attention cores
# --------------------------------------------------------------------------

def dot_product_attention(q, k, v, mask=None, bias=None):
    """test_utils/test_grid_attn.py:262-279.

    q [..., Q, d], k/v [..., K, d]; bias broadcastable to [..., Q, K];
    mask boolean/0-1, broadcastable to [..., Q, K]; masked logits are
    REPLACED by -1e9 after the bias has been added.
    """
    logits = _r(q * (q.shape[-1] ** -0.5)) @ _r(k).transpose(-1, -2)
    if bias is not None:
        logits = logits + bias.to(logits.dtype)
    if mask is not None:
        logits = logits.masked_fill(~mask.to(torch.bool), MASK_FILL)
    if _EMULATE:   # un-normalised probabilities are rounded before they meet v
        e = _r(torch.exp(logits - logits.amax(dim=-1, keepdim=True)))
        return (e @ _r(v)) / e.sum(dim=-1, keepdim=True)
    weights = torch.softmax(logits, dim=-1)
    return weights @ v


def attention_weights(q, k, mask=None, bias=None):
    """The softmax weights dot_product_attention uses (for mask checks)."""
    logits = (q * (q.shape[-1] ** -0.5)) @ k.transpose(-1, -2)
    if bias is not None:
        logits = logits + bias.to(logits.dtype)
    if mask is not None:
        logits = logits.masked_fill(~mask.to(torch.bool), MASK_FILL)
    return torch.softmax(logits, dim=-1)


def gating_attention(q_data, m_data, bias, nonbatched_bias, query_w, key_w,
                     value_w, gating_w, output_w=None, query_b=None):
    """kernel_test/grid_self_attenion.py:61-95 (and, with query_b and no
    output_w, kernel_test/batch_diffusion_cross_attention.py:62-84).

    q_data [B, Q, C], m_data [B, K, C]; bias broadcastable to [B, H, Q, K]
    (ADDED, not filled); nonbatched_bias [H, Q, K] or None; weights in the
    fused-op layout query_w/key_w/value_w/gating_w [C, H, d], output_w
    [H, d, C_out].  Returns [B, Q, C_out] or, without output_w, [B, Q, H, d].
    """
    dt = q_data.dtype
    d = query_w.shape[-1]
    q = torch.einsum("bqa,ahc->bqhc", q_data, query_w.to(dt))
    if query_b is not None:
        q = q + query_b.to(dt)
    q = q * d ** (-0.5)
    k = torch.einsum("bka,ahc->bkhc", m_data, key_w.to(dt))
    v = torch.einsum("bka,ahc->bkhc", m_data, value_w.to(dt))
    logits = torch.einsum("bqhc,bkhc->bhqk", q, k) + bias.to(dt)
    if nonbatched_bias is not None and nonbatched_bias.numel() > 0:
        logits = logits + nonbatched_bias.to(dt)[None]
    weights = torch.softmax(logits, dim=-1)
    avg = torch.einsum("bhqk,bkhc->bqhc", weights, v)
    gate = torch.sigmoid(torch.einsum("bqc,chv->bqhv", q_data, gating_w.to(dt)))
    avg = avg * gate
    if output_w is None:
        return avg
    return torch.einsum("bqhc,hco->bqo", avg, output_w.to(dt))


# --------------------------------------------------------------------------
# a2  triangle (grid) self-attention
# --------------------------------------------------------------------------

def grid_self_attention(pair, mask, p: Params, num_head: int, transpose: bool,
                        full_pair=None):
    """nn/d_attention.py:88-111 with the base class' `_attention`
    (LN -> 128->H pair bias -> optional transpose -> per-row gated attention ->
    output projection -> un-transpose).  mask [N, N] indexes (row, key) of the
    tensor AFTER the optional transpose and is itself never transposed
    (d_attention.py:63 builds the key bias before the permute).
    """
    if full_pair is None:
        full_pair = pair
    w, b = p["act_norm.weight"], p["act_norm.bias"]
    x = _r(layer_norm(pair, w, b))
    nb = _r(linear(_r(layer_norm(full_pair, w, b)), p["pair_bias_projection.weight"]))
    nb = nb.permute(2, 0, 1)                                         # [H, Q, K]
    if transpose:
        x = x.permute(1, 0, 2)
    n_row, n_key, c = x.shape
    d = c // num_head

    def heads(t):                                                    # [B,S,C] -> [B,H,S,d]
        return t.reshape(n_row, n_key, num_head, d).permute(0, 2, 1, 3)

    q = heads(linear(x, p["q_projection.weight"]))
    k = heads(linear(x, p["k_projection.weight"]))
    v = heads(linear(x, p["v_projection.weight"]))
    key_mask = mask.to(torch.bool)[:, None, None, :]
    avg = dot_product_attention(q, k, v, mask=key_mask, bias=nb[None])
    avg = avg.permute(0, 2, 1, 3).reshape(n_row, n_key, c)
    # (emulation: the attention output is stored in bf16, the gate meets it in fp32)
    avg = _r(_r(avg) * torch.sigmoid(linear(x, p["gating_query.weight"])))
    out = linear(avg, p["output_projection.weight"])
    if transpose:
        out = out.permute(1, 0, 2)
    return out


# --------------------------------------------------------------------------
# a3  transition (SwiGLU)
# --------------------------------------------------------------------------

def gated_linear_unit(x, weight_t):
    """kernel_test/transition.py:40-42: y = x @ W; silu(first half) * second half."""
    y = x @ weight_t.to(x.dtype)
    a, b = torch.chunk(y, 2, dim=-1)
    return _r(torch.nn.functional.silu(a) * b)


def transition(x, p: Params):
    """nn/d_primitives.py:31-35: LN -> GLU(transition1) -> transition2; no biases."""
    x = _r(layer_norm(x, p["input_layer_norm.weight"], p["input_layer_norm.bias"]))
    c = gated_linear_unit(x, p["transition1.weight"].transpose(0, 1))
    return linear(c, p["transition2.weight"])


# --------------------------------------------------------------------------
# a6, a7  adaptive LayerNorm and AdaLN-Zero
# --------------------------------------------------------------------------

def adaptive_layer_norm(x, single_cond, p: Params):
    """nn/d_diffusion_transformer.py:61-74.

    With conditioning: sigmoid(scale(LN_w(s))) * LN_plain(x) + bias(LN_w(s)),
    where LN_plain has no affine parameters, LN_w has a weight but no bias,
    single_cond_scale has a bias and single_cond_bias has none (:49-57).
    Without: an ordinary affine LayerNorm.
    """
    if single_cond is None:
        return _r(layer_norm(x, p["layer_norm.weight"], p.get("layer_norm.bias")))
    xn = layer_norm(x)
    s = _r(layer_norm(single_cond.to(x.dtype), p["single_cond_layer_norm.weight"]))
    scale = linear(s, p["single_cond_scale.weight"], p["single_cond_scale.bias"])
    shift = linear(s, p["single_cond_bias.weight"])
    return _r(torch.sigmoid(scale) * xn + shift)


def adaln_zero(x, single_cond, p: Params):
    """nn/d_diffusion_transformer.py:99-118: transition2(x), times
    sigmoid(adaptive_zero_cond(single_cond)) when conditioned."""
    out = linear(x, p["transition2.weight"])
    if single_cond is not None:
        cond = linear(_r(single_cond.to(x.dtype)), p["adaptive_zero_cond.weight"],
                      p.get("adaptive_zero_cond.bias"))
        out = torch.sigmoid(cond) * out
    return out


# --------------------------------------------------------------------------
# a4, a8  pair-biased self-attention (Pairformer single / diffusion)
# --------------------------------------------------------------------------

def self_attention(x, mask, pair_logits, single_cond, p: Params, num_head: int):
    """nn/d_diffusion_transformer.py:221-265.

    x [N, c] or [B, N, c]; mask [N] over keys; pair_logits [H, N, N] shared by
    the batch; q has a bias, k/v/gate have none (test_grid_attn.py:139-149).
    """
    batched = x.dim() == 3
    xa = adaptive_layer_norm(x, single_cond, _sub(p, "adaptive_layernorm"))
    q = linear(xa, p["q_projection.weight"], p["q_projection.bias"])
    k = linear(xa, p["k_projection.weight"])
    v = linear(xa, p["v_projection.weight"])
    xb = xa if batched else xa[None]
    B, N, c = xb.shape
    d = c // num_head

    def heads(t):
        return t.reshape(B, N, num_head, d).permute(0, 2, 1, 3)

    q, k, v = (heads(t if batched else t[None]) for t in (q, k, v))
    key_mask = None if mask is None else mask.to(torch.bool)[None, None, None, :]
    bias = None if pair_logits is None else pair_logits[None]
    avg = dot_product_attention(q, k, v, mask=key_mask, bias=bias)
    avg = avg.permute(0, 2, 1, 3).reshape(B, N, c)
    if not batched:
        avg = avg[0]
    avg = _r(avg * _r(torch.sigmoid(linear(xa, p["gating_query.weight"]))))
    return adaln_zero(avg, single_cond, _sub(p, "adaptive_zero_init"))


def diffusion_transition(x, single_cond, p: Params):
    """nn/d_diffusion_transformer.py:142-145."""
    xa = adaptive_layer_norm(x, single_cond, _sub(p, "adaptive_layernorm"))
    c = gated_linear_unit(xa, p["transition1.weight"].transpose(0, 1))
    return adaln_zero(c, single_cond, _sub(p, "adaptive_zero_init"))


def diffusion_transformer(act, mask, single_cond, pair_cond, p: Params,
                          num_head: int = 16, num_blocks: int = 24,
                          super_block_size: int = 4):
    """nn/d_diffusion_transformer.py:294-310.  act is updated out of place."""
    pair_act = layer_norm(pair_cond.to(act.dtype), p["pair_input_layer_norm.weight"],
                          p.get("pair_input_layer_norm.bias"))
    act = act.clone()
    for sb in range(num_blocks // super_block_size):
        logits = linear(pair_act, p[f"pair_logits_projection.{sb}.weight"])
        n, s, _ = logits.shape
        # 'n s (b h) -> b h n s'
        logits = logits.reshape(n, s, super_block_size, num_head).permute(2, 3, 0, 1)
        for j in range(super_block_size):
            i = sb * super_block_size + j
            act = act + self_attention(act, mask, logits[j], single_cond,
                                       _sub(p, f"self_attention.{i}"), num_head)
            act = act + diffusion_transition(act, single_cond,
                                             _sub(p, f"transition_block.{i}"))
    return act


# --------------------------------------------------------------------------
# a11  windowed atom cross-attention
# --------------------------------------------------------------------------

def cross_attention(x_q, x_k, mask_q, mask_k, pair_logits, single_cond_q,
                    single_cond_k, p: Params, num_head: int = 4):
    """nn/d_diffusion_transformer.py:433-464 with _attention :364-383.

    x_q [..., Q, c], x_k [..., K, c]; mask_q [..., Q], mask_k [..., K];
    pair_logits [..., H, Q, K].  The bias is +1e9 where BOTH the query and the
    key are padding (:448-452) and zero elsewhere.
    """
    dt = x_q.dtype
    bias = (1e9 * (~mask_q.to(torch.bool))[..., None, :, None].to(dt)
            * (~mask_k.to(torch.bool))[..., None, None, :].to(dt))
    xq = adaptive_layer_norm(x_q, single_cond_q, _sub(p, "q_adaptive_layernorm"))
    xk = adaptive_layer_norm(x_k, single_cond_k, _sub(p, "k_adaptive_layernorm"))
    if pair_logits is not None:
        bias = bias + pair_logits.to(dt)
    q = linear(xq, p["q_projection.weight"], p["q_projection.bias"])
    k = linear(xk, p["k_projection.weight"])
    v = linear(xk, p["v_projection.weight"])
    dk = q.shape[-1] // num_head
    dv = v.shape[-1] // num_head
    q = q.reshape(q.shape[:-1] + (num_head, dk))
    k = k.reshape(k.shape[:-1] + (num_head, dk))
    v = v.reshape(v.shape[:-1] + (num_head, dv))
    logits = torch.einsum("...qhc,...khc->...hqk", _r(q * dk ** -0.5), _r(k)) + bias
    if _EMULATE:
        e = _r(torch.exp(logits - logits.amax(dim=-1, keepdim=True)))
        weights = e / e.sum(dim=-1, keepdim=True)
    else:
        weights = torch.softmax(logits, dim=-1)
    avg = torch.einsum("...hqk,...khc->...qhc", weights, _r(v))
    avg = avg.reshape(avg.shape[:-2] + (-1,))
    avg = _r(avg * _r(torch.sigmoid(linear(xq, p["gating_query.weight"]))))
    return adaln_zero(avg, single_cond_q, _sub(p, "adaptive_zero_init"))


def gather_keys(queries_act, gather_idxs, gather_mask):
    """Stand-in for xfold's atom_layout.convert(queries_to_keys, queries_act,
    layout_axes=(-3, -2)): keys[..., s, k, :] = flat(queries)[..., idx[s, k], :]
    zeroed where gather_mask is false.  gather_idxs index the flattened
    (subset, query) axis."""
    lead = queries_act.shape[:-3]
    S, Q, C = queries_act.shape[-3:]
    flat = queries_act.reshape(lead + (S * Q, C))
    out = flat[..., gather_idxs.reshape(-1), :].reshape(lead + tuple(gather_idxs.shape) + (C,))
    return out * gather_mask.to(out.dtype)[..., None]


def cross_att_transformer(queries_act, queries_mask, gather_idxs, gather_mask,
                          keys_mask, queries_single_cond, keys_single_cond,
                          pair_cond, p: Params, num_blocks: int = 3,
                          num_head: int = 4):
    """nn/d_diffusion_transformer.py:495-543."""
    dt = queries_act.dtype
    pair_act = layer_norm(pair_cond.to(dt), p["pair_input_layer_norm.weight"],
                          p.get("pair_input_layer_norm.bias"))
    logits = linear(pair_act, p["pair_logits_projection.weight"])    # [S,Q,K,(b h)]
    S, Q, K, _ = logits.shape
    logits = logits.reshape(S, Q, K, num_blocks, num_head).permute(3, 0, 4, 1, 2)
    act = queries_act.clone()
    for blk in range(num_blocks):
        keys_act = gather_keys(act, gather_idxs, gather_mask)
        act = act + cross_attention(act, keys_act, queries_mask, keys_mask,
                                    logits[blk], queries_single_cond,
                                    keys_single_cond,
                                    _sub(p, f"cross_attention.{blk}"), num_head)
        act = act + diffusion_transition(act, queries_single_cond,
                                         _sub(p, f"transition_block.{blk}"))
    return act


# --------------------------------------------------------------------------
# a5  Pairformer block
# --------------------------------------------------------------------------

def pairformer_block(pair, pair_mask, single, seq_mask, p: Params,
                     n_heads: int = 16, n_heads_pair: int = 4,
                     with_single: bool = True):
    """nn/d_pairformer.py:99-171 with dp=1: seven residual sub-operations."""
    pair = pair + triangle_multiplication(
        pair, pair_mask, _sub(p, "triangle_multiplication_outgoing"), True)
    pair = pair + triangle_multiplication(
        pair, pair_mask, _sub(p, "triangle_multiplication_incoming"), False)
    pair = pair + grid_self_attention(
        pair, pair_mask, _sub(p, "pair_attention1"), n_heads_pair, False)
    pair = pair + grid_self_attention(
        pair, pair_mask, _sub(p, "pair_attention2"), n_heads_pair, True)
    pair = pair + transition(pair, _sub(p, "pair_transition"))
    if not with_single:
        return pair
    logits = linear(
        layer_norm(pair, p["single_pair_logits_norm.weight"],
                   p["single_pair_logits_norm.bias"]),
        p["single_pair_logits_projection.weight"]).permute(2, 0, 1)
    single = single + self_attention(single, seq_mask, logits, None,
                                     _sub(p, "single_attention_"), n_heads)
    single = single + transition(single, _sub(p, "single_transition"))
    return pair, single


def pairformer_stack(pair, pair_mask, single, seq_mask, blocks):
    """d_alphafold3.py:242-244: the trunk loop over Pairformer blocks."""
    for p in blocks:
        pair, single = pairformer_block(pair, pair_mask, single, seq_mask, p)
    return pair, single


# --------------------------------------------------------------------------
# synthetic parameters (shared by tests and the benchmark's CPU leg)
# --------------------------------------------------------------------------

def _randn(gen, *shape, std=1.0, mean=0.0, dtype=torch.float32):
    return (torch.randn(*shape, generator=gen, dtype=torch.float32) * std + mean).to(dtype)


def make_ln(gen, c, bias=True, std=0.02, dtype=torch.float32):
    d = {"weight": _randn(gen, c, std=std, mean=1.0, dtype=dtype)}
    if bias:
        d["bias"] = _randn(gen, c, std=std, dtype=dtype)
    return d


def _put(dst, prefix, src):
    for k, v in src.items():
        dst[f"{prefix}.{k}"] = v


def make_triangle_multiplication_params(gen, c=128, std=0.02, dtype=torch.float32):
    p = {}
    _put(p, "left_norm_input", make_ln(gen, c, dtype=dtype))
    p["projection.weight"] = _randn(gen, 2 * c, c, std=std, dtype=dtype)
    p["gate.weight"] = _randn(gen, 2 * c, c, std=std, dtype=dtype)
    _put(p, "center_norm", make_ln(gen, c, dtype=dtype))
    p["output_projection.weight"] = _randn(gen, c, c, std=std, dtype=dtype)
    p["gating_linear.weight"] = _randn(gen, c, c, std=std, dtype=dtype)
    return p


def make_grid_self_attention_params(gen, c=128, num_head=4, std=0.02, dtype=torch.float32):
    p = {}
    _put(p, "act_norm", make_ln(gen, c, dtype=dtype))
    p["pair_bias_projection.weight"] = _randn(gen, num_head, c, std=std, dtype=dtype)
    for n in ("q_projection", "k_projection", "v_projection", "gating_query",
              "output_projection"):
        p[f"{n}.weight"] = _randn(gen, c, c, std=std, dtype=dtype)
    return p


def make_transition_params(gen, c, factor=4, std=0.02, dtype=torch.float32):
    p = {}
    _put(p, "input_layer_norm", make_ln(gen, c, dtype=dtype))
    p["transition1.weight"] = _randn(gen, 2 * factor * c, c, std=std, dtype=dtype)
    p["transition2.weight"] = _randn(gen, c, factor * c, std=std, dtype=dtype)
    return p


def make_adaptive_layer_norm_params(gen, c_x, c_cond, use_cond, std=0.02, dtype=torch.float32):
    p = {}
    if use_cond:
        _put(p, "single_cond_layer_norm", make_ln(gen, c_cond, bias=False, dtype=dtype))
        p["single_cond_scale.weight"] = _randn(gen, c_x, c_cond, std=std, dtype=dtype)
        p["single_cond_scale.bias"] = _randn(gen, c_x, std=std, dtype=dtype)
        p["single_cond_bias.weight"] = _randn(gen, c_x, c_cond, std=std, dtype=dtype)
    else:
        _put(p, "layer_norm", make_ln(gen, c_x, dtype=dtype))
    return p


def make_adaln_zero_params(gen, c_in, c_out, c_cond, use_cond, std=0.02, dtype=torch.float32):
    p = {"transition2.weight": _randn(gen, c_out, c_in, std=std, dtype=dtype)}
    if use_cond:
        p["adaptive_zero_cond.weight"] = _randn(gen, c_out, c_cond, std=std, dtype=dtype)
        p["adaptive_zero_cond.bias"] = _randn(gen, c_out, std=std, dtype=dtype)
    return p


def make_self_attention_params(gen, c_x=768, c_cond=384, use_cond=False, std=0.02,
                               dtype=torch.float32):
    p = {}
    _put(p, "adaptive_layernorm",
         make_adaptive_layer_norm_params(gen, c_x, c_cond, use_cond, std, dtype))
    p["q_projection.weight"] = _randn(gen, c_x, c_x, std=std, dtype=dtype)
    p["q_projection.bias"] = _randn(gen, c_x, std=std, dtype=dtype)
    for n in ("k_projection", "v_projection", "gating_query"):
        p[f"{n}.weight"] = _randn(gen, c_x, c_x, std=std, dtype=dtype)
    _put(p, "adaptive_zero_init",
         make_adaln_zero_params(gen, c_x, c_x, c_cond, use_cond, std, dtype))
    return p


def make_diffusion_transition_params(gen, c_x=768, c_cond=384, factor=2, use_cond=True,
                                     std=0.02, dtype=torch.float32):
    p = {}
    _put(p, "adaptive_layernorm",
         make_adaptive_layer_norm_params(gen, c_x, c_cond, use_cond, std, dtype))
    p["transition1.weight"] = _randn(gen, 2 * factor * c_x, c_x, std=std, dtype=dtype)
    _put(p, "adaptive_zero_init",
         make_adaln_zero_params(gen, factor * c_x, c_x, c_cond, use_cond, std, dtype))
    return p


def make_diffusion_transformer_params(gen, c_act=768, c_cond=384, c_pair=128, num_head=16,
                                      num_blocks=24, super_block_size=4, std=0.02,
                                      dtype=torch.float32):
    p = {}
    _put(p, "pair_input_layer_norm", make_ln(gen, c_pair, bias=False, dtype=dtype))
    for sb in range(num_blocks // super_block_size):
        p[f"pair_logits_projection.{sb}.weight"] = _randn(
            gen, super_block_size * num_head, c_pair, std=std, dtype=dtype)
    for i in range(num_blocks):
        _put(p, f"self_attention.{i}",
             make_self_attention_params(gen, c_act, c_cond, True, std, dtype))
        _put(p, f"transition_block.{i}",
             make_diffusion_transition_params(gen, c_act, c_cond, 2, True, std, dtype))
    return p


def make_cross_attention_params(gen, c=128, c_cond=128, std=0.02, dtype=torch.float32):
    p = {}
    _put(p, "q_adaptive_layernorm",
         make_adaptive_layer_norm_params(gen, c, c_cond, True, std, dtype))
    _put(p, "k_adaptive_layernorm",
         make_adaptive_layer_norm_params(gen, c, c_cond, True, std, dtype))
    p["q_projection.weight"] = _randn(gen, c, c, std=std, dtype=dtype)
    p["q_projection.bias"] = _randn(gen, c, std=std, dtype=dtype)
    for n in ("k_projection", "v_projection", "gating_query"):
        p[f"{n}.weight"] = _randn(gen, c, c, std=std, dtype=dtype)
    _put(p, "adaptive_zero_init", make_adaln_zero_params(gen, c, c, c_cond, True, std, dtype))
    return p


def make_cross_att_transformer_params(gen, c=128, c_cond=128, c_pair=16, num_blocks=3,
                                      num_head=4, std=0.02, dtype=torch.float32):
    p = {}
    _put(p, "pair_input_layer_norm", make_ln(gen, c_pair, bias=False, dtype=dtype))
    p["pair_logits_projection.weight"] = _randn(gen, num_blocks * num_head, c_pair,
                                                std=std, dtype=dtype)
    for i in range(num_blocks):
        _put(p, f"cross_attention.{i}", make_cross_attention_params(gen, c, c_cond, std, dtype))
        _put(p, f"transition_block.{i}",
             make_diffusion_transition_params(gen, c, c_cond, 2, True, std, dtype))
    return p


def make_pairformer_block_params(gen, c_pair=128, c_single=384, n_heads=16, n_heads_pair=4,
                                 factor=4, with_single=True, std=0.02, dtype=torch.float32):
    p = {}
    _put(p, "triangle_multiplication_outgoing",
         make_triangle_multiplication_params(gen, c_pair, std, dtype))
    _put(p, "triangle_multiplication_incoming",
         make_triangle_multiplication_params(gen, c_pair, std, dtype))
    _put(p, "pair_attention1", make_grid_self_attention_params(gen, c_pair, n_heads_pair, std, dtype))
    _put(p, "pair_attention2", make_grid_self_attention_params(gen, c_pair, n_heads_pair, std, dtype))
    _put(p, "pair_transition", make_transition_params(gen, c_pair, factor, std, dtype))
    if with_single:
        _put(p, "single_pair_logits_norm", make_ln(gen, c_pair, dtype=dtype))
        p["single_pair_logits_projection.weight"] = _randn(gen, n_heads, c_pair, std=std, dtype=dtype)
        _put(p, "single_attention_",
             make_self_attention_params(gen, c_single, c_single, False, std, dtype))
        _put(p, "single_transition", make_transition_params(gen, c_single, 4, std, dtype))
    return p


def cast_params(p: Params, dtype) -> dict:
    return {k: v.to(dtype) for k, v in p.items()}


def round_bf16(t: torch.Tensor) -> torch.Tensor:
    """Round to bf16 and back, keeping the dtype: the values a bf16 kernel sees."""
    return t.to(torch.bfloat16).to(t.dtype)


def rel_err(got: torch.Tensor, want: torch.Tensor) -> float:
    """max |err| / RMS(want): the parity figure of merit."""
    want = want.double()
    rms = float(torch.sqrt((want * want).mean()))
    return float((got.double() - want).abs().max()) / max(rms, 1e-30)
