"""fp32 check mode: every operator of the hot path composed a second time from
plain fp32 kernels (csrc/check_f32.hip), reading the modules' nn.Parameters
directly (no packing).  Inputs and outputs are fp32 GPU tensors.

This path exists to check the bf16 kernels: it follows the same reference
formulas (the file:line citations are on the bf16 modules in nn/) through
independent code, matches the CPU oracle to 1e-4, and runs at sizes the CPU
oracle cannot reach.  It is slow by design and allocates freely.
"""

from __future__ import annotations

import torch

from . import ops

SPLIT, CHAN_TO_PIX, TRANSPOSE_PIX, SWIGLU, BINARY = 0, 1, 2, 3, 4


def _w(p):
    return p.detach().to(torch.float32).contiguous()


def _req(t, name):
    if not (isinstance(t, torch.Tensor) and t.is_cuda and t.dtype == torch.float32):
        raise ValueError(f"{name}: the fp32 check mode takes fp32 GPU tensors")
    return t.contiguous()


def _mul(a, b):
    y = torch.empty_like(a)
    ops.ck_elementwise(BINARY, a, b, None, y, None, a.numel(), 0, 0)
    return y


def _add(a, b):
    y = torch.empty_like(a)
    ops.ck_elementwise(BINARY, a, b, None, y, None, a.numel(), 0, 1)
    return y


def _transpose_pix(x):
    n, _, c = x.shape
    y = torch.empty_like(x)
    ops.ck_elementwise(TRANSPOSE_PIX, x, None, None, y, None, n, c, 0)
    return y


def _ln(x, norm, scale=None, shift=None):
    w = None if getattr(norm, "weight", None) is None else _w(norm.weight)
    b = None if getattr(norm, "bias", None) is None else _w(norm.bias)
    return ops.ck_layer_norm(x, w, b, scale, shift)


def _lin(x, layer, **kw):
    b = None if layer.bias is None else _w(layer.bias)
    return ops.ck_linear(x, _w(layer.weight), bias=b, **kw)


# ------------------------------------------------------------------ pair path
def triangle_multiplication(mod, pair, mask):
    pair = _req(pair, "pair")
    n = pair.shape[0]
    x = _ln(pair, mod.left_norm_input)
    proj = _lin(x, mod.projection)
    gate = _lin(x, mod.gate)
    c = pair.shape[-1]
    a = torch.empty((c, n, n), dtype=torch.float32, device=pair.device)
    b = torch.empty_like(a)
    maskf = None if mask is None else mask.to(torch.float32).contiguous()
    incoming = 0 if mod._outgoing else 1
    ops.ck_elementwise(SPLIT, proj, gate, maskf, a, b, n, c, incoming)
    # outgoing: t[c] = a[c] b[c]^T ; incoming (operands stored transposed): t[c] = b'[c] a'[c]^T
    lhs, rhs = (a, b) if mod._outgoing else (b, a)
    t = ops.ck_gemm(lhs, rhs, m=n, n=n, k=n, batch=c, lda=n, ldb=n, sa=n * n, sb=n * n)
    tp = torch.empty((n, n, c), dtype=torch.float32, device=pair.device)
    ops.ck_elementwise(CHAN_TO_PIX, t, None, None, tp, None, n, c, 0)
    y = _ln(tp, mod.center_norm)
    out_gate = _lin(x, mod.gating_linear, sigmoid=True)
    return _lin(y, mod.output_projection, mul=out_gate)


def grid_self_attention(mod, pair, mask):
    pair = _req(pair, "pair")
    n, h = pair.shape[0], mod.num_head
    x = _ln(pair, mod.act_norm)
    nb = _lin(x, mod.pair_bias_projection)                    # [q, k, h]
    if mod.transpose:
        x = _transpose_pix(x)
    d = pair.shape[-1] // h
    q = _lin(x, mod.q_projection, alpha=d ** -0.5)
    k = _lin(x, mod.k_projection)
    v = _lin(x, mod.v_projection)
    g = _lin(x, mod.gating_query, sigmoid=True)
    avg = ops.ck_attention(q, k, v, h, bias=nb, bias_strides=(0, 1, n * h, h), key_mask=mask, km_sb=n)
    out = _lin(_mul(avg, g), mod.output_projection)
    return _transpose_pix(out) if mod.transpose else out


def transition(mod, x):
    x = _req(x, "x")
    xn = _ln(x, mod.input_layer_norm)
    y = _lin(xn, mod.transition1)
    f = y.shape[-1] // 2
    hdn = torch.empty(tuple(y.shape[:-1]) + (f,), dtype=torch.float32, device=x.device)
    ops.ck_elementwise(SWIGLU, y, None, None, hdn, None, y.numel() // (2 * f), f, 0)
    return _lin(hdn, mod.transition2)


# ------------------------------------------------------- diffusion-style modules
def adaptive_layer_norm(mod, x, single_cond):
    x = _req(x, "x")
    if not mod.use_single_cond:
        return _ln(x, mod.layer_norm)
    s = _ln(_req(single_cond, "single_cond"), mod.single_cond_layer_norm)
    scale = _lin(s, mod.single_cond_scale).reshape(-1, mod.c_x)
    shift = _lin(s, mod.single_cond_bias).reshape(-1, mod.c_x)
    return ops.ck_layer_norm(x, None, None, scale, shift)


def adaln_zero(mod, x, single_cond):
    if not mod.use_single_cond:
        return _lin(x, mod.transition2)
    gate = _lin(_req(single_cond, "single_cond"), mod.adaptive_zero_cond, sigmoid=True)
    return _lin(x, mod.transition2, mul=gate.reshape(-1, mod.c_out))


def self_attention(mod, x, mask, pair_logits, single_cond, bias_view=None):
    """pair_logits [H, N, N] contiguous, or bias_view = (tensor, strides) for a strided bias."""
    xa = adaptive_layer_norm(mod.adaptive_layernorm, x, single_cond)
    batched = xa.dim() == 3
    xb = xa if batched else xa.unsqueeze(0)
    n = xb.shape[1]
    q = _lin(xb, mod.q_projection, alpha=mod.qkv_dim ** -0.5)
    k = _lin(xb, mod.k_projection)
    v = _lin(xb, mod.v_projection)
    g = _lin(xb, mod.gating_query, sigmoid=True)
    bias, strides = None, (0, 0, 0, 1)
    if bias_view is not None:
        bias, strides = bias_view
    elif pair_logits is not None:
        bias, strides = _req(pair_logits, "pair_logits"), (0, n * n, n, 1)
    avg = ops.ck_attention(q, k, v, mod.num_head, bias=bias, bias_strides=strides, key_mask=mask, km_sb=0)
    out = adaln_zero(mod.adaptive_zero_init, _mul(avg, g), single_cond)
    return out if batched else out.squeeze(0)


def diffusion_transition(mod, x, single_cond):
    xa = adaptive_layer_norm(mod.adaptive_layernorm, x, single_cond)
    y = _lin(xa, mod.transition1)
    f = y.shape[-1] // 2
    hdn = torch.empty(tuple(y.shape[:-1]) + (f,), dtype=torch.float32, device=x.device)
    ops.ck_elementwise(SWIGLU, y, None, None, hdn, None, y.numel() // (2 * f), f, 0)
    return adaln_zero(mod.adaptive_zero_init, hdn, single_cond)


def diffusion_transformer(mod, act, mask, single_cond, pair_cond):
    act = _req(act, "act")
    pair_act = _ln(_req(pair_cond, "pair_cond"), mod.pair_input_layer_norm)
    n = pair_act.shape[0]
    width = mod.super_block_size * mod.num_head
    for sb in range(mod.num_super_blocks):
        logits = _lin(pair_act, mod.pair_logits_projection[sb])           # [n, s, (b h)]
        for j in range(mod.super_block_size):
            i = sb * mod.super_block_size + j
            view = (logits.reshape(-1)[j * mod.num_head:], (0, 1, n * width, width))
            act = _add(act, self_attention(mod.self_attention[i], act, mask, None, single_cond, bias_view=view))
            act = _add(act, diffusion_transition(mod.transition_block[i], act, single_cond))
    return act


def cross_attention(mod, x_q, x_k, mask_q, mask_k, pair_logits, single_cond_q, single_cond_k):
    n_q, c = x_q.shape[-2:]
    n_k = x_k.shape[-2]
    xq = adaptive_layer_norm(mod.q_adaptive_layernorm, x_q, single_cond_q).reshape(-1, n_q, c)
    xk = adaptive_layer_norm(mod.k_adaptive_layernorm, x_k, single_cond_k).reshape(-1, n_k, c)
    h = mod.num_head
    q = _lin(xq, mod.q_projection, alpha=mod.key_dim_per_head ** -0.5)
    k = _lin(xk, mod.k_projection)
    v = _lin(xk, mod.v_projection)
    g = _lin(xq, mod.gating_query, sigmoid=True)
    mq, mk = mask_q.reshape(-1, n_q), mask_k.reshape(-1, n_k)
    bias, strides = None, (0, 0, 0, 1)
    if pair_logits is not None:
        bias = _req(pair_logits, "pair_logits").reshape(-1, h, n_q, n_k)
        strides = (h * n_q * n_k, n_q * n_k, n_k, 1)
    avg = ops.ck_attention(q, k, v, h, bias=bias, bias_strides=strides, bias_mod=mq.shape[0], qpad=mq, kpad=mk)
    out = adaln_zero(mod.adaptive_zero_init, _mul(avg, g).reshape(x_q.shape), single_cond_q)
    return out


def cross_att_transformer(mod, queries_act, queries_mask, queries_to_keys, keys_mask, queries_single_cond,
                          keys_single_cond, pair_cond):
    act = _req(queries_act, "queries_act")
    pair_act = _ln(_req(pair_cond, "pair_cond"), mod.pair_input_layer_norm)
    logits = _lin(pair_act, mod.pair_logits_projection)                   # [S, Q, K, (b h)]
    s, q, k, _ = logits.shape
    logits = logits.reshape(s, q, k, mod.num_blocks, mod.num_head).permute(3, 0, 4, 1, 2).contiguous()
    for blk in range(mod.num_blocks):
        keys_act = mod._gather(queries_to_keys, act)
        act = _add(act, cross_attention(mod.cross_attention[blk], act, keys_act, queries_mask, keys_mask,
                                        logits[blk], queries_single_cond, keys_single_cond))
        act = _add(act, diffusion_transition(mod.transition_block[blk], act, queries_single_cond))
    return act


def pairformer_block(mod, pair, pair_mask, single=None, seq_mask=None):
    pair = _req(pair, "pair")
    pair = _add(pair, triangle_multiplication(mod.triangle_multiplication_outgoing, pair, pair_mask))
    pair = _add(pair, triangle_multiplication(mod.triangle_multiplication_incoming, pair, pair_mask))
    pair = _add(pair, grid_self_attention(mod.pair_attention1, pair, pair_mask))
    pair = _add(pair, grid_self_attention(mod.pair_attention2, pair, pair_mask))
    pair = _add(pair, transition(mod.pair_transition, pair))
    if not mod.with_single:
        return pair
    n, h = pair.shape[0], mod.n_heads
    logits = _lin(_ln(pair, mod.single_pair_logits_norm), mod.single_pair_logits_projection)   # [q, k, h]
    view = (logits, (0, 1, n * h, h))
    single = _req(single, "single")
    single = _add(single, self_attention(mod.single_attention_, single, seq_mask, None, None, bias_view=view))
    single = _add(single, transition(mod.single_transition, single))
    return pair, single
