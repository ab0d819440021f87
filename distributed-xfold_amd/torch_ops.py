"""The reference's fused operators under their own names, for GPU tensors.

The reference defines five operators in the dispatcher library `_alpha_attention`
(src/distributed_xfold/xsmm_kernels/csrc/Alpha_Attention.cpp:181-211) and gives them
CPU kernels (:215-222).  `register()` gives the same operators kernels for the CUDA
(= HIP) dispatch key, backed by libaf3hip.so, so that the reference's own call sites

    torch.ops._alpha_attention.traingle_multiplication_forward(...)      prototypes/TriangleMultiplication.py:40
    torch.ops._alpha_attention.grid_self_attn_forward(...)               prototypes/GridSelfAttention.py:35
    torch.ops._alpha_attention.batch_diffusion_self_attention_forward    prototypes/Batched_DiffusionSelfAttention.py
    torch.ops._alpha_attention.batch_diffusion_cross_attention_forward   prototypes/Batched_DiffusionCrossAttention.py
    torch.ops._alpha_attention.transition_forward(...)                   prototypes/Transition.py:30

run on the GPU when they are handed GPU tensors, with the operands exactly as
`load_xsmm_params()` prepares them.  If the reference's extension is loaded as well
the two coexist: it owns the schemas and the CPU kernels, this module adds the CUDA
ones.  If it is not, the schemas are defined here (same strings).

Differences from the CPU kernels, all inside what the call sites accept:
  * results come back with their exact extents (the CPU kernels pad the sequence to
    a multiple of 64 and the callers narrow, which is then a no-op);
  * the additive key bias `[B, 1, 1, S]` of the two self-attention operators must be
    what the callers build, `1e9 * (mask - 1)`: it is read back as the 0/1 mask;
  * one GPU holds the whole operand: `grid_self_attn_forward` and
    `traingle_multiplication_forward` want the square [N, N, 128] pair tensor.

The weights arrive in the reference's layouts on every call; their repacked forms
are cached per source tensor object and version.
"""

from __future__ import annotations

import weakref
from typing import Dict, Tuple

import torch

from . import ops

NAMESPACE = "_alpha_attention"

# Alpha_Attention.cpp:182-211, verbatim
SCHEMAS: Dict[str, str] = {
    "grid_self_attn_forward":
        "grid_self_attn_forward(Tensor q_data, Tensor bias, Tensor nonbatched_bias, "
        "Tensor query_w, Tensor key_w, Tensor value_w, Tensor gating_w, Tensor output_w, "
        "int key_dim, int value_dim) -> Tensor",
    "transition_forward":
        "transition_forward(Tensor act, Tensor transition1, Tensor transition2, "
        "Tensor layernorm_weight, Tensor layernorm_bias) -> Tensor",
    "batch_diffusion_self_attention_forward":
        "batch_diffusion_self_attention_forward(Tensor q_data, Tensor bias, Tensor nonbatched_bias, "
        "Tensor query_w, Tensor query_b, Tensor key_w, Tensor value_w, Tensor gating_w, "
        "int key_dim, int value_dim) -> Tensor",
    "batch_diffusion_cross_attention_forward":
        "batch_diffusion_cross_attention_forward(Tensor q_data, Tensor m_data, Tensor batched_bias, "
        "Tensor query_w, Tensor query_b, Tensor key_w, Tensor value_w, Tensor gating_w, "
        "int key_dim, int value_dim) -> Tensor",
    "traingle_multiplication_forward":
        "traingle_multiplication_forward(Tensor act, Tensor mask, int equation_flag, "
        "Tensor left_norm_input_weight, Tensor left_norm_input_bias, Tensor projection_weight, "
        "Tensor gate_weight, Tensor center_norm_weight, Tensor center_norm_bias, "
        "Tensor output_projection_weight, Tensor gating_linear_weight) -> Tensor",
}

_CACHE: Dict[Tuple, object] = {}
_CACHE_LIMIT = 4096
_libs = []          # torch.library.Library objects must stay alive
_registered = False


def _version_of(t):
    """The tensor's modification counter, or None where it has none to offer (tensors created under
    torch.inference_mode() refuse to tell)."""
    try:
        return t._version
    except RuntimeError:
        return None


def _cached(role, tensors, build):
    """`build()` once per (role, set of source tensors).  `role` names what is built: the same tensor may
    reach two builders (an fp32 copy here, a repacked bf16 weight there) and each needs its own entry.  An
    entry holds weak references to its sources and is only good while they are the very same tensor objects,
    unmodified (`_version`): an address alone may have been handed to another tensor in the meantime.
    Sources without a version counter are not cached."""
    versions = tuple(_version_of(t) for t in tensors)
    if any(v is None for v in versions):
        return build()
    key = (role,) + tuple((id(t), v) for t, v in zip(tensors, versions))
    hit = _CACHE.get(key)
    if hit is not None and all(r() is t for r, t in zip(hit[0], tensors)):
        return hit[1]
    if len(_CACHE) >= _CACHE_LIMIT:
        _CACHE.clear()
    value = build()
    _CACHE[key] = (tuple(weakref.ref(t) for t in tensors), value)
    return value


def clear_cache() -> None:
    _CACHE.clear()


def _f32(t: torch.Tensor) -> torch.Tensor:
    return _cached("f32", (t,), lambda: t.detach().to(torch.float32).contiguous())


def _bf16(t: torch.Tensor) -> torch.Tensor:
    return _cached("bf16", (t,), lambda: t.detach().to(torch.bfloat16).contiguous())


def _linear_weight(w_chd: torch.Tensor) -> torch.Tensor:
    """[c_in, heads, dim] as load_xsmm_params stores a projection (weight.T reshaped) -> [heads * dim, c_in]."""
    return w_chd.detach().reshape(w_chd.shape[0], -1).t()


def _key_mask(bias: torch.Tensor, batch: int, seq: int) -> torch.Tensor:
    """The operators' additive `bias` argument, `1e9 * (mask - 1)` of shape [B or 1, 1, 1, S]
    (d_attention.py:63, d_diffusion_transformer.py:206), back to the 0/1 key mask [B, S] the kernels take.
    The kernels replace a masked key's logit by -1e9 and add nothing to the others, so any other additive
    value cannot be honoured: a tensor that holds anything but 0 and -1e9 is refused.  One reduction on
    the device per tensor version (the result is cached with the mask)."""
    def build():
        flat = bias.detach().reshape(-1, seq).to(torch.float32)
        if flat.shape[0] not in (1, batch):
            raise ValueError(f"bias: expected [{batch}, 1, 1, {seq}] or [1, 1, 1, {seq}], got {tuple(bias.shape)}")
        # (-1e9 as fp32 holds it, or as a bf16 / fp16-free cast chain may have rounded it: within 2^-8)
        if not bool(((flat == 0) | ((flat + 1e9).abs() <= 4e6)).all()):
            raise ValueError("bias: only the key-mask form 1e9 * (mask - 1), i.e. values 0 and -1e9, is supported "
                             "on the GPU path; other additive biases belong in nonbatched_bias")
        return (flat == 0).to(torch.float32).expand(batch, seq).contiguous()
    return _cached(("key_mask", batch, seq), (bias,), build)


def _activations(x: torch.Tensor) -> torch.Tensor:
    return x if x.dtype in (torch.bfloat16, torch.float32) else x.to(torch.float32)


# --------------------------------------------------------------------------- CUDA kernels
def traingle_multiplication_forward(act, mask, equation_flag, left_norm_input_weight, left_norm_input_bias,
                                    projection_weight, gate_weight, center_norm_weight, center_norm_bias,
                                    output_projection_weight, gating_linear_weight):
    """projection / gate weights de-interleaved as d_triangle_multiplication.py:128-129 leaves them:
    rows 0..c-1 make operand a, rows c..2c-1 operand b."""
    c = act.shape[-1]
    if c != 128:
        raise ValueError("traingle_multiplication_forward on the GPU: 128 pair channels")

    def pack():
        p, g = projection_weight.detach(), gate_weight.detach()
        chunks = [torch.cat([p[h * c + lo:h * c + lo + 64], g[h * c + lo:h * c + lo + 64]], dim=0)
                  for h in (0, 1) for lo in (0, 64)]
        return torch.stack(chunks).to(torch.bfloat16).contiguous()

    w_pg = _cached("trimul_proj_gate", (projection_weight, gate_weight), pack)
    n = act.shape[0]
    return ops.triangle_multiplication(
        _activations(act).contiguous(), mask.reshape(n, -1), int(equation_flag), _f32(left_norm_input_weight),
        _f32(left_norm_input_bias), w_pg, _f32(center_norm_weight), _f32(center_norm_bias),
        _bf16(output_projection_weight), _bf16(gating_linear_weight), residual=False)


def grid_self_attn_forward(q_data, bias, nonbatched_bias, query_w, key_w, value_w, gating_w, output_w,
                           key_dim, value_dim):
    """q_data [B, S, 128] already normalised (and transposed by the caller for the ending node),
    B = S; nonbatched_bias [H, S, S]; weights [128, H, d] and [H, d, 128] (d_attention.py:38-56)."""
    b, s, c = q_data.shape
    num_head = query_w.shape[1]
    if key_dim != value_dim or num_head * key_dim != c:
        raise ValueError("grid_self_attn_forward on the GPU: key_dim = value_dim = channels / heads")

    def pack():
        return torch.stack([_linear_weight(w) for w in (query_w, key_w, value_w, gating_w)]) \
            .to(torch.bfloat16).contiguous()

    w_qkvg = _cached("grid_qkvg", (query_w, key_w, value_w, gating_w), pack)
    w_out = _cached("attn_output_w", (output_w,), lambda: output_w.detach().reshape(-1, output_w.shape[-1]).t()
                    .to(torch.bfloat16).contiguous())
    nb = nonbatched_bias.to(torch.float32).contiguous() if nonbatched_bias.numel() else None
    return ops.grid_self_attn(_activations(q_data).contiguous(), _key_mask(bias, b, s), False, None, None, None, nb,
                              w_qkvg, w_out, num_head, residual=False)


def batch_diffusion_self_attention_forward(q_data, bias, nonbatched_bias, query_w, query_b, key_w, value_w,
                                           gating_w, key_dim, value_dim):
    """q_data [B, S, C] after the adaptive LayerNorm; returns [B, S, H, d] (d_diffusion_transformer.py:197-216)."""
    b, s, c = q_data.shape
    num_head = query_w.shape[1]

    def pack():
        return torch.cat([_linear_weight(w) for w in (query_w, key_w, value_w, gating_w)], dim=0) \
            .to(torch.bfloat16).contiguous()

    w_qkvg = _cached("self_qkvg", (query_w, key_w, value_w, gating_w), pack)
    q_b = _cached("query_b", (query_b,), lambda: query_b.detach().reshape(-1).to(torch.float32).contiguous()) \
        if query_b.numel() else None
    nb = nonbatched_bias.to(torch.float32).contiguous() if nonbatched_bias.numel() else None
    out = ops.batch_diffusion_self_attention(q_data.to(torch.bfloat16).contiguous(), _key_mask(bias, b, s), nb,
                                             w_qkvg, q_b, num_head)
    return out.to(q_data.dtype)


def batch_diffusion_cross_attention_forward(q_data, m_data, batched_bias, query_w, query_b, key_w, value_w,
                                            gating_w, key_dim, value_dim):
    """q_data [B, Q, C], m_data [B, K, C]; batched_bias [B, H or 1, Q, K], any values
    (d_diffusion_transformer.py:385-422); returns [B, Q, H, d]."""
    b, sq, c = q_data.shape
    sk = m_data.shape[1]
    num_head = query_w.shape[1]
    w_qg = _cached("cross_qg", (query_w, gating_w), lambda: torch.cat([_linear_weight(query_w), _linear_weight(gating_w)], dim=0)
                   .to(torch.bfloat16).contiguous())
    w_kv = _cached("cross_kv", (key_w, value_w), lambda: torch.cat([_linear_weight(key_w), _linear_weight(value_w)], dim=0)
                   .to(torch.bfloat16).contiguous())
    q_b = _cached("query_b", (query_b,), lambda: query_b.detach().reshape(-1).to(torch.float32).contiguous()) \
        if query_b.numel() else None
    logits = batched_bias.to(torch.float32).reshape(-1, batched_bias.shape[-3], sq, sk)
    logits = logits.expand(logits.shape[0], num_head, sq, sk).contiguous()
    if b % logits.shape[0]:
        raise ValueError("batched_bias: its batch must divide that of q_data")
    out = ops.batch_diffusion_cross_attention(q_data.to(torch.bfloat16).contiguous(),
                                              m_data.to(torch.bfloat16).contiguous(), logits, None, None,
                                              w_qg, w_kv, q_b, num_head)
    return out.to(q_data.dtype)


def transition_forward(act, transition1, transition2, layernorm_weight, layernorm_bias):
    """act [..., 128]; transition1 [c, 2 f c] and transition2 [f c, c], the transposes of the Linear
    weights (prototypes/Transition.py:71-76); silu half first (d_primitives.py:33)."""
    c = act.shape[-1]
    if c != 128:
        raise ValueError("transition_forward on the GPU: 128 channels")
    from .nn.base import pack_swiglu
    hidden = transition2.shape[0]
    w1 = _cached("transition1", (transition1,), lambda: pack_swiglu(transition1.detach().t(), 64).to(torch.bfloat16)
                 .reshape(hidden // 64, 128, 128).contiguous())
    w2 = _cached("transition2", (transition2,), lambda: transition2.detach().t().to(torch.bfloat16).contiguous())
    x = _activations(act).contiguous()
    return ops.transition128(x.view(-1, c), _f32(layernorm_weight), _f32(layernorm_bias), w1, w2,
                             residual=False).view(act.shape)


_CUDA_IMPLS = {
    "grid_self_attn_forward": grid_self_attn_forward,
    "transition_forward": transition_forward,
    "batch_diffusion_self_attention_forward": batch_diffusion_self_attention_forward,
    "batch_diffusion_cross_attention_forward": batch_diffusion_cross_attention_forward,
    "traingle_multiplication_forward": traingle_multiplication_forward,
}


# --------------------------------------------------------------------------- shapes for tracing
def _fake_grid(q_data, bias, nonbatched_bias, query_w, key_w, value_w, gating_w, output_w, key_dim, value_dim):
    return torch.empty_like(q_data)


def _fake_transition(act, transition1, transition2, layernorm_weight, layernorm_bias):
    return torch.empty_like(act)


def _fake_self(q_data, bias, nonbatched_bias, query_w, query_b, key_w, value_w, gating_w, key_dim, value_dim):
    return q_data.new_empty((q_data.shape[0], q_data.shape[1], query_w.shape[-2], query_w.shape[-1]))


def _fake_cross(q_data, m_data, batched_bias, query_w, query_b, key_w, value_w, gating_w, key_dim, value_dim):
    return q_data.new_empty((q_data.shape[0], q_data.shape[1], query_w.shape[-2], query_w.shape[-1]))


def _fake_trimul(act, mask, equation_flag, left_norm_input_weight, left_norm_input_bias, projection_weight,
                 gate_weight, center_norm_weight, center_norm_bias, output_projection_weight,
                 gating_linear_weight):
    return torch.empty_like(act)


_FAKES = {
    "grid_self_attn_forward": _fake_grid,
    "transition_forward": _fake_transition,
    "batch_diffusion_self_attention_forward": _fake_self,
    "batch_diffusion_cross_attention_forward": _fake_cross,
    "traingle_multiplication_forward": _fake_trimul,
}


def _defined(name: str) -> bool:
    try:
        getattr(getattr(torch.ops, NAMESPACE), name)
        return True
    except (AttributeError, RuntimeError):
        return False


def register() -> None:
    """Define the operators that are not defined yet and give all five a CUDA kernel
    and, where none is registered, a shape function for FakeTensor tracing.  Idempotent."""
    global _registered
    if _registered:
        return
    lib = torch.library.Library(NAMESPACE, "FRAGMENT")
    _libs.append(lib)
    for name, schema in SCHEMAS.items():
        if not _defined(name):
            lib.define(schema)
    for name, fn in _CUDA_IMPLS.items():
        lib.impl(name, fn, "CUDA")
    for name, fn in _FAKES.items():
        try:
            torch.library.register_fake(f"{NAMESPACE}::{name}", fn, lib=lib)
        except RuntimeError:
            pass    # the reference's prototypes/register_fake_kernels.py got there first
    _registered = True
