"""ctypes binding of libaf3hip.so (C ABI declared in include/af3_hip.h)."""

from __future__ import annotations

import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libaf3hip.so")

AF3_BF16, AF3_F32 = 0, 1
STATIC_SCRATCH_BYTES = 32 << 20      # AF3_STATIC_SCRATCH_BYTES
LINEAR_PLAIN, LINEAR_SWIGLU, LINEAR_GATE_RES, LINEAR_REGROUP32, LINEAR_ROWGATE_RES = 0, 2, 3, 4, 5

_vp, _i, _i64, _sz, _f = C.c_void_p, C.c_int, C.c_int64, C.c_size_t, C.c_float

# name -> (restype, argtypes); must list every symbol include/af3_hip.h declares
SIGNATURES = {
    "af3_abi_version": (_i, []),
    "af3_error_string": (C.c_char_p, [_i]),
    "af3_triangle_multiplication_workspace_bytes": (_sz, [_i64]),
    "af3_triangle_multiplication_forward": (
        _i, [_vp, _i, _vp, _i, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i64, _vp, _sz, _vp]),
    "af3_grid_self_attn_workspace_bytes": (_sz, [_i64, _i]),
    "af3_grid_self_attn_forward": (
        _i, [_vp, _i, _vp, _i, _vp, _vp, _vp, _vp, _vp, _vp, _i, _vp, _i, _i64, _vp, _sz, _vp]),
    "af3_transition_forward": (_i, [_vp, _i, _vp, _vp, _vp, _vp, _i, _vp, _i, _i64, _vp]),
    "af3_triangle_multiplication_forward_padded": (
        _i, [_vp, _i, _vp, _i, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i64, _i, _vp, _sz, _vp]),
    "af3_grid_self_attn_forward_padded": (
        _i, [_vp, _i, _vp, _i, _vp, _vp, _vp, _vp, _vp, _vp, _i, _vp, _i, _i64, _i, _vp, _sz, _vp]),
    "af3_transition_forward_padded": (_i, [_vp, _i, _vp, _vp, _vp, _vp, _i, _vp, _i, _i64, _i, _vp]),
    "af3_batch_diffusion_self_attention_workspace_bytes": (_sz, [_i64, _i64, _i]),
    "af3_batch_diffusion_self_attention_forward": (
        _i, [_vp, _vp, _i64, _vp, _i, _vp, _vp, _i, _vp, _i, _i64, _i64, _i, _vp, _sz, _vp]),
    "af3_batch_diffusion_self_attention_forward_static": (
        _i, [_vp, _vp, _i64, _vp, _i, _vp, _vp, _i, _vp, _i, _i64, _i64, _i, _vp]),
    "af3_batched_nt_product_forward": (_i, [_vp, _vp, _vp, _i64, _i64, _i64, _i64, _vp]),
    "af3_transpose_bf16_forward": (_i, [_vp, _vp, _i64, _i64, _vp]),
    "af3_atom_position_features_forward": (_i, [_vp, _vp, _vp, _vp, _vp, _i, _i64, _i64, _i64, _i, _vp]),
    "af3_gather_rows_add_forward": (_i, [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _i, _vp]),
    "af3_position_update_forward": (_i, [_vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i, _vp]),
    "af3_gathered_relu_mean_forward": (_i, [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _i, _i, _vp]),
    "af3_batch_diffusion_cross_attention_workspace_bytes": (_sz, [_i64, _i64, _i64, _i]),
    "af3_batch_diffusion_cross_attention_forward": (
        _i, [_vp, _vp, _vp, _vp, _vp, _i64, _vp, _vp, _vp, _i, _vp, _i, _i64, _i64, _i64, _i, _vp, _sz, _vp]),
    "af3_gathered_cross_attention_workspace_bytes": (_sz, [_i64, _i64, _i64, _i64, _i]),
    "af3_gathered_cross_attention_forward": (
        _i, [_vp, _vp, _vp, _vp, _vp, _vp, _i64, _vp, _vp, _vp, _i, _vp, _i, _i64, _i64, _i64, _i64, _i64, _i,
             _vp, _sz, _vp]),
    "af3_pair_logits_forward": (_i, [_vp, _i, _vp, _vp, _vp, _i, _vp, _i64, _vp]),
    "af3_layer_norm_forward": (_i, [_vp, _i, _vp, _i64, _i, _vp, _vp, _vp, _vp, _i64, _i64, _vp]),
    "af3_linear_forward": (
        _i, [_vp, _vp, _vp, _vp, _i, _i64, _i, _i, _i, _f, _i, _vp, _i64, _i64, _vp, _i, _vp]),
    "af3_triangle_contraction_forward": (_i, [_vp, _vp, _vp, _i64, _vp]),
    "af3_masked_softmax_rows_forward": (_i, [_vp, _vp, _vp, _i64, _i64, _i64, _vp]),
    "af3_narrow_linear_f32_forward": (_i, [_vp, _vp, _vp, _vp, _i64, _i, _i, _i, _vp]),
    "af3_atom_pair_cond_forward": (_i, [_vp, _vp, _vp, _vp, _vp, _i64, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp,
                                        _i64, _i64, _i64, _vp]),
    "af3_atom_pair_logits_forward": (_i, [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _i, _i, _vp]),
    "af3_pair_cond_init_forward": (_i, [_vp, _i, _f, _vp, _vp, _vp, _vp, _vp, _i, _i, _vp, _vp, _vp, _vp, _vp, _i64, _vp]),
    "af3_linear_bias_span": (_i, [_i64, _i, _i, _i, _i, _vp, _vp]),
    "af3_grid_attention_core_forward": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _i64, _vp]),
    "af3_check_gemm_f32": (
        _i, [_vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _i64, _i64, _i64, _i64, _i64, _i64, _i64,
             _vp, _f, _i, _vp, _i64, _i64, _vp, _i64, _i64, _vp]),
    "af3_check_layer_norm_f32": (_i, [_vp, _vp, _i64, _i, _vp, _vp, _vp, _vp, _i64, _i64, _vp]),
    "af3_check_elementwise_f32": (_i, [_i, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i, _vp]),
    "af3_check_attention_f32": (
        _i, [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _i64, _i64, _i64, _i64, _i, _i64, _i64, _i,
             _vp, _i64, _i64, _i64, _i64, _i64, _vp, _i64, _vp, _vp, _vp]),
}

_lib = None


class Af3Error(RuntimeError):
    pass


def load():
    """Load libaf3hip.so; raises if it has not been built (no fallback)."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise Af3Error(
            f"{LIB_PATH} is missing: build it with `make -C {os.path.join(_HERE, 'csrc')}` "
            "(or __graft_entry__.build()); there is no CPU fallback")
    lib = C.CDLL(LIB_PATH)
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)          # AttributeError if a declared symbol is absent
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib


def check(rc: int, what: str):
    if rc != 0:
        msg = load().af3_error_string(rc).decode()
        raise Af3Error(f"{what} failed: {msg} (code {rc})")
