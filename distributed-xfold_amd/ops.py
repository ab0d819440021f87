"""Operator layer: torch tensors in, C ABI calls out.

These functions stand where the reference's `torch.ops._alpha_attention.*`
operators and their Python wrappers stand (src/distributed_xfold/xsmm_kernels/
prototypes/*.py): they check dtype / shape / device / contiguity (ValueError),
own the output and scratch allocation through torch's caching allocator, pass
raw device pointers and the current HIP stream to libaf3hip.so, and turn a
non-zero return code into a RuntimeError.  No arithmetic happens here.
"""

from __future__ import annotations

from typing import Optional

import torch

from . import lib as _L

_workspaces: dict = {}


def _ws(nbytes: int, device) -> torch.Tensor:
    """Scratch buffer per device and stream, grown on demand and reused between
    calls (calls on one stream are ordered, so reuse is safe; calls on different
    streams may run at the same time and get different buffers)."""
    key = (device.type, device.index, torch.cuda.current_stream(device).cuda_stream)
    buf = _workspaces.get(key)
    if buf is None or buf.numel() < nbytes:
        buf = torch.empty(max(nbytes, 1), dtype=torch.uint8, device=device)
        _workspaces[key] = buf
    return buf


def release_workspaces():
    _workspaces.clear()


def _dt(t: torch.Tensor) -> int:
    if t.dtype == torch.bfloat16:
        return _L.AF3_BF16
    if t.dtype == torch.float32:
        return _L.AF3_F32
    raise ValueError(f"activation dtype must be bfloat16 or float32, got {t.dtype}")


def _gpu(t: torch.Tensor, name: str, dtype=None, shape=None) -> torch.Tensor:
    if not isinstance(t, torch.Tensor):
        raise ValueError(f"{name}: expected a tensor")
    if not t.is_cuda:
        raise ValueError(f"{name}: tensor must live on the GPU (got {t.device}); there is no CPU path")
    if dtype is not None and t.dtype != dtype:
        raise ValueError(f"{name}: expected dtype {dtype}, got {t.dtype}")
    if shape is not None and tuple(t.shape) != tuple(shape):
        raise ValueError(f"{name}: expected shape {tuple(shape)}, got {tuple(t.shape)}")
    if not t.is_contiguous():
        raise ValueError(f"{name}: tensor must be contiguous")
    return t


def _p(t: Optional[torch.Tensor]):
    return None if t is None else t.data_ptr()


def _stream(device) -> int:
    return torch.cuda.current_stream(device).cuda_stream


def _mask_f32(mask: Optional[torch.Tensor], shape, name: str):
    if mask is None:
        return None
    if not mask.is_cuda:
        raise ValueError(f"{name}: tensor must live on the GPU")
    if tuple(mask.shape) != tuple(shape):
        raise ValueError(f"{name}: expected shape {tuple(shape)}, got {tuple(mask.shape)}")
    return mask.to(torch.float32).contiguous()


# --------------------------------------------------------------------------
def triangle_multiplication(act, mask, equation_flag, left_norm_input_weight, left_norm_input_bias,
                            w_proj_gate, center_norm_weight, center_norm_bias,
                            w_output_projection, w_gating_linear, residual=False, out=None, valid_channels=128):
    """traingle_multiplication_forward (csrc/Alpha_Attention.cpp:148-169); returns
    the update, or act + update written in place when residual=True.
    `valid_channels` < 128: tensor and weights are zero-padded to 128 channels."""
    lib = _L.load()
    _gpu(act, "act")
    if act.dim() != 3 or act.shape[0] != act.shape[1] or act.shape[2] != 128:
        raise ValueError(f"act: expected [N, N, 128], got {tuple(act.shape)}")
    n = act.shape[0]
    io = _dt(act)
    maskf = _mask_f32(mask, (n, n), "mask")
    for nm, t in (("left_norm_input_weight", left_norm_input_weight), ("left_norm_input_bias", left_norm_input_bias),
                  ("center_norm_weight", center_norm_weight), ("center_norm_bias", center_norm_bias)):
        _gpu(t, nm, torch.float32, (128,))
    _gpu(w_proj_gate, "w_proj_gate", torch.bfloat16, (4, 128, 128))
    _gpu(w_output_projection, "w_output_projection", torch.bfloat16, (128, 128))
    _gpu(w_gating_linear, "w_gating_linear", torch.bfloat16, (128, 128))
    if out is None:
        out = act if residual else torch.empty_like(act)
    else:
        _gpu(out, "out", act.dtype, act.shape)
    nbytes = lib.af3_triangle_multiplication_workspace_bytes(n)
    ws = _ws(nbytes, act.device)
    if valid_channels != 128:
        rc = lib.af3_triangle_multiplication_forward_padded(
            _p(act), io, _p(maskf), int(equation_flag), _p(left_norm_input_weight), _p(left_norm_input_bias),
            _p(w_proj_gate), _p(center_norm_weight), _p(center_norm_bias), _p(w_output_projection),
            _p(w_gating_linear), _p(out), int(bool(residual)), n, int(valid_channels), _p(ws), ws.numel(),
            _stream(act.device))
        _L.check(rc, "af3_triangle_multiplication_forward_padded")
        return out
    rc = lib.af3_triangle_multiplication_forward(
        _p(act), io, _p(maskf), int(equation_flag), _p(left_norm_input_weight), _p(left_norm_input_bias),
        _p(w_proj_gate), _p(center_norm_weight), _p(center_norm_bias), _p(w_output_projection),
        _p(w_gating_linear), _p(out), int(bool(residual)), n, _p(ws), ws.numel(), _stream(act.device))
    _L.check(rc, "af3_triangle_multiplication_forward")
    return out


def grid_self_attn(pair, mask, transpose, act_norm_weight, act_norm_bias, w_pair_bias, nonbatched_bias,
                   w_qkvg, w_output, num_head, residual=False, out=None, valid_channels=128):
    """grid_self_attn_forward (csrc/Alpha_Attention.cpp:50-70) fused with the steps
    of DistributeGridSelfAttention.xsmm_forward (nn/d_attention.py:58-85).
    `valid_channels` < 128: tensor and weights are zero-padded to 128 channels."""
    lib = _L.load()
    _gpu(pair, "pair")
    if pair.dim() != 3 or pair.shape[0] != pair.shape[1] or pair.shape[2] != 128:
        raise ValueError(f"pair: expected [N, N, 128], got {tuple(pair.shape)}")
    n = pair.shape[0]
    io = _dt(pair)
    maskf = _mask_f32(mask, (n, n), "mask")
    if act_norm_weight is not None:
        _gpu(act_norm_weight, "act_norm_weight", torch.float32, (128,))
        _gpu(act_norm_bias, "act_norm_bias", torch.float32, (128,))
    if w_pair_bias is not None:
        _gpu(w_pair_bias, "w_pair_bias", torch.bfloat16)
        if w_pair_bias.dim() != 2 or w_pair_bias.shape[1] != 128 or w_pair_bias.shape[0] % 32 \
                or w_pair_bias.shape[0] < num_head:
            raise ValueError("w_pair_bias: expected [roundup(num_head, 32), 128]")
    if nonbatched_bias is not None:
        _gpu(nonbatched_bias, "nonbatched_bias", torch.float32, (num_head, n, n))
    _gpu(w_qkvg, "w_qkvg", torch.bfloat16, (4, 128, 128))
    _gpu(w_output, "w_output", torch.bfloat16, (128, 128))
    if out is None:
        out = pair if residual else torch.empty_like(pair)
    else:
        _gpu(out, "out", pair.dtype, pair.shape)
    nbytes = lib.af3_grid_self_attn_workspace_bytes(n, num_head)
    ws = _ws(nbytes, pair.device)
    if valid_channels != 128:
        rc = lib.af3_grid_self_attn_forward_padded(
            _p(pair), io, _p(maskf), int(bool(transpose)), _p(act_norm_weight), _p(act_norm_bias),
            _p(w_pair_bias), _p(nonbatched_bias), _p(w_qkvg), _p(w_output), int(num_head),
            _p(out), int(bool(residual)), n, int(valid_channels), _p(ws), ws.numel(), _stream(pair.device))
        _L.check(rc, "af3_grid_self_attn_forward_padded")
        return out
    rc = lib.af3_grid_self_attn_forward(
        _p(pair), io, _p(maskf), int(bool(transpose)), _p(act_norm_weight), _p(act_norm_bias),
        _p(w_pair_bias), _p(nonbatched_bias), _p(w_qkvg), _p(w_output), int(num_head),
        _p(out), int(bool(residual)), n, _p(ws), ws.numel(), _stream(pair.device))
    _L.check(rc, "af3_grid_self_attn_forward")
    return out


def transition128(act, layernorm_weight, layernorm_bias, w1_packed, w2, residual=False, out=None, valid_channels=128):
    """transition_forward (csrc/Alpha_Attention.cpp:116-125) for 128-channel rows.
    `valid_channels` < 128: rows and weights are zero-padded to 128 channels."""
    lib = _L.load()
    _gpu(act, "act")
    if act.shape[-1] != 128:
        raise ValueError("act: last dimension must be 128")
    io = _dt(act)
    hidden = w2.shape[1]
    _gpu(layernorm_weight, "layernorm_weight", torch.float32, (128,))
    _gpu(layernorm_bias, "layernorm_bias", torch.float32, (128,))
    _gpu(w1_packed, "w1_packed", torch.bfloat16, (hidden // 64, 128, 128))
    _gpu(w2, "w2", torch.bfloat16, (128, hidden))
    rows = act.numel() // 128
    if out is None:
        out = act if residual else torch.empty_like(act)
    else:
        _gpu(out, "out", act.dtype, act.shape)
    if valid_channels != 128:
        rc = lib.af3_transition_forward_padded(_p(act), io, _p(layernorm_weight), _p(layernorm_bias), _p(w1_packed),
                                               _p(w2), int(hidden), _p(out), int(bool(residual)), rows,
                                               int(valid_channels), _stream(act.device))
        _L.check(rc, "af3_transition_forward_padded")
        return out
    rc = lib.af3_transition_forward(_p(act), io, _p(layernorm_weight), _p(layernorm_bias), _p(w1_packed),
                                    _p(w2), int(hidden), _p(out), int(bool(residual)), rows,
                                    _stream(act.device))
    _L.check(rc, "af3_transition_forward")
    return out


def batch_diffusion_self_attention(q_data, key_mask, nonbatched_bias, w_qkvg, query_b, num_head,
                                   out_dtype=torch.bfloat16, out=None, static_scratch=False):
    """batch_diffusion_self_attention_forward (csrc/Alpha_Attention.cpp:72-92).
    With `static_scratch` (and a caller-provided `out`) the call goes to the
    allocation-free entry point, whose scratch is a device array the library owns.
    q_data [B, S, C] bf16 (already normalised); key_mask [S] (shared) or [B, S];
    nonbatched_bias [H, S, S] fp32, or [H, S/4, S, 4] as `quad_major_bias` makes it;
    returns [B, S, H, C/H]."""
    lib = _L.load()
    _gpu(q_data, "q_data", torch.bfloat16)
    if q_data.dim() != 3:
        raise ValueError("q_data: expected [B, S, C]")
    b, s, c = q_data.shape
    mask_batches = 1
    if key_mask is not None and key_mask.dim() == 2:
        mask_batches = b
        km = _mask_f32(key_mask, (b, s), "key_mask")
    else:
        km = _mask_f32(key_mask, (s,), "key_mask")
    quad_major = 0
    if nonbatched_bias is not None and nonbatched_bias.dim() == 4:
        quad_major = 1
        _gpu(nonbatched_bias, "nonbatched_bias", torch.float32, (num_head, s // 4, s, 4))
    elif nonbatched_bias is not None:
        _gpu(nonbatched_bias, "nonbatched_bias", torch.float32, (num_head, s, s))
    _gpu(w_qkvg, "w_qkvg", torch.bfloat16, (4 * c, c))
    if query_b is not None:
        _gpu(query_b, "query_b", torch.float32, (c,))
    if out is None:
        out = torch.empty((b, s, num_head, c // num_head), dtype=out_dtype, device=q_data.device)
    else:
        _gpu(out, "out", out_dtype, (b, s, num_head, c // num_head))
    if static_scratch:
        # allocation-free entry point: the scratch is the library's own device array
        rc = lib.af3_batch_diffusion_self_attention_forward_static(
            _p(q_data), _p(km), mask_batches, _p(nonbatched_bias), quad_major, _p(w_qkvg), _p(query_b),
            int(num_head), _p(out), _dt(out), b, s, c, _stream(q_data.device))
        _L.check(rc, "af3_batch_diffusion_self_attention_forward_static")
        return out
    nbytes = lib.af3_batch_diffusion_self_attention_workspace_bytes(b, s, c)
    ws = _ws(nbytes, q_data.device)
    rc = lib.af3_batch_diffusion_self_attention_forward(
        _p(q_data), _p(km), mask_batches, _p(nonbatched_bias), quad_major, _p(w_qkvg), _p(query_b), int(num_head), _p(out),
        _dt(out), b, s, c, _p(ws), ws.numel(), _stream(q_data.device))
    _L.check(rc, "af3_batch_diffusion_self_attention_forward")
    return out


def atom_position_features(positions, rows, weight, cond, out_dtype=torch.bfloat16):
    """out[b, q] = cond[q] + weight @ positions[b, rows[q]] (rows[q] < 0: cond[q] only)
    (af3_atom_position_features_forward).  positions [B, n_slots, 3] fp32, rows [Q] int32,
    weight [C, 3] fp32, cond [Q, C] fp32 -> [B, Q, C]."""
    lib = _L.load()
    _gpu(positions, "positions", torch.float32)
    if positions.dim() != 3 or positions.shape[-1] != 3:
        raise ValueError("positions: expected [B, n_slots, 3]")
    b, n_slots = positions.shape[:2]
    if rows.dtype != torch.int32 or rows.dim() != 1 or not rows.is_contiguous() or rows.device != positions.device:
        raise ValueError("rows: expected a contiguous int32 [Q] tensor on the device of positions")
    q = rows.shape[0]
    c = weight.shape[0]
    _gpu(weight, "weight", torch.float32, (c, 3))
    _gpu(cond, "cond", torch.float32, (q, c))
    if c % 8:
        raise ValueError("channels must be a multiple of 8")
    if getattr(rows, "_af3_checked_rows", None) != n_slots:
        if int(rows.max()) >= n_slots:
            raise ValueError("rows: slot index beyond positions")
        rows._af3_checked_rows = n_slots
    out = torch.empty((b, q, c), dtype=out_dtype, device=positions.device)
    rc = lib.af3_atom_position_features_forward(_p(positions), _p(rows), _p(weight), _p(cond), _p(out), _dt(out),
                                                b, n_slots, q, c, _stream(positions.device))
    _L.check(rc, "af3_atom_position_features_forward")
    return out


def _rows32(rows, n_src, device, name="rows"):
    if rows.dtype != torch.int32 or rows.dim() != 1 or not rows.is_contiguous() or rows.device != device:
        raise ValueError(f"{name}: expected a contiguous int32 vector on the device of the data")
    if getattr(rows, "_af3_checked_rows", None) != n_src:
        if int(rows.max()) >= n_src:
            raise ValueError(f"{name}: row index beyond the source")
        rows._af3_checked_rows = n_src             # one device round trip per index tensor


def gather_rows_add(src, rows, add):
    """out[b, q] = (src[b, rows[q]] if rows[q] >= 0 else 0) + add[b, q], all bf16
    (af3_gather_rows_add_forward).  src [B, n_src, C], rows [Q] int32, add [B, Q, C]."""
    lib = _L.load()
    _gpu(src, "src", torch.bfloat16)
    if src.dim() != 3:
        raise ValueError("src: expected [B, n_src, C]")
    b, n_src, c = src.shape
    _rows32(rows, n_src, src.device)
    q = rows.shape[0]
    _gpu(add, "add", torch.bfloat16, (b, q, c))
    if c % 8:
        raise ValueError("channels must be a multiple of 8")
    out = torch.empty_like(add)
    rc = lib.af3_gather_rows_add_forward(_p(src), _p(rows), _p(add), _p(out), b, n_src, q, c, _stream(src.device))
    _L.check(rc, "af3_gather_rows_add_forward")
    return out


def position_update(x, rows, ln_weight, weight):
    """out[b, t] = weight @ bf16(LayerNorm(x[b, rows[t]]) * ln_weight), zeros where rows[t] < 0
    (af3_position_update_forward).  x [B, n_src, 128] bf16, rows [T] int32, ln_weight [128],
    weight [3, 128] fp32 -> [B, T, 3] fp32."""
    lib = _L.load()
    _gpu(x, "x", torch.bfloat16)
    if x.dim() != 3 or x.shape[-1] != 128:
        raise ValueError("x: expected [B, n_src, 128]")
    b, n_src, c = x.shape
    _rows32(rows, n_src, x.device)
    _gpu(ln_weight, "ln_weight", torch.float32, (c,))
    _gpu(weight, "weight", torch.float32, (3, c))
    out = torch.empty((b, rows.shape[0], 3), dtype=torch.float32, device=x.device)
    rc = lib.af3_position_update_forward(_p(x), _p(rows), _p(ln_weight), _p(weight), _p(out), b, n_src,
                                         rows.shape[0], c, _stream(x.device))
    _L.check(rc, "af3_position_update_forward")
    return out


def gathered_relu_mean(src, idx, count):
    """out[b, t] = sum_a relu(src[b, idx[t, a]]) / count[t] over the slots with idx >= 0
    (af3_gathered_relu_mean_forward).  src [B, n_src, C] bf16, idx [T, A] int32,
    count [T] fp32 -> [B, T, C] fp32."""
    lib = _L.load()
    _gpu(src, "src", torch.bfloat16)
    if src.dim() != 3:
        raise ValueError("src: expected [B, n_src, C]")
    b, n_src, c = src.shape
    if idx.dtype != torch.int32 or idx.dim() != 2 or not idx.is_contiguous() or idx.device != src.device:
        raise ValueError("idx: expected a contiguous int32 [T, A] tensor on the device of src")
    t, a = idx.shape
    if a > 32 or c % 8:
        raise ValueError("at most 32 slots, channels a multiple of 8")
    if not getattr(idx, "_af3_checked_rows", None) == n_src:
        if int(idx.max()) >= n_src:
            raise ValueError("idx: row index beyond src")
        idx._af3_checked_rows = n_src          # one device round trip per index tensor
    _gpu(count, "count", torch.float32, (t,))
    out = torch.empty((b, t, c), dtype=torch.float32, device=src.device)
    rc = lib.af3_gathered_relu_mean_forward(_p(src), _p(idx), _p(count), _p(out), b, n_src, t, a, c,
                                            _stream(src.device))
    _L.check(rc, "af3_gathered_relu_mean_forward")
    return out


def quad_major_bias(bias):
    """[..., Sq, Sk] -> [..., Sk/4, Sq, 4]: the pair-bias order in which the
    attention kernel's loads are contiguous (Sk a multiple of 4).  One strided
    copy: for a bias that is computed once and used by many attention calls."""
    sq, sk = bias.shape[-2:]
    if sk % 4:
        raise ValueError("quad-major bias needs a key count that is a multiple of 4")
    lead = tuple(bias.shape[:-2])
    k = len(lead)
    return bias.reshape(lead + (sq, sk // 4, 4)).permute(*range(k), k + 1, k, k + 2).contiguous()


def batch_diffusion_cross_attention(q_data, m_data, pair_logits, mask_q, mask_k, w_qg, w_kv, query_b,
                                    num_head, out_dtype=torch.bfloat16):
    """batch_diffusion_cross_attention_forward (csrc/Alpha_Attention.cpp:127-146).
    q_data [B, Sq, C], m_data [B, Sk, C] bf16; pair_logits [Bb, H, Sq, Sk] fp32 and
    masks [Bb, Sq] / [Bb, Sk] with B a multiple of Bb; returns [B, Sq, H, C/H]."""
    lib = _L.load()
    _gpu(q_data, "q_data", torch.bfloat16)
    _gpu(m_data, "m_data", torch.bfloat16)
    b, sq, c = q_data.shape
    sk = m_data.shape[1]
    if m_data.shape[0] != b or m_data.shape[2] != c:
        raise ValueError("m_data: batch / channel mismatch with q_data")
    bias_batches = b
    if pair_logits is not None:
        _gpu(pair_logits, "pair_logits", torch.float32)
        bias_batches = pair_logits.shape[0]
        if tuple(pair_logits.shape[1:]) != (num_head, sq, sk):
            raise ValueError("pair_logits: expected [Bb, H, Sq, Sk]")
    mq = mk = None
    if mask_q is not None:
        bias_batches = mask_q.shape[0]
        mq = _mask_f32(mask_q, (bias_batches, sq), "mask_q")
        mk = _mask_f32(mask_k, (bias_batches, sk), "mask_k")
    if pair_logits is not None and pair_logits.shape[0] != bias_batches:
        raise ValueError("pair_logits and masks must share their batch size")
    _gpu(w_qg, "w_qg", torch.bfloat16, (2 * c, c))
    _gpu(w_kv, "w_kv", torch.bfloat16, (2 * c, c))
    if query_b is not None:
        _gpu(query_b, "query_b", torch.float32, (c,))
    out = torch.empty((b, sq, num_head, c // num_head), dtype=out_dtype, device=q_data.device)
    nbytes = lib.af3_batch_diffusion_cross_attention_workspace_bytes(b, sq, sk, c)
    ws = _ws(nbytes, q_data.device)
    rc = lib.af3_batch_diffusion_cross_attention_forward(
        _p(q_data), _p(m_data), _p(pair_logits), _p(mq), _p(mk), bias_batches, _p(w_qg), _p(w_kv),
        _p(query_b), int(num_head), _p(out), _dt(out), b, sq, sk, c, _p(ws), ws.numel(),
        _stream(q_data.device))
    _L.check(rc, "af3_batch_diffusion_cross_attention_forward")
    return out


def gathered_cross_attention(q_data, atom_data, key_rows, pair_logits, mask_q, mask_k, w_qg, w_kv, query_b,
                             num_head, out_dtype=torch.bfloat16):
    """The cross-attention above with the key windows looked up inside the
    kernel (af3_gathered_cross_attention_forward).  q_data [samples * Bb, Sq, C]
    bf16; atom_data [samples, n_atoms, C] bf16; key_rows [Bb, Sk] int32 (row of
    atom_data, negative for a masked slot); pair_logits [Bb, H, Sq, Sk] fp32 or
    None; masks [Bb, Sq] / [Bb, Sk] or None.  Returns [samples * Bb, Sq, H, C/H]."""
    lib = _L.load()
    _gpu(q_data, "q_data", torch.bfloat16)
    _gpu(atom_data, "atom_data", torch.bfloat16)
    _gpu(key_rows, "key_rows", torch.int32)
    b, sq, c = q_data.shape
    if atom_data.dim() != 3 or atom_data.shape[2] != c:
        raise ValueError("atom_data: expected [samples, n_atoms, C]")
    samples, n_atoms = atom_data.shape[:2]
    bb, sk = key_rows.shape
    if b != samples * bb:
        raise ValueError("q_data: batch must be samples * windows")
    if getattr(key_rows, "_af3_checked_rows", None) != n_atoms:
        # (one device round trip; the tensor is marked so that it is paid once)
        if int(key_rows.max()) >= n_atoms:
            raise ValueError("key_rows: row index beyond atom_data")
        key_rows._af3_checked_rows = n_atoms
    if pair_logits is not None:
        _gpu(pair_logits, "pair_logits", torch.float32, (bb, num_head, sq, sk))
    mq = mk = None
    if mask_q is not None:
        mq = _mask_f32(mask_q, (bb, sq), "mask_q")
        mk = _mask_f32(mask_k, (bb, sk), "mask_k")
    _gpu(w_qg, "w_qg", torch.bfloat16, (2 * c, c))
    _gpu(w_kv, "w_kv", torch.bfloat16, (2 * c, c))
    if query_b is not None:
        _gpu(query_b, "query_b", torch.float32, (c,))
    out = torch.empty((b, sq, num_head, c // num_head), dtype=out_dtype, device=q_data.device)
    ws = _ws(lib.af3_gathered_cross_attention_workspace_bytes(b, sq, samples, n_atoms, c), q_data.device)
    rc = lib.af3_gathered_cross_attention_forward(
        _p(q_data), _p(atom_data), _p(key_rows), _p(pair_logits), _p(mq), _p(mk), bb, _p(w_qg), _p(w_kv),
        _p(query_b), int(num_head), _p(out), _dt(out), b, sq, sk, samples, n_atoms, c, _p(ws), ws.numel(),
        _stream(q_data.device))
    _L.check(rc, "af3_gathered_cross_attention_forward")
    return out


def transpose2d(x):
    """out[c, r] = x[r, c] for a contiguous bf16 GPU matrix (af3_transpose_bf16_forward);
    both sizes multiples of 8."""
    lib = _L.load()
    _gpu(x, "x", torch.bfloat16)
    if x.dim() != 2 or x.shape[0] % 8 or x.shape[1] % 8:
        raise ValueError("expected a 2-D tensor with both sizes multiples of 8")
    out = torch.empty((x.shape[1], x.shape[0]), dtype=torch.bfloat16, device=x.device)
    rc = lib.af3_transpose_bf16_forward(_p(x), _p(out), x.shape[0], x.shape[1], _stream(x.device))
    _L.check(rc, "af3_transpose_bf16_forward")
    return out


def masked_softmax_rows(logits, key_mask, pad_to: int = 8):
    """softmax over the last axis of fp32 `logits` [..., rows, cols] plus the additive key mask
    1e9 * (key_mask - 1) (key_mask [cols] 0/1 or None) -> bf16 [..., rows, ld], ld = cols rounded up to
    `pad_to`, tail columns zero (af3_masked_softmax_rows_forward)."""
    lib = _L.load()
    _gpu(logits, "logits", torch.float32)
    cols = logits.shape[-1]
    rows = logits.numel() // cols
    maskf = _mask_f32(key_mask, (cols,), "key_mask")
    ld = (cols + pad_to - 1) // pad_to * pad_to
    out = torch.empty(logits.shape[:-1] + (ld,), dtype=torch.bfloat16, device=logits.device)
    rc = lib.af3_masked_softmax_rows_forward(_p(logits), _p(maskf), _p(out), rows, cols, ld, _stream(logits.device))
    _L.check(rc, "af3_masked_softmax_rows_forward")
    return out


def narrow_linear_f32(x, w, relu_input: bool = False, residual=None):
    """y = (residual or 0) + relu?(x) @ w.T in fp32 for the narrow layers of the atom conditioning:
    x [..., k] fp32, w [n_out, k] fp32 with n_out 16 or 3 and k a multiple of 4 up to 128
    (af3_narrow_linear_f32_forward)."""
    lib = _L.load()
    _gpu(x, "x", torch.float32)
    _gpu(w, "w", torch.float32)
    n_out, k = w.shape
    if x.shape[-1] != k:
        raise ValueError(f"x: last axis {x.shape[-1]} != {k}")
    rows = x.numel() // k
    out = torch.empty(x.shape[:-1] + (n_out,), dtype=torch.float32, device=x.device)
    if residual is not None:
        _gpu(residual, "residual", torch.float32, out.shape)
    rc = lib.af3_narrow_linear_f32_forward(_p(x), _p(w), _p(residual), _p(out), rows, k, n_out, int(bool(relu_input)),
                                           _stream(x.device))
    _L.check(rc, "af3_narrow_linear_f32_forward")
    return out


def atom_pair_cond(row, col, token_pair, query_token, key_token, query_pos, key_pos, query_uid, key_uid,
                   w_offsets, w_distances, w_valid, w_mlp1, w_mlp2, w_mlp3):
    """The [S, Q, K, 16] pair conditioning of the windowed atom attention with its three-layer MLP in one
    pass (af3_atom_pair_cond_forward).  row [S, Q, 16], col [S, K, 16], token_pair [N, N, 16] or None,
    query_token [S, Q] / key_token [S, K] int32 (negative: empty slot), positions [S, Q, 3] / [S, K, 3],
    uids int32, weights fp32 in nn.Linear layout."""
    lib = _L.load()
    _gpu(row, "row", torch.float32)
    s, q, _ = row.shape
    k = col.shape[1]
    _gpu(col, "col", torch.float32, (s, k, 16))
    n_tok = 0
    if token_pair is not None:
        _gpu(token_pair, "token_pair", torch.float32)
        n_tok = token_pair.shape[0]
        if tuple(token_pair.shape) != (n_tok, n_tok, 16):
            raise ValueError(f"token_pair: expected [N, N, 16], got {tuple(token_pair.shape)}")
        _gpu(query_token, "query_token", torch.int32, (s, q))
        _gpu(key_token, "key_token", torch.int32, (s, k))
        if int(query_token.max()) >= n_tok or int(key_token.max()) >= n_tok:
            raise ValueError("token index beyond token_pair")
    _gpu(query_pos, "query_pos", torch.float32, (s, q, 3))
    _gpu(key_pos, "key_pos", torch.float32, (s, k, 3))
    _gpu(query_uid, "query_uid", torch.int32, (s, q))
    _gpu(key_uid, "key_uid", torch.int32, (s, k))
    _gpu(w_offsets, "w_offsets", torch.float32, (16, 3))
    _gpu(w_distances, "w_distances", torch.float32, (16, 1))
    _gpu(w_valid, "w_valid", torch.float32, (16, 1))
    for name, w in (("w_mlp1", w_mlp1), ("w_mlp2", w_mlp2), ("w_mlp3", w_mlp3)):
        _gpu(w, name, torch.float32, (16, 16))
    out = torch.empty((s, q, k, 16), dtype=torch.float32, device=row.device)
    rc = lib.af3_atom_pair_cond_forward(_p(row), _p(col), _p(token_pair), _p(query_token), _p(key_token), n_tok,
                                        _p(query_pos), _p(key_pos), _p(query_uid), _p(key_uid), _p(w_offsets),
                                        _p(w_distances), _p(w_valid), _p(w_mlp1), _p(w_mlp2), _p(w_mlp3), _p(out), s, q, k,
                                        _stream(row.device))
    _L.check(rc, "af3_atom_pair_cond_forward")
    return out


def atom_pair_logits(pair_cond, ln_w, w, num_blocks: int, num_head: int):
    """LayerNorm (weight, no bias) and 16 -> blocks x heads projection of the atom pair conditioning, written as
    the [blocks, S, heads, Q, K] fp32 bias planes of the windowed attention (af3_atom_pair_logits_forward).
    pair_cond [S, Q, K, 16] fp32; ln_w [16] fp32; w [blocks * heads, 16] fp32."""
    lib = _L.load()
    _gpu(pair_cond, "pair_cond", torch.float32)
    if pair_cond.dim() != 4 or pair_cond.shape[-1] != 16:
        raise ValueError(f"pair_cond: expected [S, Q, K, 16], got {tuple(pair_cond.shape)}")
    s, q, k, _ = pair_cond.shape
    _gpu(ln_w, "ln_w", torch.float32, (16,))
    _gpu(w, "w", torch.float32, (num_blocks * num_head, 16))
    out = torch.empty((num_blocks, s, num_head, q, k), dtype=torch.float32, device=pair_cond.device)
    rc = lib.af3_atom_pair_logits_forward(_p(pair_cond), _p(ln_w), _p(w), _p(out), s, q, k, int(num_blocks), int(num_head),
                                          _stream(pair_cond.device))
    _L.check(rc, "af3_atom_pair_logits_forward")
    return out


def pair_cond_init(pair, token_ids, ln_w, w_pair, g_hot, g_sum, in_scale: float = 1.0,
                   max_relative_idx: int = 32, max_relative_chain: int = 2):
    """Linear(LayerNorm([pair | relative encoding])) in one pass (af3_pair_cond_init_forward).
    pair [N, N, 128] fp32 or bf16; token_ids = (asym_id, residue_index, token_index, entity_id, sym_id), each
    [N] int32; ln_w [128] fp32; w_pair [128, 128] bf16; g_hot [4 r + 2 c + 7, 128] fp32 and g_sum [128] fp32
    as DiffusionHead packs them.  Returns [N, N, 128] fp32."""
    lib = _L.load()
    _gpu(pair, "pair", None)
    n = pair.shape[0]
    if pair.dim() != 3 or pair.shape[1] != n or pair.shape[2] != 128:
        raise ValueError(f"pair: expected [N, N, 128], got {tuple(pair.shape)}")
    if len(token_ids) != 5:
        raise ValueError("token_ids: (asym_id, residue_index, token_index, entity_id, sym_id)")
    for name, t in zip(("asym_id", "residue_index", "token_index", "entity_id", "sym_id"), token_ids):
        _gpu(t, name, torch.int32, (n,))
    n_rel = 4 * max_relative_idx + 2 * max_relative_chain + 7
    _gpu(ln_w, "ln_w", torch.float32, (128,))
    _gpu(w_pair, "w_pair", torch.bfloat16, (128, 128))
    _gpu(g_hot, "g_hot", torch.float32, (n_rel, 128))
    _gpu(g_sum, "g_sum", torch.float32, (128,))
    out = torch.empty((n, n, 128), dtype=torch.float32, device=pair.device)
    rc = lib.af3_pair_cond_init_forward(_p(pair), _dt(pair), float(in_scale), *[_p(t) for t in token_ids],
                                        int(max_relative_idx), int(max_relative_chain), _p(ln_w), _p(w_pair),
                                        _p(g_hot), _p(g_sum), _p(out), n, _stream(pair.device))
    _L.check(rc, "af3_pair_cond_init_forward")
    return out


def batched_nt_product(a, b, out=None):
    """out[i] = a[i] @ b[i].T for a [batch, m, k], b [batch, n, k] bf16 (af3_batched_nt_product_forward)."""
    lib = _L.load()
    _gpu(a, "a", torch.bfloat16)
    _gpu(b, "b", torch.bfloat16)
    if a.dim() != 3 or b.dim() != 3 or a.shape[0] != b.shape[0] or a.shape[2] != b.shape[2]:
        raise ValueError("expected a [batch, m, k] and b [batch, n, k]")
    batch, m, k = a.shape
    n = b.shape[1]
    if k % 8:
        raise ValueError("k must be a multiple of 8 (pad with zero columns)")
    if out is None:
        out = torch.empty((batch, m, n), dtype=torch.bfloat16, device=a.device)
    else:
        _gpu(out, "out", torch.bfloat16, (batch, m, n))
    rc = lib.af3_batched_nt_product_forward(_p(a), _p(b), _p(out), batch, m, n, k, _stream(a.device))
    _L.check(rc, "af3_batched_nt_product_forward")
    return out


def pair_logits(pair, norm_weight, norm_bias, w_padded, n_out):
    """LayerNorm + projection of the pair tensor to [n_out, N, N] fp32 logits
    (nn/d_pairformer.py:160-162, nn/d_diffusion_transformer.py:299-305)."""
    lib = _L.load()
    _gpu(pair, "pair")
    if pair.dim() != 3 or pair.shape[0] != pair.shape[1] or pair.shape[2] != 128:
        raise ValueError(f"pair: expected [N, N, 128], got {tuple(pair.shape)}")
    n = pair.shape[0]
    _gpu(norm_weight, "norm_weight", torch.float32, (128,))
    if norm_bias is not None:
        _gpu(norm_bias, "norm_bias", torch.float32, (128,))
    _gpu(w_padded, "w_padded", torch.bfloat16)
    if w_padded.dim() != 2 or w_padded.shape[1] != 128 or w_padded.shape[0] % 32 or w_padded.shape[0] < n_out:
        raise ValueError("w_padded: expected [roundup(n_out, 32), 128]")
    out = torch.empty((n_out, n, n), dtype=torch.float32, device=pair.device)
    rc = lib.af3_pair_logits_forward(_p(pair), _dt(pair), _p(norm_weight), _p(norm_bias), _p(w_padded),
                                     int(n_out), _p(out), n, _stream(pair.device))
    _L.check(rc, "af3_pair_logits_forward")
    return out


def layer_norm(x, weight=None, bias=None, scale=None, shift=None):
    """Row LayerNorm (+ optional adaptive scale/shift) -> bf16.  scale/shift are
    fp32 views [cond_rows, C] that may be column slices of one wider tensor."""
    lib = _L.load()
    _gpu(x, "x")
    c = x.shape[-1]
    rows = x.numel() // c
    for nm, t in (("weight", weight), ("bias", bias)):
        if t is not None:
            _gpu(t, nm, torch.float32, (c,))
    cond_rows = cond_ld = 0
    if scale is not None:
        for nm, t in (("scale", scale), ("shift", shift)):
            if not t.is_cuda or t.dtype != torch.float32 or t.dim() != 2 or t.shape[1] != c or t.stride(1) != 1:
                raise ValueError(f"{nm}: expected an fp32 GPU matrix [cond_rows, {c}] with unit column stride")
        if scale.stride(0) != shift.stride(0) or scale.shape[0] != shift.shape[0]:
            raise ValueError("scale and shift must share rows and row stride")
        cond_rows, cond_ld = scale.shape[0], scale.stride(0)
        if rows % cond_rows:
            raise ValueError("rows must be a multiple of the conditioning rows")
    y = torch.empty(x.shape, dtype=torch.bfloat16, device=x.device)
    rc = lib.af3_layer_norm_forward(_p(x), _dt(x), _p(y), rows, c, _p(weight), _p(bias), _p(scale), _p(shift),
                                    cond_rows, cond_ld, _stream(x.device))
    _L.check(rc, "af3_layer_norm_forward")
    return y


def linear(x, w, bias=None, out_dtype=torch.bfloat16, mode=_L.LINEAR_PLAIN, alpha=1.0, sigmoid=False,
           gate=None, residual=None, out=None):
    """y = epilogue(x @ w.T) on bf16 MFMA (af3_linear_forward)."""
    lib = _L.load()
    _gpu(x, "x", torch.bfloat16)
    _gpu(w, "w", torch.bfloat16)
    k = x.shape[-1]
    m = x.numel() // k
    n = w.shape[0]
    if w.dim() != 2 or w.shape[1] != k:
        raise ValueError(f"w: expected [N, {k}], got {tuple(w.shape)}")
    if bias is not None:
        _gpu(bias, "bias", torch.float32, (n,))
    n_out = n // 2 if mode == _L.LINEAR_SWIGLU else n
    shape = tuple(x.shape[:-1]) + (n_out,)
    if mode == _L.LINEAR_REGROUP32:
        if m % 32 or n % 32:
            raise ValueError("regrouped store: rows of x and of w must be multiples of 32")
        shape = ((m // 32) * (n // 32), 1024)
    if out is None:
        out = torch.empty(shape, dtype=out_dtype, device=x.device)
    else:
        _gpu(out, "out", None, shape)
    gate_rows = gate_ld = 0
    if gate is not None and mode == _L.LINEAR_ROWGATE_RES:
        _gpu(gate, "gate", torch.float32)
        gate_rows = gate.numel()
        if m % gate_rows:
            raise ValueError("rows must be a multiple of the gate rows")
    elif gate is not None:
        if gate.dim() == 2 and not gate.is_contiguous() and gate.stride(1) == 1 and gate.stride(0) >= n:
            # a column slice of a wider tensor, used in place: rows gate_ld floats apart
            if not gate.is_cuda or gate.dtype != torch.float32:
                raise ValueError("gate: expected an fp32 tensor on the GPU")
            gate_ld = gate.stride(0)
        else:
            _gpu(gate, "gate", torch.float32)
        if gate.shape[-1] != n:
            raise ValueError("gate: last dimension must equal the output width")
        gate_rows = gate.numel() // n
        if m % gate_rows:
            raise ValueError("rows must be a multiple of the gate rows")
    res_dt = 0
    if residual is not None:
        _gpu(residual, "residual", None, shape)
        res_dt = _dt(residual)
    rc = lib.af3_linear_forward(_p(x), _p(w), _p(bias), _p(out), _dt(out), m, n, k, int(mode), float(alpha),
                                int(bool(sigmoid)), _p(gate), gate_rows, gate_ld, _p(residual), res_dt,
                                _stream(x.device))
    _L.check(rc, "af3_linear_forward")
    return out


# ---------------------------------------------------------- kernel-level entries
def triangle_contraction(a, b, out=None):
    """t[c] = a[c] @ b[c].T for channel-major bf16 operands [128, N, ld], ld = N
    rounded up to 8 with zero padding (the contraction stage alone)."""
    lib = _L.load()
    _gpu(a, "a", torch.bfloat16)
    _gpu(b, "b", torch.bfloat16, a.shape)
    if a.dim() != 3 or a.shape[0] != 128 or a.shape[2] != (a.shape[1] + 7) // 8 * 8:
        raise ValueError("a: expected [128, N, roundup(N, 8)]")
    if out is None:
        out = torch.empty_like(a)
    else:
        _gpu(out, "out", torch.bfloat16, a.shape)
    rc = lib.af3_triangle_contraction_forward(_p(a), _p(b), _p(out), a.shape[1], _stream(a.device))
    _L.check(rc, "af3_triangle_contraction_forward")
    return out


def pack_pair_bias(bias):
    """[4, N, >=N] pair bias (already multiplied by log2(e)) -> the MFMA-fragment
    order the attention core reads: fp16 [4, ceil(N/32), ceil(N/64), 4, 32, 16] with
    packed[h, qb, kt, i, j, c] = bias[h, 32 qb + j, 64 kt + 16 i + c], zero where
    the query or key index is >= N."""
    if bias.dim() != 3 or bias.shape[0] != 4 or bias.shape[2] < bias.shape[1]:
        raise ValueError("bias: expected [4, N, >=N]")
    n = bias.shape[1]
    qb, kt = (n + 31) // 32, (n + 63) // 64
    full = torch.zeros((4, qb * 32, kt * 64), dtype=torch.float16, device=bias.device)
    full[:, :n, :n] = bias[:, :, :n].float().clamp(-65504.0, 65504.0).to(torch.float16)
    return full.view(4, qb, 32, kt, 4, 16).permute(0, 1, 3, 4, 2, 5).contiguous()


def pack_vt(vt):
    """[N, 4, 32, >=N] transposed values -> the column order the attention core reads:
    bf16 [N, 4, 32, ld], ld = N rounded up to 16, key k at column
    (k & ~12) | ((k & 8) >> 1) | ((k & 4) << 1), columns of keys >= N zero."""
    if vt.dim() != 4 or vt.shape[1] != 4 or vt.shape[2] != 32 or vt.shape[3] < vt.shape[0]:
        raise ValueError("vt: expected [N, 4, 32, >=N]")
    n = vt.shape[0]
    ld = (n + 15) // 16 * 16
    full = torch.zeros((n, 4, 32, ld), dtype=torch.bfloat16, device=vt.device)
    full[..., :n] = vt[..., :n].to(torch.bfloat16)
    # swapping the two middle quads of every group of 16 is its own inverse
    return full.view(n, 4, 32, ld // 16, 4, 4)[..., [0, 2, 1, 3], :].reshape(n, 4, 32, ld).contiguous()


def grid_attention_core(q, k, vt, pair_bias, mask, out=None):
    """The flash-attention stage of the triangle attention on projected, head-major
    operands in base-2 form: q, k bf16 [N, 4, N, 32] (q and the bias
    pre-multiplied by log2(e)), vt from pack_vt(), pair_bias from
    pack_pair_bias() or None.  Returns softmax(q k^T + bias) v as [N*N, 128]
    bf16 (the output gate belongs to the operator's last kernel)."""
    lib = _L.load()
    _gpu(q, "q", torch.bfloat16)
    if q.dim() != 4 or q.shape[1] != 4 or q.shape[3] != 32 or q.shape[0] != q.shape[2]:
        raise ValueError("q: expected [N, 4, N, 32]")
    n = q.shape[0]
    ld = (n + 15) // 16 * 16
    _gpu(k, "k", torch.bfloat16, q.shape)
    _gpu(vt, "vt", torch.bfloat16, (n, 4, 32, ld))
    if pair_bias is not None:
        _gpu(pair_bias, "pair_bias", torch.float16, (4, (n + 31) // 32, (n + 63) // 64, 4, 32, 16))
    maskf = _mask_f32(mask, (n, n), "mask")
    if out is None:
        out = torch.empty((n * n, 128), dtype=torch.bfloat16, device=q.device)
    rc = lib.af3_grid_attention_core_forward(_p(q), _p(k), _p(vt), _p(pair_bias), _p(maskf), _p(out), n,
                                             _stream(q.device))
    _L.check(rc, "af3_grid_attention_core_forward")
    return out


# --------------------------------------------------------------- fp32 check mode
def _f32(t, name):
    _gpu(t, name, torch.float32)
    return t


def ck_gemm(a, b, *, m, n, k, batch=1, lda, ldb, ka=1, kb=1, sa=0, sb=0, out=None, bias=None, alpha=1.0,
            sigmoid=False, mul=None, add=None):
    """fp32 C[b][m][n] = epi(sum_k A(b,m,k) B(b,n,k)) with explicit element strides
    (af3_check_gemm_f32); C is dense [batch, m, n]."""
    lib = _L.load()
    if not (a.is_cuda and b.is_cuda and a.dtype == torch.float32 and b.dtype == torch.float32):
        raise ValueError("ck_gemm: operands must be fp32 GPU tensors")
    if out is None:
        out = torch.empty((batch, m, n) if batch > 1 else (m, n), dtype=torch.float32, device=a.device)
    mul_rows = ld_mul = 0
    if mul is not None:
        _f32(mul, "mul")
        mul_rows, ld_mul = mul.numel() // n, n
    ld_add = s_add = 0
    if add is not None:
        _f32(add, "add")
        ld_add, s_add = n, m * n
    if bias is not None:
        _f32(bias, "bias")
    rc = lib.af3_check_gemm_f32(_p(a), _p(b), _p(out), m, n, k, batch, lda, ka, ldb, kb, n, sa, sb, m * n,
                                _p(bias), float(alpha), int(bool(sigmoid)), _p(mul), mul_rows, ld_mul,
                                _p(add), ld_add, s_add, _stream(a.device))
    _L.check(rc, "af3_check_gemm_f32")
    return out


def ck_linear(x, w, bias=None, alpha=1.0, sigmoid=False, mul=None, add=None):
    """fp32 y = epi(x @ w.T) for contiguous x [..., K], w [N, K]."""
    _f32(x, "x")
    _f32(w, "w")
    k = x.shape[-1]
    m = x.numel() // k
    n = w.shape[0]
    y = ck_gemm(x, w, m=m, n=n, k=k, lda=k, ldb=k, bias=bias, alpha=alpha, sigmoid=sigmoid, mul=mul, add=add)
    return y.reshape(tuple(x.shape[:-1]) + (n,))


def ck_layer_norm(x, weight=None, bias=None, scale=None, shift=None):
    lib = _L.load()
    _f32(x, "x")
    c = x.shape[-1]
    rows = x.numel() // c
    cond_rows = cond_ld = 0
    if scale is not None:
        cond_rows, cond_ld = scale.shape[0], scale.stride(0)
    y = torch.empty_like(x)
    rc = lib.af3_check_layer_norm_f32(_p(x), _p(y), rows, c, _p(weight), _p(bias), _p(scale), _p(shift),
                                      cond_rows, cond_ld, _stream(x.device))
    _L.check(rc, "af3_check_layer_norm_f32")
    return y


def ck_elementwise(op, x0, x1, x2, y0, y1, n0, n1, flag):
    lib = _L.load()
    rc = lib.af3_check_elementwise_f32(int(op), _p(x0), _p(x1), _p(x2), _p(y0), _p(y1), int(n0), int(n1), int(flag),
                                       _stream(x0.device))
    _L.check(rc, "af3_check_elementwise_f32")


def ck_attention(q, k, v, num_head, bias=None, bias_strides=(0, 0, 0, 1), bias_mod=0, key_mask=None, km_sb=0,
                 qpad=None, kpad=None):
    """fp32 attention; q [B, Sq, H*d], k / v [B, Sk, H*d] (any batch / position
    strides, unit channel stride); bias addressed with explicit element strides
    (batch, head, query, key)."""
    lib = _L.load()
    for nm, t in (("q", q), ("k", k), ("v", v)):
        if not (t.is_cuda and t.dtype == torch.float32 and t.dim() == 3 and t.stride(2) == 1):
            raise ValueError(f"{nm}: expected an fp32 GPU tensor [B, S, C] with unit channel stride")
    b, sq, c = q.shape
    sk = k.shape[1]
    d = c // num_head
    out = torch.empty((b, sq, c), dtype=torch.float32, device=q.device)
    km = None if key_mask is None else key_mask.to(torch.float32).contiguous()
    qp = None if qpad is None else qpad.to(torch.float32).contiguous()
    kp = None if kpad is None else kpad.to(torch.float32).contiguous()
    rc = lib.af3_check_attention_f32(
        _p(q), _p(k), _p(v), _p(out), q.stride(0), q.stride(1), k.stride(0), k.stride(1), v.stride(0), v.stride(1),
        out.stride(0), out.stride(1), b, int(num_head), sq, sk, d, _p(bias), *[int(s) for s in bias_strides],
        int(bias_mod), _p(km), int(km_sb), _p(qp), _p(kp), _stream(q.device))
    _L.check(rc, "af3_check_attention_f32")
    return out
