"""Shared plumbing of the drop-in modules."""

from __future__ import annotations

import torch
import torch.nn as nn


_CHECK_MODE = False


class check_mode:
    """Context manager / switch for the fp32 check mode: inside it every module's
    `forward` runs the plain fp32 kernels of `check.py` (fp32 tensors in and out,
    results returned as new tensors) instead of the bf16 MFMA path."""

    def __init__(self, enabled: bool = True):
        self.enabled = enabled

    def __enter__(self):
        global _CHECK_MODE
        self._old, _CHECK_MODE = _CHECK_MODE, self.enabled
        return self

    def __exit__(self, *exc):
        global _CHECK_MODE
        _CHECK_MODE = self._old


def in_check_mode() -> bool:
    return _CHECK_MODE


def drop_mesh(args):
    """The reference's distributed classes take a device mesh as their first
    positional argument (e.g. nn/d_attention.py:24); on one GPU it carries no
    information, so it is accepted and ignored."""
    if args and not isinstance(args[0], (int, bool, float)):
        return args[1:]
    return args


def bf16(t: torch.Tensor) -> torch.Tensor:
    return t.detach().to(torch.bfloat16).contiguous()


def f32(t: torch.Tensor) -> torch.Tensor:
    return t.detach().to(torch.float32).contiguous()


def pad_to(w: torch.Tensor, *shape: int) -> torch.Tensor:
    """`w` in the leading corner of a zero tensor of `shape`."""
    out = torch.zeros(shape, dtype=w.dtype, device=w.device)
    out[tuple(slice(0, d) for d in w.shape)] = w.detach()
    return out


def pad_channels(x: torch.Tensor, width: int = 128) -> torch.Tensor:
    """[..., c] -> [..., width] with zeros behind the c real channels (a new tensor)."""
    return torch.nn.functional.pad(x, (0, width - x.shape[-1])).contiguous()


def pad_rows(w: torch.Tensor, multiple: int) -> torch.Tensor:
    rows = w.shape[0]
    target = (rows + multiple - 1) // multiple * multiple
    if target == rows:
        return w.contiguous()
    out = torch.zeros((target,) + tuple(w.shape[1:]), dtype=w.dtype, device=w.device)
    out[:rows] = w
    return out


def pack_swiglu(w1: torch.Tensor, block: int) -> torch.Tensor:
    """Re-order the rows of a GLU weight [2*hidden, c] (silu half first, linear
    half second) into alternating blocks of `block` silu rows and the `block`
    matching linear rows."""
    hidden = w1.shape[0] // 2
    if hidden % block:
        raise ValueError(f"hidden size {hidden} is not a multiple of {block}")
    a = w1[:hidden].reshape(hidden // block, block, -1)
    b = w1[hidden:].reshape(hidden // block, block, -1)
    return torch.cat([a, b], dim=1).reshape(2 * hidden, -1).contiguous()


class HipModule(nn.Module):
    """A module whose `forward` runs on the HIP kernels.

    The packed device-side weights are derived from the nn.Parameters by
    `load_hip_params()` (the counterpart of the reference's
    `load_xsmm_params()`, e.g. nn/d_triangle_multiplication.py:126-138); it runs
    lazily on the first forward and again after `invalidate()`.  `xsmm_forward`
    and `load_xsmm_params` are kept as aliases so that the reference's plug-in
    loop (run_inference.py:197-218) binds these modules unchanged.
    """

    def __init__(self):
        super().__init__()
        self._packed = None

    def invalidate(self):
        """Drop the packed weights of this module and of every HIP module below
        it, however deeply nested (blocks usually sit in an nn.ModuleList)."""
        for m in self.modules():
            if isinstance(m, HipModule):
                m._packed = None

    def _apply(self, fn, *a, **k):  # .to() / .cuda() move parameters: repack afterwards
        self._packed = None
        return super()._apply(fn, *a, **k)

    def load_state_dict(self, *a, **k):
        self.invalidate()
        return super().load_state_dict(*a, **k)

    def _pack(self):
        raise NotImplementedError

    def load_hip_params(self):
        for m in self.modules():
            if isinstance(m, HipModule):
                m._packed = m._pack()
        return self

    def packed(self):
        if self._packed is None:
            self._packed = self._pack()
        return self._packed

    # reference plug-in protocol
    def load_xsmm_params(self):
        return self.load_hip_params()

    def hip_forward(self, *a, **k):
        return self.forward(*a, **k)

    def xsmm_forward(self, *a, **k):
        return self.forward(*a, **k)


def enable_hip(model: nn.Module) -> int:
    """Counterpart of ModelRunner.enable_xsmm (run_inference.py:197-218): packs
    the weights of every HIP module under `model`.  Returns how many were bound."""
    n = 0
    for m in model.modules():
        if isinstance(m, HipModule):
            m._packed = m._pack()
            n += 1
    return n
