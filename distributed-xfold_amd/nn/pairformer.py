"""Pairformer block (AF3 Algorithm 17, lines 2-8) and the trunk stack."""

from __future__ import annotations

from typing import Optional

import torch
import torch.nn as nn

from .. import check, ops
from .attention import GridSelfAttention
from .base import HipModule, bf16, drop_mesh, f32, in_check_mode, pad_channels, pad_rows
from .diffusion_transformer import SelfAttention
from .primitives import Transition
from .triangle_multiplication import TriangleMultiplication


class PairformerBlock(HipModule):
    """Same constructor keywords, sub-module names and call signature as the
    reference's DistributePairformerBlock (nn/d_pairformer.py:32-106).

    As in the reference, `pair` and `single` are updated IN PLACE (`pair +=`,
    nn/d_pairformer.py:122-168) and returned; each of the seven sub-operations
    adds its update inside its last kernel instead of a separate pass."""

    def __init__(self, *args, n_heads: int = 16, c_pair: int = 128, c_single: int = 384,
                 c_hidden_mul: int = 128, n_heads_pair: int = 4, num_intermediate_factor: int = 4,
                 with_single: bool = True) -> None:
        super().__init__()
        args = drop_mesh(args)
        vals = list(args) + [n_heads, c_pair, c_single, c_hidden_mul, n_heads_pair, num_intermediate_factor,
                             with_single][len(args):]
        n_heads, c_pair, c_single, c_hidden_mul, n_heads_pair, num_intermediate_factor, with_single = vals[:7]
        self.n_heads, self.c_pair, self.c_single = n_heads, c_pair, c_single
        self.with_single, self.num_intermediate_factor = with_single, num_intermediate_factor
        self.triangle_multiplication_outgoing = TriangleMultiplication(c_pair=c_pair, _outgoing=True)
        self.triangle_multiplication_incoming = TriangleMultiplication(c_pair=c_pair, _outgoing=False)
        self.pair_attention1 = GridSelfAttention(c_pair=c_pair, num_head=n_heads_pair, transpose=False)
        self.pair_attention2 = GridSelfAttention(c_pair=c_pair, num_head=n_heads_pair, transpose=True)
        self.pair_transition = Transition(c_x=c_pair, num_intermediate_factor=num_intermediate_factor)
        if with_single:
            self.single_pair_logits_norm = nn.LayerNorm(c_pair)
            self.single_pair_logits_projection = nn.Linear(c_pair, n_heads, bias=False)
            self.single_attention_ = SelfAttention(c_x=c_single, num_head=n_heads, use_single_cond=False,
                                                   use_batch_infer=False)
            self.single_transition = Transition(c_x=c_single)

    def _pack(self):
        if not self.with_single:
            return {}
        return dict(ln_w=f32(self.single_pair_logits_norm.weight), ln_b=f32(self.single_pair_logits_norm.bias),
                    w_logits=pad_rows(bf16(self.single_pair_logits_projection.weight), 32))

    def forward(self, pair: torch.Tensor, pair_mask: torch.Tensor, single: Optional[torch.Tensor] = None,
                seq_mask: Optional[torch.Tensor] = None, head: int = 0,
                single_stream: Optional["torch.cuda.Stream"] = None):
        """pair [N, N, c_pair], pair_mask [N, N], single [N, c_single], seq_mask [N].

        `single_stream` (not in the reference): run the update of `single` (attention and
        transition, a chain of small kernels that leave most of the GPU idle) on that
        stream, behind the pair-bias projection, and return without waiting for it.  The
        caller then owns the ordering: `single` may only be touched on that stream until
        the caller's stream has waited for it (PairformerStack does both)."""
        if in_check_mode():
            return check.pairformer_block(self, pair, pair_mask, single, seq_mask)
        if not pair.is_contiguous():
            raise ValueError("pair must be contiguous (it is updated in place)")
        if self.c_pair < 128 and not self.with_single and self.pair_attention1.padded:
            # the 64-channel block of the template embedding (nn/d_template.py:198-201): the five operators run
            # on the 128-channel kernels over one zero-padded copy of the tensor, which stays padded in between
            x = pad_channels(pair)
            self.triangle_multiplication_outgoing.run_padded(x, pair_mask, residual=True)
            self.triangle_multiplication_incoming.run_padded(x, pair_mask, residual=True)
            self.pair_attention1.run_padded(x, pair_mask, residual=True)
            self.pair_attention2.run_padded(x, pair_mask, residual=True)
            self.pair_transition.run_padded(x, residual=True)
            pair.copy_(x[..., :self.c_pair])
            return pair
        self.triangle_multiplication_outgoing.run(pair, pair_mask, residual=True)
        self.triangle_multiplication_incoming.run(pair, pair_mask, residual=True)
        self.pair_attention1.run(pair, pair_mask, residual=True)
        self.pair_attention2.run(pair, pair_mask, residual=True)
        self.pair_transition.run(pair, residual=True)
        if not self.with_single:
            return pair
        if not single.is_contiguous():
            raise ValueError("single must be contiguous (it is updated in place)")
        p = self.packed()
        # the only reader of `pair` on the single path: it stays on the caller's stream, in front of
        # whatever updates `pair` next
        logits = ops.pair_logits(pair, p["ln_w"], p["ln_b"], p["w_logits"], self.n_heads)
        if single_stream is None:
            self.single_attention_.run(single, seq_mask, logits, None, residual=True)
            self.single_transition.run(single, residual=True)
            return pair, single
        single_stream.wait_stream(torch.cuda.current_stream(pair.device))
        logits.record_stream(single_stream)
        with torch.cuda.stream(single_stream):
            self.single_attention_.run(single, seq_mask, logits, None, residual=True)
            self.single_transition.run(single, residual=True)
        return pair, single


_SIDE_STREAMS = {}


def _side_stream(device) -> "torch.cuda.Stream":
    """One extra stream per device (default priority), shared by every trunk loop of the process."""
    key = torch.device(device).index or 0
    if key not in _SIDE_STREAMS:
        _SIDE_STREAMS[key] = torch.cuda.Stream(device=device)
    return _SIDE_STREAMS[key]


def pairformer_loop(blocks, pair, pair_mask, single, seq_mask, overlap_single: bool = True):
    """Run Pairformer blocks one after the other (the loop of d_alphafold3.py:242-244).

    `overlap_single`: inside the loop nothing reads `single` but the next block's own
    single update, so each block's single update runs on a second stream while the next
    block's pair operators, which fill the GPU, run on the caller's; the caller's stream
    waits for the second one before the loop returns.  The results are the same bits
    either way."""
    if in_check_mode() or not overlap_single or not pair.is_cuda:
        for blk in blocks:
            pair, single = blk(pair, pair_mask, single, seq_mask)
        return pair, single
    main = torch.cuda.current_stream(pair.device)
    side = _side_stream(pair.device)
    side.wait_stream(main)          # whatever produced `single` and `seq_mask`
    for blk in blocks:
        pair, single = blk(pair, pair_mask, single, seq_mask, single_stream=side)
    main.wait_stream(side)
    return pair, single


class PairformerStack(HipModule):
    """The trunk loop of DistributeEvoformer.forward (d_alphafold3.py:242-244); see pairformer_loop."""

    def __init__(self, num_blocks: int = 48, overlap_single: bool = True, **block_kwargs) -> None:
        super().__init__()
        self.trunk_pairformer = nn.ModuleList([PairformerBlock(**block_kwargs) for _ in range(num_blocks)])
        self.overlap_single = overlap_single

    def _pack(self):
        return {}

    def forward(self, pair, pair_mask, single, seq_mask):
        return pairformer_loop(self.trunk_pairformer, pair, pair_mask, single, seq_mask, self.overlap_single)
