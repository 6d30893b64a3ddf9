"""Decoder block with the norm after the sum, on an fp32 residual stream:

    x <- norm(alpha x + mixer(shift(x))),   x <- norm(alpha x + ff(x))

``norm`` is an RMS norm taken over each of ``groups`` equal consecutive parts of the row and multiplied by a weight;
``shift`` replaces what the mixer reads by ``x_t + (x_{t-1} - x_t) mix`` (zeros before a sequence's first token), so the
last row of every sequence is part of its state.  The stream stays fp32 whatever the activation type; a sublayer reads
and returns activations (bf16 or fp32).  Beside ``StreamBlock`` (``stream_block.py``: norms on both sides of a sublayer,
added to the stream) and ``DecoderBlock`` (``block.py``: a bf16 stream with the add folded into the next norm).
"""

from __future__ import annotations

from typing import Optional

import torch

from .. import hip_ops
from .stream_block import StepLayout


class TokenShift(torch.nn.Module):
    def __init__(self, mix: torch.Tensor):
        super().__init__()
        self.register_buffer("mix", mix.float().contiguous())

    def forward(self, x: torch.Tensor, out_dtype: torch.dtype, layout: StepLayout, state: Optional[torch.Tensor]) -> torch.Tensor:
        """``state`` fp32 ``[slots, W]``: every sequence's last row, read and rewritten."""
        return hip_ops.token_shift(x, self.mix, state, out_dtype, layout.query_start_loc, layout.context_lens, layout.slot_idx)


class AddGroupNorm(torch.nn.Module):
    """``x <- norm(alpha x + y (+ y2))`` in place on the stream; ``copy_dtype``: also returns the result rounded to that type."""

    def __init__(self, weight: torch.Tensor, groups: int, eps: float, alpha: float = 1.0):
        super().__init__()
        self.register_buffer("weight", weight.float().contiguous())
        self.groups, self.eps, self.alpha = int(groups), float(eps), float(alpha)

    def forward(self, x: torch.Tensor, y: Optional[torch.Tensor], y2: Optional[torch.Tensor] = None,
                copy_dtype: Optional[torch.dtype] = None, in_place: bool = True) -> torch.Tensor:
        return hip_ops.add_group_norm(x, y, self.weight, self.groups, self.eps, self.alpha, y2, in_place, copy_dtype)


class PostNormBlock(torch.nn.Module):
    """One decoder layer: token shift, mixer, norm; then (optionally) feed-forward, norm.  ``mixer(h, layout, state)``
    returns activations; ``mlp(h)`` returns activations or a pair of them (routed and shared experts) that the norm adds."""

    def __init__(self, shift: Optional[TokenShift], mixer: torch.nn.Module, mixer_norm: AddGroupNorm,
                 mlp: Optional[torch.nn.Module] = None, mlp_norm: Optional[AddGroupNorm] = None):
        super().__init__()
        self.shift, self.mixer, self.mixer_norm, self.mlp, self.mlp_norm = shift, mixer, mixer_norm, mlp, mlp_norm

    def forward(self, x: torch.Tensor, act_dtype: torch.dtype, layout: StepLayout, mixer_state, shift_state: Optional[torch.Tensor]) -> torch.Tensor:
        if self.shift is not None:
            h = self.shift(x, act_dtype, layout, shift_state)
        else:
            h = x if act_dtype == torch.float32 else x.to(act_dtype)
        y = self.mixer(h, layout, mixer_state)
        if self.mlp is None:
            return self.mixer_norm(x, y)
        if act_dtype == torch.float32:
            h = self.mixer_norm(x, y)                        # the feed-forward reads the stream itself
        else:
            h = self.mixer_norm(x, y, copy_dtype=act_dtype)   # ... or its rounded copy, written by the same launch
        y = self.mlp(h)
        y, y2 = y if isinstance(y, tuple) else (y, None)
        self.mlp_norm(x, y, y2)
        return x
