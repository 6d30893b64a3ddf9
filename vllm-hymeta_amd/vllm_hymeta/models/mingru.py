"""minGRU mixer: a gated recurrence whose gates read only the current token,

    z = sigmoid(W_z h + b_z),  u = W_x h + b_x,  cand = u + 1/2 (u >= 0) | sigmoid(u) (u < 0)
    S_t = (1 - z) S_{t-1} + z cand,   out = W_o (S_t * silu(W_g h))

(the recurrence of "Were RNNs All We Needed?", Feng et al. 2024, with its piecewise candidate activation).  The three
input projections are one linear layer; the recurrence runs in ``hip_ops.mingru`` with the state fp32, one slot per
sequence.  Beside ``GatedLinearAttention`` (``model_for_7B/gla_attention.py``), whose state is a matrix per head.
"""

from __future__ import annotations

import torch

from .. import hip_ops
from ..linear import HymetaLinear


class MinGRUMixer(torch.nn.Module):
    def __init__(self, zug_proj: HymetaLinear, o_proj: HymetaLinear, width: int):
        """``zug_proj``: rows = update gate, candidate, output gate (``3 * width`` outputs, biases folded in)."""
        super().__init__()
        self.zug_proj, self.o_proj, self.width = zug_proj, o_proj, width

    def forward(self, h: torch.Tensor, layout, state: torch.Tensor) -> torch.Tensor:
        """``state`` fp32 ``[slots, width]``, updated in place for the step's sequences."""
        zug = self.zug_proj(h)
        y = hip_ops.mingru(zug, state, layout.query_start_loc, layout.context_lens, layout.slot_idx, layout.max_query_len)
        return self.o_proj(y)
