"""Lightning attention mixer: linear attention whose state decays by a constant per head,

    q, k, v = silu(W_q h), silu(W_k h), silu(W_v h);   S_t = decay_h S_{t-1} + k_t v_t^T;   o_t = S_t^T q_t
    out = W_o (norm(concat_h o_t) * sigmoid(W_g h))

(linear attention with a fixed decay per head, as in "Lightning Attention-2: A Free Lunch for Handling Unlimited Sequence
Lengths in Large Language Models", Qin et al. 2024).  The four input projections are one linear layer; the
recurrence runs in ``hip_ops.lightning_attention`` with the state fp32 ``[slots, H, D, Dv]``, one slot per sequence.
Beside ``GatedLinearAttention`` (``model_for_7B/gla_attention.py``), whose decay is computed per token and channel, and
``MinGRUMixer`` (``mingru.py``), whose state is a vector.
"""

from __future__ import annotations

import torch

from .. import hip_ops
from ..linear import HymetaLinear


class LightningAttentionMixer(torch.nn.Module):
    def __init__(self, in_proj: HymetaLinear, o_proj: HymetaLinear, num_heads: int, dim: int, vdim: int, decay: torch.Tensor,
                 norm_weight: torch.Tensor, eps: float):
        """``in_proj``: rows = queries, keys, values, output gate (``2 H dim + 2 H vdim`` outputs)."""
        super().__init__()
        self.in_proj, self.o_proj = in_proj, o_proj
        self.H, self.D, self.Dv, self.eps = num_heads, dim, vdim, float(eps)
        self.register_buffer("decay", decay.float().contiguous())
        self.register_buffer("norm_weight", norm_weight.float().contiguous())

    def forward(self, h: torch.Tensor, layout, state: torch.Tensor) -> torch.Tensor:
        """``state`` fp32 ``[slots, H, D, Dv]``, updated in place for the step's sequences."""
        H, D, Dv = self.H, self.D, self.Dv
        proj = self.in_proj(h)
        o = hip_ops.lightning_attention(proj, state, self.decay, H, D, Dv, layout.query_start_loc, layout.context_lens,
                                        layout.slot_idx, layout.max_query_len)
        y = hip_ops.gated_rms_norm(o, proj[:, 2 * H * D + H * Dv:], self.norm_weight, self.eps)
        return self.o_proj(y)
