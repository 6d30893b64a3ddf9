"""Mixture of experts without a router network: a table gives every token id its experts, each weighing ``1 / top``
(hash-style routing).  The experts are gated feed-forward layers, ``W_down (silu(W_gate h) * (W_up h))``, held as the
stacks ``w13 [E, 2I, H]`` / ``w2 [E, H, I]`` that ``HymetaMoE`` (``moe.py``) holds; only the choice of the experts
differs, and with it the first launch of the block (``hip_ops.moe_table_forward``).
"""

from __future__ import annotations

import torch

from .. import hip_ops


class TableMoE(torch.nn.Module):
    def __init__(self, table: torch.Tensor, w13: torch.Tensor, w2: torch.Tensor):
        super().__init__()
        if table.dim() != 2 or int(table.max()) >= w13.shape[0] or int(table.min()) < 0:
            raise ValueError("table must be [vocab, top] with entries that name experts")
        self.register_buffer("table", table.to(torch.int32).contiguous())
        self.register_buffer("w13", w13.contiguous())
        self.register_buffer("w2", w2.contiguous())

    def forward(self, h: torch.Tensor, layout) -> torch.Tensor:
        return hip_ops.moe_table_forward(h, layout.token_ids, self.table, self.w13, self.w2)
