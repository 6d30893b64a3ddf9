"""Causal softmax attention over a paged cache with per-head query / key norms, a distance bias in place of a rotation,
and a sink:

    s_ij = scale * q_i . k_j - a_h ln(1 + b_h (i - j)),   p_ij = exp(s_ij) / (1 + sum_j exp(s_ij)),   out_i = sum_j p_ij v_j

The key size and the value size may differ, so a page holds rows of ``head_dim + v_dim`` per key/value head (a key
followed by its value) instead of the ``[2, ...]`` pair of ``MetaAttention`` (``attention.py``), whose kernels are built
for one head size, equal for keys and values.  ``PagedBiasAttention`` is the cache-owning object an engine finds by name
and binds a cache to, as it does with ``MetaAttention``; ``BiasSinkAttentionMixer`` is the sublayer around it.
"""

from __future__ import annotations

from typing import List, Optional, Tuple

import torch

from .. import hip_ops
from ..linear import HymetaLinear
from . import attention as _registry


class PagedBiasAttention(torch.nn.Module):
    def __init__(self, num_heads: int, num_kv_heads: int, head_dim: int, v_dim: int, scale: float, prefix: str,
                 bias_a: Optional[torch.Tensor] = None, bias_b: Optional[torch.Tensor] = None, sink: bool = True,
                 sliding_window: Optional[int] = None, dtype: torch.dtype = torch.bfloat16):
        super().__init__()
        self.num_heads, self.num_kv_heads, self.head_size, self.v_size = num_heads, num_kv_heads, head_dim, v_dim
        self.scale, self.sink, self.dtype = float(scale), bool(sink), dtype
        self.window_left = -1 if sliding_window is None else sliding_window - 1
        self.register_buffer("bias_a", None if bias_a is None else bias_a.float().contiguous())
        self.register_buffer("bias_b", None if bias_b is None else bias_b.float().contiguous())
        if prefix in _registry._LAYERS:
            raise ValueError(f"Duplicate layer name: {prefix}")
        _registry._LAYERS[prefix] = self
        self.layer_name = prefix
        self.kv_cache: List[torch.Tensor] = [torch.tensor([])]

    def kv_cache_shape(self, num_blocks: int, block_size: int) -> Tuple[int, ...]:
        return (num_blocks, block_size, self.num_kv_heads, self.head_size + self.v_size)

    def forward(self, qkv: torch.Tensor, layout, q_weight: Optional[torch.Tensor], k_weight: Optional[torch.Tensor],
                eps: float) -> torch.Tensor:
        """``qkv [T, H D + G D + G Dv]`` of the step's rows -> ``[T, H Dv]``.  Norms the queries and keys, stores the keys and
        values in the bound cache, attends through the block tables."""
        kv = self.kv_cache[0]
        if kv.numel() == 0:
            raise RuntimeError(f"{self.layer_name}: no KV cache bound")
        H, G, D, Dv = self.num_heads, self.num_kv_heads, self.head_size, self.v_size
        hip_ops.qk_norm_cache_(qkv, H, G, D, Dv, q_weight, k_weight, eps, kv, layout.slot_mapping)
        q = qkv[:, :H * D].view(-1, H, D)
        out = hip_ops.sink_attention(q, kv, layout.block_tables, layout.query_start_loc, layout.seq_lens, G, D, Dv, self.scale,
                                     layout.max_query_len, layout.max_seq_len, self.bias_a, self.bias_b, self.sink, self.window_left)
        return out.view(-1, H * Dv)


class BiasSinkAttentionMixer(torch.nn.Module):
    def __init__(self, qkv_proj: HymetaLinear, o_proj: HymetaLinear, attn: PagedBiasAttention,
                 q_norm_weight: Optional[torch.Tensor], k_norm_weight: Optional[torch.Tensor], eps: float):
        super().__init__()
        self.qkv_proj, self.o_proj, self.eps = qkv_proj, o_proj, float(eps)
        self.register_buffer("q_norm_weight", None if q_norm_weight is None else q_norm_weight.float().contiguous())
        self.register_buffer("k_norm_weight", None if k_norm_weight is None else k_norm_weight.float().contiguous())
        self._attn = (attn,)          # owned (and registered as a module) by the model, one per pass through the layer

    def forward(self, h: torch.Tensor, layout, attn: Optional[PagedBiasAttention] = None) -> torch.Tensor:
        """``attn``: the cache-owning layer of this pass (a layer inside a loop has one per pass)."""
        attn = attn or self._attn[0]
        qkv = self.qkv_proj(h)
        return self.o_proj(attn(qkv, layout, self.q_norm_weight, self.k_norm_weight, self.eps))
