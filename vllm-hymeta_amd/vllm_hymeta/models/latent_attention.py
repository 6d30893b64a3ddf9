"""Latent attention: queries, keys and values go through low-rank latents, and every head's key has a rotated part that
all heads share,

    c_q = norm(W_dq h),  q_h = W_uq,h c_q = (q_h^nope, q_h^rot)
    (c, k^rot) = W_dkv h,  c <- norm(c),   k_h = (W_uk,h c, rot(k^rot)),  v_h = W_uv,h c
    s_ij = scale (q_i^nope . k_j^nope + rot(q_i^rot) . rot(k_j^rot)),  softmax over j <= i (optionally with a sink logit
    per head in the denominator), out = W_o concat_h(sum_j p_ij v_j,h) (optionally times sigmoid(W_g h))

(multi-head latent attention: "DeepSeek-V2: A Strong, Economical, and Efficient Mixture-of-Experts Language Model",
DeepSeek-AI 2024).  Only ``(c, rot(k^rot))`` is cached, one row per token for all heads,
and the products with ``W_uk`` / ``W_uv`` are moved to the query and the output: ``q_h^nope . W_uk,h c = (W_uk,h^T q_h^nope)
. c`` and ``sum_j p_j W_uv,h c_j = W_uv,h sum_j p_j c_j``.  The attention kernel then sees one key/value head of size
``kv_rank + rot_dim`` whose first ``kv_rank`` elements are also its value, shared by all query heads.

``PagedLatentAttention`` is the cache-owning object an engine finds by name and binds a cache to (as ``MetaAttention``,
``attention.py``, and ``PagedBiasAttention``, ``sink_attention.py``); ``LatentAttentionMixer`` is the sublayer around it.
"""

from __future__ import annotations

from typing import List, Optional, Tuple

import torch

from .. import hip_ops
from ..linear import HymetaLinear
from . import attention as _registry


class PagedLatentAttention(torch.nn.Module):
    def __init__(self, num_heads: int, kv_rank: int, rot_dim: int, scale: float, prefix: str,
                 sink_logits: Optional[torch.Tensor] = None, dtype: torch.dtype = torch.bfloat16):
        super().__init__()
        self.num_heads, self.num_kv_heads, self.kv_rank, self.rot_dim = num_heads, 1, kv_rank, rot_dim
        self.head_size, self.v_size = kv_rank + rot_dim, kv_rank
        self.scale, self.dtype = float(scale), dtype
        self.register_buffer("sink_logits", None if sink_logits is None else sink_logits.float().contiguous())
        if prefix in _registry._LAYERS:
            raise ValueError(f"Duplicate layer name: {prefix}")
        _registry._LAYERS[prefix] = self
        self.layer_name = prefix
        self.kv_cache: List[torch.Tensor] = [torch.tensor([])]

    def kv_cache_shape(self, num_blocks: int, block_size: int) -> Tuple[int, ...]:
        return (num_blocks, block_size, 1, self.kv_rank + self.rot_dim)

    def cache(self) -> torch.Tensor:
        kv = self.kv_cache[0]
        if kv.numel() == 0:
            raise RuntimeError(f"{self.layer_name}: no KV cache bound")
        return kv

    def forward(self, q: torch.Tensor, layout) -> torch.Tensor:
        """``q [T, H, kv_rank + rot_dim]`` (absorbed and rotated) against the cached rows (this step's are stored already)
        -> ``[T, H, kv_rank]``: the heads' weighted sums of the latents."""
        return hip_ops.sink_attention(q, self.cache(), layout.block_tables, layout.query_start_loc, layout.seq_lens, 1, self.head_size,
                                      self.v_size, self.scale, layout.max_query_len, layout.max_seq_len, sink=self.sink_logits is not None,
                                      sink_logits=self.sink_logits, value_in_key=True)


class LatentAttentionMixer(torch.nn.Module):
    def __init__(self, down_proj: HymetaLinear, uq_proj: HymetaLinear, uk: torch.Tensor, uv: torch.Tensor, o_proj: HymetaLinear,
                 attn: PagedLatentAttention, num_heads: int, dim: int, rot_dim: int, vdim: int, kv_rank: int, q_rank: int,
                 q_norm_weight: torch.Tensor, kv_norm_weight: torch.Tensor, eps: float, rot_dims: int, rot_freqs: torch.Tensor,
                 rot_mag: float, gate: bool):
        """``down_proj``: rows = query latent, key/value latent, rotated key part (and, with ``gate``, the output gate);
        ``uk [H, dim, kv_rank]`` and ``uv [H, kv_rank, vdim]``: the keys' and values' up projections per head, laid out for
        the two batched products."""
        super().__init__()
        self.down_proj, self.uq_proj, self.o_proj = down_proj, uq_proj, o_proj
        self.register_buffer("uk", uk.contiguous())
        self.register_buffer("uv", uv.contiguous())
        self.register_buffer("q_norm_weight", q_norm_weight.float().contiguous())
        self.register_buffer("kv_norm_weight", kv_norm_weight.float().contiguous())
        self.register_buffer("rot_freqs", rot_freqs.to(torch.float64).contiguous())
        self.H, self.D, self.R, self.Dv, self.C, self.Q = num_heads, dim, rot_dim, vdim, kv_rank, q_rank
        self.eps, self.rot_dims, self.rot_mag, self.gate = float(eps), int(rot_dims), float(rot_mag), bool(gate)
        self._attn = (attn,)          # owned (and registered as a module) by the model, one per layer that runs these weights

    def forward(self, h: torch.Tensor, layout, attn: Optional[PagedLatentAttention] = None) -> torch.Tensor:
        attn = attn or self._attn[0]
        H, D, R, Dv, C, Q = self.H, self.D, self.R, self.Dv, self.C, self.Q
        T = h.shape[0]
        proj = self.down_proj(h)
        hip_ops.latent_kv_prep_(proj, 0, Q, Q, C, R, self.rot_dims, self.q_norm_weight, self.kv_norm_weight, self.eps, self.rot_freqs,
                                self.rot_mag, attn.cache(), layout.slot_mapping, layout.query_start_loc, layout.seq_lens)
        q = self.uq_proj(proj[:, :Q]).view(T, H, D + R)
        q_abs = torch.bmm(q[:, :, :D].transpose(0, 1), self.uk)                       # [H, T, C]
        q_full = hip_ops.latent_q_assemble(q, q_abs, D, R, self.rot_dims, self.rot_freqs, self.rot_mag, layout.query_start_loc,
                                           layout.seq_lens)
        o_lat = attn(q_full, layout)                                                  # [T, H, C]
        o = torch.bmm(o_lat.transpose(0, 1), self.uv).transpose(0, 1).reshape(T, H * Dv)
        if self.gate:
            o = hip_ops.sigmoid_gate_mul(o, proj[:, Q + C + R:])
        return self.o_proj(o)
