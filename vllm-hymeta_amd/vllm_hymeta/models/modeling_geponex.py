"""The Geponex decoder: an fp32 residual stream through post-norm layers (``x <- norm(alpha x + sublayer(x))``, a grouped
RMS norm) whose mixer reads a token-shifted input and is a latent attention (plain, with YaRN-scaled rotation; or with a
sink logit per head and an output gate) or a lightning attention; the feed-forward is dense (xIELU) or a sigmoid-routed
mixture of clamped gated experts beside a shared expert.  A layer may run with an earlier layer's weights and a cache and
state of its own.  The output projection is the embedding table.

The class has the surface of the package's other model classes (``GLAswaForCausalLM``, ``SonuzenForCausalLM``):
``forward(input_ids, positions, attn_metadata=..., request_ids_to_seq_ids=..., finished_requests_ids=...)`` returns the
final hidden states of the step's rows, ``compute_logits`` the fp32 logits of the rows asked for, ``load_weights`` takes
the checkpoint as a stream of named tensors; the attention layers are found by name and bound to paged caches by whoever
drives the model, the recurrent and shift states live in a slot-indexed cache that follows the requests' ids.
"""

from __future__ import annotations

from typing import Dict, Iterable, List, Optional, Set, Tuple

import torch

from .. import hip_ops
from .._compat import HasInnerState, IsHybrid
from ..linear import HymetaLinear
from ..lm_head import lm_head_logits
from ..state_cache import ConstantSizeStateCache
from .attention import bind_kv_cache, current_attn_metadata, standalone_prefix
from .configuration_geponex import DenseMlpSpec, GeponexConfig, LatentAttentionSpec, LightningSpec, MoeMlpSpec
from .feed_forward import ClampedGluMLP, SigmoidRoutedMoE, XieluMLP
from .latent_attention import LatentAttentionMixer, PagedLatentAttention
from .lightning_attention import LightningAttentionMixer
from .post_norm_block import AddGroupNorm, PostNormBlock, TokenShift
from .stream_block import StepLayout


class GeponexStateCache(ConstantSizeStateCache):
    """``shift [layers, slots, W]`` fp32: the last stream row every layer's token shift has seen; ``recurrent[r]
    [1, slots, H, D, Dv]`` fp32: the state of the ``r``-th lightning layer."""

    def __init__(self, num_layers: int, width: int, recurrent_shapes: List[Tuple[int, int, int]], max_batch_size: int, device):
        super().__init__(max_batch_size, device)
        self.shift = torch.zeros(max(num_layers, 1), max_batch_size, width, dtype=torch.float32, device=self.device)
        self.recurrent = [torch.zeros(1, max_batch_size, *s, dtype=torch.float32, device=self.device) for s in recurrent_shapes]

    @property
    def cache(self):
        return (self.shift, self.recurrent)

    def _slot_tensors(self):
        return (self.shift,) + tuple(self.recurrent)


class GeponexModel(torch.nn.Module):
    def __init__(self, config: GeponexConfig, max_num_seqs: int = 256, dtype: torch.dtype = torch.bfloat16, device="cuda",
                 prefix: Optional[str] = None):
        super().__init__()
        if dtype not in (torch.bfloat16, torch.float32):
            raise ValueError("Geponex runs in bfloat16 or float32")
        self.config, self.dtype, self.device = config, dtype, torch.device(device)
        self.prefix = standalone_prefix("model") if prefix is None else prefix
        # the cache-owning attention layers exist from construction on (an engine sizes its pages from them); a layer that
        # runs with another's weights still has a cache of its own
        self.attn_layers = torch.nn.ModuleDict()
        self._recurrent_index: Dict[int, int] = {}
        shapes: List[Tuple[int, int, int]] = []
        for i, spec in enumerate(config.layers):
            m = spec.mixer
            if isinstance(m, LatentAttentionSpec):
                self.attn_layers[str(i)] = PagedLatentAttention(m.heads, m.kv_rank, m.rot_dim, m.scale, f"{self.prefix}.layers.{i}.attn", dtype=dtype)
            else:
                self._recurrent_index[i] = len(shapes)
                shapes.append((m.heads, m.dim, m.vdim))
        self.state_cache = GeponexStateCache(config.num_hidden_layers, config.hidden_size, shapes, max_num_seqs, self.device)
        self.embed: Optional[torch.Tensor] = None
        self.blocks = torch.nn.ModuleDict()          # by the index of the layer that owns the tensors
        self.final_norm: Optional[AddGroupNorm] = None

    def layout_of(self, attn_metadata, slot_idx: torch.Tensor, token_ids: torch.Tensor) -> StepLayout:
        md = attn_metadata
        max_seq = max(md.seq_lens) if md.seq_lens else max(md.max_prefill_seq_len, md.max_decode_seq_len)
        return StepLayout(query_start_loc=md.query_start_loc, context_lens=md.context_lens_tensor, seq_lens=md.seq_lens_tensor,
                          slot_idx=slot_idx, block_tables=md.block_tables, slot_mapping=md.slot_mapping,
                          max_query_len=int(md.max_query_len or 1), max_seq_len=int(max_seq), token_ids=token_ids)

    def forward(self, input_ids: torch.Tensor, positions: Optional[torch.Tensor] = None, attn_metadata=None,
                kv_caches: Optional[List[torch.Tensor]] = None, residual_out: Optional[List[torch.Tensor]] = None,
                **kwargs) -> torch.Tensor:
        """``positions`` are not read: a row's position is its sequence's length minus the rows behind it.  ``kv_caches``:
        one page tensor per attention layer, in layer order, bound before the step (callers without an engine).
        ``residual_out``: a list that receives a copy of the stream after every layer (debugging)."""
        if kv_caches is not None:
            for layer, kv in zip(self.attn_layers.values(), kv_caches):
                bind_kv_cache(layer, kv)
        md = attn_metadata if attn_metadata is not None else current_attn_metadata()
        if md is None:
            raise RuntimeError("GeponexModel.forward needs the step's attention metadata")
        kwargs.setdefault("request_ids_to_seq_ids", {})
        kwargs.setdefault("finished_requests_ids", [])
        (shift, recurrent), slot_idx = self.state_cache.current_run_tensors(**kwargs)
        input_ids = input_ids.to(torch.int64).contiguous()
        layout = self.layout_of(md, slot_idx, input_ids)
        x = hip_ops.embed_rows(input_ids, self.embed)
        for i, spec in enumerate(self.config.layers):
            block = self.blocks[str(spec.weights_of)]
            mixer_state = self.attn_layers[str(i)] if str(i) in self.attn_layers else recurrent[self._recurrent_index[i]][0]
            x = block(x, self.dtype, layout, mixer_state, shift[i])
            if residual_out is not None:
                residual_out.append(x.clone())
        return self.final_norm(x, None, copy_dtype=self.dtype, in_place=False)


class GeponexForCausalLM(torch.nn.Module, HasInnerState, IsHybrid):
    # csrc/*.hip sources whose kernels this class calls (a first run in a fresh checkout builds these, see _C.build_library)
    kernel_sources = ("api_misc", "norm_conv", "post_norm", "latent_attn", "sink_attn", "lightning", "gated_ops", "moe_sigmoid",
                      "moe_table", "moe", "glue", "dense_gemm", "stream_gemm", "tall_gemm")

    def __init__(self, config: Optional[GeponexConfig] = None, max_num_seqs: int = 256, dtype: torch.dtype = torch.bfloat16,
                 device="cuda", *, vllm_config=None, prefix: Optional[str] = None):
        super().__init__()
        if vllm_config is not None:
            mc = vllm_config.model_config
            config = mc.hf_config if isinstance(mc.hf_config, GeponexConfig) else GeponexConfig(mc.hf_config.to_dict())
            max_num_seqs = int(vllm_config.scheduler_config.max_num_seqs)
            dtype = getattr(mc, "dtype", dtype)
            device = getattr(getattr(vllm_config, "device_config", None), "device", None) or device
            prefix = f"{prefix}.model" if prefix else "model"
        if config is None:
            raise TypeError("GeponexForCausalLM needs vllm_config= or a GeponexConfig")
        self.config = config
        self.model = GeponexModel(config, max_num_seqs=max_num_seqs, dtype=dtype, device=device, prefix=prefix)

    # what an engine asks a model with states of its own (the package's other model classes answer the same calls)
    def copy_inputs_before_cuda_graphs(self, input_buffers, **kwargs):
        return self.model.state_cache.copy_inputs_before_cuda_graphs(input_buffers, **kwargs)

    def get_seqlen_agnostic_capture_inputs(self, batch_size: int):
        return self.model.state_cache.get_seqlen_agnostic_capture_inputs(batch_size)

    def forward(self, input_ids, positions=None, intermediate_tensors=None, inputs_embeds=None, **kwargs):
        return self.model(input_ids, positions, **kwargs)

    def compute_logits(self, hidden_states: torch.Tensor, sampling_metadata=None) -> torch.Tensor:
        """The output projection is the embedding table."""
        idx = getattr(sampling_metadata, "selected_token_indices", None)
        if idx is not None:
            hidden_states = hidden_states.index_select(0, idx)
        return lm_head_logits(hidden_states, self.model.embed)

    # ------------------------------------------------------------------ weights
    def load_weights(self, weights: Iterable[Tuple[str, torch.Tensor]]) -> Set[str]:
        """Checkpoint names: ``embed``, ``final.norm``, and per layer with tensors of its own ``l<i>.norm1|norm2|shift``,
        ``l<i>.mix.<dq|dq.norm|uq|dkv|dkv.norm|uk|uv|o>`` (+ ``sink``, ``g``) for a latent attention or
        ``l<i>.mix.<q|k|v|g|o|norm>`` for a lightning attention, ``l<i>.mlp.<up|up.b|down|down.b|act>`` (dense) or
        ``l<i>.mlp.<router|e<j>.gate|e<j>.up|e<j>.down|shared.gate|shared.up|shared.down>``.  Linear weights ``[out, in]``."""
        cfg, m = self.config, self.model
        dev, dt = m.device, m.dtype
        got: Dict[str, torch.Tensor] = dict(weights)
        loaded: Set[str] = set()

        def take(name: str) -> torch.Tensor:
            if name not in got:
                raise KeyError(f"checkpoint has no tensor {name!r}")
            loaded.add(name)
            return got[name]

        def act(name: str, shape: Optional[Tuple[int, ...]] = None) -> torch.Tensor:
            t = take(name)
            if shape is not None and tuple(t.shape) != tuple(shape):
                raise ValueError(f"{name} is {tuple(t.shape)}, the configuration says {tuple(shape)}")
            return t.to(device=dev, dtype=dt).contiguous()

        def f32(name: str, shape: Optional[Tuple[int, ...]] = None) -> torch.Tensor:
            t = take(name)
            if shape is not None and tuple(t.shape) != tuple(shape):
                raise ValueError(f"{name} is {tuple(t.shape)}, the configuration says {tuple(shape)}")
            return t.to(device=dev, dtype=torch.float32).contiguous()

        def linear(parts: List[torch.Tensor], bias: Optional[torch.Tensor] = None) -> HymetaLinear:
            return HymetaLinear.from_weight(parts[0] if len(parts) == 1 else torch.cat(parts, 0).contiguous(), bias)

        W = cfg.hidden_size
        m.embed = act("embed", (cfg.vocab_size, W))
        m.final_norm = AddGroupNorm(f32("final.norm", (W,)), cfg.norm_groups, cfg.norm_eps, 1.0)
        m.blocks = torch.nn.ModuleDict()
        for i, spec in enumerate(cfg.layers):
            if spec.weights_of != i:
                continue
            p, a = f"l{i}.", spec.mixer
            if isinstance(a, LatentAttentionSpec):
                H, D, R, Dv, C, Q = a.heads, a.dim, a.rot_dim, a.vdim, a.kv_rank, a.q_rank
                sink = f32(p + "mix.sink", (H,)) if a.sink else None
                for j, other in enumerate(cfg.layers):            # every layer that runs these weights has the heads' constants
                    if other.weights_of == i:
                        m.attn_layers[str(j)].sink_logits = sink
                down = [act(p + "mix.dq", (Q, W)), act(p + "mix.dkv", (C + R, W))] + ([act(p + "mix.g", (H * Dv, W))] if a.gate else [])
                freqs, mag = a.rot.frequencies()
                mixer = LatentAttentionMixer(
                    linear(down), linear([act(p + "mix.uq", (H * (D + R), Q))]), act(p + "mix.uk", (H * D, C)).view(H, D, C),
                    act(p + "mix.uv", (H * Dv, C)).view(H, Dv, C).transpose(1, 2).contiguous(), linear([act(p + "mix.o", (W, H * Dv))]),
                    m.attn_layers[str(i)], H, D, R, Dv, C, Q, f32(p + "mix.dq.norm", (Q,)), f32(p + "mix.dkv.norm", (C,)), cfg.norm_eps,
                    a.rot.dims, torch.tensor(freqs, dtype=torch.float64, device=dev), mag, a.gate)
            else:
                assert isinstance(a, LightningSpec)
                H, D, Dv = a.heads, a.dim, a.vdim
                parts = [act(p + "mix.q", (H * D, W)), act(p + "mix.k", (H * D, W)), act(p + "mix.v", (H * Dv, W)), act(p + "mix.g", (H * Dv, W))]
                mixer = LightningAttentionMixer(linear(parts), linear([act(p + "mix.o", (W, H * Dv))]), H, D, Dv,
                                                torch.tensor(a.decay, dtype=torch.float32, device=dev), f32(p + "mix.norm", (H * Dv,)), cfg.norm_eps)
            mlp = mlp_norm = None
            e = spec.mlp
            if isinstance(e, DenseMlpSpec):
                pq = take(p + "mlp.act").float().tolist()
                mlp = XieluMLP(linear([act(p + "mlp.up", (e.ff, W))], act(p + "mlp.up.b", (e.ff,))),
                               linear([act(p + "mlp.down", (W, e.ff))], act(p + "mlp.down.b", (W,))), pq[0], pq[1])
            elif isinstance(e, MoeMlpSpec):
                F = e.expert.ff
                w13 = torch.stack([torch.cat([act(f"{p}mlp.e{j}.gate", (F, W)), act(f"{p}mlp.e{j}.up", (F, W))], 0) for j in range(e.experts)])
                w2 = torch.stack([act(f"{p}mlp.e{j}.down", (W, F)) for j in range(e.experts)])
                shared = None
                if e.shared is not None:
                    Fs = e.shared.ff
                    shared = ClampedGluMLP(linear([act(p + "mlp.shared.gate", (Fs, W)), act(p + "mlp.shared.up", (Fs, W))]),
                                           linear([act(p + "mlp.shared.down", (W, Fs))]), e.shared.limit)
                mlp = SigmoidRoutedMoE(f32(p + "mlp.router", (e.experts, W)), w13, w2, e.top, e.route_scale, e.expert.limit, shared)
            if mlp is not None:
                mlp_norm = AddGroupNorm(f32(p + "norm2", (W,)), cfg.norm_groups, cfg.norm_eps, cfg.postln_alpha)
            m.blocks[str(i)] = PostNormBlock(TokenShift(f32(p + "shift", (W,))), mixer,
                                             AddGroupNorm(f32(p + "norm1", (W,)), cfg.norm_groups, cfg.norm_eps, cfg.postln_alpha), mlp, mlp_norm)
        return loaded
