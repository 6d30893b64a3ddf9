"""The Sonuzen decoder: an fp32 residual stream through layers whose mixer is either a minGRU or a causal attention
with a log-distance bias and a sink, each followed by a table-routed mixture of experts; a run of layers may be looped
(passed through several times with the same weights, every pass with its own caches and states and its own vector
added to the stream before it); every sublayer reads its input through a short causal convolution over time.

The class has the surface of the package's other model classes (``GLAswaForCausalLM``): ``forward(input_ids, positions,
attn_metadata=..., request_ids_to_seq_ids=..., finished_requests_ids=...)`` returns the final hidden states of the
step's rows, ``compute_logits`` the fp32 logits of the rows asked for, ``load_weights`` takes the checkpoint as a stream
of named tensors; the attention layers are found by name and bound to paged caches by whoever drives the model, the
recurrent and convolution states live in a slot-indexed cache that follows the requests' ids.
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
from .configuration_sonuzen import SonuzenConfig
from .mingru import MinGRUMixer
from .sink_attention import BiasSinkAttentionMixer, PagedBiasAttention
from .stream_block import NormConvIn, NormOutResidual, StepLayout, StreamBlock
from .table_moe import TableMoE


class SonuzenStateCache(ConstantSizeStateCache):
    """``recurrent[r] [1, slots, width_r]`` fp32: the minGRU state of the ``r``-th (minGRU layer, pass); ``conv
    [C, slots, taps - 1, W]`` in the activation type: the last inputs of every sublayer's convolution, per (layer, pass,
    sublayer)."""

    def __init__(self, recurrent_widths: List[int], num_conv: int, max_batch_size: int, width: int, history: int, dtype, device):
        super().__init__(max_batch_size, device)
        self.recurrent = [torch.zeros(1, max_batch_size, w, dtype=torch.float32, device=self.device) for w in recurrent_widths]
        self.conv = torch.zeros(max(num_conv, 1), max_batch_size, max(history, 1), width, dtype=dtype, device=self.device)

    @property
    def cache(self):
        return (self.recurrent, self.conv)

    def _slot_tensors(self):
        return tuple(self.recurrent) + (self.conv,)


class SonuzenModel(torch.nn.Module):
    def __init__(self, config: SonuzenConfig, max_num_seqs: int = 256, dtype: torch.dtype = torch.bfloat16, device="cuda",
                 prefix: Optional[str] = None):
        super().__init__()
        if dtype not in (torch.bfloat16, torch.float32):
            raise ValueError("Sonuzen runs in bfloat16 or float32")
        self.config, self.dtype, self.device = config, dtype, torch.device(device)
        self.prefix = standalone_prefix("model") if prefix is None else prefix
        self.runs: List[Tuple[int, int]] = config.layer_runs()
        # the cache-owning attention layers exist from construction on (an engine sizes its pages from them); a layer
        # inside the loop has one per pass
        self.attn_layers = torch.nn.ModuleDict()
        self._attn_key: Dict[Tuple[int, int], str] = {}
        self._recurrent_index: Dict[Tuple[int, int], int] = {}
        for (i, t) in self.runs:
            spec = config.layers[i]
            if spec.type == "attention":
                key = f"{i}_{t}"
                m = spec.mixer
                self.attn_layers[key] = PagedBiasAttention(m.heads, m.kv_heads, m.dim, m.vdim, m.scale,
                                                           f"{self.prefix}.layers.{i}.pass{t}.attn", dtype=dtype)
                self._attn_key[(i, t)] = key
            else:
                self._recurrent_index[(i, t)] = len(self._recurrent_index)
        self.history = max(config.conv_taps - 1, 0) if config.has_conv else 0
        self._conv_index: Dict[Tuple[int, int], int] = {}
        n_conv = 0
        for (i, t) in self.runs:
            self._conv_index[(i, t)] = n_conv
            n_conv += (1 + int(config.layers[i].mlp is not None)) if self.history else 0
        widths = [config.layers[i].mixer.width for (i, t) in self.runs if (i, t) in self._recurrent_index]
        self.state_cache = SonuzenStateCache(widths, n_conv, max_num_seqs, config.hidden_size, self.history, dtype, self.device)
        self.embed: Optional[torch.Tensor] = None
        self.loop_step: Optional[torch.Tensor] = None        # fp32 [times, W]
        self.layers = torch.nn.ModuleList()
        self.final_norm: Optional[NormConvIn] = None

    # ------------------------------------------------------------------ the step
    def _post_add(self, n: int) -> Optional[torch.Tensor]:
        """The vector added to the stream after run ``n``: the next pass's vector when run ``n + 1`` starts a pass."""
        cfg = self.config
        if not cfg.has_loop or self.loop_step is None or n + 1 >= len(self.runs):
            return None
        i, t = self.runs[n + 1]
        return self.loop_step[t] if i == cfg.loop_start else None

    def layout_of(self, attn_metadata, slot_idx: torch.Tensor, token_ids: torch.Tensor) -> StepLayout:
        md = attn_metadata
        max_seq = max(md.seq_lens) if md.seq_lens else max(md.max_prefill_seq_len, md.max_decode_seq_len)
        return StepLayout(query_start_loc=md.query_start_loc, context_lens=md.context_lens_tensor, seq_lens=md.seq_lens_tensor,
                          slot_idx=slot_idx, block_tables=md.block_tables, slot_mapping=md.slot_mapping,
                          max_query_len=int(md.max_query_len or 1), max_seq_len=int(max_seq), token_ids=token_ids)

    def forward(self, input_ids: torch.Tensor, positions: Optional[torch.Tensor] = None, attn_metadata=None,
                kv_caches: Optional[List[torch.Tensor]] = None, residual_out: Optional[List[torch.Tensor]] = None,
                **kwargs) -> torch.Tensor:
        """``positions`` are not read: a row's position is its sequence's length minus the rows behind it, and enters only
        through the attention's distance bias.  ``kv_caches``: one page tensor per attention layer and pass, in execution
        order, bound before the step (callers without an engine).  ``residual_out``: a list that receives a copy of the
        stream after every layer run (debugging)."""
        if kv_caches is not None:
            for layer, kv in zip(self.attn_layers.values(), kv_caches):
                bind_kv_cache(layer, kv)
        md = attn_metadata if attn_metadata is not None else current_attn_metadata()
        if md is None:
            raise RuntimeError("SonuzenModel.forward needs the step's attention metadata")
        kwargs.setdefault("request_ids_to_seq_ids", {})
        kwargs.setdefault("finished_requests_ids", [])
        (recurrent, conv), slot_idx = self.state_cache.current_run_tensors(**kwargs)
        input_ids = input_ids.to(torch.int64).contiguous()
        layout = self.layout_of(md, slot_idx, input_ids)
        cfg = self.config
        first_add = self.loop_step[0] if (cfg.has_loop and cfg.loop_start == 0 and self.loop_step is not None) else None
        x = hip_ops.embed_rows(input_ids, self.embed, first_add)
        for n, (i, t) in enumerate(self.runs):
            block = self.layers[i]
            if (i, t) in self._attn_key:
                mixer_state = self.attn_layers[self._attn_key[(i, t)]]
            else:
                mixer_state = recurrent[self._recurrent_index[(i, t)]][0]
            c0 = self._conv_index[(i, t)]
            x = block(x, self.dtype, layout, mixer_state, [conv[c0 + j] for j in range(block.conv_states)], self._post_add(n))
            if residual_out is not None:
                pa = self._post_add(n)
                residual_out.append(x.clone() if pa is None else x - pa)
        return self.final_norm(x, self.dtype)


class SonuzenForCausalLM(torch.nn.Module, HasInnerState, IsHybrid):
    # csrc/*.hip sources whose kernels this class calls (a first run in a fresh checkout builds these, see _C.build_library)
    kernel_sources = ("api_misc", "norm_conv", "mingru", "sink_attn", "moe_table", "moe", "glue", "dense_gemm", "stream_gemm", "tall_gemm")

    def __init__(self, config: Optional[SonuzenConfig] = None, max_num_seqs: int = 256, dtype: torch.dtype = torch.bfloat16,
                 device="cuda", *, vllm_config=None, prefix: Optional[str] = None):
        super().__init__()
        if vllm_config is not None:
            mc = vllm_config.model_config
            config = mc.hf_config if isinstance(mc.hf_config, SonuzenConfig) else SonuzenConfig(mc.hf_config.to_dict())
            max_num_seqs = int(vllm_config.scheduler_config.max_num_seqs)
            dtype = getattr(mc, "dtype", dtype)
            device = getattr(getattr(vllm_config, "device_config", None), "device", None) or device
            prefix = f"{prefix}.model" if prefix else "model"
        if config is None:
            raise TypeError("SonuzenForCausalLM needs vllm_config= or a SonuzenConfig")
        self.config = config
        self.model = SonuzenModel(config, max_num_seqs=max_num_seqs, dtype=dtype, device=device, prefix=prefix)
        self.lm_head: Optional[torch.Tensor] = None

    # what an engine asks a model with states of its own (the package's other model classes answer the same calls)
    def copy_inputs_before_cuda_graphs(self, input_buffers, **kwargs):
        return self.model.state_cache.copy_inputs_before_cuda_graphs(input_buffers, **kwargs)

    def get_seqlen_agnostic_capture_inputs(self, batch_size: int):
        return self.model.state_cache.get_seqlen_agnostic_capture_inputs(batch_size)

    def forward(self, input_ids, positions=None, intermediate_tensors=None, inputs_embeds=None, **kwargs):
        return self.model(input_ids, positions, **kwargs)

    def compute_logits(self, hidden_states: torch.Tensor, sampling_metadata=None) -> torch.Tensor:
        idx = getattr(sampling_metadata, "selected_token_indices", None)
        if idx is not None:
            hidden_states = hidden_states.index_select(0, idx)
        logits = lm_head_logits(hidden_states, self.lm_head)
        return logits.mul_(self.config.logit_scale) if self.config.logit_scale != 1.0 else logits

    # ------------------------------------------------------------------ weights
    def load_weights(self, weights: Iterable[Tuple[str, torch.Tensor]]) -> Set[str]:
        """Checkpoint names: ``embed``, ``head``, ``final.norm``, ``loop.step``, and per layer ``l<i>.norm1|norm1b|norm2|norm2b``,
        ``l<i>.canon1|canon2``, ``l<i>.mix.<q|k|v|o|q.norm|k.norm|r1|r2>`` (attention) or ``l<i>.mix.<z|z.b|x|x.b|g|o>`` (minGRU),
        ``l<i>.mlp.table`` and ``l<i>.mlp.e<j>.<gate|up|down>``.  Linear weights ``[out, in]``."""
        cfg, m = self.config, self.model
        dev, dt = m.device, m.dtype
        got: Dict[str, torch.Tensor] = {}
        for name, tensor in weights:
            got[name] = tensor
        loaded: Set[str] = set()

        def take(name: str) -> torch.Tensor:
            if name not in got:
                raise KeyError(f"checkpoint has no tensor {name!r}")
            loaded.add(name)
            return got[name]

        def act(name: str) -> torch.Tensor:
            return take(name).to(device=dev, dtype=dt).contiguous()

        def f32(name: str) -> torch.Tensor:
            return take(name).to(device=dev, dtype=torch.float32).contiguous()

        def linear(names: List[str], biases: Optional[List[Optional[str]]] = None) -> HymetaLinear:
            ws = [act(n) for n in names]
            w = ws[0] if len(ws) == 1 else torch.cat(ws, 0).contiguous()
            b = None
            if biases is not None and any(biases):
                b = torch.cat([act(bn) if bn else torch.zeros(wi.shape[0], dtype=dt, device=dev) for bn, wi in zip(biases, ws)]).contiguous()
            return HymetaLinear.from_weight(w, b)

        W = cfg.hidden_size
        m.embed = act("embed")
        if m.embed.shape != (cfg.vocab_size, W):
            raise ValueError(f"embed is {tuple(m.embed.shape)}, config says {(cfg.vocab_size, W)}")
        self.lm_head = act("head")
        m.final_norm = NormConvIn(f32("final.norm"), cfg.norm_eps)
        if cfg.has_loop:
            m.loop_step = f32("loop.step")
            if m.loop_step.shape != (cfg.loop_times, W):
                raise ValueError(f"loop.step is {tuple(m.loop_step.shape)}, the loop runs {cfg.loop_times} times over width {W}")
        m.layers = torch.nn.ModuleList()
        conv = cfg.has_conv
        for i, spec in enumerate(cfg.layers):
            p = f"l{i}."
            if spec.type == "attention":
                a = spec.mixer
                first_pass = min(t for (j, t) in m.runs if j == i)
                for (j, t) in m.runs:       # every pass's cache owner gets the heads' constants
                    if j == i:
                        layer = m.attn_layers[m._attn_key[(j, t)]]
                        layer.bias_a, layer.bias_b = f32(p + "mix.r1"), f32(p + "mix.r2")
                mixer = BiasSinkAttentionMixer(linear([p + "mix.q", p + "mix.k", p + "mix.v"]), linear([p + "mix.o"]),
                                               m.attn_layers[m._attn_key[(i, first_pass)]], f32(p + "mix.q.norm"),
                                               f32(p + "mix.k.norm"), cfg.norm_eps)
                want = ((a.heads + a.kv_heads) * a.dim + a.kv_heads * a.vdim, W)
                if tuple(mixer.qkv_proj.weight.shape) != want or tuple(mixer.o_proj.weight.shape) != (W, a.heads * a.vdim):
                    raise ValueError(f"layer {i}: attention projections do not have the configured sizes")
            else:
                mixer = MinGRUMixer(linear([p + "mix.z", p + "mix.x", p + "mix.g"], [p + "mix.z.b", p + "mix.x.b", None]),
                                    linear([p + "mix.o"]), spec.mixer.width)
                if tuple(mixer.zug_proj.weight.shape) != (3 * spec.mixer.width, W) or tuple(mixer.o_proj.weight.shape) != (W, spec.mixer.width):
                    raise ValueError(f"layer {i}: minGRU projections do not have the configured sizes")
            mixer_in = NormConvIn(f32(p + "norm1"), cfg.norm_eps, f32(p + "canon1") if conv else None)
            mixer_out = NormOutResidual(f32(p + "norm1b"), cfg.norm_eps, cfg.residual_mult)
            mlp_in = mlp = mlp_out = None
            if spec.mlp is not None:
                e = spec.mlp
                w13 = torch.stack([torch.cat([act(f"{p}mlp.e{j}.gate"), act(f"{p}mlp.e{j}.up")], 0) for j in range(e.experts)])
                w2 = torch.stack([act(f"{p}mlp.e{j}.down") for j in range(e.experts)])
                if tuple(w13.shape) != (e.experts, 2 * e.ff, W) or tuple(w2.shape) != (e.experts, W, e.ff):
                    raise ValueError(f"layer {i}: expert weights do not have the configured sizes")
                table = take(p + "mlp.table").to(device=dev)
                if tuple(table.shape) != (cfg.vocab_size, e.top):
                    raise ValueError(f"layer {i}: the expert table is {tuple(table.shape)}, config says {(cfg.vocab_size, e.top)}")
                mlp = TableMoE(table, w13, w2)
                mlp_in = NormConvIn(f32(p + "norm2"), cfg.norm_eps, f32(p + "canon2") if conv else None)
                mlp_out = NormOutResidual(f32(p + "norm2b"), cfg.norm_eps, cfg.residual_mult)
            m.layers.append(StreamBlock(mixer_in, mixer, mixer_out, mlp_in, mlp, mlp_out))
        return loaded
