"""A small serving engine of the package's own: request queue, page and state-slot bookkeeping, continuous batching
with portions of prompts beside single decoded tokens, greedy (or temperature) sampling.  It drives a model class
through the calls vLLM's V0 engine makes (the step's ``MetaAttentionMetadata`` in the forward context,
``request_ids_to_seq_ids`` / ``finished_requests_ids`` for the state slots, ``compute_logits`` on selected rows, paged
caches bound to the attention layers found by name), so a model class serves under either.

``LLMEngine.execute`` is the one step function: the scheduler's batches (``step`` / ``generate``) and batches given
from outside (``run_batch``: a replayed trace) go through it.
"""

from __future__ import annotations

import os
from collections import deque
from dataclasses import dataclass, field
from itertools import accumulate
from typing import Deque, Dict, Iterable, Iterator, List, Optional, Sequence, Tuple

import torch

from . import hip_ops, registry
from .attention.meta_attention import MetaAttentionMetadata
from .models import attention as layer_registry
from .models.attention import bind_kv_cache, forward_context


@dataclass
class SamplingParams:
    max_tokens: int = 16
    temperature: float = 0.0          # 0: greedy
    seed: Optional[int] = None
    stop_token_ids: Tuple[int, ...] = ()


@dataclass
class Request:
    request_id: str
    token_ids: List[int]                              # prompt, then generated tokens
    num_prompt_tokens: int
    params: SamplingParams = field(default_factory=SamplingParams)
    num_computed: int = 0                             # tokens whose keys / states are in the caches
    blocks: List[int] = field(default_factory=list)
    finished: bool = False
    state_key: str = ""                               # the name the model's state cache knows the request by

    @property
    def output_token_ids(self) -> List[int]:
        return self.token_ids[self.num_prompt_tokens:]


class BlockPool:
    """Pages of the paged caches: a free list, last freed first reused."""

    def __init__(self, num_blocks: int, block_size: int):
        self.num_blocks, self.block_size = int(num_blocks), int(block_size)
        self._free: List[int] = list(range(self.num_blocks - 1, -1, -1))

    @property
    def num_free(self) -> int:
        return len(self._free)

    def blocks_for(self, num_tokens: int) -> int:
        return (num_tokens + self.block_size - 1) // self.block_size

    def grow(self, blocks: List[int], num_tokens: int) -> None:
        need = self.blocks_for(num_tokens) - len(blocks)
        if need > len(self._free):
            raise RuntimeError(f"out of cache pages: {need} needed, {len(self._free)} free")
        for _ in range(max(need, 0)):
            blocks.append(self._free.pop())

    def release(self, blocks: List[int]) -> None:
        self._free.extend(reversed(blocks))
        blocks.clear()


class Scheduler:
    """Continuous batching: every running request gets its next token (or the next portion of its prompt) each step,
    decodes first, within ``max_num_batched_tokens``; waiting requests are admitted while a state slot and pages for
    their next portion are free."""

    def __init__(self, pool: BlockPool, max_num_seqs: int, max_num_batched_tokens: int):
        self.pool, self.max_num_seqs, self.max_num_batched_tokens = pool, max_num_seqs, max_num_batched_tokens
        self.waiting: Deque[Request] = deque()
        self.running: List[Request] = []

    def add(self, request: Request) -> None:
        self.waiting.append(request)

    def has_work(self) -> bool:
        return bool(self.waiting or self.running)

    def schedule(self) -> List[Tuple[Request, int]]:
        budget = self.max_num_batched_tokens
        batch: List[Tuple[Request, int]] = []
        pages = self.pool.num_free
        order = sorted(self.running, key=lambda r: len(r.token_ids) - r.num_computed)     # single tokens before portions
        for r in order:
            n = min(len(r.token_ids) - r.num_computed, budget)
            need = self.pool.blocks_for(r.num_computed + n) - len(r.blocks)
            if n <= 0 or need > pages:
                continue
            batch.append((r, n))
            budget -= n
            pages -= need
        while self.waiting and len(self.running) < self.max_num_seqs and budget > 0:
            r = self.waiting[0]
            n = min(len(r.token_ids), budget)
            need = self.pool.blocks_for(n)
            if need > pages:
                break
            self.waiting.popleft()
            self.running.append(r)
            batch.append((r, n))
            budget -= n
            pages -= need
        return batch

    def retire(self, request: Request) -> None:
        if request in self.running:
            self.running.remove(request)


class LLMEngine:
    def __init__(self, model: torch.nn.Module, num_blocks: int, block_size: int = 64, max_num_seqs: int = 4,
                 max_num_batched_tokens: int = 8192, device="cuda"):
        self.model, self.device = model, torch.device(device)
        self.pool = BlockPool(num_blocks, block_size)
        self.scheduler = Scheduler(self.pool, max_num_seqs, max_num_batched_tokens)
        self.requests: Dict[str, Request] = {}
        self._finished_since_last_step: List[str] = []
        self._generators: Dict[str, torch.Generator] = {}
        self._serial = 0
        prefix = getattr(getattr(model, "model", model), "prefix", None)
        if prefix is None:
            raise ValueError("the model does not say under which prefix its attention layers are registered")
        # the cache-owning layers of this model, by name; each says what a page of its cache looks like
        self.attn_layers = {name: layer for name, layer in layer_registry.registered_layers().items() if name.startswith(prefix + ".")}
        self.kv_caches: Dict[str, torch.Tensor] = {}
        for name, layer in self.attn_layers.items():
            if hasattr(layer, "kv_cache_shape"):
                shape, dtype = layer.kv_cache_shape(num_blocks, block_size), layer.dtype
            else:      # MetaAttention: the backend's [2, blocks, block_size, Hkv, D] pair, bf16
                from .attention.meta_attention import MetaAttentionBackend
                shape = MetaAttentionBackend.get_kv_cache_shape(num_blocks, block_size, layer.num_kv_heads, layer.head_size)
                dtype = torch.bfloat16
            self.kv_caches[name] = torch.zeros(shape, dtype=dtype, device=self.device)
            bind_kv_cache(layer, self.kv_caches[name])

    # ------------------------------------------------------------------ construction from a checkpoint folder
    @classmethod
    def from_pretrained(cls, model_dir: str, dtype: torch.dtype = torch.bfloat16, max_tokens: int = 8192, block_size: int = 64,
                        max_num_seqs: int = 4, max_num_batched_tokens: int = 8192, device="cuda") -> "LLMEngine":
        """The model class is chosen by ``config.json``; the page pool holds ``max_tokens`` tokens (each request's count
        rounded up to whole pages), the state cache ``max_num_seqs`` sequences."""
        model_cls, config = registry.resolve(model_dir)
        try:
            model = model_cls(config, max_num_seqs=max_num_seqs, dtype=dtype, device=device)
        except TypeError:
            if dtype != torch.bfloat16:
                raise ValueError(f"{model_cls.__name__} runs in bfloat16 only")
            model = model_cls(config, max_num_seqs=max_num_seqs, device=device)
        model.load_weights(iter_safetensors(model_dir))
        return cls(model, num_blocks=(max_tokens + block_size - 1) // block_size, block_size=block_size,
                   max_num_seqs=max_num_seqs, max_num_batched_tokens=max_num_batched_tokens, device=device)

    # ------------------------------------------------------------------ requests
    def add_request(self, request_id: str, prompt_token_ids: Sequence[int], params: Optional[SamplingParams] = None,
                    schedule: bool = True) -> Request:
        if request_id in self.requests:
            raise ValueError(f"request {request_id!r} is live already")
        r = Request(request_id, list(prompt_token_ids), len(prompt_token_ids), params or SamplingParams())
        # a name of its own for the state cache: a request id that comes back after its first owner ended is a new request
        self._serial += 1
        r.state_key = f"{request_id}#{self._serial}"
        self.requests[request_id] = r
        if schedule:
            self.scheduler.add(r)
        return r

    def finish_request(self, request_id: str) -> None:
        """Give back what the request holds: its pages now, its state slot at the start of the next step (the model's
        state cache releases the ids it is told have finished)."""
        r = self.requests.pop(request_id)
        r.finished = True
        self.pool.release(r.blocks)
        self.scheduler.retire(r)
        self._finished_since_last_step.append(r.state_key)
        self._generators.pop(request_id, None)

    # ------------------------------------------------------------------ the step function
    @torch.inference_mode()
    def execute(self, batch: Sequence[Tuple[Request, int]], want: Optional[Sequence[Sequence[int]]] = None) -> torch.Tensor:
        """Run the next ``n`` tokens of every ``(request, n)`` of the batch in one model step, from the caches and states
        the earlier steps left.  Returns the fp32 logits of the rows asked for, in the batch's order: ``want[b]`` lists
        the places among request ``b``'s tokens of this step (default: its last)."""
        if want is None:
            want = [[n - 1] for _, n in batch]
        # vLLM's row order: portions of prompts first, then the single decoded tokens
        order = sorted(range(len(batch)), key=lambda b: (batch[b][1] == 1 and batch[b][0].num_computed > 0, b))
        bs = self.pool.block_size
        tokens: List[int] = []
        positions: List[int] = []
        slot_mapping: List[int] = []
        query_lens, seq_lens, context_lens, tables = [], [], [], []
        row_of: Dict[Tuple[int, int], int] = {}
        ids: Dict[str, List[int]] = {}
        num_prefills = num_prefill_tokens = 0
        for b in order:
            r, n = batch[b]
            if n <= 0 or r.num_computed + n > len(r.token_ids):
                raise ValueError(f"request {r.request_id!r}: {n} tokens asked, {len(r.token_ids) - r.num_computed} left")
            ctx = r.num_computed
            self.pool.grow(r.blocks, ctx + n)
            for w in want[b]:
                if not 0 <= w < n:
                    raise ValueError(f"request {r.request_id!r}: place {w} is not among the step's {n} tokens")
                row_of[(b, w)] = len(tokens) + w
            tokens.extend(r.token_ids[ctx:ctx + n])
            positions.extend(range(ctx, ctx + n))
            slot_mapping.extend(r.blocks[p // bs] * bs + p % bs for p in range(ctx, ctx + n))
            query_lens.append(n), seq_lens.append(ctx + n), context_lens.append(ctx), tables.append(list(r.blocks))
            ids[r.state_key] = [0]
            if not (n == 1 and ctx > 0):
                num_prefills += 1
                num_prefill_tokens += n
        dev = self.device

        def i32(v):
            return torch.tensor(v, dtype=torch.int32, device=dev)

        width = max(len(t) for t in tables)
        block_tables = torch.zeros(len(tables), width, dtype=torch.int32)
        for k, t in enumerate(tables):
            block_tables[k, :len(t)] = torch.tensor(t, dtype=torch.int32)
        decode_lens = seq_lens[num_prefills:]
        md = MetaAttentionMetadata(
            num_prefills=num_prefills, num_prefill_tokens=num_prefill_tokens, num_decode_tokens=len(tokens) - num_prefill_tokens,
            slot_mapping=torch.tensor(slot_mapping, dtype=torch.int64, device=dev), multi_modal_placeholder_index_maps=None,
            enable_kv_scales_calculation=False, seq_lens=seq_lens, seq_lens_tensor=i32(seq_lens),
            max_prefill_seq_len=max(seq_lens[:num_prefills], default=0), max_decode_seq_len=max(decode_lens, default=0),
            context_lens_tensor=i32(context_lens), block_tables=block_tables.to(dev), use_cuda_graph=False,
            max_query_len=max(query_lens), max_decode_query_len=1,
            query_start_loc=i32(list(accumulate(query_lens, initial=0))), seq_start_loc=i32(list(accumulate(seq_lens, initial=0))))
        input_ids = torch.tensor(tokens, dtype=torch.int64, device=dev)
        pos = torch.tensor(positions, dtype=torch.int64, device=dev)
        finished, self._finished_since_last_step = self._finished_since_last_step, []
        with forward_context(md):
            hidden = self.model(input_ids, pos, request_ids_to_seq_ids=ids, finished_requests_ids=finished)
        for r, n in batch:
            r.num_computed += n
        rows = [row_of[(b, w)] for b in range(len(batch)) for w in want[b]]
        if not rows:
            return torch.empty(0, 0, dtype=torch.float32, device=dev)
        return self.model.compute_logits(hidden.index_select(0, torch.tensor(rows, dtype=torch.int64, device=dev)), None)

    def run_batch(self, entries: Sequence[Tuple[str, Sequence[int], Sequence[int]]]) -> torch.Tensor:
        """A batch given from outside: ``(request id, its next tokens, places whose logits are wanted)``.  A request is
        admitted at its first entry; its tokens are appended and run.  Returns ``[wanted rows, vocab]`` fp32."""
        batch, want = [], []
        for rid, toks, places in entries:
            r = self.requests.get(rid)
            if r is None:
                r = self.add_request(rid, [], schedule=False)
            r.token_ids.extend(int(t) for t in toks)
            r.num_prompt_tokens = len(r.token_ids)
            batch.append((r, len(toks)))
            want.append(list(places))
        return self.execute(batch, want)

    # ------------------------------------------------------------------ generation
    def _sample(self, logits: torch.Tensor, requests: Sequence[Request]) -> List[int]:
        greedy = hip_ops.argmax_rows(logits).tolist()
        out = []
        for k, r in enumerate(requests):
            if r.params.temperature <= 0:
                out.append(int(greedy[k]))
                continue
            g = self._generators.get(r.request_id)
            if g is None:
                g = self._generators[r.request_id] = torch.Generator(device=self.device)
                g.manual_seed(r.params.seed if r.params.seed is not None else hash(r.request_id) & 0x7fffffff)
            p = torch.softmax(logits[k] / r.params.temperature, -1)
            out.append(int(torch.multinomial(p, 1, generator=g)))
        return out

    def step(self) -> List[Request]:
        """One scheduler step: run the batch, sample a token for every request whose last known token it computed, retire
        the finished.  Returns the requests that finished in this step."""
        batch = self.scheduler.schedule()
        if not batch:
            if self.scheduler.has_work():
                raise RuntimeError("nothing can be scheduled: the page pool is too small for the waiting requests")
            return []
        sampling = [b for b, (r, n) in enumerate(batch) if r.num_computed + n == len(r.token_ids)]
        logits = self.execute(batch, [[n - 1] if b in sampling else [] for b, (r, n) in enumerate(batch)])
        done: List[Request] = []
        if sampling:
            rs = [batch[b][0] for b in sampling]
            for r, tok in zip(rs, self._sample(logits, rs)):
                r.token_ids.append(tok)
                if len(r.output_token_ids) >= r.params.max_tokens or tok in r.params.stop_token_ids:
                    done.append(r)
        for r in done:
            self.finish_request(r.request_id)
        return done

    def generate(self, prompts: Sequence[Sequence[int]], params: Optional[SamplingParams] = None) -> List[List[int]]:
        """Token ids generated for every prompt (lists of token ids), through the scheduler."""
        rs = [self.add_request(f"gen-{id(prompts)}-{k}", p, params) for k, p in enumerate(prompts)]
        while self.scheduler.has_work():
            self.step()
        return [r.output_token_ids for r in rs]


def iter_safetensors(model_dir: str) -> Iterator[Tuple[str, torch.Tensor]]:
    """``(name, tensor)`` of every ``*.safetensors`` file of a checkpoint folder, one tensor at a time."""
    from safetensors import safe_open
    files = sorted(f for f in os.listdir(model_dir) if f.endswith(".safetensors"))
    if not files:
        raise FileNotFoundError(f"{model_dir}: no .safetensors file")
    for fn in files:
        with safe_open(os.path.join(model_dir, fn), framework="pt", device="cpu") as f:
            for name in f.keys():
                yield name, f.get_tensor(name)
