"""Side benchmark of the Sonuzen design (``bench.py --design sonuzen``): prefill and decode throughput of a Sonuzen
stack at the layer sizes of a real model (random weights), beside the package's closest existing model, the 7B
"gla_swa" hybrid (recurrent layers + softmax attention layers + gated feed-forward), at equal sizes -- same width,
heads, head size, layers, and as many feed-forward weights ACTIVE per token -- and, kernel by kernel, how far each new
kernel is from its roofline next to the like kernel of that model.

Not the headline benchmark: ``bench.py`` without ``--design`` is unchanged.  Prints one JSON line.
"""
from __future__ import annotations

import json
import time

import torch

HBM_GBS = 8000.0          # MI355X HBM3E peak
MFMA_TFLOPS = 2500.0      # dense bf16 peak
BLOCK = 256


def _events_ms(fn, iters=20, warm=3):
    for _ in range(warm):
        fn()
    torch.cuda.synchronize()
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    a.record()
    for _ in range(iters):
        fn()
    b.record()
    torch.cuda.synchronize()
    return a.elapsed_time(b) / iters


def sonuzen_config(width, heads, kv_heads, dim, layers, experts, top, ff, vocab, taps=3):
    ls = []
    for kind in layers:
        mixer = dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=dim, scale=dim ** -0.5) if kind == "attention" else dict(width=width)
        ls.append(dict(type=kind, mixer=mixer, mlp=dict(kind="moe", expert=dict(ff=ff), router=dict(experts=experts, top=top))))
    return dict(architecture="Sonuzen", vocab=vocab, width=width, layers=ls, norm=dict(eps=1e-5), residual_mult=0.5, logit_scale=1.0,
                canon=dict(taps=taps))


def sonuzen_checkpoint(cfg, dev, seed=0):
    g = torch.Generator(device=dev)
    g.manual_seed(seed)
    W, V = cfg["width"], cfg["vocab"]

    def rnd(*shape, std=1.0):
        return (torch.randn(*shape, device=dev, generator=g, dtype=torch.float32) * std).to(torch.bfloat16)

    yield "embed", rnd(V, W, std=0.5)
    yield "head", rnd(V, W, std=0.02)
    yield "final.norm", rnd(W, std=0.05)
    taps = cfg["canon"]["taps"]
    for i, spec in enumerate(cfg["layers"]):
        p = f"l{i}."
        for n in ("norm1", "norm1b", "norm2", "norm2b"):
            yield p + n, rnd(W, std=0.05)
        yield p + "canon1", rnd(W, taps, std=0.2)
        yield p + "canon2", rnd(W, taps, std=0.2)
        mx = spec["mixer"]
        if spec["type"] == "attention":
            H, G, D, Dv = mx["heads"], mx["kv_heads"], mx["dim"], mx["vdim"]
            yield p + "mix.q", rnd(H * D, W, std=W ** -0.5)
            yield p + "mix.k", rnd(G * D, W, std=W ** -0.5)
            yield p + "mix.v", rnd(G * Dv, W, std=W ** -0.5)
            yield p + "mix.o", rnd(W, H * Dv, std=(H * Dv) ** -0.5)
            yield p + "mix.q.norm", torch.ones(D, dtype=torch.bfloat16, device=dev)
            yield p + "mix.k.norm", torch.ones(D, dtype=torch.bfloat16, device=dev)
            yield p + "mix.r1", torch.full((H,), 0.5, dtype=torch.bfloat16, device=dev)
            yield p + "mix.r2", torch.full((H,), 0.1, dtype=torch.bfloat16, device=dev)
        else:
            for n in ("z", "x", "g"):
                yield p + "mix." + n, rnd(W, W, std=W ** -0.5)
            yield p + "mix.z.b", rnd(W, std=0.3)
            yield p + "mix.x.b", rnd(W, std=0.3)
            yield p + "mix.o", rnd(W, W, std=W ** -0.5)
        E, top, ff = spec["mlp"]["router"]["experts"], spec["mlp"]["router"]["top"], spec["mlp"]["expert"]["ff"]
        for e in range(E):
            yield f"{p}mlp.e{e}.gate", rnd(ff, W, std=W ** -0.5)
            yield f"{p}mlp.e{e}.up", rnd(ff, W, std=W ** -0.5)
            yield f"{p}mlp.e{e}.down", rnd(W, ff, std=ff ** -0.5)
        yield p + "mlp.table", torch.rand(V, E, device=dev, generator=g).argsort(1)[:, :top].to(torch.int32).contiguous()


class SonuzenRunner:
    """The model class under static metadata: a decode batch replayed from one HIP graph (as ``bench.DecodeRunner`` replays the
    7B step), or one prompt run eagerly."""

    def __init__(self, model, dev):
        self.model, self.dev = model, dev
        self.layers = list(model.model.attn_layers.values())

    def _bind(self, nblk):
        from vllm_hymeta.models.attention import bind_kv_cache
        self.kv = [torch.randn(l.kv_cache_shape(nblk, BLOCK), device=self.dev, dtype=torch.float32).to(torch.bfloat16) for l in self.layers]
        for l, kv in zip(self.layers, self.kv):
            bind_kv_cache(l, kv)

    def _metadata(self, S, q, ctx, block_tables, slot_mapping, seq_lens, context_lens, max_seq):
        from vllm_hymeta.attention.meta_attention import MetaAttentionMetadata
        qsl = torch.arange(0, (S + 1) * q, q, dtype=torch.int32, device=self.dev)
        return MetaAttentionMetadata(
            num_prefills=S if q > 1 else 0, num_prefill_tokens=S * q if q > 1 else 0, num_decode_tokens=S if q == 1 else 0,
            slot_mapping=slot_mapping, multi_modal_placeholder_index_maps=None, enable_kv_scales_calculation=False, seq_lens=None,
            seq_lens_tensor=seq_lens, max_prefill_seq_len=max_seq if q > 1 else 0, max_decode_seq_len=max_seq if q == 1 else 0,
            context_lens_tensor=context_lens, block_tables=block_tables, use_cuda_graph=q == 1, max_query_len=q, max_decode_query_len=1,
            query_start_loc=qsl, seq_start_loc=None)

    def decode(self, B, ctx, steps, warmup):
        from vllm_hymeta import hip_ops
        dev = self.dev
        bps = (ctx + steps + warmup + 8 + BLOCK - 1) // BLOCK
        self._bind(B * bps)
        g = torch.Generator(device="cpu")
        g.manual_seed(1)
        bt = torch.randperm(B * bps, generator=g).to(torch.int32).view(B, bps).to(dev)
        positions = torch.full((B,), ctx, dtype=torch.int64, device=dev)
        seq_lens = torch.full((B,), ctx + 1, dtype=torch.int32, device=dev)
        context_lens = torch.full((B,), ctx, dtype=torch.int32, device=dev)
        slot_mapping = (torch.gather(bt.long(), 1, (positions // BLOCK).unsqueeze(1)).squeeze(1) * BLOCK + positions % BLOCK).contiguous()
        ids = torch.randint(0, self.model.config.vocab_size, (B,), generator=g).to(dev)
        md = self._metadata(B, 1, ctx, bt, slot_mapping, seq_lens, context_lens, ctx + steps + warmup + 8)
        cache, idx = self.model.get_seqlen_agnostic_capture_inputs(B)
        idx.copy_(torch.arange(B, dtype=torch.int32, device=dev))

        def step():
            h = self.model(ids, positions, attn_metadata=md, seqlen_agnostic_capture_inputs=(cache, idx))
            hip_ops.argmax_rows(self.model.compute_logits(h), out=ids)

        for _ in range(2):
            step()
        torch.cuda.synchronize()
        side, graph = torch.cuda.Stream(), torch.cuda.CUDAGraph()
        with torch.cuda.stream(side):
            step()
            with torch.cuda.graph(graph, stream=side):
                step()
        torch.cuda.synchronize()

        def advance():
            hip_ops.advance_step(B, B, BLOCK, seq_lens, slot_mapping, bt, input_positions=positions)
            context_lens.add_(1)

        for _ in range(warmup):
            advance()
            graph.replay()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            advance()
            graph.replay()
        torch.cuda.synchronize()
        ms = (time.perf_counter() - t0) * 1e3 / steps
        del graph
        return ms

    def prefill(self, L, runs=3):
        from vllm_hymeta import hip_ops
        dev = self.dev
        nblk = (L + BLOCK - 1) // BLOCK
        self._bind(nblk)
        bt = torch.arange(nblk, dtype=torch.int32, device=dev).view(1, nblk)
        md = self._metadata(1, L, 0, bt, torch.arange(L, dtype=torch.int64, device=dev), torch.tensor([L], dtype=torch.int32, device=dev),
                            torch.zeros(1, dtype=torch.int32, device=dev), L)
        ids = torch.randint(0, self.model.config.vocab_size, (L,), device=dev)
        pos = torch.arange(L, dtype=torch.int64, device=dev)
        cache, idx = self.model.get_seqlen_agnostic_capture_inputs(1)
        idx.zero_()

        def run():
            h = self.model(ids, pos, attn_metadata=md, seqlen_agnostic_capture_inputs=(cache, idx))
            return hip_ops.argmax_rows(self.model.compute_logits(h[-1:]))

        run()
        torch.cuda.synchronize()
        ts = []
        for _ in range(runs):
            t0 = time.perf_counter()
            run()
            torch.cuda.synchronize()
            ts.append((time.perf_counter() - t0) * 1e3)
        return sorted(ts)[len(ts) // 2]


def kernel_table(dev, W, H, G, D, B, ctx, L, E, top, ff):
    """(name, ms, fraction of the roofline that bounds it) for each new kernel and the like kernel of the 7B model."""
    from vllm_hymeta import _C, hip_ops
    rows = []
    bf = torch.bfloat16

    def rnd(*shape, std=1.0, dtype=bf):
        return (torch.randn(*shape, device=dev, dtype=torch.float32) * std).to(dtype)

    def i32(v):
        return torch.tensor(v, dtype=torch.int32, device=dev)

    def add(name, fn, nbytes=0, flops=0, iters=20):
        ms = _events_ms(fn, iters=iters)
        t_mem, t_mma = nbytes / (HBM_GBS * 1e9) * 1e3, flops / (MFMA_TFLOPS * 1e12) * 1e3
        rows.append(dict(kernel=name, ms=round(ms, 4), roofline_ms=round(max(t_mem, t_mma), 4), bound="hbm" if t_mem >= t_mma else "mfma",
                         fraction_of_roofline=round(max(t_mem, t_mma) / ms, 3)))

    # ---- attention, one prompt of L tokens
    nblk = (L + BLOCK - 1) // BLOCK
    q = rnd(L, H, D)
    kvc = rnd(nblk, BLOCK, G, 2 * D)
    bt = torch.arange(nblk, dtype=torch.int32, device=dev).view(1, nblk)
    r1, r2 = torch.full((H,), 0.5, device=dev), torch.full((H,), 0.1, device=dev)
    causal_flops = 2 * H * D * L * L            # QK^T and PV over the causal half
    add(f"sink_attention prefill L={L}", lambda: hip_ops.sink_attention(q, kvc, bt, i32([0, L]), i32([L]), G, D, D, D ** -0.5, L, L, r1, r2),
        flops=causal_flops, iters=5)
    k7, v7 = rnd(L, G, D), rnd(L, G, D)
    cu = i32([0, L])
    add(f"meta_swa_prefill (7B, full causal) L={L}", lambda: hip_ops.meta_swa_prefill(q, cu, L, key=k7, value=v7, cu_seqlens_k=cu, window_left=-1),
        flops=causal_flops, iters=5)
    # ---- attention, B decode rows at context ctx
    bps = (ctx + 1 + BLOCK - 1) // BLOCK
    kvd = rnd(B * bps, BLOCK, G, 2 * D)
    btd = torch.randperm(B * bps).to(torch.int32).view(B, bps).to(dev)
    qd = rnd(B, H, D)
    sl = torch.full((B,), ctx + 1, dtype=torch.int32, device=dev)
    qsl = torch.arange(B + 1, dtype=torch.int32, device=dev)
    kv_bytes = B * G * (ctx + 1) * 2 * D * 2
    add(f"sink_attention decode B={B} ctx={ctx}", lambda: hip_ops.sink_attention(qd, kvd, btd, qsl, sl, G, D, D, D ** -0.5, 1, ctx + 1, r1, r2),
        nbytes=kv_bytes)
    kv7 = rnd(2, B * bps, BLOCK, G, D)
    add(f"meta_swa_paged_decode (7B) B={B} ctx={ctx}", lambda: hip_ops.meta_swa_paged_decode(qd, kv7[0], kv7[1], sl, btd, window_left=-1,
                                                                                          max_seqlen_k=ctx + 1), nbytes=kv_bytes)
    # ---- recurrences
    zug = rnd(L, 3 * W)
    st = torch.zeros(4, W, device=dev)
    add(f"mingru prefill L={L}", lambda: hip_ops.mingru(zug, st, i32([0, L]), i32([0]), i32([1]), L), nbytes=L * W * 4 * 2)
    qg, kg, vg, gg = rnd(L, H, D), rnd(L, G, D), rnd(L, G, D), -torch.rand(L, G, D, device=dev) / 16
    st7 = torch.zeros(2, G, D, D, dtype=bf, device=dev)
    # chunked gated linear attention: per token and head 2 D^2 (state) + the in-chunk products; its bytes: q, k, v, g, out
    add(f"gla_prefill_varlen (7B) L={L}", lambda: hip_ops.gla_prefill_varlen(qg, kg, vg, gg, st7, i32([1]), i32([0, L]), L, context_lens=i32([0])),
        nbytes=L * (2 * H * D * 2 + 2 * G * D * 2 + G * D * 4), flops=L * H * 4 * D * D, iters=5)
    zd = rnd(B, 3 * W)
    std_ = torch.zeros(B, W, device=dev)
    sidx = torch.arange(B, dtype=torch.int32, device=dev)
    ones = torch.ones(B, dtype=torch.int32, device=dev)
    add(f"mingru decode B={B}", lambda: hip_ops.mingru(zd, std_, qsl, ones, sidx, 1), nbytes=B * W * (4 * 2 + 8))
    qs, ks, vs, gs = rnd(B, H, D), rnd(B, G, D), rnd(B, G, D), -torch.rand(B, G, D, device=dev) / 16
    st7d = torch.zeros(B, G, D, D, dtype=bf, device=dev)
    add(f"gla_decode (7B) B={B}", lambda: hip_ops.gla_decode(qs, ks, vs, gs, st7d, sidx), nbytes=B * (2 * G * D * D * 2 + 2 * H * D * 2))
    # ---- norms
    for T in (B, L):
        x = rnd(T, W, dtype=torch.float32)
        wn, cw = rnd(W, std=0.1, dtype=torch.float32), rnd(W, 3, std=0.2, dtype=torch.float32).contiguous()
        cs = torch.zeros(max(T, 4), 2, W, dtype=bf, device=dev)
        if T == B:
            lay = (qsl, ones, sidx)
        else:
            lay = (i32([0, T]), i32([0]), i32([1]))
        add(f"norm_conv T={T}", lambda: hip_ops.norm_conv(x, wn, 1e-5, bf, 1.0, cw, cs, *lay), nbytes=T * W * (4 + 2))
        y = rnd(T, W)
        add(f"norm_residual T={T}", lambda: hip_ops.norm_residual_(x, y, wn, 1e-5, 0.5, 1.0), nbytes=T * W * (2 + 4 + 4))
        xb, res, w7 = rnd(T, W), rnd(T, W), torch.ones(W, dtype=bf, device=dev)
        add(f"add_rmsnorm (7B) T={T}", lambda: hip_ops.add_rmsnorm(xb, w7, 1e-6, residual=res), nbytes=T * W * (2 + 2 + 2 + 2))
    # ---- experts
    w13, w2 = rnd(E, 2 * ff, W, std=W ** -0.5), rnd(E, W, ff, std=ff ** -0.5)
    table = torch.rand(1024, E, device=dev).argsort(1)[:, :top].to(torch.int32).contiguous()
    for T in (B, L):
        xm = rnd(T, W)
        ids = torch.randint(0, 1024, (T,), device=dev)
        lg = rnd(T, E)
        wbytes = min(E, T * top) * 3 * ff * W * 2
        fl = T * top * 3 * ff * W * 2
        add(f"moe_table_forward T={T} (E={E}, top {top})", lambda: hip_ops.moe_table_forward(xm, ids, table, w13, w2), nbytes=wbytes, flops=fl,
            iters=10 if T > 256 else 20)
        add(f"moe_forward (routed block) T={T} (E={E}, top {top})", lambda: hip_ops.moe_forward(xm, lg, w13, w2, top_k=top), nbytes=wbytes,
            flops=fl, iters=10 if T > 256 else 20)
    return rows


def main(args):
    import bench
    from vllm_hymeta.model_for_7B.configuration_gla_swa import GLAswaConfig
    from vllm_hymeta.model_for_7B.modeling_gla_swa import GLAswaForCausalLM
    from vllm_hymeta.models.configuration_sonuzen import SonuzenConfig
    from vllm_hymeta.models.modeling_sonuzen import SonuzenForCausalLM

    torch.cuda.set_device(0)
    dev = torch.device("cuda", 0)
    B, ctx, L = args.batch, args.ctx if args.ctx_given else 4096, min(args.prefill_ctx, 8192)
    vocab, layers = 32768, 4
    out = {"metric": "sonuzen_vs_gla_swa_tokens_per_s", "dtype": "bf16", "data": "synthetic", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
           "sizes": []}
    for (W, H, G, inter) in ((2048, 16, 4, 8192), (3584, 28, 4, 18944)):
        D, E, top = 128, 8, 2
        ff = inter // top
        # ---- the 7B family at this geometry: GLA, attention, GLA, attention; window beyond the context = full causal attention
        cfg7 = GLAswaConfig(vocab_size=vocab, hidden_size=W, num_hidden_layers=layers, num_attention_heads=H, num_key_value_heads=G,
                            intermediate_size=inter, sliding_window=1 << 20)
        m7 = GLAswaForCausalLM(cfg7, max_num_seqs=B, device=dev)
        m7.load_weights(bench.synthetic_checkpoint_7b(cfg7, dev, "bf16"))
        total = args.warmup + args.steps
        r7 = bench.DecodeRunner(m7, B, ctx, total, dev)
        r7.capture()
        for _ in range(args.warmup):
            r7.step()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            r7.step()
        torch.cuda.synchronize()
        dec7 = (time.perf_counter() - t0) * 1e3 / args.steps
        del r7
        pre7 = bench.ttft_only(m7, dev, L)
        del m7
        torch.cuda.empty_cache()
        # ---- Sonuzen: attention, minGRU, attention, minGRU; E experts of ff, top active = the dense MLP's weights per token
        cfg = sonuzen_config(W, H, G, D, ("attention", "mingru", "attention", "mingru"), E, top, ff, vocab)
        ms = SonuzenForCausalLM(SonuzenConfig(cfg), max_num_seqs=max(B, 4), dtype=torch.bfloat16, device=dev)
        ms.load_weights(sonuzen_checkpoint(cfg, dev))
        run = SonuzenRunner(ms, dev)
        dec = run.decode(B, ctx, args.steps, args.warmup)
        pre = run.prefill(L)
        del run, ms
        torch.cuda.empty_cache()
        out["sizes"].append({"width": W, "heads": H, "kv_heads": G, "head_dim": D, "layers": layers, "active_ff": inter,
                             "experts": E, "top": top, "batch": B, "ctx": ctx, "prompt": L,
                             "sonuzen": {"decode_ms_per_step": round(dec, 3), "decode_tokens_per_s": round(B / dec * 1e3, 1),
                                         "prefill_ms": round(pre, 2), "prefill_tokens_per_s": round(L / pre * 1e3, 1)},
                             "gla_swa": {"decode_ms_per_step": round(dec7, 3), "decode_tokens_per_s": round(B / dec7 * 1e3, 1),
                                         "prefill_ms": round(pre7, 2), "prefill_tokens_per_s": round(L / pre7 * 1e3, 1)}})
        print(json.dumps(out["sizes"][-1]), flush=True)
    out["kernels"] = kernel_table(dev, 3584, 28, 4, 128, B, ctx, L, 8, 2, 9472)
    s = out["sizes"][-1]
    out["value"], out["unit"] = s["sonuzen"]["decode_tokens_per_s"], "tokens/s"
    out["config"] = {"model": "Sonuzen 4 layers at the 7B layer geometry", "global_batch": B, "seq_len": ctx, "parallelism": "tp1"}
    print(json.dumps(out))
