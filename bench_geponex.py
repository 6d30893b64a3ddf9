"""Side benchmark of the Geponex design (``bench.py --design geponex``): prefill and decode throughput of a Geponex
stack at layer sizes that resemble a real model's (random weights), beside the package's closest existing model, Sonuzen
(fp32 stream, softmax attention over pages + a recurrent mixer + routed experts), at equal sizes -- same width, heads,
layers, experts and expert size -- and, kernel by kernel, how far each new kernel is from its roofline next to the like
kernel of that model.

Not the headline benchmark: ``bench.py`` without ``--design`` is unchanged.  Prints one JSON line.
"""
from __future__ import annotations

import json

import torch

from bench_sonuzen import BLOCK, HBM_GBS, MFMA_TFLOPS, SonuzenRunner, _events_ms, sonuzen_checkpoint, sonuzen_config


def geponex_config(width, heads, layers, experts, top, ff, vocab, kv_rank=128, rot_dim=64, dim=64, vdim=128, lin_dim=128, lin_vdim=128):
    ls = []
    for kind in layers:
        if kind == "lightning":
            mixer = dict(heads=heads, dim=lin_dim, vdim=lin_vdim, decay=[1.0 - 2.0 ** (-5 - 3 * h / max(heads - 1, 1)) for h in range(heads)])
        else:
            mixer = dict(heads=heads, dim=dim, rot_dim=rot_dim, vdim=vdim, kv_rank=kv_rank, q_rank=width // 4, scale=(dim + rot_dim) ** -0.5,
                         rot=dict(base=10000.0, dims=rot_dim))
            if kind == "latent_attention":
                mixer["rot"]["scaling"] = dict(factor=8.0, original=4096, fast=32.0, slow=1.0)
        mlp = dict(kind="moe", expert=dict(ff=ff, limit=7.0), router=dict(experts=experts, top=top, scale=1.0), shared=dict(ff=ff // 4, limit=7.0))
        ls.append(dict(type=kind, mixer=mixer, mlp=mlp))
    return dict(architecture="Geponex", vocab=vocab, width=width, layers=ls, norm=dict(eps=1e-6, groups=2), postln_alpha=2.0)


def geponex_checkpoint(cfg, dev, seed=0):
    g = torch.Generator(device=dev)
    g.manual_seed(seed)
    W, V = cfg["width"], cfg["vocab"]

    def rnd(*shape, std=1.0):
        return (torch.randn(*shape, device=dev, generator=g, dtype=torch.float32) * std).to(torch.bfloat16)

    def lin(o, i):
        return rnd(o, i, std=i ** -0.5)

    yield "embed", rnd(V, W, std=0.5)
    yield "final.norm", 1 + rnd(W, std=0.05)
    for i, spec in enumerate(cfg["layers"]):
        p, m = f"l{i}.", spec["mixer"]
        yield p + "norm1", 1 + rnd(W, std=0.05)
        yield p + "norm2", 1 + rnd(W, std=0.05)
        yield p + "shift", torch.rand(W, device=dev, generator=g).to(torch.bfloat16)
        H = m["heads"]
        if spec["type"] == "lightning":
            D, Dv = m["dim"], m["vdim"]
            for n, o in (("q", H * D), ("k", H * D), ("v", H * Dv), ("g", H * Dv)):
                yield p + "mix." + n, lin(o, W)
            yield p + "mix.o", lin(W, H * Dv)
            yield p + "mix.norm", 1 + rnd(H * Dv, std=0.05)
        else:
            D, R, Dv, C, Q = m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"], m["q_rank"]
            yield p + "mix.dq", lin(Q, W)
            yield p + "mix.dq.norm", 1 + rnd(Q, std=0.05)
            yield p + "mix.uq", lin(H * (D + R), Q)
            yield p + "mix.dkv", lin(C + R, W)
            yield p + "mix.dkv.norm", 1 + rnd(C, std=0.05)
            yield p + "mix.uk", lin(H * D, C)
            yield p + "mix.uv", lin(H * Dv, C)
            yield p + "mix.o", lin(W, H * Dv)
            if spec["type"] == "latent_attention_2":
                yield p + "mix.sink", rnd(H)
                yield p + "mix.g", lin(H * Dv, W)
        e = spec["mlp"]
        F, Fs = e["expert"]["ff"], e["shared"]["ff"]
        for j in range(e["router"]["experts"]):
            yield f"{p}mlp.e{j}.gate", lin(F, W)
            yield f"{p}mlp.e{j}.up", lin(F, W)
            yield f"{p}mlp.e{j}.down", lin(W, F)
        yield p + "mlp.router", lin(e["router"]["experts"], W)
        yield p + "mlp.shared.gate", lin(Fs, W)
        yield p + "mlp.shared.up", lin(Fs, W)
        yield p + "mlp.shared.down", lin(W, Fs)


def kernel_table(dev, W, H, B, ctx, L, E, top, ff, C=128, R=64, D=128):
    """(name, ms, fraction of the roofline that bounds it) for each new kernel and the like kernel of Sonuzen."""
    from vllm_hymeta import hip_ops
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

    # ---- attention over one prompt of L tokens: latent rows (one shared key/value head of C + R, value inside the key)
    # beside Sonuzen's attention with 4 key/value heads of D
    nblk = (L + BLOCK - 1) // BLOCK
    bt = torch.arange(nblk, dtype=torch.int32, device=dev).view(1, nblk)
    ql, kvl = rnd(L, H, C + R), rnd(nblk, BLOCK, 1, C + R)
    sink = rnd(H, dtype=torch.float32)
    add(f"latent attention prefill L={L} (H={H}, {C}+{R})",
        lambda: hip_ops.sink_attention(ql, kvl, bt, i32([0, L]), i32([L]), 1, C + R, C, 0.1, L, L, sink=True, sink_logits=sink, value_in_key=True),
        flops=H * L * L * (2 * C + R), iters=5)
    G = 4
    qs, kvs = rnd(L, H, D), rnd(nblk, BLOCK, G, 2 * D)
    r1, r2 = torch.full((H,), 0.5, device=dev), torch.full((H,), 0.1, device=dev)
    add(f"sink_attention prefill (Sonuzen) L={L} (H={H}, D={D})",
        lambda: hip_ops.sink_attention(qs, kvs, bt, i32([0, L]), i32([L]), G, D, D, D ** -0.5, L, L, r1, r2), flops=2 * H * D * L * L, iters=5)
    # ---- decode rows at context ctx
    bps = (ctx + 1 + BLOCK - 1) // BLOCK
    btd = torch.randperm(B * bps).to(torch.int32).view(B, bps).to(dev)
    sl = torch.full((B,), ctx + 1, dtype=torch.int32, device=dev)
    qsl = torch.arange(B + 1, dtype=torch.int32, device=dev)
    qd, kvd = rnd(B, H, C + R), rnd(B * bps, BLOCK, 1, C + R)
    add(f"latent attention decode B={B} ctx={ctx}",
        lambda: hip_ops.sink_attention(qd, kvd, btd, qsl, sl, 1, C + R, C, 0.1, 1, ctx + 1, sink=True, sink_logits=sink, value_in_key=True),
        nbytes=B * (ctx + 1) * (C + R) * 2)
    qd2, kvd2 = rnd(B, H, D), rnd(B * bps, BLOCK, G, 2 * D)
    add(f"sink_attention decode (Sonuzen) B={B} ctx={ctx}",
        lambda: hip_ops.sink_attention(qd2, kvd2, btd, qsl, sl, G, D, D, D ** -0.5, 1, ctx + 1, r1, r2), nbytes=B * G * (ctx + 1) * 2 * D * 2)
    # ---- a latent of 512 + 64 (value slices of 128, each launch repeats the scores), 16 heads
    Cw, Hw = 512, 16
    qw, kvw = rnd(L, Hw, Cw + R), rnd(nblk, BLOCK, 1, Cw + R)
    sinkw = rnd(Hw, dtype=torch.float32)
    add(f"latent attention prefill L={L} (H={Hw}, {Cw}+{R})",
        lambda: hip_ops.sink_attention(qw, kvw, bt, i32([0, L]), i32([L]), 1, Cw + R, Cw, 0.05, L, L, sink=True, sink_logits=sinkw, value_in_key=True),
        flops=Hw * L * L * (2 * Cw + R), iters=3)
    qwd, kvwd = rnd(B, Hw, Cw + R), rnd(B * bps, BLOCK, 1, Cw + R)
    add(f"latent attention decode B={B} ctx={ctx} (H={Hw}, {Cw}+{R})",
        lambda: hip_ops.sink_attention(qwd, kvwd, btd, qsl, sl, 1, Cw + R, Cw, 0.05, 1, ctx + 1, sink=True, sink_logits=sinkw, value_in_key=True),
        nbytes=B * (ctx + 1) * (Cw + R) * 2)
    # ---- the rest of the latent attention around its matrix products
    Q = W // 4
    proj = rnd(L, Q + C + R)
    freqs = torch.tensor([10000.0 ** (-2.0 * i / R) for i in range(R // 2)], dtype=torch.float64, device=dev)
    wq, wkv = torch.ones(Q, device=dev), torch.ones(C, device=dev)
    sm = torch.arange(L, dtype=torch.int64, device=dev)
    add(f"latent_kv_prep T={L}", lambda: hip_ops.latent_kv_prep_(proj, 0, Q, Q, C, R, R, wq, wkv, 1e-6, freqs, 1.0, kvl, sm, i32([0, L]), i32([L])),
        nbytes=L * ((2 * Q + C + R) * 2 + (C + R) * 2))
    qn, qa = rnd(L, H, 64 + R), rnd(H, L, C)
    add(f"latent_q_assemble T={L}", lambda: hip_ops.latent_q_assemble(qn, qa, 64, R, R, freqs, 1.0, i32([0, L]), i32([L])),
        nbytes=L * H * ((R + C) * 2 * 2))
    # ---- recurrences
    Dl = 128
    qkv = rnd(L, 2 * H * Dl + 2 * H * Dl)
    st = torch.zeros(2, H, Dl, Dl, device=dev)
    decay = torch.full((H,), 0.99, device=dev)
    add(f"lightning_attention prefill L={L} (H={H}, {Dl}x{Dl})",
        lambda: hip_ops.lightning_attention(qkv, st, decay, H, Dl, Dl, i32([0, L]), i32([0]), i32([1]), L),
        nbytes=L * H * (3 * Dl * 2 + Dl * 4), flops=L * H * (4 * Dl * Dl + 4 * 64 * Dl), iters=5)
    zug = rnd(L, 3 * W)
    stg = torch.zeros(4, W, device=dev)
    add(f"mingru prefill (Sonuzen) L={L}", lambda: hip_ops.mingru(zug, stg, i32([0, L]), i32([0]), i32([1]), L), nbytes=L * W * 4 * 2)
    qkvd = rnd(B, 4 * H * Dl)
    std_ = torch.zeros(B, H, Dl, Dl, device=dev)
    sidx = torch.arange(B, dtype=torch.int32, device=dev)
    ones = torch.ones(B, dtype=torch.int32, device=dev)
    add(f"lightning_attention decode B={B}", lambda: hip_ops.lightning_attention(qkvd, std_, decay, H, Dl, Dl, qsl, ones, sidx, 1),
        nbytes=B * H * (2 * Dl * Dl * 4 + 3 * Dl * 2 + Dl * 4))
    zd, stm = rnd(B, 3 * W), torch.zeros(B, W, device=dev)
    add(f"mingru decode (Sonuzen) B={B}", lambda: hip_ops.mingru(zd, stm, qsl, ones, sidx, 1), nbytes=B * W * (4 * 2 + 8))
    # ---- stream kernels
    for T in (B, L):
        x = rnd(T, W, dtype=torch.float32)
        wn = 1 + rnd(W, std=0.1, dtype=torch.float32)
        lay = (qsl, ones, sidx) if T == B else (i32([0, T]), i32([0]), i32([1]))
        shift_state = torch.zeros(max(B, 4), W, device=dev)
        mix = torch.rand(W, device=dev)
        add(f"token_shift T={T}", lambda: hip_ops.token_shift(x, mix, shift_state, bf, *lay), nbytes=T * W * (4 + 2))
        y = rnd(T, W)
        add(f"add_group_norm T={T}", lambda: hip_ops.add_group_norm(x, y, wn, 2, 1e-6, 2.0, out_dtype=bf), nbytes=T * W * (2 + 4 + 4 + 2))
        o, gt = rnd(T, H * Dl, dtype=torch.float32), rnd(T, H * Dl)
        wg = torch.ones(H * Dl, device=dev)
        add(f"gated_rms_norm T={T}", lambda: hip_ops.gated_rms_norm(o, gt, wg, 1e-6), nbytes=T * H * Dl * (4 + 2 + 2))
        cw = rnd(W, 3, std=0.2, dtype=torch.float32).contiguous()
        cs = torch.zeros(max(T, 4), 2, W, dtype=bf, device=dev)
        add(f"norm_conv (Sonuzen) T={T}", lambda: hip_ops.norm_conv(x, wn, 1e-5, bf, 1.0, cw, cs, *lay), nbytes=T * W * (4 + 2))
        add(f"norm_residual (Sonuzen) T={T}", lambda: hip_ops.norm_residual_(x, y, wn, 1e-5, 0.5, 1.0), nbytes=T * W * (2 + 4 + 4))
    # ---- experts
    w13, w2 = rnd(E, 2 * ff, W, std=W ** -0.5), rnd(E, W, ff, std=ff ** -0.5)
    router = rnd(E, W, std=W ** -0.5, dtype=torch.float32)
    table = torch.rand(1024, E, device=dev).argsort(1)[:, :top].to(torch.int32).contiguous()
    for T in (B, L):
        xm = rnd(T, W)
        ids = torch.randint(0, 1024, (T,), device=dev)
        wbytes = min(E, T * top) * 3 * ff * W * 2
        fl = T * top * 3 * ff * W * 2
        add(f"moe_sigmoid_forward T={T} (E={E}, top {top})", lambda: hip_ops.moe_sigmoid_forward(xm, router, w13, w2, top, 1.0, 7.0), nbytes=wbytes,
            flops=fl, iters=10 if T > 256 else 20)
        add(f"moe_table_forward (Sonuzen) T={T} (E={E}, top {top})", lambda: hip_ops.moe_table_forward(xm, ids, table, w13, w2), nbytes=wbytes,
            flops=fl, iters=10 if T > 256 else 20)
    return rows


def main(args):
    from vllm_hymeta.models.configuration_geponex import GeponexConfig
    from vllm_hymeta.models.configuration_sonuzen import SonuzenConfig
    from vllm_hymeta.models.modeling_geponex import GeponexForCausalLM
    from vllm_hymeta.models.modeling_sonuzen import SonuzenForCausalLM

    torch.cuda.set_device(0)
    dev = torch.device("cuda", 0)
    B, ctx, L = args.batch, args.ctx if args.ctx_given else 4096, min(args.prefill_ctx, 8192)
    vocab = 32768
    out = {"metric": "geponex_vs_sonuzen_tokens_per_s", "dtype": "bf16", "data": "synthetic", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
           "sizes": []}
    for (W, H, inter) in ((2048, 16, 8192), (3584, 28, 18944)):
        E, top = 8, 2
        ff = inter // top
        res = {}
        for name in ("sonuzen", "geponex"):
            if name == "sonuzen":
                cfg = sonuzen_config(W, H, 4, 128, ("attention", "mingru", "attention", "mingru"), E, top, ff, vocab)
                model = SonuzenForCausalLM(SonuzenConfig(cfg), max_num_seqs=max(B, 4), dtype=torch.bfloat16, device=dev)
                model.load_weights(sonuzen_checkpoint(cfg, dev))
            else:
                cfg = geponex_config(W, H, ("latent_attention_2", "lightning", "latent_attention", "lightning"), E, top, ff, vocab)
                model = GeponexForCausalLM(GeponexConfig(cfg), max_num_seqs=max(B, 4), dtype=torch.bfloat16, device=dev)
                model.load_weights(geponex_checkpoint(cfg, dev))
            run = SonuzenRunner(model, dev)
            dec = run.decode(B, ctx, args.steps, args.warmup)
            pre = run.prefill(L)
            res[name] = {"decode_ms_per_step": round(dec, 3), "decode_tokens_per_s": round(B / dec * 1e3, 1), "prefill_ms": round(pre, 2),
                         "prefill_tokens_per_s": round(L / pre * 1e3, 1)}
            del run, model
            torch.cuda.empty_cache()
        out["sizes"].append({"width": W, "heads": H, "layers": 4, "experts": E, "top": top, "expert_ff": ff, "batch": B, "ctx": ctx, "prompt": L,
                             "latent": {"kv_rank": 128, "rot_dim": 64, "dim": 64, "vdim": 128}, "lightning": {"dim": 128, "vdim": 128}, **res})
        print(json.dumps(out["sizes"][-1]), flush=True)
    out["kernels"] = kernel_table(dev, 3584, 28, B, ctx, L, 8, 2, 9472)
    s = out["sizes"][-1]
    out["value"], out["unit"] = s["geponex"]["decode_tokens_per_s"], "tokens/s"
    out["config"] = {"model": "Geponex 4 layers (latent attention / lightning, routed + shared experts)", "global_batch": B, "seq_len": ctx,
                     "parallelism": "tp1"}
    print(json.dumps(out))
