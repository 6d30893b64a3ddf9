"""Plain, slow CPU statement of the Sonuzen decoder, one function per mechanism, in whatever float type the inputs
have (the tests use float64).  TEST INFRASTRUCTURE ONLY: written from the model's equations, shares no code with the
product path, and also makes the random checkpoints the tests load into the product.

Every function sees ONE whole sequence from its first token: no cache, no state, no batching.
"""
from __future__ import annotations

import math
from typing import Dict, List, Optional

import torch


def rms_unit(x: torch.Tensor, eps: float) -> torch.Tensor:
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def norm_one_plus_ref(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    """RMS norm whose stored weight lies around zero."""
    return rms_unit(x, eps) * (1.0 + w)


def causal_conv_add_ref(h: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
    """``h [T, W]``, ``w [W, taps]``: ``h_t + sum_j w[:, j] h_{t - taps + 1 + j}``, zeros before the sequence."""
    T, taps = h.shape[0], w.shape[1]
    out = h.clone()
    for t in range(T):
        for j in range(taps):
            src = t - taps + 1 + j
            if src >= 0:
                out[t] = out[t] + w[:, j] * h[src]
    return out


def mingru_ref(h: torch.Tensor, wz, bz, wx, bx, wg, wo) -> torch.Tensor:
    S = torch.zeros(wz.shape[0], dtype=h.dtype)
    rows = []
    for t in range(h.shape[0]):
        z = torch.sigmoid(wz @ h[t] + bz)
        u = wx @ h[t] + bx
        cand = torch.where(u >= 0, u + 0.5, torch.sigmoid(u))
        S = (1 - z) * S + z * cand
        g = wg @ h[t]
        rows.append(wo @ (S * (g * torch.sigmoid(g))))
    return torch.stack(rows)


def sink_attention_ref(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, scale: float, r1: Optional[torch.Tensor],
                       r2: Optional[torch.Tensor], sink: bool = True, window_left: int = -1) -> torch.Tensor:
    """``q [T, H, D]``, ``k [T, G, D]``, ``v [T, G, Dv]`` (already normed) -> ``[T, H, Dv]``.  Row by row, key by key."""
    T, H, _ = q.shape
    G = k.shape[1]
    out = torch.zeros(T, H, v.shape[2], dtype=q.dtype)
    for h in range(H):
        g = h // (H // G)
        for i in range(T):
            lo = 0 if window_left < 0 else max(0, i - window_left)
            s = (k[lo:i + 1, g] @ q[i, h]) * scale                      # one score per visible key j = lo .. i
            if r1 is not None:
                s = s - r1[h] * torch.log1p(r2[h] * (i - torch.arange(lo, i + 1)).to(q.dtype))
            e = torch.exp(s)
            p = e / ((1.0 if sink else 0.0) + e.sum())
            out[i, h] = (p[:, None] * v[lo:i + 1, g]).sum(0)
    return out


def attention_mixer_ref(h: torch.Tensor, wq, wk, wv, wo, q_norm, k_norm, r1, r2, heads: int, kv_heads: int, dim: int, vdim: int,
                        scale: float, eps: float) -> torch.Tensor:
    T = h.shape[0]
    q = (h @ wq.T).view(T, heads, dim)
    k = (h @ wk.T).view(T, kv_heads, dim)
    v = (h @ wv.T).view(T, kv_heads, vdim)
    q = rms_unit(q, eps) * q_norm
    k = rms_unit(k, eps) * k_norm
    return sink_attention_ref(q, k, v, scale, r1, r2).reshape(T, heads * vdim) @ wo.T


def table_moe_ref(h: torch.Tensor, tokens: List[int], table: torch.Tensor, gates, ups, downs) -> torch.Tensor:
    top = table.shape[1]
    out = torch.zeros(h.shape[0], downs[0].shape[0], dtype=h.dtype)
    for t, tok in enumerate(tokens):
        for e in table[tok].tolist():
            g = gates[e] @ h[t]
            out[t] = out[t] + (downs[e] @ ((g * torch.sigmoid(g)) * (ups[e] @ h[t]))) / top
    return out


def layer_runs_ref(cfg: dict) -> List[tuple]:
    """``(layer, number of the pass it starts or None)`` in execution order."""
    n = len(cfg["layers"])
    loop = cfg.get("loop")
    if not loop or loop["stop"] <= loop["start"]:
        return [(i, None) for i in range(n)]
    runs = [(i, None) for i in range(loop["start"])]
    for t in range(loop["times"]):
        runs += [(i, t if i == loop["start"] else None) for i in range(loop["start"], loop["stop"])]
    return runs + [(i, None) for i in range(loop["stop"], n)]


def sonuzen_ref(cfg: dict, weights: Dict[str, torch.Tensor], tokens: List[int], dtype=torch.float64,
                residual_out: Optional[list] = None) -> torch.Tensor:
    """Logits ``[T, vocab]`` of one sequence."""
    W = {k: (v.to(dtype) if v.dtype.is_floating_point else v.long()) for k, v in weights.items()}
    eps, m = cfg["norm"]["eps"], cfg["residual_mult"]
    x = W["embed"][tokens]
    for i, starts_pass in layer_runs_ref(cfg):
        if starts_pass is not None:
            x = x + W["loop.step"][starts_pass]
        spec, p = cfg["layers"][i], f"l{i}."
        h = norm_one_plus_ref(x, W[p + "norm1"], eps)
        if cfg.get("canon"):
            h = causal_conv_add_ref(h, W[p + "canon1"])
        if spec["type"] == "mingru":
            y = mingru_ref(h, W[p + "mix.z"], W[p + "mix.z.b"], W[p + "mix.x"], W[p + "mix.x.b"], W[p + "mix.g"], W[p + "mix.o"])
        else:
            a = spec["mixer"]
            y = attention_mixer_ref(h, W[p + "mix.q"], W[p + "mix.k"], W[p + "mix.v"], W[p + "mix.o"], W[p + "mix.q.norm"],
                                    W[p + "mix.k.norm"], W[p + "mix.r1"], W[p + "mix.r2"], a["heads"], a["kv_heads"], a["dim"],
                                    a["vdim"], a["scale"], eps)
        x = x + m * norm_one_plus_ref(y, W[p + "norm1b"], eps)
        if spec["mlp"] is not None:
            h = norm_one_plus_ref(x, W[p + "norm2"], eps)
            if cfg.get("canon"):
                h = causal_conv_add_ref(h, W[p + "canon2"])
            E = spec["mlp"]["router"]["experts"]
            y = table_moe_ref(h, tokens, W[p + "mlp.table"], [W[f"{p}mlp.e{e}.gate"] for e in range(E)],
                              [W[f"{p}mlp.e{e}.up"] for e in range(E)], [W[f"{p}mlp.e{e}.down"] for e in range(E)])
            x = x + m * norm_one_plus_ref(y, W[p + "norm2b"], eps)
        if residual_out is not None:
            residual_out.append(x.clone())
    return (norm_one_plus_ref(x, W["final.norm"], eps) @ W["head"].T) * cfg["logit_scale"]


# --------------------------------------------------------------------------- random checkpoints for the tests
def sonuzen_config(vocab=96, width=64, layers=("attention", "mingru"), heads=4, kv_heads=2, dim=16, vdim=24, mingru_width=None,
                   experts=4, top=2, ff=32, taps=3, loop=None, residual_mult=0.5, logit_scale=0.75, eps=1e-5, scale=None,
                   no_mlp=()) -> dict:
    ls = []
    for i, kind in enumerate(layers):
        if kind == "attention":
            mixer = dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, scale=scale if scale is not None else dim ** -0.5)
        else:
            mixer = dict(width=mingru_width or width)
        mlp = None if i in no_mlp else dict(kind="moe", expert=dict(ff=ff), router=dict(experts=experts, top=top))
        ls.append(dict(type=kind, mixer=mixer, mlp=mlp))
    cfg = dict(architecture="Sonuzen", vocab=vocab, width=width, layers=ls, norm=dict(eps=eps), residual_mult=residual_mult,
               logit_scale=logit_scale)
    if taps:
        cfg["canon"] = dict(taps=taps)
    if loop:
        cfg["loop"] = dict(start=loop[0], stop=loop[1], times=loop[2])
    return cfg


def sonuzen_random_weights(cfg: dict, seed: int = 0) -> Dict[str, torch.Tensor]:
    """bf16 tensors (int32 tables) under the checkpoint's names."""
    g = torch.Generator().manual_seed(seed)
    W, V = cfg["width"], cfg["vocab"]

    def rnd(*shape, std=1.0):
        return (torch.randn(*shape, generator=g) * std).to(torch.bfloat16)

    out = {"embed": rnd(V, W), "head": rnd(V, W, std=W ** -0.5), "final.norm": rnd(W, std=0.1)}
    if cfg.get("loop"):
        out["loop.step"] = rnd(cfg["loop"]["times"], W, std=0.3)
    taps = (cfg.get("canon") or {}).get("taps", 0)
    for i, spec in enumerate(cfg["layers"]):
        p = f"l{i}."
        for n in ("norm1", "norm1b") + (("norm2", "norm2b") if spec["mlp"] is not None else ()):
            out[p + n] = rnd(W, std=0.1)
        if taps:
            out[p + "canon1"] = rnd(W, taps, std=0.3)
            if spec["mlp"] is not None:
                out[p + "canon2"] = rnd(W, taps, std=0.3)
        mx = spec["mixer"]
        if spec["type"] == "attention":
            H, G, D, Dv = mx["heads"], mx["kv_heads"], mx["dim"], mx["vdim"]
            out[p + "mix.q"], out[p + "mix.k"] = rnd(H * D, W, std=W ** -0.5), rnd(G * D, W, std=W ** -0.5)
            out[p + "mix.v"], out[p + "mix.o"] = rnd(G * Dv, W, std=W ** -0.5), rnd(W, H * Dv, std=(H * Dv) ** -0.5)
            out[p + "mix.q.norm"], out[p + "mix.k.norm"] = 1 + rnd(D, std=0.2), 1 + rnd(D, std=0.2)
            out[p + "mix.r1"] = (torch.rand(H, generator=g) * 1.5 + 0.1).to(torch.bfloat16)
            out[p + "mix.r2"] = (torch.rand(H, generator=g) * 0.5 + 0.02).to(torch.bfloat16)
        else:
            M = mx["width"]
            for n in ("z", "x", "g"):
                out[p + "mix." + n] = rnd(M, W, std=W ** -0.5)
            out[p + "mix.z.b"], out[p + "mix.x.b"] = rnd(M, std=0.5), rnd(M, std=0.5)
            out[p + "mix.o"] = rnd(W, M, std=M ** -0.5)
        if spec["mlp"] is not None:
            E, top, ff = spec["mlp"]["router"]["experts"], spec["mlp"]["router"]["top"], spec["mlp"]["expert"]["ff"]
            for e in range(E):
                out[f"{p}mlp.e{e}.gate"], out[f"{p}mlp.e{e}.up"] = rnd(ff, W, std=W ** -0.5), rnd(ff, W, std=W ** -0.5)
                out[f"{p}mlp.e{e}.down"] = rnd(W, ff, std=ff ** -0.5)
            out[p + "mlp.table"] = torch.stack([torch.randperm(E, generator=g)[:top] for _ in range(V)]).to(torch.int32)
    return out
