"""Plain, slow CPU statement of the Geponex decoder, one function per mechanism, in whatever float type the inputs
have (the tests use float64).  TEST INFRASTRUCTURE ONLY: written from the model's equations, shares no code with the
product path, and also makes the random checkpoints the tests load into the product.

Every function sees ONE whole sequence from its first token: no cache, no state, no batching.

The design: a post-norm decoder (``x <- norm(alpha x + sublayer(x))``, grouped RMS norm) whose mixers read a token-shifted
input and are either a latent attention (queries and keys/values through low-rank latents, a rotated key part shared by the
heads; optionally with YaRN-scaled frequencies, or with a per-head sink logit and an output gate) or a lightning attention
(linear attention with a constant decay per head); the feed-forward is dense (xIELU) or a sigmoid-routed mixture of clamped
gated experts with a shared expert.
"""
from __future__ import annotations

import math
from typing import Dict, List, Optional

import torch


# ------------------------------------------------------------------------------------------------ norms, shift
def rms_unit(x: torch.Tensor, eps: float) -> torch.Tensor:
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def group_norm_ref(x: torch.Tensor, w: torch.Tensor, groups: int, eps: float) -> torch.Tensor:
    """``x [..., W]`` split into ``groups`` consecutive parts, each divided by its own root mean square; times ``w``."""
    parts = x.reshape(*x.shape[:-1], groups, x.shape[-1] // groups)
    return rms_unit(parts, eps).reshape(x.shape) * w


def token_shift_ref(h: torch.Tensor, mu: torch.Tensor) -> torch.Tensor:
    """``h_t + (h_{t-1} - h_t) mu`` with zeros before the first token."""
    prev = torch.cat([torch.zeros_like(h[:1]), h[:-1]], 0)
    return h + (prev - h) * mu


# ------------------------------------------------------------------------------------------------ rotation
def rotary_frequencies_ref(dims: int, base: float, scaling: Optional[dict]):
    """Frequencies ``[dims / 2]`` (float64) and the factor on cos and sin."""
    f = torch.tensor([base ** (-2.0 * i / dims) for i in range(dims // 2)], dtype=torch.float64)
    if not scaling:
        return f, 1.0
    factor, orig = float(scaling["factor"]), float(scaling["original"])

    def turn_dim(turns):
        return dims * math.log(orig / (2 * math.pi * turns)) / (2 * math.log(base))

    lo = max(math.floor(turn_dim(float(scaling["fast"]))), 0)
    hi = min(math.ceil(turn_dim(float(scaling["slow"]))), dims - 1)
    ramp = torch.tensor([min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0) for i in range(dims // 2)], dtype=torch.float64)
    return f / factor * ramp + f * (1 - ramp), 0.1 * math.log(factor) + 1.0


def rotate_pairs_ref(x: torch.Tensor, positions: torch.Tensor, freqs: torch.Tensor, mag: float) -> torch.Tensor:
    """``x [T, ..., dims]``: the pair (2i, 2i + 1) turned by ``positions * freqs[i]``, cos and sin times ``mag``."""
    T = x.shape[0]
    ang = positions.to(torch.float64)[:, None] * freqs[None, :]
    shape = [T] + [1] * (x.dim() - 2) + [freqs.shape[0]]
    c, s = (torch.cos(ang) * mag).to(x.dtype).reshape(shape), (torch.sin(ang) * mag).to(x.dtype).reshape(shape)
    u, v = x[..., 0::2], x[..., 1::2]
    out = torch.empty_like(x)
    out[..., 0::2] = u * c - v * s
    out[..., 1::2] = v * c + u * s
    return out


# ------------------------------------------------------------------------------------------------ mixers
def latent_attention_ref(h: torch.Tensor, w: Dict[str, torch.Tensor], m: dict, eps: float) -> torch.Tensor:
    """``w``: the mixer's tensors by their short names (``dq``, ``dq.norm``, ``uq``, ``dkv``, ``dkv.norm``, ``uk``, ``uv``,
    ``o``, and for the gated form with a sink ``sink`` and ``g``).  Keys and values are written out per head: no absorbed
    products, no cache."""
    T = h.shape[0]
    H, D, R, Dv, C = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    cq = rms_unit(h @ w["dq"].T, eps) * w["dq.norm"]
    q = (cq @ w["uq"].T).reshape(T, H, D + R)
    ckv = h @ w["dkv"].T
    c = rms_unit(ckv[:, :C], eps) * w["dkv.norm"]
    k_rot = ckv[:, C:]
    k_nope = (c @ w["uk"].T).reshape(T, H, D)
    v = (c @ w["uv"].T).reshape(T, H, Dv)
    freqs, mag = rotary_frequencies_ref(m["rot"]["dims"], m["rot"]["base"], m["rot"].get("scaling"))
    pos = torch.arange(T)
    q_rot = rotate_pairs_ref(q[..., D:], pos, freqs, mag)
    k_rot = rotate_pairs_ref(k_rot, pos, freqs, mag)
    out = torch.zeros(T, H, Dv, dtype=h.dtype)
    for hh in range(H):
        for i in range(T):
            s = (k_nope[:i + 1, hh] @ q[i, hh, :D] + k_rot[:i + 1] @ q_rot[i, hh]) * m["scale"]
            if "sink" in w:
                mx = torch.maximum(s.max(), w["sink"][hh])
                e = torch.exp(s - mx)
                p = e / (e.sum() + torch.exp(w["sink"][hh] - mx))
            else:
                p = torch.softmax(s, 0)
            out[i, hh] = p @ v[:i + 1, hh]
    out = out.reshape(T, H * Dv)
    if "g" in w:
        out = out * torch.sigmoid(h @ w["g"].T)
    return out @ w["o"].T


def lightning_ref(h: torch.Tensor, w: Dict[str, torch.Tensor], m: dict, eps: float) -> torch.Tensor:
    T = h.shape[0]
    H, D, Dv = m["heads"], m["dim"], m["vdim"]
    silu = torch.nn.functional.silu
    q, k, v = silu(h @ w["q"].T).reshape(T, H, D), silu(h @ w["k"].T).reshape(T, H, D), silu(h @ w["v"].T).reshape(T, H, Dv)
    S = torch.zeros(H, D, Dv, dtype=h.dtype)
    decay = torch.tensor(m["decay"], dtype=h.dtype)
    rows = []
    for t in range(T):
        S = decay[:, None, None] * S + k[t][:, :, None] * v[t][:, None, :]
        rows.append(torch.einsum("hdv,hd->hv", S, q[t]).reshape(H * Dv))
    o = rms_unit(torch.stack(rows), eps) * w["norm"]
    return (o * torch.sigmoid(h @ w["g"].T)) @ w["o"].T


# ------------------------------------------------------------------------------------------------ feed-forward
def xielu_ref(z: torch.Tensor, p: torch.Tensor, q: torch.Tensor) -> torch.Tensor:
    sp = torch.nn.functional.softplus
    pos = sp(p) * z * z + z / 2
    neg = (0.5 + sp(q)) * (torch.exp(torch.clamp(z, max=0.0)) - 1 - z) + z / 2
    return torch.where(z > 0, pos, neg)


def dense_ff_ref(h: torch.Tensor, w: Dict[str, torch.Tensor]) -> torch.Tensor:
    z = h @ w["up"].T + w["up.b"]
    return xielu_ref(z, w["act"][0], w["act"][1]) @ w["down"].T + w["down.b"]


def clamped_expert_ref(h: torch.Tensor, gate: torch.Tensor, up: torch.Tensor, down: torch.Tensor, limit: float) -> torch.Tensor:
    g = torch.clamp(h @ gate.T, max=limit)
    u = torch.clamp(h @ up.T, -limit, limit)
    return (g * torch.sigmoid(1.702 * g) * (u + 1)) @ down.T


def moe_ff_ref(h: torch.Tensor, w: Dict[str, torch.Tensor], mlp: dict) -> torch.Tensor:
    E, top, scale = mlp["router"]["experts"], mlp["router"]["top"], mlp["router"]["scale"]
    s = torch.sigmoid(h @ w["router"].T)
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        order = sorted(range(E), key=lambda e: (-float(s[t, e]), e))[:top]
        total = sum(s[t, e] for e in order) + 1e-20
        for e in order:
            out[t] = out[t] + (s[t, e] / total * scale) * clamped_expert_ref(h[t:t + 1], w[f"e{e}.gate"], w[f"e{e}.up"], w[f"e{e}.down"],
                                                                            mlp["expert"]["limit"])[0]
    if mlp.get("shared"):
        out = out + clamped_expert_ref(h, w["shared.gate"], w["shared.up"], w["shared.down"], mlp["shared"]["limit"])
    return out


# ------------------------------------------------------------------------------------------------ the model
def _sub(weights: Dict[str, torch.Tensor], prefix: str, dtype) -> Dict[str, torch.Tensor]:
    return {k[len(prefix):]: v.to(dtype) for k, v in weights.items() if k.startswith(prefix)}


def geponex_ref(cfg: dict, weights: Dict[str, torch.Tensor], tokens: List[int], dtype=torch.float64,
                residual_out: Optional[list] = None) -> torch.Tensor:
    """Logits ``[T, vocab]`` of one sequence."""
    eps, groups, alpha = cfg["norm"]["eps"], cfg["norm"]["groups"], cfg["postln_alpha"]
    x = weights["embed"].to(dtype)[torch.tensor(tokens)]
    for i, entry in enumerate(cfg["layers"]):
        j = entry.get("weights_of", i)
        p = f"l{j}."
        h = token_shift_ref(x, weights[p + "shift"].to(dtype))
        mw = _sub(weights, p + "mix.", dtype)
        if entry["type"] == "lightning":
            y = lightning_ref(h, mw, entry["mixer"], eps)
        elif entry["type"] in ("latent_attention", "latent_attention_2"):
            y = latent_attention_ref(h, mw, entry["mixer"], eps)
        else:
            raise ValueError(entry["type"])
        x = group_norm_ref(alpha * x + y, weights[p + "norm1"].to(dtype), groups, eps)
        if entry.get("mlp") is not None:
            fw = _sub(weights, p + "mlp.", dtype)
            y = dense_ff_ref(x, fw) if entry["mlp"]["kind"] == "dense" else moe_ff_ref(x, fw, entry["mlp"])
            x = group_norm_ref(alpha * x + y, weights[p + "norm2"].to(dtype), groups, eps)
        if residual_out is not None:
            residual_out.append(x.clone())
    x = group_norm_ref(x, weights["final.norm"].to(dtype), groups, eps)
    return x @ weights["embed"].to(dtype).T


# ------------------------------------------------------------------------------------------------ test checkpoints
def latent_mixer_config(heads=3, dim=16, rot_dim=8, vdim=24, kv_rank=40, q_rank=48, base=10000.0, scale=None, scaling=None):
    rot = {"base": base, "dims": rot_dim}
    if scaling:
        rot["scaling"] = dict(scaling)
    return {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank, "q_rank": q_rank, "rot": rot,
            "scale": float(scale if scale is not None else (dim + rot_dim) ** -0.5)}


def lightning_mixer_config(heads=3, dim=16, vdim=24, decay=None):
    return {"heads": heads, "dim": dim, "vdim": vdim, "decay": list(decay) if decay is not None else [0.5 + 0.49 * (h + 1) / heads for h in range(heads)]}


def moe_config(experts=6, top=2, ff=40, limit=1.5, scale=1.75, shared_ff=24, shared_limit=2.5):
    mlp = {"kind": "moe", "expert": {"ff": ff, "limit": limit}, "router": {"experts": experts, "top": top, "scale": scale}}
    if shared_ff:
        mlp["shared"] = {"ff": shared_ff, "limit": shared_limit}
    return mlp


def geponex_config(vocab=80, width=48, layers=None, groups=3, eps=1e-5, alpha=1.5) -> dict:
    """``layers``: a list of ``(type, mixer config, mlp config or None)`` or ``("weights_of", j)``."""
    if layers is None:
        layers = [("latent_attention_2", latent_mixer_config(), {"kind": "dense", "ff": 72}),
                  ("lightning", lightning_mixer_config(), moe_config()),
                  ("latent_attention", latent_mixer_config(scaling={"factor": 4.0, "original": 64, "fast": 16.0, "slow": 2.0}), moe_config()),
                  ("weights_of", 1)]
    out = []
    for entry in layers:
        if entry[0] == "weights_of":
            src = dict(out[entry[1]])
            src["weights_of"] = entry[1]
            out.append(src)
        else:
            out.append({"type": entry[0], "mixer": entry[1], "mlp": entry[2]})
    return {"architecture": "Geponex", "vocab": vocab, "width": width, "norm": {"eps": eps, "groups": groups}, "postln_alpha": alpha,
            "layers": out}


def geponex_random_weights(cfg: dict, seed: int = 0, std: float = 1.0) -> Dict[str, torch.Tensor]:
    """bf16-representable random tensors under the checkpoint's names (fp32 tensors whose values survive a bf16 round trip)."""
    g = torch.Generator().manual_seed(seed)
    W = cfg["width"]

    def rnd(*shape, s=1.0):
        return (torch.randn(*shape, generator=g) * s * std).to(torch.bfloat16).float()

    def lin(o, i):
        return rnd(o, i, s=i ** -0.5)

    w: Dict[str, torch.Tensor] = {"embed": rnd(cfg["vocab"], W), "final.norm": 1 + rnd(W, s=0.1)}
    for i, entry in enumerate(cfg["layers"]):
        if "weights_of" in entry:
            continue
        p, m = f"l{i}.", entry["mixer"]
        w[p + "norm1"], w[p + "shift"] = 1 + rnd(W, s=0.1), torch.rand(W, generator=g).to(torch.bfloat16).float()
        if entry["type"] == "lightning":
            H, D, Dv = m["heads"], m["dim"], m["vdim"]
            w[p + "mix.q"], w[p + "mix.k"], w[p + "mix.v"] = lin(H * D, W), lin(H * D, W), lin(H * Dv, W)
            w[p + "mix.g"], w[p + "mix.o"], w[p + "mix.norm"] = lin(H * Dv, W), lin(W, H * Dv), 1 + rnd(H * Dv, s=0.1)
        else:
            H, D, R, Dv, C, Q = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"], m["q_rank"]
            w[p + "mix.dq"], w[p + "mix.dq.norm"], w[p + "mix.uq"] = lin(Q, W), 1 + rnd(Q, s=0.1), lin(H * (D + R), Q)
            w[p + "mix.dkv"], w[p + "mix.dkv.norm"] = lin(C + R, W), 1 + rnd(C, s=0.1)
            w[p + "mix.uk"], w[p + "mix.uv"], w[p + "mix.o"] = lin(H * D, C), lin(H * Dv, C), lin(W, H * Dv)
            if entry["type"] == "latent_attention_2":
                w[p + "mix.sink"], w[p + "mix.g"] = rnd(H), lin(H * Dv, W)
        mlp = entry.get("mlp")
        if mlp is None:
            continue
        w[p + "norm2"] = 1 + rnd(W, s=0.1)
        if mlp["kind"] == "dense":
            F = mlp["ff"]
            w[p + "mlp.up"], w[p + "mlp.up.b"], w[p + "mlp.down"], w[p + "mlp.down.b"] = lin(F, W), rnd(F, s=0.1), lin(W, F), rnd(W, s=0.1)
            w[p + "mlp.act"] = rnd(2)
        else:
            F = mlp["expert"]["ff"]
            for e in range(mlp["router"]["experts"]):
                w[f"{p}mlp.e{e}.gate"], w[f"{p}mlp.e{e}.up"], w[f"{p}mlp.e{e}.down"] = lin(F, W), lin(F, W), lin(W, F)
            w[p + "mlp.router"] = lin(mlp["router"]["experts"], W)
            if mlp.get("shared"):
                Fs = mlp["shared"]["ff"]
                w[p + "mlp.shared.gate"], w[p + "mlp.shared.up"], w[p + "mlp.shared.down"] = lin(Fs, W), lin(Fs, W), lin(W, Fs)
    return w


def shared_row_attention_ref(q: torch.Tensor, rows: torch.Tensor, v_dim: int, scale: float, sink: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Causal attention of ``q [T, H, Dk]`` over ``rows [T, Dk]`` that all heads share as keys, the first ``v_dim`` elements
    of a row being its value; ``sink [H]``: a logit per head in the denominator.  -> ``[T, H, v_dim]``."""
    T, H, _ = q.shape
    out = torch.zeros(T, H, v_dim, dtype=q.dtype)
    for h in range(H):
        for i in range(T):
            s = (rows[:i + 1] @ q[i, h]) * scale
            mx = s.max() if sink is None else torch.maximum(s.max(), sink[h])
            e = torch.exp(s - mx)
            den = e.sum() + (0 if sink is None else torch.exp(sink[h] - mx))
            out[i, h] = (e / den) @ rows[:i + 1, :v_dim]
    return out
