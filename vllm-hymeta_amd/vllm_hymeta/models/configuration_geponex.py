"""Configuration of the Geponex family (``"architecture": "Geponex"`` in ``config.json``).

The file is nested: ``layers`` lists the decoder layers in order, each with the ``type`` of its mixer
(``"latent_attention"``, ``"latent_attention_2"`` or ``"lightning"``), the mixer's sizes and constants (``mixer``) and its
feed-forward (``mlp``: ``{"kind": "dense", ...}``, ``{"kind": "moe", ...}`` or ``null``); an entry with ``weights_of: j``
runs with layer ``j``'s tensors and a cache and state of its own.  Everything that can differ between two checkpoints of
the family is read from the file; this class only names and checks the fields.
"""

from __future__ import annotations

import json
import math
import os
from dataclasses import dataclass
from typing import Any, Dict, List, Optional, Tuple


@dataclass
class RotarySpec:
    """Pairs (2i, 2i + 1), i < dims / 2, turn by ``position * base^(-2i / dims)``; with ``scaling`` (YaRN) the frequency
    of pair i is blended towards ``f_i / factor`` along a ramp between the pairs that make ``fast`` and ``slow`` turns
    over ``original`` positions, and cos and sin grow by ``0.1 ln(factor) + 1``."""
    dims: int
    base: float
    scaling: Optional[Dict[str, float]] = None

    def frequencies(self) -> Tuple[List[float], float]:
        """``(frequency per pair, factor on cos and sin)`` in double precision."""
        n = self.dims // 2
        f = [self.base ** (-2.0 * i / self.dims) for i in range(n)]
        if not self.scaling:
            return f, 1.0
        factor, original = float(self.scaling["factor"]), float(self.scaling["original"])

        def pair_of(turns: float) -> float:
            return self.dims * math.log(original / (2.0 * math.pi * turns)) / (2.0 * math.log(self.base))

        lo = max(math.floor(pair_of(float(self.scaling["fast"]))), 0)
        hi = min(math.ceil(pair_of(float(self.scaling["slow"]))), self.dims - 1)
        span = max(hi - lo, 0.001)
        out = []
        for i in range(n):
            ramp = min(max((i - lo) / span, 0.0), 1.0)
            out.append(f[i] / factor * ramp + f[i] * (1.0 - ramp))
        return out, 0.1 * math.log(factor) + 1.0


@dataclass
class LatentAttentionSpec:
    heads: int
    dim: int              # unrotated query / key size per head
    rot_dim: int          # rotated size per head (the key's rotated part is shared by the heads)
    vdim: int
    kv_rank: int
    q_rank: int
    scale: float
    rot: RotarySpec
    sink: bool            # a learned sink logit per head in the softmax's denominator
    gate: bool            # sigmoid output gate on the concatenated heads


@dataclass
class LightningSpec:
    heads: int
    dim: int
    vdim: int
    decay: List[float]


@dataclass
class DenseMlpSpec:
    ff: int


@dataclass
class ClampedExpertSpec:
    ff: int
    limit: float


@dataclass
class MoeMlpSpec:
    experts: int
    top: int
    route_scale: float
    expert: ClampedExpertSpec
    shared: Optional[ClampedExpertSpec]


@dataclass
class GeponexLayerSpec:
    type: str
    mixer: Any
    mlp: Any                      # DenseMlpSpec, MoeMlpSpec or None
    weights_of: int               # the layer whose tensors this one uses (itself unless the entry says otherwise)


# what the two latent-attention types add to the common form
_LATENT_TYPES = {"latent_attention": dict(sink=False, gate=False), "latent_attention_2": dict(sink=True, gate=True)}


class GeponexConfig:
    model_type = "geponex"
    architectures = ["GeponexForCausalLM"]

    def __init__(self, raw: Dict[str, Any]):
        self.raw = raw
        self.vocab_size = int(raw["vocab"])
        self.hidden_size = int(raw["width"])
        self.norm_eps = float(raw["norm"]["eps"])
        self.norm_groups = int(raw["norm"].get("groups", 1))
        self.postln_alpha = float(raw.get("postln_alpha", 1.0))
        if self.norm_groups < 1 or self.hidden_size % self.norm_groups:
            raise ValueError(f"width {self.hidden_size} does not split into {self.norm_groups} norm groups")
        self.layers: List[GeponexLayerSpec] = []
        for i, entry in enumerate(raw["layers"]):
            kind, mx = entry["type"], entry.get("mixer") or {}
            if kind in _LATENT_TYPES:
                rot = mx.get("rot") or {}
                rot_dim = int(mx.get("rot_dim", 0))
                spec = RotarySpec(dims=int(rot.get("dims", rot_dim)), base=float(rot.get("base", 10000.0)), scaling=rot.get("scaling"))
                if spec.dims % 2 or rot_dim % 2 or spec.dims > rot_dim:
                    raise ValueError(f"layer {i}: {spec.dims} rotated dimensions do not fit a rotated part of {rot_dim}")
                mixer = LatentAttentionSpec(heads=int(mx["heads"]), dim=int(mx["dim"]), rot_dim=rot_dim, vdim=int(mx["vdim"]),
                                            kv_rank=int(mx["kv_rank"]), q_rank=int(mx["q_rank"]), scale=float(mx["scale"]), rot=spec,
                                            **_LATENT_TYPES[kind])
            elif kind == "lightning":
                mixer = LightningSpec(heads=int(mx["heads"]), dim=int(mx["dim"]), vdim=int(mx["vdim"]), decay=[float(d) for d in mx["decay"]])
                if len(mixer.decay) != mixer.heads:
                    raise ValueError(f"layer {i}: {len(mixer.decay)} decays for {mixer.heads} heads")
            else:
                raise ValueError(f"layer {i}: unknown mixer type {kind!r}")
            mlp = entry.get("mlp")
            if mlp is not None:
                fk = mlp.get("kind", "dense")
                if fk == "dense":
                    mlp = DenseMlpSpec(ff=int(mlp["ff"]))
                elif fk == "moe":
                    sh = mlp.get("shared")
                    mlp = MoeMlpSpec(experts=int(mlp["router"]["experts"]), top=int(mlp["router"]["top"]),
                                     route_scale=float(mlp["router"].get("scale", 1.0)),
                                     expert=ClampedExpertSpec(int(mlp["expert"]["ff"]), float(mlp["expert"]["limit"])),
                                     shared=None if not sh else ClampedExpertSpec(int(sh["ff"]), float(sh["limit"])))
                    if not 1 <= mlp.top <= mlp.experts:
                        raise ValueError(f"layer {i}: top {mlp.top} of {mlp.experts} experts")
                else:
                    raise ValueError(f"layer {i}: unknown feed-forward kind {fk!r}")
            src = int(entry.get("weights_of", i))
            if not 0 <= src < len(raw["layers"]) or (src != i and "weights_of" in raw["layers"][src]):
                raise ValueError(f"layer {i}: weights_of {src} must name a layer with tensors of its own")
            self.layers.append(GeponexLayerSpec(kind, mixer, mlp, src))
        self.num_hidden_layers = len(self.layers)

    @classmethod
    def from_pretrained(cls, model_dir: str) -> "GeponexConfig":
        with open(os.path.join(model_dir, "config.json")) as f:
            return cls(json.load(f))
