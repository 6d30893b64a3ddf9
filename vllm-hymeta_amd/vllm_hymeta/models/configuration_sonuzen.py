"""Configuration of the Sonuzen family (``"architecture": "Sonuzen"`` in ``config.json``).

The file is nested: ``layers`` lists the decoder layers in order, each with the ``type`` of its mixer (``"attention"``
or ``"mingru"``), the mixer's sizes and its feed-forward (``mlp``, ``null`` for none); ``loop`` says which run of layers
is passed through several times with the same weights.  Everything that can differ between two checkpoints of the
family is read from it; this class only names and checks the fields.
"""

from __future__ import annotations

import json
import os
from dataclasses import dataclass
from typing import Any, Dict, List, Optional, Tuple


@dataclass
class SonuzenAttentionSpec:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float


@dataclass
class SonuzenMinGruSpec:
    width: int


@dataclass
class SonuzenMoeSpec:
    experts: int
    top: int
    ff: int


@dataclass
class SonuzenLayerSpec:
    type: str
    mixer: Any
    mlp: Optional[SonuzenMoeSpec]


class SonuzenConfig:
    model_type = "sonuzen"
    architectures = ["SonuzenForCausalLM"]

    def __init__(self, raw: Dict[str, Any]):
        self.raw = raw
        self.vocab_size = int(raw["vocab"])
        self.hidden_size = int(raw["width"])
        self.norm_eps = float(raw["norm"]["eps"])
        self.residual_mult = float(raw.get("residual_mult", 1.0))
        self.logit_scale = float(raw.get("logit_scale", 1.0))
        self.has_conv = bool(raw.get("canon"))
        self.conv_taps = int(raw["canon"]["taps"]) if self.has_conv else 1
        self.layers: List[SonuzenLayerSpec] = []
        for i, entry in enumerate(raw["layers"]):
            kind, mx = entry["type"], entry.get("mixer") or {}
            if kind == "attention":
                mixer = SonuzenAttentionSpec(heads=int(mx["heads"]), kv_heads=int(mx.get("kv_heads", mx["heads"])), dim=int(mx["dim"]),
                                             vdim=int(mx.get("vdim", mx["dim"])), scale=float(mx["scale"]))
                if mixer.heads % mixer.kv_heads:
                    raise ValueError(f"layer {i}: {mixer.heads} query heads do not divide over {mixer.kv_heads} key/value heads")
            elif kind == "mingru":
                mixer = SonuzenMinGruSpec(width=int(mx.get("width", self.hidden_size)))
            else:
                raise ValueError(f"layer {i}: unknown mixer type {kind!r}")
            mlp = entry.get("mlp")
            if mlp is not None:
                if mlp.get("kind", "moe") != "moe":
                    raise ValueError(f"layer {i}: unknown feed-forward kind {mlp.get('kind')!r}")
                mlp = SonuzenMoeSpec(experts=int(mlp["router"]["experts"]), top=int(mlp["router"]["top"]), ff=int(mlp["expert"]["ff"]))
                if not 1 <= mlp.top <= mlp.experts:
                    raise ValueError(f"layer {i}: top {mlp.top} of {mlp.experts} experts")
            self.layers.append(SonuzenLayerSpec(kind, mixer, mlp))
        self.num_hidden_layers = len(self.layers)
        loop = raw.get("loop")
        self.loop_start, self.loop_stop, self.loop_times = 0, 0, 1
        if loop:
            self.loop_start, self.loop_stop, self.loop_times = int(loop["start"]), int(loop["stop"]), int(loop["times"])
            if not (0 <= self.loop_start <= self.loop_stop <= self.num_hidden_layers) or self.loop_times < 1:
                raise ValueError(f"loop {loop} does not fit {self.num_hidden_layers} layers")
            if self.loop_start == self.loop_stop:
                self.loop_times = 1

    @property
    def has_loop(self) -> bool:
        return self.loop_stop > self.loop_start

    def layer_runs(self) -> List[Tuple[int, int]]:
        """``(layer, pass)`` in execution order: the layers before the loop, the looped run ``loop_times`` times, the rest."""
        runs = [(i, 0) for i in range(self.loop_start)]
        for t in range(self.loop_times if self.has_loop else 0):
            runs += [(i, t) for i in range(self.loop_start, self.loop_stop)]
        runs += [(i, 0) for i in range(self.loop_stop if self.has_loop else self.loop_start, self.num_hidden_layers)]
        return runs

    @classmethod
    def from_pretrained(cls, model_dir: str) -> "SonuzenConfig":
        with open(os.path.join(model_dir, "config.json")) as f:
            return cls(json.load(f))
