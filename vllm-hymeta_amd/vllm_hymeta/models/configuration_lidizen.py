"""Configuration of the Lidizen family (``"architecture": "Lidizen"`` in ``config.json``).

The file is nested: ``layers`` lists the decoder layers in order, each with the ``type`` of its mixer (``"attention"``),
the mixer's sizes and constants (``mixer``) and its feed-forward (``mlp``: ``{"kind": "dense", ...}``, ``{"kind": "moe",
...}`` or ``null``); ``streams`` is the number of residual streams (absent: one plain residual), ``embedding.bigram`` the
hashed pair table beside the token table (absent: none).  Everything that can differ between two checkpoints of the
family is read from the file; this class only names and checks the fields.
"""

from __future__ import annotations

import json
import os
from dataclasses import dataclass
from typing import Any, Dict, List, Optional


@dataclass
class PairEmbeddingSpec:
    """Row ``(previous token * mul_prev + token * mul_cur) mod buckets`` of a table of ``buckets + 1`` rows (the last row:
    a sequence's first token)."""
    buckets: int
    mul_prev: int
    mul_cur: int


@dataclass
class TalkingAttentionSpec:
    heads: int
    kv_heads: int
    dim: int              # query / key size per head
    vdim: int
    scale: float
    rot_dims: int         # leading dimensions of a head that turn, in interleaved pairs
    rot_base: float
    window: Optional[int]     # a query sees the keys less than this far back (None: all)
    keep_first: int           # ... and the first keep_first keys of its sequence
    v_mix: bool               # values blended with those of the first layer that says so

    def frequencies(self) -> List[float]:
        return [self.rot_base ** (-2.0 * i / self.rot_dims) for i in range(self.rot_dims // 2)]


@dataclass
class SiluMlpSpec:
    ff: int


@dataclass
class Relu2MoeSpec:
    experts: int
    top: int
    ff: int


@dataclass
class LidizenLayerSpec:
    type: str
    mixer: TalkingAttentionSpec
    mlp: Any                  # SiluMlpSpec, Relu2MoeSpec or None


class LidizenConfig:
    model_type = "lidizen"
    architectures = ["LidizenForCausalLM"]

    def __init__(self, raw: Dict[str, Any]):
        self.raw = raw
        self.vocab_size = int(raw["vocab"])
        self.hidden_size = int(raw["width"])
        self.norm_eps = float(raw["norm"]["eps"])
        self.streams = int(raw.get("streams") or 0)          # 0: a plain residual, no stream weights in the checkpoint
        if self.streams < 0:
            raise ValueError("streams counts residual streams")
        big = (raw.get("embedding") or {}).get("bigram")
        self.bigram = None if not big else PairEmbeddingSpec(int(big["buckets"]), int(big["mul_prev"]), int(big["mul_cur"]))
        if self.bigram is not None and self.bigram.buckets < 1:
            raise ValueError("the pair table needs at least one bucket")
        self.layers: List[LidizenLayerSpec] = []
        for i, entry in enumerate(raw["layers"]):
            kind, mx = entry["type"], entry.get("mixer") or {}
            if kind != "attention":
                raise ValueError(f"layer {i}: unknown mixer type {kind!r}")
            rot, mask = mx.get("rot") or {}, mx.get("mask") or {}
            mixer = TalkingAttentionSpec(
                heads=int(mx["heads"]), kv_heads=int(mx.get("kv_heads", mx["heads"])), dim=int(mx["dim"]), vdim=int(mx.get("vdim", mx["dim"])),
                scale=float(mx["scale"]), rot_dims=int(rot.get("dims", 0)), rot_base=float(rot.get("base", 10000.0)),
                window=int(mask["size"]) if mask.get("size") is not None else None, keep_first=int(mask.get("keep_first", 0)),
                v_mix=bool(mx.get("v_mix", False)))
            if mixer.heads % mixer.kv_heads:
                raise ValueError(f"layer {i}: {mixer.heads} query heads do not split over {mixer.kv_heads} key/value heads")
            if mixer.rot_dims % 2 or not 0 <= mixer.rot_dims <= mixer.dim:
                raise ValueError(f"layer {i}: {mixer.rot_dims} rotated dimensions do not fit a head of {mixer.dim}")
            if (mixer.window is not None and mixer.window < 1) or mixer.keep_first < 0:
                raise ValueError(f"layer {i}: the window and the kept tokens count tokens")
            mlp = entry.get("mlp")
            if mlp is not None:
                fk = mlp.get("kind", "dense")
                if fk == "dense":
                    mlp = SiluMlpSpec(ff=int(mlp["ff"]))
                elif fk == "moe":
                    mlp = Relu2MoeSpec(experts=int(mlp["router"]["experts"]), top=int(mlp["router"]["top"]), ff=int(mlp["expert"]["ff"]))
                    if not 1 <= mlp.top <= mlp.experts:
                        raise ValueError(f"layer {i}: top {mlp.top} of {mlp.experts} experts")
                else:
                    raise ValueError(f"layer {i}: unknown feed-forward kind {fk!r}")
            self.layers.append(LidizenLayerSpec(kind, mixer, mlp))
        self.num_hidden_layers = len(self.layers)
        blended = [l.mixer for l in self.layers if l.mixer.v_mix]
        if any(m.kv_heads * m.vdim != blended[0].kv_heads * blended[0].vdim for m in blended):
            raise ValueError("layers that blend their values must have values of one size")

    @classmethod
    def from_pretrained(cls, model_dir: str) -> "LidizenConfig":
        with open(os.path.join(model_dir, "config.json")) as f:
            return cls(json.load(f))
