"""Configuration of the Dapuzen family (``"architecture": "Dapuzen"`` in ``config.json``).

The file is nested: ``layers`` lists the decoder layers in order, each with the ``type`` of its mixer (``"attention"``,
``"retention"`` or ``"parallel"``: an attention and a state-space layer side by side), the mixer's sizes and constants
(``mixer``) and its feed-forward (``mlp``: ``{"kind": "dense", ...}``, ``{"kind": "moe", ...}`` or ``null``); an entry with
``weights_of: j`` runs with layer ``j``'s tensors and a cache and state of its own.  Everything that can differ between two
checkpoints of the family is read from the file; this class only names and checks the fields.
"""

from __future__ import annotations

import json
import os
from dataclasses import dataclass
from typing import Any, Dict, List, Optional


@dataclass
class WindowAttentionSpec:
    """Softmax attention over grouped key/value heads.  ``rot_dims`` leading dimensions of a head turn in half-split pairs
    (i with i + rot_dims / 2); ``window``: a query sees itself and the ``window - 1`` keys before it (None: all);
    ``softcap``: scores become ``softcap tanh(score / softcap)`` (None: as they are); ``bias``: the four projections have
    biases; ``gate``: a sigmoid gate per head on the heads' outputs."""
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    rot_dims: int
    rot_base: float
    window: Optional[int]
    softcap: Optional[float]
    bias: bool
    gate: bool

    def frequencies(self) -> List[float]:
        return [self.rot_base ** (-2.0 * i / self.rot_dims) for i in range(self.rot_dims // 2)]


@dataclass
class RetentionSpec:
    heads: int
    dim: int
    vdim: int
    decay: List[float]
    rot_dims: int
    rot_base: float

    def frequencies(self) -> List[float]:
        return [self.rot_base ** (-2.0 * i / self.rot_dims) for i in range(self.rot_dims // 2)]


@dataclass
class StateSpaceSpec:
    """Mamba-2: ``heads`` heads of ``vdim`` channels, a state of ``state`` rows per head, ``groups`` B / C groups, a
    convolution of ``conv`` taps, the output norm in ``norm_groups`` parts."""
    heads: int
    vdim: int
    state: int
    groups: int
    norm_groups: int
    conv: int

    @property
    def inner(self) -> int:
        return self.heads * self.vdim

    @property
    def conv_channels(self) -> int:
        return self.inner + 2 * self.groups * self.state


@dataclass
class SideBySideSpec:
    left: WindowAttentionSpec
    right: StateSpaceSpec
    left_scale: float
    right_scale: float


@dataclass
class DenseMlpSpec:
    ff: int


@dataclass
class GroupedMoeSpec:
    experts: int          # experts with tensors
    identity: int         # router outputs behind them whose expert is the identity
    top: int
    groups: int
    keep: int
    ff: int
    shared_ff: int        # 0: no shared expert


@dataclass
class DapuzenLayerSpec:
    type: str
    mixer: Any
    mlp: Any                      # DenseMlpSpec, GroupedMoeSpec or None
    weights_of: int               # the layer whose tensors this one uses (itself unless the entry says otherwise)


def _attention(i: int, mx: Dict[str, Any], bias: bool, gate: bool) -> WindowAttentionSpec:
    rot, mask = mx.get("rot") or {}, mx.get("mask") or {}
    a = WindowAttentionSpec(
        heads=int(mx["heads"]), kv_heads=int(mx.get("kv_heads", mx["heads"])), dim=int(mx["dim"]), vdim=int(mx.get("vdim", mx["dim"])),
        scale=float(mx["scale"]), rot_dims=int(rot.get("dims", 0)), rot_base=float(rot.get("base", 10000.0)),
        window=int(mask["size"]) if mask.get("size") is not None else None,
        softcap=float(mx["softcap"]) if mx.get("softcap") else None, bias=bias, gate=gate)
    if a.heads % a.kv_heads:
        raise ValueError(f"layer {i}: {a.heads} query heads do not split over {a.kv_heads} key/value heads")
    if a.rot_dims % 2 or not 0 <= a.rot_dims <= a.dim:
        raise ValueError(f"layer {i}: {a.rot_dims} rotated dimensions do not fit a head of {a.dim}")
    if a.window is not None and a.window < 1:
        raise ValueError(f"layer {i}: the window counts tokens")
    return a


class DapuzenConfig:
    model_type = "dapuzen"
    architectures = ["DapuzenForCausalLM"]

    def __init__(self, raw: Dict[str, Any]):
        self.raw = raw
        self.vocab_size = int(raw["vocab"])
        self.hidden_size = int(raw["width"])
        self.norm_eps = float(raw["norm"]["eps"])
        self.embedding_scale = float((raw.get("embedding") or {}).get("scale", 1.0))
        self.layers: List[DapuzenLayerSpec] = []
        for i, entry in enumerate(raw["layers"]):
            kind, mx = entry["type"], entry.get("mixer") or {}
            if kind == "attention":
                mixer = _attention(i, mx, bias=False, gate=True)
            elif kind == "retention":
                rot = mx.get("rot") or {}
                mixer = RetentionSpec(heads=int(mx["heads"]), dim=int(mx["dim"]), vdim=int(mx.get("vdim", mx["dim"])),
                                      decay=[float(d) for d in mx["decay"]], rot_dims=int(rot.get("dims", 0)), rot_base=float(rot.get("base", 10000.0)))
                if len(mixer.decay) != mixer.heads:
                    raise ValueError(f"layer {i}: {len(mixer.decay)} decays for {mixer.heads} heads")
                if mixer.rot_dims % 2 or not 0 <= mixer.rot_dims <= mixer.dim:
                    raise ValueError(f"layer {i}: {mixer.rot_dims} rotated dimensions do not fit a head of {mixer.dim}")
            elif kind == "parallel":
                r = mx["right"]
                right = StateSpaceSpec(heads=int(r["heads"]), vdim=int(r["vdim"]), state=int(r["state"]), groups=int(r.get("groups", 1)),
                                       norm_groups=int(r.get("norm_groups", 1)), conv=int(r["conv"]))
                if right.heads % right.groups or right.inner % right.norm_groups or right.conv < 1:
                    raise ValueError(f"layer {i}: the state-space heads do not split into its groups")
                mixer = SideBySideSpec(_attention(i, mx["left"], bias=True, gate=False), right,
                                       float(mx.get("left_scale", 1.0)), float(mx.get("right_scale", 1.0)))
            else:
                raise ValueError(f"layer {i}: unknown mixer type {kind!r}")
            mlp = entry.get("mlp")
            if mlp is not None:
                fk = mlp.get("kind", "dense")
                if fk == "dense":
                    mlp = DenseMlpSpec(ff=int(mlp["ff"]))
                elif fk == "moe":
                    r, grp = mlp["router"], mlp["router"].get("groups") or {}
                    mlp = GroupedMoeSpec(experts=int(r["experts"]), identity=int(r.get("identity", 0)), top=int(r["top"]),
                                         groups=int(grp.get("count", 1)), keep=int(grp.get("keep", grp.get("count", 1))),
                                         ff=int(mlp["expert"]["ff"]), shared_ff=int((mlp.get("shared") or {}).get("ff", 0)))
                    outputs = mlp.experts + mlp.identity
                    if not 1 <= mlp.top <= outputs:
                        raise ValueError(f"layer {i}: top {mlp.top} of {outputs} router outputs")
                    if mlp.groups < 1 or outputs % mlp.groups or not 1 <= mlp.keep <= mlp.groups:
                        raise ValueError(f"layer {i}: {outputs} router outputs do not form {mlp.groups} equal groups of which {mlp.keep} are kept")
                    if mlp.keep * (outputs // mlp.groups) < mlp.top:
                        raise ValueError(f"layer {i}: the kept groups hold fewer outputs than top {mlp.top}")
                else:
                    raise ValueError(f"layer {i}: unknown feed-forward kind {fk!r}")
            src = int(entry.get("weights_of", i))
            if not 0 <= src < len(raw["layers"]) or (src != i and "weights_of" in raw["layers"][src]):
                raise ValueError(f"layer {i}: weights_of {src} must name a layer with tensors of its own")
            self.layers.append(DapuzenLayerSpec(kind, mixer, mlp, src))
        self.num_hidden_layers = len(self.layers)

    @classmethod
    def from_pretrained(cls, model_dir: str) -> "DapuzenConfig":
        with open(os.path.join(model_dir, "config.json")) as f:
            return cls(json.load(f))
