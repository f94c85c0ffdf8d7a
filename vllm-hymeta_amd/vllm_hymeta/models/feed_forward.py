"""Feed-forward sublayers of the designs on fp32 residual streams:

``XieluMLP``        ``W_down xielu(W_up h + b_up) + b_down`` with ``xielu(z) = a_pos z^2 + z / 2`` for ``z > 0`` and
                    ``a_neg (exp(z) - 1 - z) + z / 2`` otherwise, ``a_pos = softplus(p)``, ``a_neg = 1/2 + softplus(q)``
``ClampedGluMLP``   ``W_down (g sigmoid(alpha g) (u + 1))`` with ``g = min(W_gate h, limit)``, ``u = clamp(W_up h, +-limit)``
``SigmoidRoutedMoE``  experts of the second form chosen by the largest ``sigmoid`` router scores, weighing their scores
                    over the chosen's sum times a constant, beside an optional shared expert that every token runs
``SiluGluMLP``      ``W_down (silu(W_gate h + b_gate) (W_up h + b_up)) + b_down``, bf16 or fp32
``Relu2RoutedMoE``  experts ``W_down max(W_up h, 0)^2`` chosen by the largest router logits ``W_r h + b_r``, weighing the
                    softmax over the chosen logits alone
``GroupedSoftmaxMoE``  silu-gated experts weighed by the softmax over ALL router outputs (not renormalised), chosen by
                    corrected scores within the best groups of outputs; the last outputs are identity experts; a shared
                    expert behind a sigmoid gate of one number per token

Beside ``HymetaMoE`` (``moe.py``: softmax router, silu experts) and ``TableMoE`` (``table_moe.py``: no router network);
the expert stacks ``w13 [E, 2I, H]`` / ``w2 [E, H, I]`` are theirs.
"""

from __future__ import annotations

import math
from typing import Optional, Tuple

import torch

from .. import hip_ops
from ..linear import HymetaLinear

GLU_ALPHA = 1.702       # the sigmoid's slope in the clamped gated unit


def _softplus(v: float) -> float:
    return max(v, 0.0) + math.log1p(math.exp(-abs(v)))


class XieluMLP(torch.nn.Module):
    def __init__(self, up_proj: HymetaLinear, down_proj: HymetaLinear, p: float, q: float):
        super().__init__()
        self.up_proj, self.down_proj = up_proj, down_proj
        self.a_pos, self.a_neg = _softplus(float(p)), 0.5 + _softplus(float(q))

    def forward(self, h: torch.Tensor) -> torch.Tensor:
        return self.down_proj(hip_ops.xielu(self.up_proj(h), self.a_pos, self.a_neg))


class ClampedGluMLP(torch.nn.Module):
    def __init__(self, gate_up_proj: HymetaLinear, down_proj: HymetaLinear, limit: float, alpha: float = GLU_ALPHA):
        """``gate_up_proj``: rows = gate, then up."""
        super().__init__()
        self.gate_up_proj, self.down_proj, self.limit, self.alpha = gate_up_proj, down_proj, float(limit), float(alpha)

    def forward(self, h: torch.Tensor) -> torch.Tensor:
        return self.down_proj(hip_ops.clamped_glu(self.gate_up_proj(h), self.limit, self.alpha))


class SigmoidRoutedMoE(torch.nn.Module):
    def __init__(self, router_weight: torch.Tensor, w13: torch.Tensor, w2: torch.Tensor, top_k: int, route_scale: float, limit: float,
                 shared: Optional[ClampedGluMLP] = None, alpha: float = GLU_ALPHA):
        super().__init__()
        self.register_buffer("router_weight", router_weight.float().contiguous())     # the router runs in fp32
        self.register_buffer("w13", w13.contiguous())
        self.register_buffer("w2", w2.contiguous())
        self.top_k, self.route_scale, self.limit, self.alpha, self.shared = int(top_k), float(route_scale), float(limit), float(alpha), shared

    def forward(self, h: torch.Tensor) -> Tuple[torch.Tensor, Optional[torch.Tensor]]:
        """``(routed experts' weighted sum, shared expert's output or None)``: whoever adds them to the stream adds both."""
        y = hip_ops.moe_sigmoid_forward(h, self.router_weight, self.w13, self.w2, self.top_k, self.route_scale, self.limit, self.alpha)
        return y, (None if self.shared is None else self.shared(h))


class SiluGluMLP(torch.nn.Module):
    def __init__(self, gate_up_proj: HymetaLinear, down_proj: HymetaLinear):
        """``gate_up_proj``: rows = gate, then up (with their biases)."""
        super().__init__()
        self.gate_up_proj, self.down_proj = gate_up_proj, down_proj

    def forward(self, h: torch.Tensor) -> torch.Tensor:
        return self.down_proj(hip_ops.silu_mul(self.gate_up_proj(h)))


class Relu2RoutedMoE(torch.nn.Module):
    def __init__(self, router_weight: torch.Tensor, router_bias: Optional[torch.Tensor], w1: torch.Tensor, w2: torch.Tensor, top_k: int):
        """``w1 [E, I, H]`` (up projections), ``w2 [E, H, I]``."""
        super().__init__()
        self.register_buffer("router_weight", router_weight.float().contiguous())     # the router runs in fp32
        self.register_buffer("router_bias", None if router_bias is None else router_bias.float().contiguous())
        self.register_buffer("w1", w1.contiguous())
        self.register_buffer("w2", w2.contiguous())
        self.top_k = int(top_k)

    def forward(self, h: torch.Tensor) -> torch.Tensor:
        return hip_ops.moe_routed_forward(h, self.router_weight, self.router_bias, self.w1, self.w2, self.top_k,
                                          hip_ops.ROUTE_SOFTMAX_CHOSEN, 1.0, "relu2")


class GroupedSoftmaxMoE(torch.nn.Module):
    """``s = softmax(W_r h)`` over ``experts + identity`` outputs; the ``top_k`` largest ``s + correction`` among the outputs
    of the ``keep`` groups (of ``groups`` equal runs of neighbours) whose best corrected score is largest are chosen; the
    output is ``sum_chosen s_e expert_e(h)`` with ``expert_e(h) = W_down (silu(W_gate h) W_up h)``, or ``h`` itself for the
    last ``identity`` outputs, plus ``sigmoid(w_sg . h) shared(h)``."""

    def __init__(self, router_weight: torch.Tensor, correction: Optional[torch.Tensor], w13: torch.Tensor, w2: torch.Tensor, top_k: int,
                 groups: int, keep: int, identity: int, shared: Optional[SiluGluMLP] = None, shared_gate: Optional[torch.Tensor] = None):
        """``router_weight [experts + identity, H]``, ``shared_gate [1, H]`` (with ``shared``)."""
        super().__init__()
        if (shared is None) != (shared_gate is None):
            raise ValueError("the shared expert comes with its gate")
        rows = router_weight.float() if shared_gate is None else torch.cat([router_weight.float(), shared_gate.float().reshape(1, -1)], 0)
        self.register_buffer("router_rows", rows.contiguous())           # the router runs in fp32; the gate's row rides behind it
        self.register_buffer("correction", None if correction is None else correction.float().contiguous())
        self.register_buffer("w13", w13.contiguous())
        self.register_buffer("w2", w2.contiguous())
        self.top_k, self.groups, self.keep, self.identity, self.shared = int(top_k), int(groups), int(keep), int(identity), shared

    def forward(self, h: torch.Tensor):
        """Terms for whoever adds them to the stream: the routed sum, ``identity_weight[t] h[t]``, the gated shared expert."""
        choice = hip_ops.GroupedChoice(self.correction, self.groups, self.keep, self.identity, 0 if self.shared is None else 1)
        y, identity_weight, gate = hip_ops.moe_routed_forward(h, self.router_rows, None, self.w13, self.w2, self.top_k,
                                                              hip_ops.ROUTE_SOFTMAX_GROUPED, 1.0, "silu_glu", choice=choice)
        terms = [(y, 1.0, None)]
        if identity_weight is not None:
            terms.append((h, 1.0, identity_weight))
        if self.shared is not None:
            terms.append((self.shared(h), 1.0, gate))
        return terms
