"""Decoder block whose mixer and feed-forward read ONE norm of the fp32 residual stream and are added together:

    h = x / sqrt(mean(x^2) + eps) * g        (g: one number for all columns)
    x <- x + mixer(h) + ff(h)

A sublayer returns an activation tensor or a list of terms ``(y, coefficient, per-row fp32 scale or None)``: two mixers side
by side with their constants, a mixture's routed sum beside its identity experts' share of ``h`` and its gated shared
expert.  All terms of a layer are added in one launch (``hip_ops.stream_add_norm_``) that also writes the NEXT block's
``h`` (or the model's final norm), so the stream is read and written once per layer.  Beside ``StreamBlock``
(``stream_block.py``: norms on both sides of every sublayer), ``PostNormBlock`` and ``HyperStreamBlock``.
"""

from __future__ import annotations

from typing import List, Optional, Tuple, Union

import torch

from .. import hip_ops
from .stream_block import StepLayout

Term = Tuple[torch.Tensor, float, Optional[torch.Tensor]]


def as_terms(y: Union[torch.Tensor, List[Term]]) -> List[Term]:
    return [(y, 1.0, None)] if isinstance(y, torch.Tensor) else list(y)


class SideBySideMixer(torch.nn.Module):
    """Two mixers on the same input, ``left_scale * left(h) + right_scale * right(h)``: the sum is left to the block's add."""

    def __init__(self, left: torch.nn.Module, right: torch.nn.Module, left_scale: float, right_scale: float):
        super().__init__()
        self.left, self.right, self.left_scale, self.right_scale = left, right, float(left_scale), float(right_scale)

    def forward(self, h: torch.Tensor, layout: StepLayout, state) -> List[Term]:
        """``state``: ``(left's, right's)``."""
        return [(self.left(h, layout, state[0]), self.left_scale, None), (self.right(h, layout, state[1]), self.right_scale, None)]


class ParallelBlock(torch.nn.Module):
    """``mixer(h, layout, state)`` and ``mlp(h)`` return activations or lists of terms.  ``norm_scale``: the block's ``g``."""

    def __init__(self, norm_scale: float, mixer: torch.nn.Module, mlp: Optional[torch.nn.Module], eps: float):
        super().__init__()
        self.norm_scale, self.mixer, self.mlp, self.eps = float(norm_scale), mixer, mlp, float(eps)

    def read(self, x: torch.Tensor, act_dtype: torch.dtype) -> torch.Tensor:
        """``h`` of a stream that nothing is waiting to be added to (the first block)."""
        return hip_ops.stream_add_norm_(x, [], self.norm_scale, self.eps, act_dtype)

    def forward(self, x: torch.Tensor, h: torch.Tensor, layout: StepLayout, mixer_state, next_norm_scale: Optional[float]) -> Optional[torch.Tensor]:
        """Adds the block to the stream in place; returns the next reader's ``h`` (``next_norm_scale``: its ``g``; None:
        nobody reads on)."""
        terms = as_terms(self.mixer(h, layout, mixer_state))
        if self.mlp is not None:
            terms += as_terms(self.mlp(h))
        return hip_ops.stream_add_norm_(x, terms, next_norm_scale, self.eps, h.dtype)
