"""Pre-norm decoder block on several fp32 residual streams ("hyper-connections"):

    u = sum_s in[s] x_s,   y = sublayer(norm(u)),   x_t <- sum_s mix[s, t] x_s + out[t] y   (all streams from the old ones)

(learned read weights, write weights and a remix of the streams per sublayer; "Hyper-Connections", Zhu et al. 2024).  One
stream with ``in = out = mix = 1`` is the plain pre-norm residual ``x <- x + sublayer(norm(x))``, which is how a model
without streams runs here.  ``norm`` is a layer norm with a weight and no bias.  The streams stay fp32 whatever the
activation type; a sublayer reads and returns activations (bf16 or fp32).

The write of one sublayer and the read of the next are ONE launch (``hip_ops.hyper_stream_``): a sublayer's output is
kept as *pending* until the next read (or the end of the model) applies it.  Beside ``StreamBlock`` (``stream_block.py``:
one stream, norms on both sides of a sublayer), ``PostNormBlock`` (``post_norm_block.py``) and ``DecoderBlock``
(``block.py``: a bf16 stream).
"""

from __future__ import annotations

from typing import Optional, Tuple

import torch

from .. import hip_ops
from .stream_block import StepLayout


class HyperConnection(torch.nn.Module):
    """The stream weights of one sublayer: ``in_w [S]``, ``out_w [S]``, ``mix [S, S]`` indexed [from, to]."""

    def __init__(self, in_w: torch.Tensor, out_w: torch.Tensor, mix: torch.Tensor):
        super().__init__()
        S = in_w.numel()
        if out_w.numel() != S or tuple(mix.shape) != (S, S):
            raise ValueError("in_w [S], out_w [S] and mix [S, S] must agree")
        self.register_buffer("in_w", in_w.float().contiguous())
        self.register_buffer("out_w", out_w.float().contiguous())
        self.register_buffer("mix", mix.float().contiguous())

    @classmethod
    def plain(cls, device) -> "HyperConnection":
        one = torch.ones(1, dtype=torch.float32, device=device)
        return cls(one, one.clone(), one.clone().view(1, 1))

    @classmethod
    def summing(cls, streams: int, device) -> "HyperConnection":
        """Reads the sum of the streams (what the model's last norm sees); never written through."""
        return cls(torch.ones(streams, dtype=torch.float32, device=device), torch.zeros(streams, dtype=torch.float32, device=device),
                   torch.eye(streams, dtype=torch.float32, device=device))


Pending = Optional[Tuple[torch.Tensor, HyperConnection]]      # a sublayer's output and the weights that will spread it


class StreamNormRead(torch.nn.Module):
    """``norm(sum_s in[s] x_s)`` of the streams, after whatever is pending has been written into them (same launch)."""

    def __init__(self, hc: HyperConnection, weight: torch.Tensor, eps: float):
        super().__init__()
        self.hc = hc
        self.register_buffer("weight", weight.float().contiguous())
        self.eps = float(eps)

    def forward(self, x: torch.Tensor, pending: Pending, out_dtype: torch.dtype) -> torch.Tensor:
        y, w = pending if pending is not None else (None, None)
        return hip_ops.hyper_stream_(x, y, None if w is None else w.mix, None if w is None else w.out_w, self.hc.in_w, self.weight,
                                     self.eps, out_dtype)


def flush_pending(x: torch.Tensor, pending: Pending) -> None:
    """Write a pending sublayer output into the streams without reading them."""
    if pending is not None:
        y, w = pending
        hip_ops.hyper_stream_(x, y, w.mix, w.out_w, None, None, 0.0, None)


class HyperStreamBlock(torch.nn.Module):
    """One decoder layer: mixer sublayer, then (optionally) feed-forward sublayer.  ``mixer(h, layout, state, carry)``
    returns ``(activations, carry)`` (``carry``: what later layers' mixers want from earlier ones); ``mlp(h)`` returns
    activations."""

    def __init__(self, mixer_in: StreamNormRead, mixer: torch.nn.Module, mlp_in: Optional[StreamNormRead] = None,
                 mlp: Optional[torch.nn.Module] = None):
        super().__init__()
        self.mixer_in, self.mixer, self.mlp_in, self.mlp = mixer_in, mixer, mlp_in, mlp

    def forward(self, x: torch.Tensor, pending: Pending, act_dtype: torch.dtype, layout: StepLayout, mixer_state, carry):
        """``x [T, S, W]`` fp32, updated in place up to the block's last sublayer, whose output is returned pending."""
        h = self.mixer_in(x, pending, act_dtype)
        y, carry = self.mixer(h, layout, mixer_state, carry)
        pending = (y, self.mixer_in.hc)
        if self.mlp is not None:
            h = self.mlp_in(x, pending, act_dtype)
            pending = (self.mlp(h), self.mlp_in.hc)
        return pending, carry
