"""Decoder block on an fp32 residual stream with a norm on both sides of every sublayer:

    x <- x + mult * norm_out(sublayer(conv_in(norm_in(x))))

``norm_in`` / ``norm_out`` are RMS norms whose weight is stored around zero (the kernel applies ``1 + w``);
``conv_in`` is an optional short causal convolution over time on each channel, added to its own input, whose last
``taps - 1`` input rows are part of a sequence's state.  The stream stays fp32 whatever the activation type; a
sublayer reads and returns activations (bf16 or fp32).  Beside ``DecoderBlock`` (``block.py``), which keeps a bf16
stream and folds the residual add into the next norm.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Optional

import torch

from .. import hip_ops


@dataclass
class StepLayout:
    """What the kernels need to know about a step's rows: sequence ``s`` owns rows ``query_start_loc[s] ..
    query_start_loc[s + 1] - 1``, had ``context_lens[s]`` tokens before them and ``seq_lens[s]`` with them, keeps its
    recurrent states in slot ``slot_idx[s]`` and its keys in the pages ``block_tables[s]``."""
    query_start_loc: torch.Tensor
    context_lens: torch.Tensor
    seq_lens: torch.Tensor
    slot_idx: torch.Tensor
    block_tables: Optional[torch.Tensor]
    slot_mapping: Optional[torch.Tensor]
    max_query_len: int
    max_seq_len: int
    token_ids: Optional[torch.Tensor] = None
    positions: Optional[torch.Tensor] = None      # int64 [rows], where the caller of the model gave them


class NormConvIn(torch.nn.Module):
    """``norm_in`` and ``conv_in`` of a sublayer, one launch.  ``weight`` is the stored norm weight (around zero),
    ``conv_weight [W, taps]`` or None."""

    def __init__(self, weight: torch.Tensor, eps: float, conv_weight: Optional[torch.Tensor] = None, weight_offset: float = 1.0):
        super().__init__()
        self.register_buffer("weight", weight.float().contiguous())
        self.register_buffer("conv_weight", None if conv_weight is None else conv_weight.float().contiguous())
        self.eps, self.weight_offset = float(eps), float(weight_offset)

    @property
    def history(self) -> int:
        return 0 if self.conv_weight is None else self.conv_weight.shape[1] - 1

    def forward(self, x: torch.Tensor, out_dtype: torch.dtype, layout: Optional[StepLayout] = None,
                conv_state: Optional[torch.Tensor] = None) -> torch.Tensor:
        if self.history == 0:
            return hip_ops.norm_conv(x, self.weight, self.eps, out_dtype, self.weight_offset, self.conv_weight)
        return hip_ops.norm_conv(x, self.weight, self.eps, out_dtype, self.weight_offset, self.conv_weight, conv_state,
                                 layout.query_start_loc, layout.context_lens, layout.slot_idx)


class NormOutResidual(torch.nn.Module):
    """``x += mult * norm_out(y) (+ post_add)`` on the fp32 stream, one launch, in place."""

    def __init__(self, weight: torch.Tensor, eps: float, mult: float, weight_offset: float = 1.0):
        super().__init__()
        self.register_buffer("weight", weight.float().contiguous())
        self.eps, self.mult, self.weight_offset = float(eps), float(mult), float(weight_offset)

    def forward(self, x: torch.Tensor, y: torch.Tensor, post_add: Optional[torch.Tensor] = None) -> torch.Tensor:
        return hip_ops.norm_residual_(x, y, self.weight, self.eps, self.mult, self.weight_offset, post_add)


class StreamBlock(torch.nn.Module):
    """One decoder layer: mixer sublayer, then (optionally) feed-forward sublayer.  ``mixer(h, layout, state)`` and
    ``mlp(h, layout)`` take and return activations."""

    def __init__(self, mixer_in: NormConvIn, mixer: torch.nn.Module, mixer_out: NormOutResidual,
                 mlp_in: Optional[NormConvIn] = None, mlp: Optional[torch.nn.Module] = None,
                 mlp_out: Optional[NormOutResidual] = None):
        super().__init__()
        self.mixer_in, self.mixer, self.mixer_out = mixer_in, mixer, mixer_out
        self.mlp_in, self.mlp, self.mlp_out = mlp_in, mlp, mlp_out

    @property
    def conv_states(self) -> int:
        """Convolution states a pass through this layer carries (one per sublayer with a convolution)."""
        return int(self.mixer_in.history > 0) + int(self.mlp is not None and self.mlp_in.history > 0)

    def forward(self, x: torch.Tensor, act_dtype: torch.dtype, layout: StepLayout, mixer_state, conv_states,
                post_add: Optional[torch.Tensor] = None) -> torch.Tensor:
        """``conv_states``: this pass's convolution-state tensors in sublayer order; ``mixer_state``: whatever the mixer
        carries (a recurrent state tensor, an attention layer's paged cache is its own); ``post_add``: a vector added to
        the stream after the layer (what the next layer, or pass, wants added before it starts)."""
        states = list(conv_states)
        h = self.mixer_in(x, act_dtype, layout, states.pop(0) if self.mixer_in.history else None)
        y = self.mixer(h, layout, mixer_state)
        self.mixer_out(x, y, post_add if self.mlp is None else None)
        if self.mlp is not None:
            h = self.mlp_in(x, act_dtype, layout, states.pop(0) if self.mlp_in.history else None)
            y = self.mlp(h, layout)
            self.mlp_out(x, y, post_add)
        return x
