"""Retention mixer: linear attention with a constant decay per head and neither softmax nor denominator,

    q, k = rotate(W_q h), rotate(W_k h) dim^(-1/2);   v = W_v h;   S_t = decay_h S_{t-1} + k_t v_t^T;   o_t = S_t^T q_t
    out = W_o (concat_h(o_t / rms(o_t)) * silu(W_g h))

("Retentive Network: A Successor to Transformer for Large Language Models", Sun et al. 2023).  ``rotate`` turns dimensions i
and i + rot_dims / 2 of a head together by position * base^(-2 i / rot_dims).  The four input projections are one linear
layer; the rotation is ``hip_ops.rotary_cache_`` (no cache), the recurrence ``hip_ops.decay_scan`` with the state fp32
``[slots, H, D, Dv]``, one slot per sequence; every head's output is divided by its own root mean square
(``hip_ops.gated_rms_norm`` with one group per head, no weight).  Beside ``LightningAttentionMixer``
(``lightning_attention.py``), whose inputs pass a silu and whose norm spans the heads, and ``StateSpaceMixer``
(``state_space.py``), whose decay changes from token to token.
"""

from __future__ import annotations

from typing import Optional

import torch

from .. import hip_ops
from ..linear import HymetaLinear


class RetentionMixer(torch.nn.Module):
    def __init__(self, in_proj: HymetaLinear, o_proj: HymetaLinear, num_heads: int, dim: int, vdim: int, decay: torch.Tensor,
                 rot_dims: int, rot_freqs: Optional[torch.Tensor], eps: float):
        """``in_proj``: rows = queries, keys, values, output gate (``2 H dim + 2 H vdim`` outputs)."""
        super().__init__()
        self.in_proj, self.o_proj = in_proj, o_proj
        self.H, self.D, self.Dv, self.rot_dims, self.eps = num_heads, dim, vdim, int(rot_dims), float(eps)
        self.register_buffer("decay", decay.float().contiguous())
        self.register_buffer("rot_freqs", None if rot_freqs is None else rot_freqs.to(torch.float64).contiguous())

    def forward(self, h: torch.Tensor, layout, state: torch.Tensor) -> torch.Tensor:
        """``state`` fp32 ``[slots, H, D, Dv]``, updated in place for the step's sequences."""
        H, D, Dv = self.H, self.D, self.Dv
        proj = self.in_proj(h)
        hip_ops.rotary_cache_(proj, H, H, D, Dv, self.rot_dims, self.rot_freqs, D ** -0.5, positions=layout.positions,
                              query_start_loc=layout.query_start_loc, seq_lens=layout.seq_lens)
        q, k = proj[:, :H * D].view(-1, H, D), proj[:, H * D:2 * H * D].view(-1, H, D)
        v = proj[:, 2 * H * D:2 * H * D + H * Dv].view(-1, H, Dv)
        o = hip_ops.decay_scan(q, k, v, state, layout.query_start_loc, layout.context_lens, layout.slot_idx, layout.max_query_len,
                               decay=self.decay)
        y = hip_ops.gated_rms_norm(o, proj[:, 2 * H * D + H * Dv:], None, self.eps, groups=H, gate_act="silu")
        return self.o_proj(y)
