"""State-space mixer in the state-space duality form (Mamba-2: "Transformers are SSMs", Dao and Gu 2024):

    [z | xBC | dt] = W_in h;   xBC <- silu(causal conv over time per channel, with bias);   x, B, C = split(xBC)
    dt <- softplus(dt + dt_bias);   per head (B and C shared by a group of heads):
    S_t = exp(-exp(A_log) dt_t) S_{t-1} + dt_t B_t x_t^T;   y_t = S_t^T C_t + D x_t
    out = W_o (rms_norm_in_groups(y * silu(z)) * w)                   (the gate comes before the norm)

The convolution with the step sizes is ``hip_ops.causal_conv_silu`` (its last taps - 1 input rows are part of a
sequence's state), the recurrence ``hip_ops.decay_scan`` with the state fp32 ``[slots, heads, N, P]``, the gate and the
grouped norm ``hip_ops.gated_rms_norm``.  Beside ``RetentionMixer`` (``retention.py``: a constant decay per head),
``LightningAttentionMixer`` and ``MinGRUMixer`` (``mingru.py``: a vector state).
"""

from __future__ import annotations

import torch

from .. import hip_ops
from ..linear import HymetaLinear


class StateSpaceMixer(torch.nn.Module):
    def __init__(self, in_proj: HymetaLinear, o_proj: HymetaLinear, heads: int, vdim: int, state: int, groups: int, norm_groups: int,
                 conv_weight: torch.Tensor, conv_bias: torch.Tensor, dt_bias: torch.Tensor, a_log: torch.Tensor, skip: torch.Tensor,
                 norm_weight: torch.Tensor, eps: float):
        """``in_proj``: rows = gate z (``heads vdim``), x (``heads vdim``), B and C (``groups state`` each), dt (``heads``)."""
        super().__init__()
        self.in_proj, self.o_proj = in_proj, o_proj
        self.H, self.P, self.N, self.G, self.norm_groups, self.eps = heads, vdim, state, groups, int(norm_groups), float(eps)
        for name, t in (("conv_weight", conv_weight), ("conv_bias", conv_bias), ("dt_bias", dt_bias), ("a_log", a_log), ("skip", skip),
                        ("norm_weight", norm_weight)):
            self.register_buffer(name, t.float().contiguous())

    @property
    def taps(self) -> int:
        return self.conv_weight.shape[1]

    def forward(self, h: torch.Tensor, layout, state) -> torch.Tensor:
        """``state``: ``(S fp32 [slots, heads, N, P], conv inputs [slots, taps - 1, channels] in the activations' type)``,
        updated in place for the step's sequences."""
        ssm_state, conv_state = state
        H, P, N, G = self.H, self.P, self.N, self.G
        inner, ch = H * P, H * P + 2 * G * N
        proj = self.in_proj(h)
        xbc, dt, log2_decay = hip_ops.causal_conv_silu(proj[:, inner:inner + ch], self.conv_weight, self.conv_bias, conv_state,
                                                       layout.query_start_loc, layout.context_lens, layout.slot_idx,
                                                       dt_in=proj[:, inner + ch:inner + ch + H], dt_bias=self.dt_bias, a_log=self.a_log,
                                                       max_query_len=layout.max_query_len)
        x = xbc[:, :inner].view(-1, H, P)
        b, c = xbc[:, inner:inner + G * N].view(-1, G, N), xbc[:, inner + G * N:].view(-1, G, N)
        y = hip_ops.decay_scan(c, b, x, ssm_state, layout.query_start_loc, layout.context_lens, layout.slot_idx, layout.max_query_len,
                               log2_decay=log2_decay, v_scale=dt, skip=self.skip)
        y = hip_ops.gated_rms_norm(y, proj[:, :inner], self.norm_weight, self.eps, groups=self.norm_groups, gate_act="silu", gate_first=True)
        return self.o_proj(y)
