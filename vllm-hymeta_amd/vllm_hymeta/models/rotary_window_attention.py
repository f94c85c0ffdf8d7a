"""Causal softmax attention over a paged cache with grouped key/value heads, a sliding window, half-split rotary pairs,
optionally tanh-capped scores and a sigmoid gate per head:

    q, k, v = W_q h (+ b), W_k h (+ b), W_v h (+ b);   dimensions i and i + rot_dims / 2 of every query and key head turn
    together by position * base^(-2 i / rot_dims) ("rotate half"); the rest of a head passes
    s_ij = scale q_i . k_j;   s_ij <- softcap tanh(s_ij / softcap)  (with softcap)
    query i sees keys j with 0 <= i - j < window;   p = softmax(s) over them
    out = W_o concat_h(sigmoid(W_g h)_h * sum_j p_h(i, j) v_g(h)(j))  (+ b)       (the gate: one number per head)

The gate's rows ride in the fused input projection (queries, keys, values, gates: one GEMM); the rotation, the paged write
and the attention are ``hip_ops.rotary_cache_`` and ``hip_ops.sink_attention`` (no sink, ``KV_KEY_THEN_VALUE`` rows, the
cap and the gate inside the attention kernels).  ``PagedWindowAttention`` is the cache-owning object an engine finds by
name and binds a cache to (as ``MetaAttention``, ``PagedBiasAttention``, ``PagedSharedKeyAttention``);
``WindowAttentionMixer`` is the sublayer around it.
"""

from __future__ import annotations

from typing import List, Optional, Tuple

import torch

from .. import hip_ops
from ..linear import HymetaLinear
from . import attention as _registry


class PagedWindowAttention(torch.nn.Module):
    def __init__(self, num_heads: int, num_kv_heads: int, head_dim: int, v_dim: int, scale: float, prefix: str,
                 sliding_window: Optional[int] = None, softcap: Optional[float] = None, dtype: torch.dtype = torch.bfloat16):
        super().__init__()
        self.num_heads, self.num_kv_heads, self.head_size, self.v_size = num_heads, num_kv_heads, head_dim, v_dim
        self.scale, self.softcap, self.dtype = float(scale), float(softcap or 0.0), dtype
        self.window_left = -1 if sliding_window is None else sliding_window - 1
        if prefix in _registry._LAYERS:
            raise ValueError(f"Duplicate layer name: {prefix}")
        _registry._LAYERS[prefix] = self
        self.layer_name = prefix
        self.kv_cache: List[torch.Tensor] = [torch.tensor([])]

    def kv_cache_shape(self, num_blocks: int, block_size: int) -> Tuple[int, ...]:
        return (num_blocks, block_size, self.num_kv_heads, self.head_size + self.v_size)

    def cache(self) -> torch.Tensor:
        kv = self.kv_cache[0]
        if kv.numel() == 0:
            raise RuntimeError(f"{self.layer_name}: no KV cache bound")
        return kv

    def forward(self, q: torch.Tensor, layout, head_gate: Optional[torch.Tensor] = None) -> torch.Tensor:
        """``q [T, H, D]`` against the cached rows (this step's are stored already) -> ``[T, H, Dv]``."""
        return hip_ops.sink_attention(q, self.cache(), layout.block_tables, layout.query_start_loc, layout.seq_lens, self.num_kv_heads,
                                      self.head_size, self.v_size, self.scale, layout.max_query_len, layout.max_seq_len, sink=False,
                                      window_left=self.window_left, softcap=self.softcap, head_gate=head_gate)


class WindowAttentionMixer(torch.nn.Module):
    def __init__(self, in_proj: HymetaLinear, o_proj: HymetaLinear, attn: PagedWindowAttention, rot_dims: int,
                 rot_freqs: Optional[torch.Tensor], gated: bool):
        """``in_proj``: rows = queries, keys, values and (``gated``) one gate row per head."""
        super().__init__()
        self.in_proj, self.o_proj, self.rot_dims, self.gated = in_proj, o_proj, int(rot_dims), bool(gated)
        self.register_buffer("rot_freqs", None if rot_freqs is None else rot_freqs.to(torch.float64).contiguous())
        self._attn = (attn,)          # owned (and registered as a module) by the model, one per layer that runs these weights

    def forward(self, h: torch.Tensor, layout, attn: Optional[PagedWindowAttention] = None) -> torch.Tensor:
        attn = attn or self._attn[0]
        H, G, D, Dv = attn.num_heads, attn.num_kv_heads, attn.head_size, attn.v_size
        proj = self.in_proj(h)
        hip_ops.rotary_cache_(proj, H, G, D, Dv, self.rot_dims, self.rot_freqs, 1.0, attn.cache(), layout.slot_mapping,
                              positions=layout.positions, query_start_loc=layout.query_start_loc, seq_lens=layout.seq_lens)
        gate = proj[:, (H + G) * D + G * Dv:(H + G) * D + G * Dv + H] if self.gated else None
        o = attn(proj[:, :H * D].view(-1, H, D), layout, gate)
        return self.o_proj(o.view(-1, H * Dv))
