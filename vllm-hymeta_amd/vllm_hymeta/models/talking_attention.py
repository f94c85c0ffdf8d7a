"""Softmax attention whose scores are mixed across heads before the softmax ("Talking-Heads Attention", Shazeer et al.
2020; here only the mix before the softmax), over grouped key/value heads:

    q = W_q h + b_q, k = W_k h + b_k, v = W_v h + b_v;  q, k <- RMS norm over the WHOLE projection, times a weight
    the first rot_dims dimensions of every head turn in interleaved pairs (2i, 2i + 1) by position * base^(-2i / rot_dims)
    s_h(i, j) = scale q_h(i) . k_g(h)(j),   s'_h = sum_g talk[h, g] s_g
    query i sees key j <= i if i - j < window or j < keep_first;  p = softmax(s') over the visible keys
    v <- (1 - blend) v + blend v_first  (v_first: the values the first blending layer computed for the same token)
    out = W_o concat_h(sum_j p_h(i, j) v_g(h)(j))

The mix is linear in the queries, so it is moved onto them: with the keys of a token's G key/value heads concatenated
into one row ``K(j)``, ``s'_h(i, j) = scale Q_h(i) . K(j)`` where ``Q_h(i)[g D + d] = sum over the query heads j of group g
of talk[h, j] q_j(i)[d]``.  The attention kernel then sees ONE key of ``G D`` elements per token, shared by all query heads,
followed by the G values (``hip_ops.sink_attention(shared_key=True)``), for prompts and decoding alike; what the mix costs
is a key product ``G`` times as long.

``PagedSharedKeyAttention`` is the cache-owning object an engine finds by name and binds a cache to (as ``MetaAttention``,
``PagedBiasAttention``, ``PagedLatentAttention``); ``TalkingHeadsAttentionMixer`` is the sublayer around it.
"""

from __future__ import annotations

from typing import List, Optional, Tuple

import torch

from .. import hip_ops
from ..linear import HymetaLinear
from . import attention as _registry


class PagedSharedKeyAttention(torch.nn.Module):
    def __init__(self, num_heads: int, num_kv_heads: int, head_dim: int, v_dim: int, scale: float, prefix: str,
                 sliding_window: Optional[int] = None, keep_first: int = 0, dtype: torch.dtype = torch.bfloat16):
        super().__init__()
        self.num_heads, self.num_kv_heads, self.head_dim, self.v_size = num_heads, num_kv_heads, head_dim, v_dim
        self.head_size = num_kv_heads * head_dim          # the shared key: every key/value head's key of the token
        self.scale, self.dtype = float(scale), dtype
        self.window_left = -1 if sliding_window is None else sliding_window - 1
        self.keep_first = int(keep_first) if sliding_window is not None else 0
        if prefix in _registry._LAYERS:
            raise ValueError(f"Duplicate layer name: {prefix}")
        _registry._LAYERS[prefix] = self
        self.layer_name = prefix
        self.kv_cache: List[torch.Tensor] = [torch.tensor([])]

    def kv_cache_shape(self, num_blocks: int, block_size: int) -> Tuple[int, ...]:
        return (num_blocks, block_size, 1, self.num_kv_heads * (self.head_dim + self.v_size))

    def cache(self) -> torch.Tensor:
        kv = self.kv_cache[0]
        if kv.numel() == 0:
            raise RuntimeError(f"{self.layer_name}: no KV cache bound")
        return kv

    def forward(self, q: torch.Tensor, layout) -> torch.Tensor:
        """``q [T, H, G D]`` (mixed across heads) against the cached rows (this step's are stored already) -> ``[T, H, Dv]``."""
        return hip_ops.sink_attention(q, self.cache(), layout.block_tables, layout.query_start_loc, layout.seq_lens, self.num_kv_heads,
                                      self.head_size, self.v_size, self.scale, layout.max_query_len, layout.max_seq_len, sink=False,
                                      window_left=self.window_left, shared_key=True, keep_first=self.keep_first)


class TalkingHeadsAttentionMixer(torch.nn.Module):
    def __init__(self, qkv_proj: HymetaLinear, o_proj: HymetaLinear, attn: PagedSharedKeyAttention, q_norm_weight: torch.Tensor,
                 k_norm_weight: torch.Tensor, talk: Optional[torch.Tensor], eps: float, rot_dims: int, rot_freqs: Optional[torch.Tensor],
                 blend: Optional[float]):
        """``qkv_proj``: rows = queries, keys, values.  ``talk [H, H]`` (None: the heads' scores are not mixed).  ``blend``:
        None: the layer does not blend its values; otherwise its weight on the first blending layer's values."""
        super().__init__()
        self.qkv_proj, self.o_proj = qkv_proj, o_proj
        H = attn.num_heads
        dev = q_norm_weight.device
        self.register_buffer("q_norm_weight", q_norm_weight.float().contiguous())
        self.register_buffer("k_norm_weight", k_norm_weight.float().contiguous())
        self.register_buffer("talk", (torch.eye(H, device=dev) if talk is None else talk).float().contiguous())
        self.register_buffer("rot_freqs", None if rot_freqs is None else rot_freqs.to(torch.float64).contiguous())
        self.eps, self.rot_dims, self.blend = float(eps), int(rot_dims), blend
        self._attn = (attn,)          # owned (and registered as a module) by the model

    def forward(self, h: torch.Tensor, layout, attn: Optional[PagedSharedKeyAttention] = None,
                v_first: Optional[torch.Tensor] = None) -> Tuple[torch.Tensor, Optional[torch.Tensor]]:
        """Returns ``(output, v_first)``: the first blending layer hands its own values (columns of its projection, as
        computed) to the later ones."""
        attn = attn or self._attn[0]
        H, G, D, Dv = attn.num_heads, attn.num_kv_heads, attn.head_dim, attn.v_size
        qkv = self.qkv_proj(h)
        other = v_first if self.blend is not None else None
        q = hip_ops.talk_qkv_prep(qkv, H, G, D, Dv, self.q_norm_weight, self.k_norm_weight, self.talk, self.eps, self.rot_dims,
                                  self.rot_freqs, attn.cache(), layout.slot_mapping, layout.query_start_loc, layout.seq_lens,
                                  v_other=other, v_blend=self.blend if other is not None else 0.0, positions=getattr(layout, "positions", None))
        if self.blend is not None and v_first is None:
            v_first = qkv[:, (H + G) * D:]
        o = attn(q, layout)
        return self.o_proj(o.view(-1, H * Dv)), v_first
