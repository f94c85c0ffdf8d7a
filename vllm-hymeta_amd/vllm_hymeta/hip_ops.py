"""Torch-tensor front end of the C ABI: checks tensors on the host, fills the
argument structs and enqueues the kernels on torch's current HIP stream.

torch is used for device memory and the stream handle only; every op below
runs in libhymeta_hip.so.
"""

from __future__ import annotations

import ctypes as C
import os
from typing import NamedTuple, Optional, Sequence, Tuple

import torch

from . import _C

_DT = {torch.bfloat16: _C.HYMETA_BF16, torch.float32: _C.HYMETA_F32}


def _stream(t: torch.Tensor):
    return C.c_void_p(torch.cuda.current_stream(t.device).cuda_stream)


def _p(t: Optional[torch.Tensor]):
    return None if t is None else C.c_void_p(t.data_ptr())


def _require(cond: bool, msg: str) -> None:
    if not cond:
        raise ValueError(msg)


def _dev(*ts):
    dev = None
    for t in ts:
        if t is None:
            continue
        _require(t.is_cuda, "hymeta ops need HIP device tensors")
        dev = dev or t.device
        _require(t.device == dev, "all tensors must live on one device")
    return dev


def _inner_contig(t: torch.Tensor, name: str) -> None:
    _require(t.stride(-1) == 1, f"{name}: innermost dimension must be contiguous")


# ---------------------------------------------------------------------------
# GLA decode
# ---------------------------------------------------------------------------
def gla_decode(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    g: Optional[torch.Tensor],
    state: torch.Tensor,
    slot_idx: torch.Tensor,
    scale: Optional[float] = None,
    out: Optional[torch.Tensor] = None,
    gate_mode: int = _C.GATE_NONE,
    lower_bound: Optional[torch.Tensor] = None,
    gate_normalizer: float = 16.0,
    gate_clamp: float = 0.95,
    out_norm_weight: Optional[torch.Tensor] = None,
    out_norm_eps: float = 1e-6,
    g_w1: Optional[torch.Tensor] = None,
    g_bias: Optional[torch.Tensor] = None,
    qkv_partials: Optional["PartialSums"] = None,
    qkv_cols: Optional[tuple] = None,
    g_w0: Optional[torch.Tensor] = None,
) -> torch.Tensor:
    """q [B,H,D]; k, v, g [B,Hkv,D]; state [slots,H,D,D] (one state per query head, the reference's
    layout) or [slots,Hkv,D,D] (one per key/value head; any gate but the 70B lower-bound one), updated
    in place; slot_idx [B] int32.

    Low-rank gate (7B): with ``g_w1`` bf16 [Hkv*D, 16] (and ``g_bias`` bf16 [Hkv*D]) ``g`` is the rank-16 input
    bf16 [B, 16] and the kernel applies the second linear of the gate projection itself.  With ``g_w0`` bf16
    [16, hidden] as well, ``g`` is the layer input bf16 [B, hidden] and the kernel applies both linears (state per
    key/value head only).

    ``qkv_partials`` (``PartialSums`` of the fused qkv projection) with ``qkv_cols = (q_col, k_col, v_col, g_col)``:
    q, k, v and the rank-16 gate input are read from the partial sums (the projection's reduce launch is skipped); then
    ``q`` / ``k`` / ``v`` / ``g`` are given as shapes only: ``(B, H, D)``, ``(B, Hkv, D)``, ``(B, Hkv, D)``, None.
    With ``g_w0`` as well (a quantised projection carries no rank columns; its partial sums may be the int32 ones of a
    W8A8 linear) ``g`` is the layer input bf16 [B, hidden] and ``g_col`` is unused; state per key/value head only.

    Returns out [B,H,D] bf16 (rows of skipped sequences, slot -1, are left as they were).
    """
    if qkv_partials is not None:
        return _gla_decode_from_partials(q, k, qkv_partials, qkv_cols, state, slot_idx, scale, out, gate_mode, gate_normalizer,
                                         gate_clamp, out_norm_weight, out_norm_eps, g_w1, g_bias, g, g_w0)
    _dev(q, k, v, g, state, slot_idx, lower_bound, out_norm_weight)
    B, H, D = q.shape
    Hkv = k.shape[1]
    _require(q.dtype == torch.bfloat16 and k.dtype == torch.bfloat16 and v.dtype == torch.bfloat16,
             "q, k, v must be bfloat16")
    _require(k.shape == (B, Hkv, D) and v.shape == (B, Hkv, D), "k, v must be [B, Hkv, D]")
    if g_w1 is not None:
        _dev(g_w1, g_bias, g_w0)
        width = 16 if g_w0 is None else g_w0.shape[1]
        _require(g_w0 is None or (g_w0.dtype == torch.bfloat16 and g_w0.is_contiguous() and g_w0.dim() == 2 and g_w0.shape[0] == 16
                                  and width % 8 == 0 and state.shape[1] == Hkv != H),
                 "g_w0 must be contiguous bf16 [16, hidden], with a state per key/value head")
        _require(g is not None and g.shape == (B, width) and g.dtype == torch.bfloat16 and g.stride(1) == 1 and g.stride(0) % 8 == 0,
                 "low-rank gate: g must be bf16 [B, 16] (or [B, hidden] with g_w0) with rows a multiple of 8 elements apart")
        _require(g_w1.dtype == torch.bfloat16 and g_w1.is_contiguous() and g_w1.shape == (Hkv * D, 16), "g_w1 must be contiguous bf16 [Hkv*D, 16]")
        _require(g_bias is None or (g_bias.dtype == torch.bfloat16 and g_bias.is_contiguous() and g_bias.numel() == Hkv * D),
                 "g_bias must be contiguous bf16 [Hkv*D]")
    else:
        _require(g_w0 is None, "g_w0 needs g_w1")
        _require(g is None or g.shape == (B, Hkv, D), "g must be [B, Hkv, D]")
    _require(state.dim() == 4 and state.shape[2:] == (D, D) and state.shape[1] in (H, Hkv),
             "state must be [slots, H, D, D] or [slots, Hkv, D, D]")
    _require(state.shape[1] == H or gate_mode != _C.GATE_70B_LOWER_BOUND,
             "the lower-bound gate depends on the query head: the state must be per query head")
    _require(state.stride(3) == 1 and state.stride(2) == D, "state (Dk, Dv) blocks must be contiguous")
    _require(state.dtype in _DT, "state must be bfloat16 or float32")
    _require(slot_idx.dtype == torch.int32 and slot_idx.shape == (B,) and slot_idx.is_contiguous(),
             "slot_idx must be contiguous int32 [B]")
    for name, t in (("q", q), ("k", k), ("v", v), ("g", g)):
        if t is not None:
            _inner_contig(t, name)
    if out is None:
        out = torch.empty(B, H, D, dtype=torch.bfloat16, device=q.device)
    _require(out.shape == (B, H, D) and out.dtype == torch.bfloat16 and out.stride(-1) == 1,
             "out must be bf16 [B, H, D]")
    if lower_bound is not None:
        _require(lower_bound.dtype == torch.float32 and lower_bound.is_contiguous()
                 and lower_bound.numel() == H * D, "lower_bound must be contiguous fp32 [H*D]")
    if out_norm_weight is not None:
        _require(out_norm_weight.dtype == torch.bfloat16 and out_norm_weight.is_contiguous()
                 and out_norm_weight.numel() == D, "out_norm_weight must be contiguous bf16 [D]")
    a = _C.GlaDecodeArgs()
    a.q, a.k, a.v, a.g, a.out, a.state = _p(q), _p(k), _p(v), _p(g), _p(out), _p(state)
    a.slot_idx, a.lower_bound, a.out_norm_weight = _p(slot_idx), _p(lower_bound), _p(out_norm_weight)
    a.batch, a.num_heads, a.num_kv_heads, a.head_dim = B, H, Hkv, D
    a.q_stride_b, a.q_stride_h = q.stride(0), q.stride(1)
    a.k_stride_b, a.k_stride_h = k.stride(0), k.stride(1)
    a.v_stride_b, a.v_stride_h = v.stride(0), v.stride(1)
    if g is not None:
        a.g_stride_b, a.g_stride_h = g.stride(0), g.stride(1)
        _require(g.dtype in _DT, "g must be bfloat16 or float32")
        a.g_dtype = _DT[g.dtype]
    a.g_w1, a.g_bias = _p(g_w1), _p(g_bias)
    if g_w0 is not None:
        a.g_w0, a.g_hidden = _p(g_w0), g_w0.shape[1]
    a.out_stride_b, a.out_stride_h = out.stride(0), out.stride(1)
    a.state_stride_slot, a.state_stride_h = state.stride(0), state.stride(1)
    a.state_dtype = _DT[state.dtype]
    a.state_heads = state.shape[1]
    a.gate_mode = gate_mode
    a.scale = float(scale) if scale is not None else 0.0
    a.gate_normalizer, a.gate_clamp, a.out_norm_eps = gate_normalizer, gate_clamp, out_norm_eps
    _C.check(_C.load().hymeta_gla_decode(C.byref(a), _stream(q)), "hymeta_gla_decode")
    return out


def _gla_decode_from_partials(q_shape, k_shape, partials, cols, state, slot_idx, scale, out, gate_mode, gate_normalizer,
                              gate_clamp, out_norm_weight, out_norm_eps, g_w1, g_bias, g=None, g_w0=None) -> torch.Tensor:
    partials.check_live()
    B, H, D = q_shape
    Hkv = k_shape[1]
    _dev(state, slot_idx, out_norm_weight, g_w1, g_bias, out, g, g_w0)
    _require(partials.shape[0] == B, "partial sums must be slabs of B rows")
    _require(not partials.desc.is_int32 or state.shape[1] == Hkv != H, "int32 partial sums: state per key/value head only")
    if g_w0 is not None:
        _require(g_w0.dtype == torch.bfloat16 and g_w0.is_contiguous() and g_w0.dim() == 2 and g_w0.shape[0] == 16
                 and g_w0.shape[1] % 8 == 0 and state.shape[1] == Hkv != H,
                 "g_w0 must be contiguous bf16 [16, hidden], with a state per key/value head")
        _require(g is not None and g.shape == (B, g_w0.shape[1]) and g.dtype == torch.bfloat16 and g.stride(1) == 1 and g.stride(0) % 8 == 0,
                 "with g_w0, g must be the layer input bf16 [B, hidden] with rows a multiple of 8 elements apart")
    else:
        _require(g is None, "partial-sum inputs carry the rank-16 gate input themselves (or give g_w0 and the layer input)")
    _require(gate_mode == _C.GATE_7B and g_w1 is not None, "partial-sum inputs are wired for the 7B low-rank gate")
    _require(g_w1.dtype == torch.bfloat16 and g_w1.is_contiguous() and g_w1.shape == (Hkv * D, 16), "g_w1 must be contiguous bf16 [Hkv*D, 16]")
    _require(g_bias is None or (g_bias.dtype == torch.bfloat16 and g_bias.is_contiguous() and g_bias.numel() == Hkv * D),
             "g_bias must be contiguous bf16 [Hkv*D]")
    _require(state.dim() == 4 and state.shape[2:] == (D, D) and state.shape[1] in (H, Hkv) and state.stride(3) == 1
             and state.stride(2) == D and state.dtype in _DT, "state must be [slots, H | Hkv, D, D] with contiguous blocks")
    _require(slot_idx.dtype == torch.int32 and slot_idx.shape == (B,) and slot_idx.is_contiguous(), "slot_idx must be contiguous int32 [B]")
    if out is None:
        out = torch.empty(B, H, D, dtype=torch.bfloat16, device=partials.device)
    _require(out.shape == (B, H, D) and out.dtype == torch.bfloat16 and out.stride(-1) == 1, "out must be bf16 [B, H, D]")
    if out_norm_weight is not None:
        _require(out_norm_weight.dtype == torch.bfloat16 and out_norm_weight.is_contiguous() and out_norm_weight.numel() == D,
                 "out_norm_weight must be contiguous bf16 [D]")
    a = _C.GlaDecodeArgs()
    a.out, a.state, a.slot_idx, a.out_norm_weight = _p(out), _p(state), _p(slot_idx), _p(out_norm_weight)
    a.batch, a.num_heads, a.num_kv_heads, a.head_dim = B, H, Hkv, D
    a.out_stride_b, a.out_stride_h = out.stride(0), out.stride(1)
    a.state_stride_slot, a.state_stride_h = state.stride(0), state.stride(1)
    a.state_dtype, a.g_dtype = _DT[state.dtype], _C.HYMETA_BF16
    a.state_heads = state.shape[1]
    a.gate_mode = gate_mode
    a.scale = float(scale) if scale is not None else 0.0
    a.gate_normalizer, a.gate_clamp, a.out_norm_eps = gate_normalizer, gate_clamp, out_norm_eps
    a.g_w1, a.g_bias = _p(g_w1), _p(g_bias)
    d = partials.desc
    a.qkv_slabs, a.qkv_bias, a.qkv_splits, a.qkv_n = d.slabs, d.bias, d.splits, d.N
    if d.is_int32:
        a.qkv_x_scale, a.qkv_w_scale = d.x_scale, d.w_scale
    a.q_col, a.k_col, a.v_col, a.g_col = (int(c) for c in cols)
    if g_w0 is not None:
        a.g, a.g_stride_b, a.g_w0, a.g_hidden = _p(g), g.stride(0), _p(g_w0), g_w0.shape[1]
    _C.check(_C.load().hymeta_gla_decode(C.byref(a), _stream(out)), "hymeta_gla_decode")
    return out


# ---------------------------------------------------------------------------
# GLA varlen prefill
# ---------------------------------------------------------------------------
def gla_prefill_varlen(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    g: Optional[torch.Tensor],
    state: torch.Tensor,
    slot_idx: torch.Tensor,
    cu_seqlens: torch.Tensor,
    max_seqlen: int,
    context_lens: Optional[torch.Tensor] = None,
    meta_state: Optional[torch.Tensor] = None,
    scale: Optional[float] = None,
    out: Optional[torch.Tensor] = None,
    gate_mode: int = _C.GATE_NONE,
    lower_bound: Optional[torch.Tensor] = None,
    gate_normalizer: float = 16.0,
    gate_clamp: float = 0.95,
    out_norm_weight: Optional[torch.Tensor] = None,
    out_norm_eps: float = 1e-6,
    num_segments: int = 0,
) -> torch.Tensor:
    """q [T,H,D]; k, v, g [T,Hkv,D]; cu_seqlens int32 [nseq+1]; state [slots,H,D,D] or [slots,Hkv,D,D]
    (see gla_decode) updated in place.
    ``num_segments``: 0 lets the library decide whether to cut long sequences into parallel runs,
    1 forces a single run per (sequence, head), >1 forces that many."""
    _dev(q, k, v, g, state, slot_idx, cu_seqlens, context_lens, meta_state, lower_bound, out_norm_weight)
    T, H, D = q.shape
    Hkv = k.shape[1]
    nseq = cu_seqlens.numel() - 1
    _require(q.dtype == torch.bfloat16 and k.dtype == torch.bfloat16 and v.dtype == torch.bfloat16,
             "q, k, v must be bfloat16")
    _require(k.shape == (T, Hkv, D) and v.shape == (T, Hkv, D), "k, v must be [T, Hkv, D]")
    _require(g is None or g.shape == (T, Hkv, D), "g must be [T, Hkv, D]")
    _require(state.dim() == 4 and state.shape[2:] == (D, D) and state.shape[1] in (H, Hkv),
             "state must be [slots, H, D, D] or [slots, Hkv, D, D]")
    SH = state.shape[1]
    _require(SH == H or gate_mode != _C.GATE_70B_LOWER_BOUND,
             "the lower-bound gate depends on the query head: the state must be per query head")
    _require(state.stride(3) == 1 and state.stride(2) == D, "state (Dk, Dv) blocks must be contiguous")
    _require(state.dtype in _DT, "state must be bfloat16 or float32")
    for name, t, n in (("slot_idx", slot_idx, nseq), ("cu_seqlens", cu_seqlens, nseq + 1),
                       ("context_lens", context_lens, nseq)):
        if t is not None:
            _require(t.dtype == torch.int32 and t.is_contiguous() and t.numel() == n,
                     f"{name} must be contiguous int32 [{n}]")
    for name, t in (("q", q), ("k", k), ("v", v), ("g", g)):
        if t is not None:
            _inner_contig(t, name)
    if meta_state is not None:
        _require(meta_state.shape == (SH, D, D) and meta_state.dtype == state.dtype
                 and meta_state.stride(2) == 1 and meta_state.stride(1) == D,
                 "meta_state must be [state heads, D, D] in the state dtype with contiguous blocks")
    if out is None:
        out = torch.empty(T, H, D, dtype=torch.bfloat16, device=q.device)
    _require(out.shape == (T, H, D) and out.dtype == torch.bfloat16 and out.stride(-1) == 1,
             "out must be bf16 [T, H, D]")
    a = _C.GlaPrefillArgs()
    a.q, a.k, a.v, a.g, a.out, a.state = _p(q), _p(k), _p(v), _p(g), _p(out), _p(state)
    a.slot_idx, a.cu_seqlens, a.context_lens = _p(slot_idx), _p(cu_seqlens), _p(context_lens)
    a.meta_state, a.lower_bound, a.out_norm_weight = _p(meta_state), _p(lower_bound), _p(out_norm_weight)
    a.num_seqs, a.total_tokens, a.max_seqlen = nseq, T, int(max_seqlen)
    a.num_heads, a.num_kv_heads, a.head_dim = H, Hkv, D
    a.q_stride_t, a.q_stride_h = q.stride(0), q.stride(1)
    a.k_stride_t, a.k_stride_h = k.stride(0), k.stride(1)
    a.v_stride_t, a.v_stride_h = v.stride(0), v.stride(1)
    if g is not None:
        _require(g.dtype in _DT, "g must be bfloat16 or float32")
        a.g_stride_t, a.g_stride_h = g.stride(0), g.stride(1)
        a.g_dtype = _DT[g.dtype]
    a.out_stride_t, a.out_stride_h = out.stride(0), out.stride(1)
    a.state_stride_slot, a.state_stride_h = state.stride(0), state.stride(1)
    if meta_state is not None:
        a.meta_state_stride_h = meta_state.stride(0)
    a.state_dtype = _DT[state.dtype]
    a.state_heads = SH
    a.gate_mode = gate_mode
    a.scale = float(scale) if scale is not None else 0.0
    a.gate_normalizer, a.gate_clamp, a.out_norm_eps = gate_normalizer, gate_clamp, out_norm_eps
    lib = _C.load()
    nseg = int(num_segments)
    if nseg == 0:
        nseg = int(lib.hymeta_gla_prefill_segments(nseq, SH, int(max_seqlen)))   # SH: heads that run as workgroups
    nseg = max(1, min(nseg, (int(max_seqlen) + 31) // 32))
    a.num_segments = nseg
    nbytes = int(lib.hymeta_gla_prefill_workspace_bytes(nseq, H, SH, nseg))
    if nbytes:
        ws = _workspace(q.device, nbytes, "gla_prefill")
        a.workspace, a.workspace_bytes = _p(ws), nbytes
    _C.check(lib.hymeta_gla_prefill_varlen(C.byref(a), _stream(q)), "hymeta_gla_prefill_varlen")
    return out


# ---------------------------------------------------------------------------
# Paged KV write
# ---------------------------------------------------------------------------
def reshape_and_cache(
    key: torch.Tensor,
    value: torch.Tensor,
    key_cache: torch.Tensor,
    value_cache: torch.Tensor,
    slot_mapping: torch.Tensor,
) -> None:
    """key/value [T,Hkv,D] -> caches [nblk,bs,Hkv,D] at slot_mapping [<=T] int64 (negative: skip)."""
    _dev(key, value, key_cache, value_cache, slot_mapping)
    _require(key.dtype == value.dtype == key_cache.dtype == value_cache.dtype,
             "key, value and both caches must share a dtype (kv_cache_dtype 'auto')")
    _require(key_cache.shape == value_cache.shape and key_cache.stride() == value_cache.stride(),
             "key and value caches must have identical layout")
    nblk, bs, Hkv, D = key_cache.shape
    _require(key.shape[1:] == (Hkv, D) and value.shape == key.shape, "key/value must be [T, Hkv, D]")
    _require(slot_mapping.dtype == torch.int64 and slot_mapping.is_contiguous(), "slot_mapping must be int64")
    n = slot_mapping.numel()
    _require(n <= key.shape[0], "slot_mapping longer than key")
    for name, t in (("key", key), ("value", value), ("key_cache", key_cache)):
        _inner_contig(t, name)
    a = _C.ReshapeAndCacheArgs()
    a.key, a.value, a.key_cache, a.value_cache = _p(key), _p(value), _p(key_cache), _p(value_cache)
    a.slot_mapping = _p(slot_mapping)
    a.num_tokens, a.num_kv_heads, a.head_dim, a.block_size = n, Hkv, D, bs
    a.elem_bytes = key.element_size()
    a.num_blocks = nblk
    a.key_stride_t, a.key_stride_h = key.stride(0), key.stride(1)
    a.value_stride_t, a.value_stride_h = value.stride(0), value.stride(1)
    a.cache_stride_block, a.cache_stride_pos, a.cache_stride_h = (
        key_cache.stride(0), key_cache.stride(1), key_cache.stride(2))
    _C.check(_C.load().hymeta_reshape_and_cache(C.byref(a), _stream(key)), "hymeta_reshape_and_cache")


# ---------------------------------------------------------------------------
# Paged decode attention (sliding window + meta keys)
# ---------------------------------------------------------------------------
_workspaces = {}
_retired = []
_TICKETED = ("gptq_gemm", "bf16_gemm", "w8a8_gemm", "moe_router")     # workspaces that start with split-K ticket counters


class _Workspace:
    __slots__ = ("buf", "eager_clean", "captures", "uses")

    def __init__(self, buf, eager_clean):
        self.buf, self.eager_clean, self.captures, self.uses = buf, eager_clean, set(), 0


def _capture_id(stream) -> int:
    cid = C.c_uint64(0)
    _C.check(_C.load().hymeta_stream_capture_id(C.c_void_p(stream.cuda_stream), C.byref(cid)), "hymeta_stream_capture_id")
    return int(cid.value)


def _workspace(device: torch.device, nbytes: int, tag: str = "paged_decode") -> torch.Tensor:
    """Grow-only scratch per (device, stream, op): split-KV partials, prefill segment states, split-K
    slabs.  Calls on one stream are ordered, so they share; calls of one op on two streams (a shared
    expert beside the routed ones) each get their own, ticket counters included.

    The split-K GEMMs keep ticket counters at the front of theirs, which must be zero when a call starts
    and which every completed call leaves zero.  Eagerly that is one zero fill when the buffer is made.
    Under graph capture a fill recorded once would only run when that graph is replayed, so every
    capture (told apart by its capture id) records its own clearing kernel in front of its first use of a
    ticketed workspace: each replay then starts from zero tickets whatever ran before it, and a buffer
    made during a capture is cleared eagerly before its first eager use."""
    stream = torch.cuda.current_stream(device)
    key = (device, stream.cuda_stream, tag)
    cid = _capture_id(stream) if torch.cuda.is_current_stream_capturing() else 0
    ticketed = tag in _TICKETED
    ws = _workspaces.get(key)
    if ws is None or ws.buf.numel() < nbytes:
        if ws is not None:
            _retired.append(ws.buf)     # a captured HIP graph may still hold its address: never hand it back
        size = max(nbytes, 1 << 20)
        if cid == 0:
            ws = _Workspace(torch.zeros(size, dtype=torch.uint8, device=device) if ticketed
                            else torch.empty(size, dtype=torch.uint8, device=device), True)
        else:
            ws = _Workspace(torch.empty(size, dtype=torch.uint8, device=device), False)
        _workspaces[key] = ws
    if ticketed:
        if cid != 0 and cid not in ws.captures:
            ws.buf[: _C.GEMM_TICKET_BYTES].zero_()      # a fill kernel node of this graph (no memset node)
            ws.captures.add(cid)
        elif cid == 0 and not ws.eager_clean:
            ws.buf[: _C.GEMM_TICKET_BYTES].zero_()
            ws.eager_clean = True
    ws.uses += 1
    return ws.buf


class PartialSums:
    """Result of a K-sliced linear whose slice sum is left to its consumer (``bf16_gemm`` / ``w8a8_gemm`` with
    ``defer=True``): ``add_rmsnorm`` takes it in place of ``x`` and adds the slices while it reads them, ``tensor()``
    runs the linear's own reduce launch.  The partial sums live in the linear's workspace: they must be consumed
    before the next linear of that kind on the stream (checked)."""

    def __init__(self, desc, shape, device, key, keep):
        self.desc, self.shape, self.device = desc, shape, device
        self._key, self._keep = key, keep            # keep: tensors the descriptor points into
        self._uses = _workspaces[key].uses

    def check_live(self) -> None:
        ws = _workspaces.get(self._key)
        _require(ws is not None and ws.uses == self._uses and ws.buf is self._keep[0],
                 "partial sums were overwritten: another linear used the workspace before they were consumed")

    def tensor(self, out: Optional[torch.Tensor] = None) -> torch.Tensor:
        self.check_live()
        M, N = self.shape
        if out is None:
            out = torch.empty(M, N, dtype=torch.bfloat16, device=self.device)
        _require(out.shape == (M, N) and out.dtype == torch.bfloat16 and out.stride(1) == 1, "out must be bf16 [M, N]")
        _C.check(_C.load().hymeta_gemm_partials_reduce(C.byref(self.desc), _p(out), out.stride(0),
                                                       C.c_void_p(torch.cuda.current_stream(self.device).cuda_stream)),
                 "hymeta_gemm_partials_reduce")
        return out


def _partials(desc, M, N, device, tag, *keep):
    stream = torch.cuda.current_stream(device)
    key = (device, stream.cuda_stream, tag)
    return PartialSums(desc, (M, N), device, key, (_workspaces[key].buf,) + keep)


def reset_workspace_tickets(device: Optional[torch.device] = None) -> None:
    """Zero the ticket counters of every split-K workspace (of ``device``): the recovery step after a launch
    that failed or was aborted midway, which may leave tickets drawn."""
    for (dev, _, tag), ws in _workspaces.items():
        if tag in _TICKETED and (device is None or dev == torch.device(device)):
            ws.buf[: _C.GEMM_TICKET_BYTES].zero_()


def paged_decode_splits(batch: int, num_kv_heads: int, max_seqlen_k: int, window_left: int,
                        num_meta: int) -> int:
    return int(_C.load().hymeta_meta_swa_paged_decode_splits(batch, num_kv_heads, max_seqlen_k,
                                                             window_left, num_meta))


def meta_swa_paged_decode(
    q: torch.Tensor,
    key_cache: torch.Tensor,
    value_cache: torch.Tensor,
    cache_seqlens: torch.Tensor,
    block_tables: torch.Tensor,
    meta_key: Optional[torch.Tensor] = None,
    meta_value: Optional[torch.Tensor] = None,
    window_left: int = -1,
    scale: Optional[float] = None,
    max_seqlen_k: int = 0,
    num_splits: int = 0,
    out: Optional[torch.Tensor] = None,
    workspace: Optional[torch.Tensor] = None,
    new_key: Optional[torch.Tensor] = None,
    new_value: Optional[torch.Tensor] = None,
    slot_mapping: Optional[torch.Tensor] = None,
    static_scratch: bool = False,
) -> torch.Tensor:
    """q [B,H,D]; caches [nblk,bs,Hkv,D]; cache_seqlens int32 [B]; block_tables int32 [B,maxblk];
    meta_key/meta_value [M,Hkv,D] or None.  Returns out [B,H,D] bf16.
    ``static_scratch``: run ``hymeta_meta_swa_paged_decode_static`` (split-KV partials in the library's
    own fixed device array; no workspace is allocated or passed; pass ``out`` to allocate nothing at all).
    With ``new_key`` / ``new_value`` [B,Hkv,D] and ``slot_mapping`` int64 [B] the call first writes the
    decoded tokens' K/V rows into the cache (the fused form of ``reshape_and_cache`` + decode)."""
    _dev(q, key_cache, value_cache, cache_seqlens, block_tables, meta_key, meta_value, out, workspace,
         new_key, new_value, slot_mapping)
    B, H, D = q.shape
    nblk, bs, Hkv, Dc = key_cache.shape
    _require(q.dtype == torch.bfloat16 and key_cache.dtype == torch.bfloat16
             and value_cache.dtype == torch.bfloat16, "q and the KV cache must be bfloat16")
    _require(Dc == D and value_cache.shape == key_cache.shape
             and value_cache.stride() == key_cache.stride(), "key/value cache layout mismatch")
    _require(cache_seqlens.dtype == torch.int32 and cache_seqlens.is_contiguous()
             and cache_seqlens.numel() == B, "cache_seqlens must be contiguous int32 [B]")
    _require(block_tables.dtype == torch.int32 and block_tables.dim() == 2
             and block_tables.shape[0] == B and block_tables.stride(1) == 1,
             "block_tables must be int32 [B, max_blocks]")
    _inner_contig(q, "q")
    _inner_contig(key_cache, "key_cache")
    M = 0
    if meta_key is not None:
        _require(meta_value is not None and meta_key.shape == meta_value.shape
                 and meta_key.stride() == meta_value.stride(), "meta key/value layout mismatch")
        _require(meta_key.dtype == torch.bfloat16 and meta_key.shape[1:] == (Hkv, D)
                 and meta_key.stride(-1) == 1, "meta_key must be bf16 [M, Hkv, D]")
        M = meta_key.shape[0]
    if out is None:
        out = torch.empty(B, H, D, dtype=torch.bfloat16, device=q.device)
    _require(out.shape == (B, H, D) and out.dtype == torch.bfloat16 and out.stride(-1) == 1,
             "out must be bf16 [B, H, D]")
    max_blocks = block_tables.shape[1]
    if max_seqlen_k <= 0:
        max_seqlen_k = max_blocks * bs
    lib = _C.load()
    if num_splits <= 0:
        num_splits = lib.hymeta_meta_swa_paged_decode_splits(B, Hkv, max_seqlen_k, window_left, M)
    need = 0 if static_scratch else lib.hymeta_meta_swa_paged_decode_workspace_bytes(B, H, D, num_splits)
    if need and (workspace is None or workspace.numel() * workspace.element_size() < need):
        workspace = _workspace(q.device, need)
    a = _C.PagedDecodeArgs()
    a.q, a.out, a.key_cache, a.value_cache = _p(q), _p(out), _p(key_cache), _p(value_cache)
    a.block_tables, a.cache_seqlens = _p(block_tables), _p(cache_seqlens)
    a.meta_key, a.meta_value = _p(meta_key), _p(meta_value)
    a.workspace = _p(workspace) if need else None
    a.workspace_bytes = workspace.numel() * workspace.element_size() if need else 0
    a.batch, a.num_heads, a.num_kv_heads, a.head_dim = B, H, Hkv, D
    a.block_size, a.max_blocks_per_seq, a.num_meta = bs, max_blocks, M
    a.window_left, a.max_seqlen_k, a.num_splits = int(window_left), int(max_seqlen_k), int(num_splits)
    a.q_stride_b, a.q_stride_h = q.stride(0), q.stride(1)
    a.out_stride_b, a.out_stride_h = out.stride(0), out.stride(1)
    if new_key is not None:
        _require(new_value is not None and slot_mapping is not None, "new_key needs new_value and slot_mapping")
        _require(new_key.shape == (B, Hkv, D) and new_value.shape == (B, Hkv, D)
                 and new_key.dtype == torch.bfloat16 and new_value.dtype == torch.bfloat16,
                 "new_key / new_value must be bf16 [B, Hkv, D]")
        _require(slot_mapping.dtype == torch.int64 and slot_mapping.is_contiguous() and slot_mapping.numel() == B,
                 "slot_mapping must be contiguous int64 [B]")
        _inner_contig(new_key, "new_key")
        _inner_contig(new_value, "new_value")
        a.new_key, a.new_value, a.slot_mapping = _p(new_key), _p(new_value), _p(slot_mapping)
        a.new_key_stride_b, a.new_key_stride_h = new_key.stride(0), new_key.stride(1)
        a.new_value_stride_b, a.new_value_stride_h = new_value.stride(0), new_value.stride(1)
    a.cache_stride_block, a.cache_stride_pos, a.cache_stride_h = (
        key_cache.stride(0), key_cache.stride(1), key_cache.stride(2))
    a.block_table_stride = block_tables.stride(0)
    if meta_key is not None:
        a.meta_stride_t, a.meta_stride_h = meta_key.stride(0), meta_key.stride(1)
    a.scale = float(scale) if scale is not None else 0.0
    if static_scratch:
        _C.check(lib.hymeta_meta_swa_paged_decode_static(C.byref(a), _stream(q)), "hymeta_meta_swa_paged_decode_static")
    else:
        _C.check(lib.hymeta_meta_swa_paged_decode(C.byref(a), _stream(q)), "hymeta_meta_swa_paged_decode")
    return out


# ---------------------------------------------------------------------------
# Varlen prefill attention (sliding window + meta keys)
# ---------------------------------------------------------------------------
def meta_swa_prefill(
    q: torch.Tensor,
    cu_seqlens_q: torch.Tensor,
    max_seqlen_q: int,
    key: Optional[torch.Tensor] = None,
    value: Optional[torch.Tensor] = None,
    cu_seqlens_k: Optional[torch.Tensor] = None,
    key_cache: Optional[torch.Tensor] = None,
    value_cache: Optional[torch.Tensor] = None,
    block_tables: Optional[torch.Tensor] = None,
    seq_lens_k: Optional[torch.Tensor] = None,
    meta_query: Optional[torch.Tensor] = None,
    meta_key: Optional[torch.Tensor] = None,
    meta_value: Optional[torch.Tensor] = None,
    window_left: int = -1,
    scale: Optional[float] = None,
    out: Optional[torch.Tensor] = None,
    max_seqlen_k: int = 0,
    num_splits: int = 0,
) -> torch.Tensor:
    """q [T,H,D].  Un-paged keys: key/value [Tk,Hkv,D] + cu_seqlens_k; paged keys: caches +
    block_tables + seq_lens_k.  Returns [(M if meta_query)+T, H, D] bf16, meta rows first.
    ``max_seqlen_k`` (0: unknown) and ``num_splits`` (0: library's choice) steer the key slicing of
    short chunks of long sequences."""
    _dev(q, cu_seqlens_q, key, value, cu_seqlens_k, key_cache, value_cache, block_tables,
         seq_lens_k, meta_query, meta_key, meta_value, out)
    T, H, D = q.shape
    nseq = cu_seqlens_q.numel() - 1
    paged = block_tables is not None
    _require(q.dtype == torch.bfloat16, "q must be bfloat16")
    _inner_contig(q, "q")
    _require(cu_seqlens_q.dtype == torch.int32 and cu_seqlens_q.is_contiguous(), "cu_seqlens_q must be int32")
    a = _C.SwaPrefillArgs()
    if paged:
        _require(key_cache is not None and value_cache is not None and seq_lens_k is not None,
                 "paged prefill needs key_cache, value_cache and seq_lens_k")
        nblk, bs, Hkv, Dc = key_cache.shape
        _require(Dc == D and key_cache.dtype == torch.bfloat16 and value_cache.shape == key_cache.shape
                 and value_cache.stride() == key_cache.stride() and key_cache.stride(-1) == 1,
                 "key/value cache layout mismatch")
        _require(block_tables.dtype == torch.int32 and block_tables.shape[0] == nseq
                 and block_tables.stride(1) == 1, "block_tables must be int32 [nseq, max_blocks]")
        _require(seq_lens_k.dtype == torch.int32 and seq_lens_k.is_contiguous()
                 and seq_lens_k.numel() == nseq, "seq_lens_k must be contiguous int32 [nseq]")
        a.key_cache, a.value_cache = _p(key_cache), _p(value_cache)
        a.block_tables, a.seq_lens_k = _p(block_tables), _p(seq_lens_k)
        a.block_size, a.max_blocks_per_seq = bs, block_tables.shape[1]
        a.cache_stride_block, a.cache_stride_pos, a.cache_stride_h = (
            key_cache.stride(0), key_cache.stride(1), key_cache.stride(2))
        a.block_table_stride = block_tables.stride(0)
    else:
        _require(key is not None and value is not None and cu_seqlens_k is not None,
                 "un-paged prefill needs key, value and cu_seqlens_k")
        Hkv = key.shape[1]
        _require(key.dtype == torch.bfloat16 and value.dtype == torch.bfloat16
                 and key.shape[1:] == (Hkv, D) and value.shape == key.shape, "key/value must be bf16 [Tk, Hkv, D]")
        _inner_contig(key, "key")
        _inner_contig(value, "value")
        _require(cu_seqlens_k.dtype == torch.int32 and cu_seqlens_k.is_contiguous()
                 and cu_seqlens_k.numel() == nseq + 1, "cu_seqlens_k must be contiguous int32 [nseq+1]")
        a.key, a.value, a.cu_seqlens_k = _p(key), _p(value), _p(cu_seqlens_k)
        a.k_stride_t, a.k_stride_h = key.stride(0), key.stride(1)
        a.v_stride_t, a.v_stride_h = value.stride(0), value.stride(1)
    M = 0
    if meta_key is not None:
        _require(meta_value is not None and meta_key.shape == meta_value.shape
                 and meta_key.stride() == meta_value.stride(), "meta key/value layout mismatch")
        _require(meta_key.dtype == torch.bfloat16 and meta_key.shape[1:] == (Hkv, D)
                 and meta_key.stride(-1) == 1, "meta_key must be bf16 [M, Hkv, D]")
        M = meta_key.shape[0]
        a.meta_key, a.meta_value = _p(meta_key), _p(meta_value)
        a.meta_stride_t, a.meta_stride_h = meta_key.stride(0), meta_key.stride(1)
    rows = T
    if meta_query is not None:
        _require(M > 0 and meta_query.shape == (M, H, D) and meta_query.dtype == torch.bfloat16
                 and meta_query.stride(-1) == 1, "meta_query must be bf16 [M, H, D]")
        a.meta_query = _p(meta_query)
        a.meta_q_stride_t, a.meta_q_stride_h = meta_query.stride(0), meta_query.stride(1)
        rows += M
    if out is None:
        out = torch.empty(rows, H, D, dtype=torch.bfloat16, device=q.device)
    _require(out.shape == (rows, H, D) and out.dtype == torch.bfloat16 and out.stride(-1) == 1,
             f"out must be bf16 [{rows}, H, D]")
    a.q, a.cu_seqlens_q, a.out = _p(q), _p(cu_seqlens_q), _p(out)
    a.num_seqs, a.total_q, a.max_seqlen_q = nseq, T, int(max_seqlen_q)
    a.num_heads, a.num_kv_heads, a.head_dim = H, Hkv, D
    a.num_meta, a.window_left = M, int(window_left)
    a.q_stride_t, a.q_stride_h = q.stride(0), q.stride(1)
    a.out_stride_t, a.out_stride_h = out.stride(0), out.stride(1)
    a.scale = float(scale) if scale is not None else 0.0
    lib = _C.load()
    a.max_seqlen_k = max(int(max_seqlen_k), 0)
    splits = int(num_splits) if num_splits > 0 else int(lib.hymeta_meta_swa_prefill_splits(
        T, H, M, M if meta_query is not None else 0, int(window_left), a.max_seqlen_k))
    a.num_splits = splits
    if splits > 1:
        ws = _workspace(q.device, int(lib.hymeta_meta_swa_prefill_workspace_bytes(rows, H, splits)), "swa_prefill")
        a.workspace, a.workspace_bytes = _p(ws), ws.numel()
    _C.check(lib.hymeta_meta_swa_prefill(C.byref(a), _stream(q)), "hymeta_meta_swa_prefill")
    return out


# ---------------------------------------------------------------------------
# Layer glue: rotary embedding and the 70B two-branch norm combine
# ---------------------------------------------------------------------------
def rope_neox_(positions: torch.Tensor, q: torch.Tensor, k: Optional[torch.Tensor],
               cos_sin_cache: torch.Tensor, position_offset: int = 0) -> None:
    """In-place NeoX rotary embedding.  positions int64 [T]; q [T,H,D]; k [T,Hkv,D] or None;
    cos_sin_cache bf16 [max_pos, D] (cos | sin)."""
    _dev(positions, q, k, cos_sin_cache)
    T, H, D = q.shape
    _require(q.dtype == torch.bfloat16 and (k is None or k.dtype == torch.bfloat16), "q, k must be bfloat16")
    _require(positions.dtype == torch.int64 and positions.is_contiguous() and positions.numel() == T,
             "positions must be contiguous int64 [T]")
    _require(cos_sin_cache.dtype == torch.bfloat16 and cos_sin_cache.is_contiguous()
             and cos_sin_cache.shape[1] == D, "cos_sin_cache must be contiguous bf16 [max_pos, D]")
    _inner_contig(q, "q")
    a = _C.RopeArgs()
    a.q, a.positions, a.cos_sin_cache = _p(q), _p(positions), _p(cos_sin_cache)
    a.num_tokens, a.num_heads, a.head_dim, a.rot_dim = T, H, D, D
    a.max_position = cos_sin_cache.shape[0]
    a.position_offset = int(position_offset)
    a.q_stride_t, a.q_stride_h = q.stride(0), q.stride(1)
    if k is not None:
        _require(k.shape[0] == T and k.shape[2] == D, "k must be [T, Hkv, D]")
        _inner_contig(k, "k")
        a.k, a.num_kv_heads = _p(k), k.shape[1]
        a.k_stride_t, a.k_stride_h = k.stride(0), k.stride(1)
    _C.check(_C.load().hymeta_rope_neox(C.byref(a), _stream(q)), "hymeta_rope_neox")


def rope_from_partials(partials: "PartialSums", positions: torch.Tensor, cos_sin_cache: torch.Tensor, num_heads: int,
                       num_kv_heads: int, position_offset: int = 0) -> torch.Tensor:
    """The fused qkv projection finished from its K slices' partial sums with NeoX RoPE on the q and k heads: returns
    the projection's bf16 ``[T, N]`` output (q heads, k heads, then v and whatever rides behind), the bits of the plain
    linear followed by ``rope_neox_`` in one launch instead of two."""
    partials.check_live()
    T, N = partials.shape
    D = cos_sin_cache.shape[1]
    _dev(positions, cos_sin_cache)
    _require(positions.dtype == torch.int64 and positions.is_contiguous() and positions.numel() == T,
             "positions must be contiguous int64 [T]")
    _require(cos_sin_cache.dtype == torch.bfloat16 and cos_sin_cache.is_contiguous(), "cos_sin_cache must be contiguous bf16 [max_pos, D]")
    _require((num_heads + 2 * num_kv_heads) * D <= N, "the projection is narrower than its q, k and v heads")
    out = torch.empty(T, N, dtype=torch.bfloat16, device=partials.device)
    a = _C.RopeArgs()
    a.q, a.positions, a.cos_sin_cache = _p(out), _p(positions), _p(cos_sin_cache)
    a.num_tokens, a.num_heads, a.num_kv_heads, a.head_dim, a.rot_dim = T, num_heads, num_kv_heads, D, D
    a.max_position = cos_sin_cache.shape[0]
    a.position_offset = int(position_offset)
    a.q_stride_t, a.q_stride_h = N, D
    _C.check(_C.load().hymeta_rope_neox_partials(C.byref(a), C.byref(partials.desc), _stream(out)), "hymeta_rope_neox_partials")
    return out


def _combine_args(o_attn, o_lin, weight1, weight2, stats, out, eps):
    T, Hd = o_attn.shape
    _require(o_lin.shape == (T, Hd) and o_attn.dtype == torch.bfloat16 and o_lin.dtype == torch.bfloat16,
             "o_attn, o_lin must be bf16 [T, hidden_local]")
    _require(o_attn.stride(1) == 1 and o_lin.stride(1) == 1, "branch outputs must be row-contiguous")
    a = _C.CombineArgs()
    a.o_attn, a.o_lin, a.stats, a.out = _p(o_attn), _p(o_lin), _p(stats), _p(out)
    a.weight1, a.weight2 = _p(weight1), _p(weight2)
    a.num_tokens, a.hidden_local = T, Hd
    a.attn_stride_t, a.lin_stride_t = o_attn.stride(0), o_lin.stride(0)
    if out is not None:
        a.out_stride_t = out.stride(0)
    a.eps = eps
    return a


def rms_sumsq2(o_attn: torch.Tensor, o_lin: torch.Tensor) -> torch.Tensor:
    """Local mean of squares of both branches: fp32 [T, 2] (all-reduce it, divide by tp)."""
    _dev(o_attn, o_lin)
    stats = torch.empty(o_attn.shape[0], 2, dtype=torch.float32, device=o_attn.device)
    a = _combine_args(o_attn, o_lin, None, None, stats, None, 0.0)
    _C.check(_C.load().hymeta_rms_sumsq2(C.byref(a), _stream(o_attn)), "hymeta_rms_sumsq2")
    return stats


def hybrid_combine(o_attn: torch.Tensor, o_lin: torch.Tensor, weight1: torch.Tensor, weight2: torch.Tensor,
                   eps: float = 1e-6, stats: Optional[torch.Tensor] = None,
                   out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """bf16((RMSNorm1(o_attn) + RMSNorm2(o_lin)) / 2); ``stats`` = all-reduced mean squares or None (tp=1)."""
    _dev(o_attn, o_lin, weight1, weight2, stats, out)
    for w in (weight1, weight2):
        _require(w.dtype == torch.float32 and w.is_contiguous() and w.numel() == o_attn.shape[1],
                 "norm weights must be contiguous fp32 [hidden_local]")
    if stats is not None:
        _require(stats.dtype == torch.float32 and stats.is_contiguous() and stats.shape == (o_attn.shape[0], 2),
                 "stats must be contiguous fp32 [T, 2]")
    if out is None:
        out = torch.empty_like(o_attn)
    a = _combine_args(o_attn, o_lin, weight1, weight2, stats, out, eps)
    _C.check(_C.load().hymeta_hybrid_combine(C.byref(a), _stream(o_attn)), "hymeta_hybrid_combine")
    return out


INT8_ROWS_ATTR = "_hymeta_int8_rows"


def int8_rows_of(x: torch.Tensor):
    """``(xq int8 [T, K], x_scale fp32 [T])`` a producer attached to exactly this tensor object (``add_rmsnorm(...,
    int8=True)``), or None.  A view or copy of the tensor does not carry them."""
    return getattr(x, INT8_ROWS_ATTR, None)


def add_rmsnorm(x: torch.Tensor, weight: torch.Tensor, eps: float = 1e-6, residual: Optional[torch.Tensor] = None,
                out: Optional[torch.Tensor] = None, int8: bool = False) -> torch.Tensor:
    """RMS norm of the decoder blocks.  With ``residual``: residual <- bf16(x + residual) in place
    and the norm is taken of that sum (the blocks' ``mlp_norm(hidden, residual)`` call).  ``x`` may be the
    ``PartialSums`` of a K-sliced linear (needs ``residual``): the slices are added as the input is read.

    ``int8``: the launch also writes the dynamic per-token int8 quantisation of its output (the bits ``w8a8_quantize``
    gives) and attaches ``(xq, x_scale)`` to the returned tensor (``int8_rows_of``); a W8A8 linear called on that very
    tensor skips its own quantise launch."""
    if isinstance(x, PartialSums):
        x.check_live()
        M, N = x.shape
        _dev(weight, residual, out)
        _require(residual is not None and residual.shape == (M, N) and residual.dtype == torch.bfloat16 and residual.stride(1) == 1,
                 "partial sums need a row-contiguous bf16 residual [T, hidden]")
        _require(weight.dtype == torch.bfloat16 and weight.is_contiguous() and weight.numel() == N, "weight must be contiguous bf16 [hidden]")
        if out is None:
            out = torch.empty(M, N, dtype=torch.bfloat16, device=residual.device)
        _require(out.shape == (M, N) and out.dtype == torch.bfloat16 and out.stride(1) == 1, "out must be row-contiguous bf16 [T, hidden]")
        a = _C.AddRmsNormArgs(x=None, residual=residual.data_ptr(), weight=weight.data_ptr(), out=out.data_ptr(), num_tokens=M,
                              hidden=N, x_stride_t=0, residual_stride_t=residual.stride(0), out_stride_t=out.stride(0), eps=eps)
        if int8:
            xq = torch.empty(M, N, dtype=torch.int8, device=out.device)
            xs = torch.empty(M, dtype=torch.float32, device=out.device)
            _C.check(_C.load().hymeta_add_rmsnorm_int8(C.byref(a), C.byref(x.desc), _p(xq), _p(xs), _stream(residual)),
                     "hymeta_add_rmsnorm_int8")
            setattr(out, INT8_ROWS_ATTR, (xq, xs))
            return out
        _C.check(_C.load().hymeta_add_rmsnorm_partials(C.byref(a), C.byref(x.desc), _stream(residual)), "hymeta_add_rmsnorm_partials")
        return out
    _dev(x, weight, residual, out)
    _require(x.dim() == 2 and x.dtype == torch.bfloat16 and x.stride(1) == 1, "x must be row-contiguous bf16 [T, hidden]")
    _require(weight.dtype == torch.bfloat16 and weight.is_contiguous() and weight.numel() == x.shape[1],
             "weight must be contiguous bf16 [hidden]")
    if residual is not None:
        _require(residual.shape == x.shape and residual.dtype == torch.bfloat16 and residual.stride(1) == 1,
                 "residual must be row-contiguous bf16 [T, hidden]")
    if out is None:
        out = torch.empty_like(x)
    _require(out.shape == x.shape and out.dtype == torch.bfloat16 and out.stride(1) == 1, "out must be row-contiguous bf16 [T, hidden]")
    a = _C.AddRmsNormArgs(x=x.data_ptr(), residual=residual.data_ptr() if residual is not None else None,
                          weight=weight.data_ptr(), out=out.data_ptr(), num_tokens=x.shape[0], hidden=x.shape[1],
                          x_stride_t=x.stride(0), residual_stride_t=residual.stride(0) if residual is not None else 0,
                          out_stride_t=out.stride(0), eps=eps)
    if int8:
        xq = torch.empty(x.shape, dtype=torch.int8, device=out.device)
        xs = torch.empty(x.shape[0], dtype=torch.float32, device=out.device)
        _C.check(_C.load().hymeta_add_rmsnorm_int8(C.byref(a), None, _p(xq), _p(xs), _stream(x)), "hymeta_add_rmsnorm_int8")
        setattr(out, INT8_ROWS_ATTR, (xq, xs))
        return out
    _C.check(_C.load().hymeta_add_rmsnorm(C.byref(a), _stream(x)), "hymeta_add_rmsnorm")
    return out


LOWRANK_GATE_ROWS = 256     # above this the two library GEMMs are ahead (w0 is re-read per token here)


def lowrank_gate(x: torch.Tensor, w0: torch.Tensor, w1: torch.Tensor, bias: Optional[torch.Tensor] = None,
                 out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """bf16( bf16(x w0^T) w1^T + bias ): the rank-16 gate projection of the 7B GLA layer in one launch.
    x [T, hidden]; w0 [16, hidden]; w1 [N, 16]; bias [N] -> [T, N]."""
    _dev(x, w0, w1, bias, out)
    T, hidden = x.shape
    N = w1.shape[0]
    _require(x.dtype == torch.bfloat16 and x.stride(1) == 1, "x must be row-contiguous bf16 [T, hidden]")
    _require(w0.dtype == torch.bfloat16 and w0.is_contiguous() and w0.shape == (16, hidden), "w0 must be contiguous bf16 [16, hidden]")
    _require(w1.dtype == torch.bfloat16 and w1.is_contiguous() and w1.shape == (N, 16), "w1 must be contiguous bf16 [N, 16]")
    _require(bias is None or (bias.dtype == torch.bfloat16 and bias.is_contiguous() and bias.numel() == N),
             "bias must be contiguous bf16 [N]")
    if out is None:
        out = torch.empty(T, N, dtype=torch.bfloat16, device=x.device)
    _require(out.shape == (T, N) and out.dtype == torch.bfloat16 and out.stride(1) == 1, "out must be row-contiguous bf16 [T, N]")
    a = _C.LowrankGateArgs(x=x.data_ptr(), w0=w0.data_ptr(), w1=w1.data_ptr(), bias=_p(bias), out=out.data_ptr(),
                           num_tokens=T, hidden=hidden, rank=16, out_features=N,
                           x_stride_t=x.stride(0), out_stride_t=out.stride(0))
    _C.check(_C.load().hymeta_lowrank_gate(C.byref(a), _stream(x)), "hymeta_lowrank_gate")
    return out


# ---------------------------------------------------------------------------
# Quantised linears
# ---------------------------------------------------------------------------
def gptq_gemm(x: torch.Tensor, qweight: torch.Tensor, qzeros: torch.Tensor, scales: torch.Tensor,
              bits: int, group_size: int, bias: Optional[torch.Tensor] = None, zero_offset: int = 1,
              split_k: int = 0, out: Optional[torch.Tensor] = None, defer: bool = False):
    """x bf16 [M,K] @ GPTQ(qweight int32 [K/pack,N], qzeros int32 [K/group,N/pack], scales fp16|bf16
    [K/group,N]) (+ bias bf16 [N]) -> bf16 [M,N]."""
    _dev(x, qweight, qzeros, scales, bias, out)
    M, K = x.shape
    N = qweight.shape[1]
    pack = 32 // bits
    _require(x.dtype == torch.bfloat16 and x.stride(1) == 1, "x must be row-contiguous bf16 [M, K]")
    _require(qweight.dtype == torch.int32 and qweight.is_contiguous() and qweight.shape[0] * pack == K,
             "qweight must be contiguous int32 [K/pack, N]")
    _require(qzeros.dtype == torch.int32 and qzeros.is_contiguous()
             and qzeros.shape == (K // group_size, N // pack), "qzeros must be contiguous int32 [K/group, N/pack]")
    _require(scales.dtype in (torch.float16, torch.bfloat16) and scales.is_contiguous()
             and scales.shape == (K // group_size, N), "scales must be contiguous fp16/bf16 [K/group, N]")
    if bias is not None:
        _require(bias.dtype == torch.bfloat16 and bias.is_contiguous() and bias.numel() == N, "bias must be bf16 [N]")
    if out is None:
        out = torch.empty(M, N, dtype=torch.bfloat16, device=x.device)
    _require(out.shape == (M, N) and out.dtype == torch.bfloat16 and out.stride(1) == 1, "out must be bf16 [M, N]")
    lib = _C.load()
    a = _C.GptqGemmArgs()
    # split_k <= 0: the library chooses how to cut the work; its workspace bound does not depend on K
    need = int(lib.hymeta_gptq_gemm_workspace_bytes(M, N, max(split_k, 0)))
    if need:
        ws = _workspace(x.device, need, "gptq_gemm")
        a.workspace, a.workspace_bytes = _p(ws), ws.numel()
    a.x, a.qweight, a.qzeros, a.scales, a.bias, a.out = _p(x), _p(qweight), _p(qzeros), _p(scales), _p(bias), _p(out)
    a.M, a.K, a.N, a.bits, a.group_size = M, K, N, bits, group_size
    a.scales_dtype = _C.HYMETA_F16 if scales.dtype == torch.float16 else _C.HYMETA_BF16
    a.zero_offset, a.split_k = zero_offset, max(split_k, 0)
    a.x_stride_m, a.out_stride_m = x.stride(0), out.stride(0)
    if defer and a.split_k == 0 and need:
        desc = _C.GemmPartials()
        _C.check(lib.hymeta_gptq_gemm_deferred(C.byref(a), C.byref(desc), _stream(x)), "hymeta_gptq_gemm_deferred")
        return _partials(desc, M, N, x.device, "gptq_gemm", bias) if desc.splits > 0 else out
    _C.check(lib.hymeta_gptq_gemm(C.byref(a), _stream(x)), "hymeta_gptq_gemm")
    return out


def gptq_dequant_nk_supported(qweight: torch.Tensor, bits: int) -> bool:
    """The transposed expansion covers whole 64-column x 32-packed-row tiles."""
    pack = 32 // bits
    return qweight.shape[1] % 64 == 0 and (qweight.shape[0] * pack) % (32 * pack) == 0


def gptq_dequant(qweight: torch.Tensor, qzeros: torch.Tensor, scales: torch.Tensor, bits: int, group_size: int,
                 zero_offset: int = 1, out: Optional[torch.Tensor] = None, transposed: bool = False) -> torch.Tensor:
    """GPTQ tensors -> bf16 weights [K, N] (so that y = x @ W), or with ``transposed`` [N, K] as torch stores a Linear
    weight (so that y = F.linear(x, W)): the layout the library GEMM runs faster at prefill-sized batches."""
    _dev(qweight, qzeros, scales, out)
    pack = 32 // bits
    K, N = qweight.shape[0] * pack, qweight.shape[1]
    _require(qweight.dtype == torch.int32 and qweight.is_contiguous(), "qweight must be contiguous int32 [K/pack, N]")
    _require(qzeros.dtype == torch.int32 and qzeros.is_contiguous() and qzeros.shape == (K // group_size, N // pack),
             "qzeros must be contiguous int32 [K/group, N/pack]")
    _require(scales.dtype in (torch.float16, torch.bfloat16) and scales.is_contiguous()
             and scales.shape == (K // group_size, N), "scales must be contiguous fp16/bf16 [K/group, N]")
    shape = (N, K) if transposed else (K, N)
    if out is None:
        out = torch.empty(shape, dtype=torch.bfloat16, device=qweight.device)
    _require(out.shape == shape and out.dtype == torch.bfloat16 and out.is_contiguous(),
             "out must be contiguous bf16 [K, N] ([N, K] when transposed)")
    sd = _C.HYMETA_F16 if scales.dtype == torch.float16 else _C.HYMETA_BF16
    if transposed:
        _require(gptq_dequant_nk_supported(qweight, bits), "transposed expansion needs N % 64 == 0 and K % (32 * pack) == 0")
        _C.check(_C.load().hymeta_gptq_dequant_nk(_p(qweight), _p(qzeros), _p(scales), _p(out), K, N, bits, group_size, sd,
                                                  zero_offset, _stream(qweight)), "hymeta_gptq_dequant_nk")
        return out
    _C.check(_C.load().hymeta_gptq_dequant(_p(qweight), _p(qzeros), _p(scales), _p(out), K, N, bits, group_size, sd,
                                           zero_offset, _stream(qweight)), "hymeta_gptq_dequant")
    return out


BF16_GEMM_MAX_ROWS = 128      # 65 to 128 rows: the streaming kernel only (K a multiple of 64, at least 256)
BF16_GEMM_TALL_ROWS = 256     # 129 to 256 rows: the shapes the library says it takes (hymeta_bf16_gemm_takes)


def bf16_gemm_preferred(x: torch.Tensor, weight: torch.Tensor) -> bool:
    """Where the kernel is used instead of the library GEMM: every decode-sized shape it takes (measured with
    cold weights on the 7B projections at 1 / 16 / 64 rows: ahead on all of them but the 3584 x 3584 output
    projection at 64 rows, 16 against 14 us)."""
    return bf16_gemm_supported(x, weight)


def bf16_gemm_supported(x: torch.Tensor, weight: torch.Tensor) -> bool:
    """Shapes the bf16 linear kernels take: decode-sized batches, and from 129 to 256 rows what the library's
    129..256-row kernel covers (``hymeta_bf16_gemm_takes``)."""
    if not (x.dim() == 2 and 0 < x.shape[0] <= BF16_GEMM_TALL_ROWS and x.is_cuda and x.dtype == torch.bfloat16
            and weight.dtype == torch.bfloat16 and x.stride(1) == 1 and weight.stride(1) == 1
            and weight.shape[1] % 32 == 0 and weight.shape[0] % 64 == 0
            and (x.shape[0] <= 64 or (weight.shape[1] % 64 == 0 and weight.shape[1] >= 256))
            and x.stride(0) % 8 == 0 and weight.stride(0) % 8 == 0):
        return False
    if x.shape[0] <= BF16_GEMM_MAX_ROWS:
        return True
    return bool(_C.load().hymeta_bf16_gemm_takes(x.shape[0], weight.shape[1], weight.shape[0], 0))


def bf16_gemm(x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor] = None,
              out: Optional[torch.Tensor] = None, split_k: int = 0, defer: bool = False):
    """x bf16 [M, K] @ weight bf16 [N, K]^T (+ bias bf16 [N]) -> bf16 [M, N] for the shapes of ``bf16_gemm_supported``;
    ``split_k`` 0: library's choice.
    ``defer``: when the library cuts K into slices, return their ``PartialSums`` instead of summing them."""
    _dev(x, weight, bias, out)
    M, K = x.shape
    N = weight.shape[0]
    _require(x.dtype == torch.bfloat16 and x.stride(1) == 1, "x must be row-contiguous bf16 [M, K]")
    _require(weight.dtype == torch.bfloat16 and weight.stride(1) == 1 and weight.shape == (N, K),
             "weight must be row-contiguous bf16 [N, K]")
    if bias is not None:
        _require(bias.dtype == torch.bfloat16 and bias.is_contiguous() and bias.numel() == N, "bias must be bf16 [N]")
    if out is None:
        out = torch.empty(M, N, dtype=torch.bfloat16, device=x.device)
    _require(out.shape == (M, N) and out.dtype == torch.bfloat16 and out.stride(1) == 1, "out must be bf16 [M, N]")
    a = _C.Bf16GemmArgs()
    a.x, a.weight, a.bias, a.out = _p(x), _p(weight), _p(bias), _p(out)
    a.M, a.K, a.N = M, K, N
    a.x_stride_m, a.w_stride_n, a.out_stride_m = x.stride(0), weight.stride(0), out.stride(0)
    lib = _C.load()
    a.split_k = max(int(split_k), 0)
    nbytes = int(lib.hymeta_bf16_gemm_workspace_bytes(M, N, a.split_k))
    if nbytes > 0:
        ws = _workspace(x.device, nbytes, "bf16_gemm")
        a.workspace, a.workspace_bytes = _p(ws), ws.numel()
    if defer and a.split_k == 0 and nbytes > 0:
        desc = _C.GemmPartials()
        _C.check(lib.hymeta_bf16_gemm_deferred(C.byref(a), C.byref(desc), _stream(x)), "hymeta_bf16_gemm_deferred")
        return _partials(desc, M, N, x.device, "bf16_gemm", bias) if desc.splits > 0 else out
    _C.check(lib.hymeta_bf16_gemm(C.byref(a), _stream(x)), "hymeta_bf16_gemm")
    return out


def logits_supported(x: torch.Tensor, weight: torch.Tensor) -> bool:
    """Shapes ``bf16_logits`` takes (any number of rows: they go 64 at a time)."""
    return (x.dim() == 2 and x.is_cuda and x.dtype == torch.bfloat16 and weight.dtype == torch.bfloat16 and weight.is_cuda
            and x.stride(1) == 1 and weight.stride(1) == 1 and weight.shape[1] % 64 == 0 and weight.shape[1] >= 256
            and weight.shape[0] % 64 == 0 and x.stride(0) % 8 == 0 and weight.stride(0) % 8 == 0)


def bf16_logits(x: torch.Tensor, weight: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """x bf16 [M, K] @ weight bf16 [N, K]^T -> fp32 [M, N], fp32 accumulation, result not rounded: the logits of a bf16
    lm_head (the fp32 GEMM of the operands widened to fp32, up to the order of the sums).  Rows go through the
    weight-streaming kernels 128 or 256 at a time."""
    _dev(x, weight, out)
    M, K = x.shape
    N = weight.shape[0]
    _require(logits_supported(x, weight) and weight.shape == (N, K), "bf16_logits: x bf16 [M, K], weight bf16 [N, K], K % 64 == 0, N % 64 == 0")
    if out is None:
        out = torch.empty(M, N, dtype=torch.float32, device=x.device)
    _require(out.shape == (M, N) and out.dtype == torch.float32 and out.stride(1) == 1 and out.stride(0) % 4 == 0, "out must be fp32 [M, N]")
    lib = _C.load()
    r0 = 0
    while r0 < M:
        # 256 rows at a time where the 129..256-row kernel takes the matrix (one pass over the weights instead of two)
        rows = min(M - r0, BF16_GEMM_TALL_ROWS)
        if rows > BF16_GEMM_MAX_ROWS and not lib.hymeta_bf16_gemm_takes(rows, K, N, 2):
            rows = BF16_GEMM_MAX_ROWS
        xs, os_ = x[r0:r0 + rows], out[r0:r0 + rows]
        r0 += rows
        a = _C.Bf16GemmArgs()
        a.x, a.weight, a.out = _p(xs), _p(weight), _p(os_)
        a.M, a.K, a.N = xs.shape[0], K, N
        a.x_stride_m, a.w_stride_n, a.out_stride_m = x.stride(0), weight.stride(0), out.stride(0)
        _C.check(lib.hymeta_bf16_gemm_f32out(C.byref(a), _stream(x)), "hymeta_bf16_gemm_f32out")
    return out


def advance_step(num_seqs: int, num_queries: int, block_size: int, seq_lens: torch.Tensor, slot_mapping: torch.Tensor,
                 block_tables: torch.Tensor, input_tokens: Optional[torch.Tensor] = None,
                 sampled_token_ids: Optional[torch.Tensor] = None, input_positions: Optional[torch.Tensor] = None) -> None:
    """Multi-step decoding, in place and in one launch: sequence i < num_queries gets its sampled token as input, its
    position (= its length so far), length + 1 and the cache slot of that position; padding rows get slot -1."""
    _dev(seq_lens, slot_mapping, block_tables, input_tokens, sampled_token_ids, input_positions)
    _require(seq_lens.dtype == torch.int32 and seq_lens.is_contiguous() and seq_lens.numel() >= num_seqs, "seq_lens must be contiguous int32 [num_seqs]")
    _require(slot_mapping.dtype == torch.int64 and slot_mapping.is_contiguous() and slot_mapping.numel() >= num_seqs,
             "slot_mapping must be contiguous int64 [num_seqs]")
    _require(block_tables.dtype == torch.int32 and block_tables.dim() == 2 and block_tables.stride(1) == 1
             and block_tables.shape[0] >= num_queries, "block_tables must be int32 [num_seqs, blocks]")
    for name, t in (("input_tokens", input_tokens), ("input_positions", input_positions)):
        _require(t is None or (t.dtype == torch.int64 and t.is_contiguous() and t.numel() >= num_queries), f"{name} must be contiguous int64")
    if sampled_token_ids is not None:
        sampled_token_ids = sampled_token_ids.reshape(-1)
        _require(sampled_token_ids.dtype == torch.int64 and sampled_token_ids.is_contiguous() and sampled_token_ids.numel() >= num_queries,
                 "sampled_token_ids must be contiguous int64 [num_queries(, 1)]")
    _C.check(_C.load().hymeta_advance_step(num_seqs, num_queries, block_size, _p(input_tokens), _p(sampled_token_ids), _p(input_positions),
                                           _p(seq_lens), _p(slot_mapping), _p(block_tables), block_tables.stride(0), _stream(seq_lens)),
             "hymeta_advance_step")


def argmax_rows(logits: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Greedy sampling: int64 [M] indices of the largest fp32 logit of each row (the lowest index among equals)."""
    _dev(logits, out)
    _require(logits.dim() == 2 and logits.dtype == torch.float32 and logits.stride(1) == 1, "logits must be row-contiguous fp32 [M, N]")
    M, N = logits.shape
    if out is None:
        out = torch.empty(M, dtype=torch.int64, device=logits.device)
    _require(out.shape == (M,) and out.dtype == torch.int64 and out.is_contiguous(), "out must be contiguous int64 [M]")
    lib = _C.load()
    ws = _workspace(logits.device, int(lib.hymeta_argmax_rows_workspace_bytes(M)), "argmax_rows") if M > 0 else None
    _C.check(lib.hymeta_argmax_rows(_p(logits), logits.stride(0), M, N, _p(out), _p(ws), ws.numel() if ws is not None else 0,
                                    _stream(logits)), "hymeta_argmax_rows")
    return out


def w8a8_gemm(x: torch.Tensor, qweight: torch.Tensor, w_scale: torch.Tensor,
              bias: Optional[torch.Tensor] = None, out: Optional[torch.Tensor] = None, defer: bool = False):
    """x bf16 [M,K] -> dynamic per-token int8; qweight int8 [N,K]; w_scale fp32 [N] -> bf16 [M,N].
    ``defer``: when the library cuts K into slices, return their ``PartialSums`` instead of summing them."""
    _dev(x, qweight, w_scale, bias, out)
    M, K = x.shape
    N = qweight.shape[0]
    _require(x.dtype == torch.bfloat16 and x.stride(1) == 1, "x must be row-contiguous bf16 [M, K]")
    _require(qweight.dtype == torch.int8 and qweight.is_contiguous() and qweight.shape == (N, K),
             "qweight must be contiguous int8 [N, K]")
    _require(w_scale.dtype == torch.float32 and w_scale.is_contiguous() and w_scale.numel() == N,
             "w_scale must be contiguous fp32 [N]")
    if bias is not None:
        _require(bias.dtype == torch.bfloat16 and bias.is_contiguous() and bias.numel() == N, "bias must be bf16 [N]")
    if out is None:
        out = torch.empty(M, N, dtype=torch.bfloat16, device=x.device)
    _require(out.shape == (M, N) and out.dtype == torch.bfloat16 and out.stride(1) == 1, "out must be bf16 [M, N]")
    ready = int8_rows_of(x)
    xq, xs = ready if ready is not None else (torch.empty(M, K, dtype=torch.int8, device=x.device),
                                              torch.empty(M, dtype=torch.float32, device=x.device))
    a = _C.W8A8GemmArgs()
    a.x, a.qweight, a.w_scale, a.bias, a.out, a.xq, a.x_scale = (
        None if ready is not None else _p(x), _p(qweight), _p(w_scale), _p(bias), _p(out), _p(xq), _p(xs))
    a.M, a.K, a.N = M, K, N
    a.x_stride_m, a.out_stride_m = x.stride(0), out.stride(0)
    lib = _C.load()
    a.split_k = 0        # the library chooses the kernel and the decomposition; the workspace bound covers every choice
    ws = _workspace(x.device, int(lib.hymeta_w8a8_gemm_workspace_bytes(M, N, 0)), "w8a8_gemm")
    a.workspace, a.workspace_bytes = _p(ws), ws.numel()
    if defer:
        desc = _C.GemmPartials()
        _C.check(lib.hymeta_w8a8_gemm_deferred(C.byref(a), C.byref(desc), _stream(x)), "hymeta_w8a8_gemm_deferred")
        return _partials(desc, M, N, x.device, "w8a8_gemm", xs, w_scale, bias) if desc.splits > 0 else out
    _C.check(lib.hymeta_w8a8_gemm(C.byref(a), _stream(x)), "hymeta_w8a8_gemm")
    return out


def gemm_silu_mul_supported(x: torch.Tensor, weight: torch.Tensor) -> bool:
    """Shapes the gate/up projection with the activation in its epilogue takes: decode-sized batches of a bf16
    ``[2 I, K]`` weight (gate rows, then up rows), any batch of an int8 one."""
    esize = 1 if weight.dtype == torch.int8 else 2
    rows = BF16_GEMM_TALL_ROWS if weight.dtype == torch.bfloat16 else 1 << 30      # int8: the tiled kernel above the streaming rows
    if not (x.dim() == 2 and 0 < x.shape[0] <= rows and x.is_cuda and x.dtype == torch.bfloat16
            and weight.dtype in (torch.bfloat16, torch.int8) and x.stride(1) == 1 and weight.is_contiguous()
            and (weight.shape[1] * esize) % 128 == 0 and weight.shape[1] * esize >= 512 and weight.shape[0] % 128 == 0
            and x.stride(0) % 8 == 0):
        return False
    if weight.dtype == torch.bfloat16 and x.shape[0] > BF16_GEMM_MAX_ROWS:
        return bool(_C.load().hymeta_bf16_gemm_takes(x.shape[0], weight.shape[1], weight.shape[0], 1))
    return True


def gemm_silu_mul(x: torch.Tensor, weight: torch.Tensor, w_scale: Optional[torch.Tensor] = None,
                  out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``silu(x gate^T) * (x up^T)`` in one launch: x bf16 [M, K]; weight [2 I, K] bf16 (M <= 128, wide ones to 256), or int8 with ``w_scale``
    fp32 [2 I] (dynamic per-token int8 activations; any M) -> bf16 [M, I].  Bit for bit the linear followed by
    ``silu_and_mul``."""
    _dev(x, weight, w_scale, out)
    M, K = x.shape
    N = weight.shape[0]
    _require(gemm_silu_mul_supported(x, weight) and weight.shape == (N, K), "shape not covered: run the linear and silu_and_mul")
    if out is None:
        out = torch.empty(M, N // 2, dtype=torch.bfloat16, device=x.device)
    _require(out.shape == (M, N // 2) and out.dtype == torch.bfloat16 and out.stride(1) == 1 and out.stride(0) % 8 == 0,
             "out must be row-contiguous bf16 [M, I]")
    lib = _C.load()
    if weight.dtype == torch.bfloat16:
        a = _C.Bf16GemmArgs()
        a.x, a.weight, a.out = _p(x), _p(weight), _p(out)
        a.M, a.K, a.N = M, K, N
        a.x_stride_m, a.w_stride_n, a.out_stride_m = x.stride(0), weight.stride(0), out.stride(0)
        _C.check(lib.hymeta_bf16_gemm_silu_mul(C.byref(a), _stream(x)), "hymeta_bf16_gemm_silu_mul")
        return out
    _require(w_scale is not None and w_scale.dtype == torch.float32 and w_scale.is_contiguous() and w_scale.numel() == N,
             "w_scale must be contiguous fp32 [2 I]")
    ready = int8_rows_of(x)
    xq, xs = ready if ready is not None else (torch.empty(M, K, dtype=torch.int8, device=x.device),
                                              torch.empty(M, dtype=torch.float32, device=x.device))
    a = _C.W8A8GemmArgs()
    a.x, a.qweight, a.w_scale, a.out, a.xq, a.x_scale = (None if ready is not None else _p(x), _p(weight), _p(w_scale), _p(out),
                                                         _p(xq), _p(xs))
    a.M, a.K, a.N = M, K, N
    a.x_stride_m, a.out_stride_m = x.stride(0), out.stride(0)
    _C.check(lib.hymeta_w8a8_gemm_silu_mul(C.byref(a), _stream(x)), "hymeta_w8a8_gemm_silu_mul")
    return out


def w8a8_quantize(x: torch.Tensor):
    """Dynamic per-token int8 quantisation: x bf16 [M,K] -> (xq int8 [M,K], x_scale fp32 [M])."""
    _dev(x)
    M, K = x.shape
    _require(x.dtype == torch.bfloat16 and x.stride(1) == 1, "x must be row-contiguous bf16 [M, K]")
    if int8_rows_of(x) is not None:
        return int8_rows_of(x)
    xq = torch.empty(M, K, dtype=torch.int8, device=x.device)
    xs = torch.empty(M, dtype=torch.float32, device=x.device)
    _C.check(_C.load().hymeta_w8a8_quantize(_p(x), _p(xq), _p(xs), M, K, x.stride(0), _stream(x)), "hymeta_w8a8_quantize")
    return xq, xs


def w8a8_scale_out(acc: torch.Tensor, x_scale: torch.Tensor, w_scale: torch.Tensor, bias: Optional[torch.Tensor] = None,
                   out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """acc int32 [M,N] (exact sums of int8 products) -> bf16(acc * x_scale[m] * w_scale[n] + bias[n])."""
    _dev(acc, x_scale, w_scale, bias, out)
    M, N = acc.shape
    _require(acc.dtype == torch.int32 and acc.stride(1) == 1, "acc must be row-contiguous int32 [M, N]")
    _require(x_scale.dtype == torch.float32 and x_scale.is_contiguous() and x_scale.numel() == M, "x_scale must be fp32 [M]")
    _require(w_scale.dtype == torch.float32 and w_scale.is_contiguous() and w_scale.numel() == N, "w_scale must be fp32 [N]")
    if bias is not None:
        _require(bias.dtype == torch.bfloat16 and bias.is_contiguous() and bias.numel() == N, "bias must be bf16 [N]")
    if out is None:
        out = torch.empty(M, N, dtype=torch.bfloat16, device=acc.device)
    _require(out.shape == (M, N) and out.dtype == torch.bfloat16 and out.stride(1) == 1, "out must be bf16 [M, N]")
    _C.check(_C.load().hymeta_w8a8_scale_out(_p(acc), _p(x_scale), _p(w_scale), _p(bias), _p(out), M, N, acc.stride(0),
                                             out.stride(0), _stream(acc)), "hymeta_w8a8_scale_out")
    return out


# ---------------------------------------------------------------------------
# Sparse mixture of experts
# ---------------------------------------------------------------------------
def silu_and_mul(x: torch.Tensor, out: Optional[torch.Tensor] = None, num_rows_dev: Optional[torch.Tensor] = None
                 ) -> torch.Tensor:
    """x bf16 [R, 2I] -> silu(x[:, :I]) * x[:, I:] bf16 [R, I]; ``num_rows_dev`` (int32 device scalar)
    limits the rows actually computed."""
    _dev(x, out, num_rows_dev)
    R, two_i = x.shape
    inter = two_i // 2
    _require(x.dtype == torch.bfloat16 and x.stride(1) == 1 and two_i % 2 == 0, "x must be row-contiguous bf16 [R, 2I]")
    if out is None:
        out = torch.empty(R, inter, dtype=torch.bfloat16, device=x.device)
    _require(out.shape == (R, inter) and out.dtype == torch.bfloat16 and out.stride(1) == 1, "out must be bf16 [R, I]")
    _C.check(_C.load().hymeta_silu_and_mul(_p(x), _p(out), _p(num_rows_dev), R, inter, x.stride(0), out.stride(0),
                                           _stream(x)), "hymeta_silu_and_mul")
    return out


def silu_and_mul_int8(x: torch.Tensor, num_rows_dev: Optional[torch.Tensor] = None):
    """x bf16 [R, 2I] -> the rows ``silu_and_mul`` would give, quantised per row as ``w8a8_quantize`` quantises them:
    (int8 [R, I], fp32 scales [R]) in one launch, the bf16 rows never written."""
    _dev(x, num_rows_dev)
    R, two_i = x.shape
    inter = two_i // 2
    _require(x.dtype == torch.bfloat16 and x.stride(1) == 1 and two_i % 2 == 0, "x must be row-contiguous bf16 [R, 2I]")
    q = torch.empty(R, inter, dtype=torch.int8, device=x.device)
    sc = torch.empty(R, dtype=torch.float32, device=x.device)
    _C.check(_C.load().hymeta_silu_and_mul_int8(_p(x), _p(q), _p(sc), _p(num_rows_dev), R, inter, x.stride(0), _stream(x)),
             "hymeta_silu_and_mul_int8")
    return q, sc


class GptqExperts(NamedTuple):
    """One projection of GPTQ experts, stacked: ``qweight`` int32 [E, K / pack, N], ``qzeros`` int32 [E, K / group, N / pack],
    ``scales`` fp16 | bf16 [E, K / group, N] (each expert's tensors as ``gptq_gemm`` takes them), contiguous."""
    qweight: torch.Tensor
    qzeros: torch.Tensor
    scales: torch.Tensor
    bits: int = 4
    group_size: int = 128
    zero_offset: int = 1

    @property
    def shape(self):
        """(E, N, K): the shape of the bf16 stack this stands for."""
        return (self.qweight.shape[0], self.qweight.shape[2], self.qweight.shape[1] * (32 // self.bits))


# Rows per local expert (on average) up to which GPTQ experts run the fused de-quantising grouped GEMM; above, the local
# experts are expanded to bf16 once per call and the tiled bf16 grouped GEMM runs on the expansion (the fused kernel
# re-reads an expert's weights per 32-row tile).  Measured on the 70B TP=4 shapes (16 experts, us per block, fused /
# expanded): 1024 tokens 466 / 796, 2048: 777 / 943, 4096: 1373 / 1164, 8192: 2569 / 1557.
MOE_GPTQ_FUSED_ROWS_PER_EXPERT = int(os.environ.get("HYMETA_MOE_GPTQ_FUSED_ROWS", "160"))


def moe_gptq_expand(w: GptqExperts) -> torch.Tensor:
    """GPTQ expert stack -> bf16 [E, N, K] (one launch), in a grow-only workspace of the device and stream."""
    E, N, K = w.shape
    pack = 32 // w.bits
    _require(w.qweight.dtype == torch.int32 and w.qweight.is_contiguous() and w.qzeros.is_contiguous() and w.scales.is_contiguous(),
             "GPTQ expert tensors must be contiguous")
    _require(N % 64 == 0 and K % (16 * pack) == 0, "expansion needs N % 64 == 0 and K % (16 * pack) == 0")
    ws = _workspace(w.qweight.device, E * N * K * 2, f"moe_gptq_expand_{N}x{K}")
    out = ws[: E * N * K * 2].view(torch.bfloat16).view(E, N, K)
    sd = _C.HYMETA_F16 if w.scales.dtype == torch.float16 else _C.HYMETA_BF16
    _C.check(_C.load().hymeta_moe_gptq_expand(_p(w.qweight), _p(w.qzeros), _p(w.scales), _p(out), E, K, N, w.bits, w.group_size,
                                              sd, w.zero_offset, _stream(w.qweight)), "hymeta_moe_gptq_expand")
    return out


# Switch for A/B timing and for tests of both forms: fold the combine into the experts' down GEMM at decode sizes (see
# moe_forward).
MOE_FUSE_DOWN = os.environ.get("HYMETA_MOE_FUSE_DOWN", "1") != "0"


def moe_router_fused(x: torch.Tensor, gate_weight: torch.Tensor) -> bool:
    """Whether ``moe_forward`` routes this batch with the one-launch router (linear layer + routing)."""
    per16 = 16 if gate_weight.dtype == torch.int8 else 8      # an int8 router reads the tokens' int8 rows
    return (x.is_cuda and x.dtype == torch.bfloat16 and gate_weight.dtype in (torch.bfloat16, torch.int8)
            and gate_weight.is_contiguous() and 0 < x.shape[0] <= _C.MOE_ROUTER_MAX_TOKENS and x.shape[1] % per16 == 0
            and x.stride(0) % 8 == 0 and gate_weight.shape[0] <= 64)


def moe_forward(x: torch.Tensor, router_logits: Optional[torch.Tensor], w13: torch.Tensor, w2: torch.Tensor, top_k: int = 1,
                renormalize: bool = False, shared: Optional[torch.Tensor] = None,
                local_experts: Optional[tuple] = None, out: Optional[torch.Tensor] = None,
                gate_weight: Optional[torch.Tensor] = None, logits_out: Optional[torch.Tensor] = None,
                w13_scale: Optional[torch.Tensor] = None, w2_scale: Optional[torch.Tensor] = None,
                gate_scale: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Sparse MoE block: x bf16 [T,H], router_logits [T,E] (bf16 | fp32), w13 bf16 [E,2I,H], w2 bf16
    [E,H,I] -- or W8A8 experts: w13 / w2 int8 with per-output-channel ``w13_scale`` fp32 [E,2I] / ``w2_scale`` fp32 [E,H]
    (the tokens and the activated rows are quantised per row on the way in: exact int32 sums, scales applied once);
    ``shared`` bf16 [T,H] is added to the result; ``local_experts = (lo, hi)`` computes only
    this rank's experts (the caller all-reduces); the weight tensors may then hold just those experts
    (``[hi - lo, 2I, H]`` / ``[hi - lo, H, I]``, expert ``lo`` first: an expert-parallel rank keeps nothing else), with the
    number of experts taken from the router (``gate_weight`` rows / ``router_logits`` columns).  Returns bf16 [T,H].
    With ``router_logits=None`` and ``gate_weight`` bf16 [E,H] the block computes the logits itself: decode-sized batches
    in the routing launch (``moe_router_fused``; ``logits_out`` bf16 [T,E] then receives them), larger ones through the
    linear layer.  An int8 ``gate_weight`` with ``gate_scale`` fp32 [E] (the router of a W8A8 checkpoint) is routed in
    that launch too, on the tokens' int8 rows; larger batches must come with ``router_logits``.  GPTQ experts: ``w13`` /
    ``w2`` as ``GptqExperts`` stacks -- decode-sized batches run the fused de-quantising grouped GEMM, larger ones expand
    the local experts to bf16 once per call."""
    gptq = isinstance(w13, GptqExperts)
    if gptq:
        _require(isinstance(w2, GptqExperts), "w13 and w2 must both be GPTQ stacks")
        n_local = (local_experts[1] - local_experts[0]) if local_experts is not None else w13.shape[0]
        if x.shape[0] * top_k > MOE_GPTQ_FUSED_ROWS_PER_EXPERT * max(n_local, 1):
            held = w13.shape[0]
            total = gate_weight.shape[0] if gate_weight is not None else router_logits.shape[1]
            if held == total and local_experts is not None and tuple(local_experts) != (0, total):
                lo_, hi_ = local_experts      # expand the rank's experts only
                w13 = w13._replace(qweight=w13.qweight[lo_:hi_], qzeros=w13.qzeros[lo_:hi_], scales=w13.scales[lo_:hi_])
                w2 = w2._replace(qweight=w2.qweight[lo_:hi_], qzeros=w2.qzeros[lo_:hi_], scales=w2.scales[lo_:hi_])
            return moe_forward(x, router_logits, moe_gptq_expand(w13), moe_gptq_expand(w2), top_k, renormalize, shared,
                               local_experts, out, gate_weight, logits_out)
        _dev(x, router_logits, w13.qweight, w2.qweight, shared, out, gate_weight, gate_scale)
    else:
        _dev(x, router_logits, w13, w2, shared, out, gate_weight, gate_scale)
    T, H = x.shape
    E_held, two_i, Hw = w13.shape
    inter = two_i // 2
    _require(router_logits is not None or gate_weight is not None, "router_logits or gate_weight must be given")
    E = gate_weight.shape[0] if gate_weight is not None else router_logits.shape[1]
    lo, hi = local_experts if local_experts is not None else (0, E)
    _require(0 <= lo <= hi <= E, "local_experts must lie inside the router's experts")
    compact = E_held != E                   # only the local experts are held: slot 0 = expert lo
    _require(E_held == E or E_held == hi - lo, "w13 / w2 must hold every expert or exactly the local ones")
    fused_router = router_logits is None and T > 0 and moe_router_fused(x, gate_weight)
    if gate_weight is not None and gate_weight.dtype == torch.int8 and router_logits is None:
        _require(fused_router, "an int8 router above the one-launch router's batch size needs router_logits")
        _require(gate_scale is not None and gate_scale.dtype == torch.float32 and gate_scale.is_contiguous()
                 and gate_scale.numel() == E, "gate_scale must be contiguous fp32 [E]")
    if router_logits is None and not fused_router:
        _require(gate_weight.shape == (E, H), "gate_weight must be [E, H]")
        router_logits = torch.nn.functional.linear(x, gate_weight)
        if logits_out is not None:
            logits_out.copy_(router_logits)
    _require(x.dtype == torch.bfloat16 and x.stride(1) == 1, "x must be row-contiguous bf16 [T, H]")
    i8 = not gptq and w13.dtype == torch.int8
    if gptq:
        _require(Hw == H and tuple(w2.shape) == (E_held, H, inter), "GPTQ stacks must stand for w13 [E, 2I, H] and w2 [E, H, I]")
        for w in (w13, w2):
            pk = 32 // w.bits
            _require(w.qweight.dtype == torch.int32 and w.qweight.is_contiguous() and w.qzeros.dtype == torch.int32
                     and w.qzeros.is_contiguous() and w.scales.dtype in (torch.float16, torch.bfloat16) and w.scales.is_contiguous(),
                     "GPTQ expert tensors must be contiguous int32 / int32 / fp16 | bf16")
            _require(tuple(w.qzeros.shape) == (E_held, w.shape[2] // w.group_size, w.shape[1] // pk)
                     and tuple(w.scales.shape) == (E_held, w.shape[2] // w.group_size, w.shape[1]),
                     "qzeros / scales must be [E, K / group, N / pack] / [E, K / group, N]")
    else:
        _require(w13.dtype in (torch.bfloat16, torch.int8) and w13.is_contiguous() and Hw == H,
                 "w13 must be contiguous bf16 | int8 [E, 2I, H]")
        _require(w2.dtype == w13.dtype and w2.is_contiguous() and w2.shape == (E_held, H, inter),
                 "w2 must be contiguous [E, H, I] of w13's type")
    if i8:
        _dev(w13_scale, w2_scale)
        _require(w13_scale is not None and w13_scale.dtype == torch.float32 and w13_scale.is_contiguous()
                 and w13_scale.shape == (E_held, two_i), "w13_scale must be contiguous fp32 [E, 2I]")
        _require(w2_scale is not None and w2_scale.dtype == torch.float32 and w2_scale.is_contiguous()
                 and w2_scale.shape == (E_held, H), "w2_scale must be contiguous fp32 [E, H]")
        _require(H % 128 == 0 and inter % 64 == 0, "int8 experts need H % 128 == 0 and I % 64 == 0")
    _require(fused_router or (router_logits.shape == (T, E) and router_logits.dtype in _DT and router_logits.stride(1) == 1),
             "router_logits must be [T, E] bf16 | fp32")
    dev = x.device
    P = T * top_k
    ids = torch.empty(T, top_k, dtype=torch.int32, device=dev)
    wts = torch.empty(T, top_k, dtype=torch.float32, device=dev)
    meta = torch.empty(3 * (E + 1), dtype=torch.int32, device=dev)
    counts, cursors, offsets = meta[: E + 1], meta[E + 1: 2 * (E + 1)], meta[2 * (E + 1):]
    sorted_pair = torch.empty(max(P, 1), dtype=torch.int32, device=dev)
    pair_pos = torch.empty(max(P, 1), dtype=torch.int32, device=dev)
    if out is None:
        out = torch.empty(T, H, dtype=torch.bfloat16, device=dev)
    if T == 0:
        return out
    lib, st = _C.load(), _stream(x)
    if fused_router:
        _require(gate_weight.shape == (E, H), "gate_weight must be [E, H]")
        _require(logits_out is None or (logits_out.shape == (T, E) and logits_out.dtype == torch.bfloat16 and logits_out.is_contiguous()),
                 "logits_out must be contiguous bf16 [T, E]")
        r = _C.MoeRouterArgs()
        r.x, r.gate_weight, r.logits_out = _p(x), _p(gate_weight), _p(logits_out)
        r.x_stride_t = x.stride(0)
        if gate_weight.dtype == torch.int8:
            xq_r, xs_r = w8a8_quantize(x)       # (the rows a quantising norm attached, or one launch; the experts reuse them)
            setattr(x, INT8_ROWS_ATTR, (xq_r, xs_r))
            r.x, r.x_stride_t = _p(xq_r), xq_r.stride(0)
            r.operand_dtype, r.x_scale, r.gate_scale = _C.HYMETA_I8, _p(xs_r), _p(gate_scale)
        r.topk_ids, r.topk_weights, r.expert_offsets = _p(ids), _p(wts), _p(offsets)
        r.sorted_pair, r.pair_pos = _p(sorted_pair), _p(pair_pos)
        r.ticket = _p(_workspace(dev, 64, "moe_router"))
        r.num_tokens, r.num_experts, r.top_k, r.renormalize, r.hidden = T, E, top_k, int(bool(renormalize)), H
        r.local_expert_begin, r.local_expert_end = lo, hi
        _C.check(lib.hymeta_moe_router(C.byref(r), st), "hymeta_moe_router")
    else:
        r = _C.MoeRouteArgs()
        r.router_logits, r.topk_ids, r.topk_weights = _p(router_logits), _p(ids), _p(wts)
        r.counts, r.cursors, r.expert_offsets = _p(counts), _p(cursors), _p(offsets)
        r.sorted_pair, r.pair_pos = _p(sorted_pair), _p(pair_pos)
        r.num_tokens, r.num_experts, r.top_k, r.renormalize = T, E, top_k, int(bool(renormalize))
        r.logits_dtype = _DT[router_logits.dtype]
        r.local_expert_begin, r.local_expert_end = lo, hi
        r.logits_stride_t = router_logits.stride(0)
        _C.check(lib.hymeta_moe_route(C.byref(r), st), "hymeta_moe_route")

    h13 = torch.empty(P, two_i, dtype=torch.bfloat16, device=dev)
    if gptq:
        if shared is not None:
            _require(shared.shape == (T, H) and shared.dtype == torch.bfloat16 and shared.stride(1) == 1,
                     "shared must be bf16 [T, H]")

        def gptq_gemm_args(w: GptqExperts, xin, xout, K_, N_):
            q = _C.MoeGptqGemmArgs()
            back = lo if compact else 0           # tensors that hold the local experts only: address expert 0
            per_q, per_z, per_s = w.qweight.stride(0) * 4, w.qzeros.stride(0) * 4, w.scales.stride(0) * 2
            q.qweight = C.c_void_p(w.qweight.data_ptr() - back * per_q)
            q.qzeros = C.c_void_p(w.qzeros.data_ptr() - back * per_z)
            q.scales = C.c_void_p(w.scales.data_ptr() - back * per_s)
            q.x, q.out, q.expert_offsets = _p(xin), _p(xout), _p(offsets)
            q.max_rows, q.K, q.N = P, K_, N_
            q.bits, q.group_size, q.zero_offset = w.bits, w.group_size, w.zero_offset
            q.scales_dtype = _C.HYMETA_F16 if w.scales.dtype == torch.float16 else _C.HYMETA_BF16
            q.local_expert_begin, q.local_expert_end = lo, hi
            q.x_stride_m, q.out_stride_m = xin.stride(0), xout.stride(0)
            return q

        q13 = gptq_gemm_args(w13, x, h13, H, two_i)
        q13.a_rows, q13.a_rows_div = _p(sorted_pair), top_k
        _C.check(lib.hymeta_moe_gptq_gemm(C.byref(q13), st), "hymeta_moe_gptq_gemm (w13)")
        hact = torch.empty(P, inter, dtype=torch.bfloat16, device=dev)
        silu_and_mul(h13, out=hact)
        y = torch.empty(P, H, dtype=torch.bfloat16, device=dev)
        q2 = gptq_gemm_args(w2, hact, y, inter, H)
        q2.a_rows_div, q2.scale_rows, q2.row_scale = 1, _p(sorted_pair), _p(wts)
        _C.check(lib.hymeta_moe_gptq_gemm(C.byref(q2), st), "hymeta_moe_gptq_gemm (w2)")
        c = _C.MoeCombineArgs()
        c.y, c.shared, c.out, c.pair_pos, c.topk_weights = _p(y), _p(shared), _p(out), _p(pair_pos), _p(wts)
        c.num_tokens, c.hidden, c.top_k = T, H, top_k
        c.y_stride_m, c.out_stride_m = y.stride(0), out.stride(0)
        if shared is not None:
            c.shared_stride_m = shared.stride(0)
        _C.check(lib.hymeta_moe_combine(C.byref(c), st), "hymeta_moe_combine")
        return out
    g = _C.MoeGemmArgs()
    # the kernels index the weights by the expert's number: tensors that hold the local experts only are addressed from
    # where expert 0 would lie (only experts lo .. hi - 1 are ever read)
    esize = 1 if i8 else 2
    w13_base = C.c_void_p(w13.data_ptr() - (lo * w13.stride(0) * esize if compact else 0))
    w2_base = C.c_void_p(w2.data_ptr() - (lo * w2.stride(0) * esize if compact else 0))
    xin = x
    if i8:
        xin, xs = w8a8_quantize(x)              # per token, once for all its experts
        g.operand_dtype, g.x_scale = _C.HYMETA_I8, _p(xs)
        g.w_scale = C.c_void_p(w13_scale.data_ptr() - (lo * two_i * 4 if compact else 0))
    g.x, g.weights, g.out, g.expert_offsets = _p(xin), w13_base, _p(h13), _p(offsets)
    g.a_rows, g.a_rows_div, g.max_rows, g.K, g.N = _p(sorted_pair), top_k, P, H, two_i
    g.local_expert_begin, g.local_expert_end = lo, hi
    g.x_stride_m, g.out_stride_m, g.w_stride_e = xin.stride(0), h13.stride(0), w13.stride(0)
    _C.check(lib.hymeta_moe_gemm(C.byref(g), st), "hymeta_moe_gemm (w13)")

    if shared is not None:
        _require(shared.shape == (T, H) and shared.dtype == torch.bfloat16 and shared.stride(1) == 1,
                 "shared must be bf16 [T, H]")
    # decode-sized batches with one choice per token and every expert local: the down GEMM writes its rows straight to
    # their tokens with the shared expert added -- no combine launch
    fuse_combine = (MOE_FUSE_DOWN and top_k == 1 and (lo, hi) == (0, E)
                    and bool(lib.hymeta_moe_gemm_fuses(P, hi - lo, inter // 2 if i8 else inter, H))
                    and (shared is None or shared.stride(0) % 8 == 0))
    # slots in use are a prefix only when lo == 0; otherwise act on all P rows (unused rows are never read)
    d = _C.MoeGemmArgs()
    if i8:
        hact, hs = silu_and_mul_int8(h13)       # activation and per-row quantisation in one launch
        d.operand_dtype, d.x_scale = _C.HYMETA_I8, _p(hs)
        d.w_scale = C.c_void_p(w2_scale.data_ptr() - (lo * H * 4 if compact else 0))
    else:
        hact = torch.empty(P, inter, dtype=torch.bfloat16, device=dev)
        silu_and_mul(h13, out=hact)
    d.x, d.x_stride_m = _p(hact), hact.stride(0)
    y = out if fuse_combine else torch.empty(P, H, dtype=torch.bfloat16, device=dev)
    d.weights, d.out, d.expert_offsets = w2_base, _p(y), _p(offsets)
    d.scale_rows, d.row_scale = _p(sorted_pair), _p(wts)
    d.a_rows_div, d.max_rows, d.K, d.N = 1, P, inter, H
    d.local_expert_begin, d.local_expert_end = lo, hi
    d.out_stride_m, d.w_stride_e = y.stride(0), w2.stride(0)
    if fuse_combine:
        d.combine_tokens = _p(sorted_pair)       # one choice per token: the pair index is the token
        if shared is not None:
            d.combine_shared, d.combine_shared_stride_m = _p(shared), shared.stride(0)
    _C.check(lib.hymeta_moe_gemm(C.byref(d), st), "hymeta_moe_gemm (w2)")
    if fuse_combine:
        return out

    c = _C.MoeCombineArgs()
    c.y, c.shared, c.out, c.pair_pos, c.topk_weights = _p(y), _p(shared), _p(out), _p(pair_pos), _p(wts)
    c.num_tokens, c.hidden, c.top_k = T, H, top_k
    c.y_stride_m, c.out_stride_m = y.stride(0), out.stride(0)
    if shared is not None:
        c.shared_stride_m = shared.stride(0)
    _C.check(lib.hymeta_moe_combine(C.byref(c), st), "hymeta_moe_combine")
    return out


# ---------------------------------------------------------------------------
# Building blocks of recurrent / biased-attention designs: fp32 residual stream, norm + short convolution,
# minGRU, paged attention with a distance bias and a sink, table-routed experts.  Activations bf16 or fp32.
# ---------------------------------------------------------------------------
def _act(t: torch.Tensor) -> int:
    _require(t.dtype in _DT, "activations must be bf16 or fp32")
    return _DT[t.dtype]


def _f32vec(t: Optional[torch.Tensor], n: int, name: str) -> None:
    _require(t is None or (t.dtype == torch.float32 and t.is_contiguous() and t.numel() == n), f"{name} must be contiguous fp32 [{n}]")


def _i32vec(t: torch.Tensor, n: int, name: str) -> None:
    _require(t.dtype == torch.int32 and t.is_contiguous() and t.numel() >= n, f"{name} must be contiguous int32 [{n}]")


def embed_rows(token_ids: torch.Tensor, table: torch.Tensor, add: Optional[torch.Tensor] = None, scale: float = 1.0) -> torch.Tensor:
    """fp32 ``[T, W]`` rows ``table[token_ids] * scale (+ add)``: the start of an fp32 residual stream."""
    _dev(token_ids, table, add)
    _require(token_ids.dtype == torch.int64 and token_ids.dim() == 1 and token_ids.is_contiguous(), "token_ids must be contiguous int64 [T]")
    _require(table.dim() == 2 and table.is_contiguous(), "table must be contiguous [vocab, width]")
    V, W = table.shape
    _f32vec(add, W, "add")
    out = torch.empty(token_ids.shape[0], W, dtype=torch.float32, device=table.device)
    a = _C.EmbedRowsArgs()
    a.token_ids, a.table, a.add, a.out = _p(token_ids), _p(table), _p(add), _p(out)
    a.num_tokens, a.width, a.vocab, a.act_dtype, a.scale = token_ids.shape[0], W, V, _act(table), float(scale)
    _C.check(_C.load().hymeta_embed_rows(C.byref(a), _stream(table)), "hymeta_embed_rows")
    return out


def norm_conv(x: torch.Tensor, weight: torch.Tensor, eps: float, out_dtype: torch.dtype, weight_offset: float = 0.0,
              conv_weight: Optional[torch.Tensor] = None, conv_state: Optional[torch.Tensor] = None,
              query_start_loc: Optional[torch.Tensor] = None, context_lens: Optional[torch.Tensor] = None,
              slot_idx: Optional[torch.Tensor] = None) -> torch.Tensor:
    """RMS norm of the fp32 rows ``x [T, W]`` (weight ``weight_offset + weight``), then, with ``conv_weight [W, taps]``,
    ``out[t] = n[t] + sum_j conv_weight[:, j] n[t - taps + 1 + j]`` over each sequence's rows; ``conv_state
    [slots, taps - 1, W]`` (``out_dtype``) carries a sequence's last rows between steps and is updated in place."""
    _dev(x, weight, conv_weight, conv_state, query_start_loc, context_lens, slot_idx)
    _require(x.dim() == 2 and x.dtype == torch.float32 and x.stride(1) == 1, "x must be row-contiguous fp32 [T, W]")
    T, W = x.shape
    _f32vec(weight, W, "weight")
    _require(out_dtype in _DT, "out_dtype must be bf16 or fp32")
    out = torch.empty(T, W, dtype=out_dtype, device=x.device)
    a = _C.NormConvArgs()
    a.x, a.weight, a.out = _p(x), _p(weight), _p(out)
    a.num_tokens, a.width, a.act_dtype, a.eps, a.weight_offset, a.x_stride_t = T, W, _DT[out_dtype], eps, weight_offset, x.stride(0)
    a.taps = 1
    if conv_weight is not None:
        taps = conv_weight.shape[1]
        _require(conv_weight.dtype == torch.float32 and conv_weight.is_contiguous() and conv_weight.shape == (W, taps),
                 "conv_weight must be contiguous fp32 [W, taps]")
        _require(1 <= taps <= _C.CONV_MAX_TAPS, f"taps must be 1 .. {_C.CONV_MAX_TAPS}")
        a.conv_weight, a.taps = _p(conv_weight), taps
        if taps > 1:
            _require(query_start_loc is not None and context_lens is not None, "a convolution over time needs the step's sequence layout")
            S = query_start_loc.numel() - 1
            _i32vec(query_start_loc, S + 1, "query_start_loc")
            _i32vec(context_lens, S, "context_lens")
            a.query_start_loc, a.context_lens, a.num_seqs = _p(query_start_loc), _p(context_lens), S
            if conv_state is not None:
                _require(slot_idx is not None, "conv_state needs slot_idx")
                _i32vec(slot_idx, S, "slot_idx")
                _require(conv_state.dtype == out_dtype and conv_state.is_contiguous() and conv_state.dim() == 3
                         and conv_state.shape[1:] == (taps - 1, W), "conv_state must be contiguous [slots, taps - 1, W] of out_dtype")
                a.conv_state, a.slot_idx = _p(conv_state), _p(slot_idx)
    _C.check(_C.load().hymeta_norm_conv(C.byref(a), _stream(x)), "hymeta_norm_conv")
    return out


def norm_residual_(x: torch.Tensor, y: torch.Tensor, weight: torch.Tensor, eps: float, mult: float = 1.0,
                   weight_offset: float = 0.0, post_add: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``x += mult * rmsnorm(y) * (weight_offset + weight) (+ post_add)`` on the fp32 rows ``x [T, W]``, in place."""
    _dev(x, y, weight, post_add)
    _require(x.dim() == 2 and x.dtype == torch.float32 and x.stride(1) == 1, "x must be row-contiguous fp32 [T, W]")
    T, W = x.shape
    _require(y.shape == (T, W) and y.stride(1) == 1, "y must be row-contiguous [T, W]")
    _f32vec(weight, W, "weight")
    _f32vec(post_add, W, "post_add")
    a = _C.NormResidualArgs()
    a.y, a.weight, a.post_add, a.x = _p(y), _p(weight), _p(post_add), _p(x)
    a.num_tokens, a.width, a.act_dtype = T, W, _act(y)
    a.eps, a.weight_offset, a.mult, a.y_stride_t, a.x_stride_t = eps, weight_offset, mult, y.stride(0), x.stride(0)
    _C.check(_C.load().hymeta_norm_residual(C.byref(a), _stream(x)), "hymeta_norm_residual")
    return x


def mingru(zug: torch.Tensor, state: torch.Tensor, query_start_loc: torch.Tensor, context_lens: torch.Tensor,
           slot_idx: torch.Tensor, max_query_len: int) -> torch.Tensor:
    """minGRU over a step's rows: ``zug [T, 3W]`` = the update-gate, candidate and output-gate projections;
    ``state`` fp32 ``[slots, W]`` is read (where ``context_lens > 0``) and written.  Returns ``S * silu(g)`` ``[T, W]``."""
    _dev(zug, state, query_start_loc, context_lens, slot_idx)
    _require(zug.dim() == 2 and zug.stride(1) == 1 and zug.shape[1] % 3 == 0, "zug must be row-contiguous [T, 3W]")
    T, W = zug.shape[0], zug.shape[1] // 3
    _require(state.dtype == torch.float32 and state.is_contiguous() and state.dim() == 2 and state.shape[1] == W, "state must be contiguous fp32 [slots, W]")
    S = query_start_loc.numel() - 1
    _i32vec(query_start_loc, S + 1, "query_start_loc")
    _i32vec(context_lens, S, "context_lens")
    _i32vec(slot_idx, S, "slot_idx")
    out = torch.empty(T, W, dtype=zug.dtype, device=zug.device)
    a = _C.MinGruArgs()
    a.zug, a.state, a.out = _p(zug), _p(state), _p(out)
    a.query_start_loc, a.context_lens, a.slot_idx = _p(query_start_loc), _p(context_lens), _p(slot_idx)
    a.num_tokens, a.num_seqs, a.width, a.act_dtype, a.max_query_len, a.zug_stride_t = T, S, W, _act(zug), max_query_len, zug.stride(0)
    lib = _C.load()
    nbytes = int(lib.hymeta_mingru_workspace_bytes(S, W, max_query_len))
    if nbytes:
        ws = _workspace(zug.device, nbytes, "mingru")
        a.workspace, a.workspace_bytes = _p(ws), ws.numel()
    _C.check(lib.hymeta_mingru(C.byref(a), _stream(zug)), "hymeta_mingru")
    return out


def qk_norm_cache_(qkv: torch.Tensor, num_heads: int, num_kv_heads: int, head_dim: int, v_dim: int,
                   q_weight: Optional[torch.Tensor], k_weight: Optional[torch.Tensor], eps: float,
                   kv_cache: Optional[torch.Tensor], slot_mapping: Optional[torch.Tensor]) -> None:
    """Per-head RMS norm of the query / key columns of ``qkv [T, H D + G D + G Dv]`` (queries in place) and the paged
    write of the normed keys and the values into ``kv_cache [blocks, block_size, G, D + Dv]`` at ``slot_mapping``."""
    _dev(qkv, q_weight, k_weight, kv_cache, slot_mapping)
    T = qkv.shape[0]
    _require(qkv.dim() == 2 and qkv.stride(1) == 1 and qkv.shape[1] == (num_heads + num_kv_heads) * head_dim + num_kv_heads * v_dim,
             "qkv must be row-contiguous [T, H D + G D + G Dv]")
    _f32vec(q_weight, head_dim, "q_weight")
    _f32vec(k_weight, head_dim, "k_weight")
    a = _C.QkNormCacheArgs()
    a.qkv, a.q_weight, a.k_weight = _p(qkv), _p(q_weight), _p(k_weight)
    a.num_tokens, a.num_heads, a.num_kv_heads, a.head_dim, a.v_dim = T, num_heads, num_kv_heads, head_dim, v_dim
    a.act_dtype, a.eps, a.qkv_stride_t, a.block_size = _act(qkv), eps, qkv.stride(0), 1
    if kv_cache is not None and kv_cache.numel() > 0 and slot_mapping is not None:
        _require(kv_cache.dtype == qkv.dtype and kv_cache.is_contiguous() and kv_cache.dim() == 4
                 and kv_cache.shape[2:] == (num_kv_heads, head_dim + v_dim), "kv_cache must be contiguous [blocks, block_size, G, D + Dv]")
        _require(slot_mapping.dtype == torch.int64 and slot_mapping.is_contiguous() and slot_mapping.numel() == T, "slot_mapping must be int64 [T]")
        a.kv_cache, a.slot_mapping, a.num_blocks, a.block_size = _p(kv_cache), _p(slot_mapping), kv_cache.shape[0], kv_cache.shape[1]
    _C.check(_C.load().hymeta_qk_norm_cache(C.byref(a), _stream(qkv)), "hymeta_qk_norm_cache")


def sink_attention(q: torch.Tensor, kv_cache: torch.Tensor, block_tables: torch.Tensor, query_start_loc: torch.Tensor,
                   seq_lens: torch.Tensor, num_kv_heads: int, head_dim: int, v_dim: int, scale: float,
                   max_query_len: int, max_seq_len: int, bias_a: Optional[torch.Tensor] = None,
                   bias_b: Optional[torch.Tensor] = None, sink: bool = True, window_left: int = -1,
                   sink_logits: Optional[torch.Tensor] = None, value_in_key: bool = False, shared_key: bool = False,
                   keep_first: int = 0, softcap: float = 0.0, head_gate: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Causal attention of the rows ``q [T, H, D]`` over their sequences' paged keys (this step's included):
    ``softmax`` over ``scale q.k - bias_a[h] ln(1 + bias_b[h] (i - j))`` with, for ``sink``, ``exp(sink_logits[h])`` (one
    without ``sink_logits``) added to the denominator.  ``softcap > 0``: ``scale q.k`` becomes ``softcap tanh(scale q.k /
    softcap)``.  ``head_gate [T, H]`` (a view with any row stride): head ``h``'s output is multiplied by its sigmoid.  ``value_in_key``: a cache row holds ``D`` elements per key/value
    head, the first ``Dv`` of which are also the value (a latent that keys and values share).  Returns ``[T, H, Dv]``."""
    _dev(q, kv_cache, block_tables, query_start_loc, seq_lens, bias_a, bias_b, sink_logits)
    _require(q.dim() == 3 and q.stride(2) == 1 and q.stride(1) == head_dim and q.shape[2] == head_dim, "q must be [T, H, D] with contiguous heads")
    T, H, _ = q.shape
    row = head_dim if value_in_key else head_dim + v_dim
    _require(not value_in_key or v_dim <= head_dim, "a value inside its key cannot be longer than the key")
    _require(not (value_in_key and shared_key), "one row layout at a time")
    cache_tail = (1, head_dim + num_kv_heads * v_dim) if shared_key else (num_kv_heads, row)
    _require(kv_cache.dtype == q.dtype and kv_cache.is_contiguous() and kv_cache.dim() == 4
             and kv_cache.shape[2:] == cache_tail, f"kv_cache must be contiguous [blocks, block_size, {cache_tail[0]}, {cache_tail[1]}]")
    _require(keep_first >= 0, "keep_first counts tokens")
    _f32vec(sink_logits, H, "sink_logits")
    S = query_start_loc.numel() - 1
    _i32vec(query_start_loc, S + 1, "query_start_loc")
    _i32vec(seq_lens, S, "seq_lens")
    _require(block_tables.dtype == torch.int32 and block_tables.dim() == 2 and block_tables.shape[0] >= S and block_tables.stride(1) == 1,
             "block_tables must be int32 [S, blocks]")
    _require((bias_a is None) == (bias_b is None), "bias_a and bias_b come together")
    _f32vec(bias_a, H, "bias_a")
    _f32vec(bias_b, H, "bias_b")
    out = torch.empty(T, H, v_dim, dtype=q.dtype, device=q.device)
    lib = _C.load()
    a = _C.SinkAttentionArgs()
    a.q, a.kv_cache, a.out, a.block_tables = _p(q), _p(kv_cache), _p(out), _p(block_tables)
    a.query_start_loc, a.seq_lens, a.bias_a, a.bias_b = _p(query_start_loc), _p(seq_lens), _p(bias_a), _p(bias_b)
    nbytes = int(lib.hymeta_sink_attention_workspace_bytes(S, H, num_kv_heads, v_dim, max_seq_len))
    if nbytes:
        ws = _workspace(q.device, nbytes, "sink_attention")
        a.workspace, a.workspace_bytes = _p(ws), ws.numel()
    a.num_tokens, a.num_seqs, a.num_heads, a.num_kv_heads, a.head_dim, a.v_dim = T, S, H, num_kv_heads, head_dim, v_dim
    a.block_size, a.act_dtype, a.num_blocks = kv_cache.shape[1], _act(q), kv_cache.shape[0]
    a.bias_mode = _C.BIAS_NONE if bias_a is None else _C.BIAS_LOG_DISTANCE
    a.sink, a.window_left, a.max_query_len, a.max_seq_len, a.scale = int(bool(sink)), window_left, max_query_len, max_seq_len, scale
    a.sink_logits, a.keep_first, a.softcap = _p(sink_logits), keep_first, float(softcap)
    if head_gate is not None:
        _dev(q, head_gate)
        _require(head_gate.shape == (T, H) and head_gate.stride(1) == 1 and head_gate.dtype == q.dtype, "head_gate must be [T, H] of q's type with contiguous heads")
        a.head_gate, a.head_gate_stride_t = _p(head_gate), head_gate.stride(0)
    a.kv_layout = _C.KV_SHARED_KEY if shared_key else (_C.KV_VALUE_IN_KEY if value_in_key else _C.KV_KEY_THEN_VALUE)
    a.q_stride_t, a.block_table_stride = q.stride(0), block_tables.stride(0)
    _C.check(lib.hymeta_sink_attention(C.byref(a), _stream(q)), "hymeta_sink_attention")
    return out


def moe_mfma_shapes(hidden: int, inter: int) -> bool:
    """Whether the routed block's MFMA grouped GEMMs take experts of these sizes (bf16: K in whole 32s, N in whole 64s)."""
    return hidden % 64 == 0 and inter % 32 == 0 and (2 * inter) % 64 == 0


def moe_table_forward(x: torch.Tensor, token_ids: torch.Tensor, table: torch.Tensor, w13: torch.Tensor, w2: torch.Tensor) -> torch.Tensor:
    """Experts chosen by ``table[token_id]`` (int32 ``[vocab, top]``), each weighing ``1 / top``: ``x [T, H]``, ``w13
    [E, 2I, H]`` (gate rows, then up rows), ``w2 [E, H, I]``, all bf16 or all fp32.  The counting sort by expert is
    one launch; bf16 experts in the MFMA tiles' shapes then run the routed block's grouped GEMMs, activation and
    combine, everything else the generic grouped GEMM (activation in its epilogue) and combine."""
    _dev(x, token_ids, table, w13, w2)
    T, H = x.shape
    E, two_i, _ = w13.shape
    inter = two_i // 2
    top = table.shape[1]
    _require(x.dtype in _DT and x.stride(1) == 1 and w13.dtype == x.dtype and w2.dtype == x.dtype, "x, w13 and w2 must share bf16 or fp32")
    _require(w13.is_contiguous() and w13.shape == (E, 2 * inter, H) and w2.is_contiguous() and w2.shape == (E, H, inter),
             "w13 must be contiguous [E, 2I, H] and w2 [E, H, I]")
    _require(table.dtype == torch.int32 and table.is_contiguous() and table.dim() == 2, "table must be contiguous int32 [vocab, top]")
    _require(token_ids.dtype == torch.int64 and token_ids.is_contiguous() and token_ids.numel() == T, "token_ids must be contiguous int64 [T]")
    dev = x.device
    out = torch.empty(T, H, dtype=x.dtype, device=dev)
    if T == 0:
        return out
    P = T * top
    ids = torch.empty(T, top, dtype=torch.int32, device=dev)
    wts = torch.empty(T, top, dtype=torch.float32, device=dev)
    offsets = torch.empty(E + 1, dtype=torch.int32, device=dev)
    sorted_pair = torch.empty(P, dtype=torch.int32, device=dev)
    pair_pos = torch.empty(P, dtype=torch.int32, device=dev)
    lib, st = _C.load(), _stream(x)
    r = _C.MoeRouteTableArgs()
    r.token_ids, r.table, r.topk_ids, r.topk_weights = _p(token_ids), _p(table), _p(ids), _p(wts)
    r.expert_offsets, r.sorted_pair, r.pair_pos = _p(offsets), _p(sorted_pair), _p(pair_pos)
    r.num_tokens, r.num_experts, r.top_k, r.vocab = T, E, top, table.shape[0]
    _C.check(lib.hymeta_moe_route_table(C.byref(r), st), "hymeta_moe_route_table")

    if (x.dtype == torch.bfloat16 and moe_mfma_shapes(H, inter) and E <= 64 and x.stride(0) % 8 == 0 and x.data_ptr() % 16 == 0):
        h13 = torch.empty(P, two_i, dtype=torch.bfloat16, device=dev)
        g = _C.MoeGemmArgs()
        g.x, g.weights, g.out, g.expert_offsets = _p(x), _p(w13), _p(h13), _p(offsets)
        g.a_rows, g.a_rows_div, g.max_rows, g.K, g.N = _p(sorted_pair), top, P, H, two_i
        g.local_expert_begin, g.local_expert_end = 0, E
        g.x_stride_m, g.out_stride_m, g.w_stride_e = x.stride(0), h13.stride(0), w13.stride(0)
        _C.check(lib.hymeta_moe_gemm(C.byref(g), st), "hymeta_moe_gemm (w13)")
        hact = torch.empty(P, inter, dtype=torch.bfloat16, device=dev)
        silu_and_mul(h13, out=hact)
        y = torch.empty(P, H, dtype=torch.bfloat16, device=dev)
        d = _C.MoeGemmArgs()
        d.x, d.x_stride_m, d.weights, d.out, d.expert_offsets = _p(hact), hact.stride(0), _p(w2), _p(y), _p(offsets)
        d.scale_rows, d.row_scale = _p(sorted_pair), _p(wts)
        d.a_rows_div, d.max_rows, d.K, d.N = 1, P, inter, H
        d.local_expert_begin, d.local_expert_end = 0, E
        d.out_stride_m, d.w_stride_e = y.stride(0), w2.stride(0)
        _C.check(lib.hymeta_moe_gemm(C.byref(d), st), "hymeta_moe_gemm (w2)")
        c = _C.MoeCombineArgs()
        c.y, c.out, c.pair_pos, c.topk_weights = _p(y), _p(out), _p(pair_pos), _p(wts)
        c.num_tokens, c.hidden, c.top_k = T, H, top
        c.y_stride_m, c.out_stride_m = y.stride(0), out.stride(0)
        _C.check(lib.hymeta_moe_combine(C.byref(c), st), "hymeta_moe_combine")
        return out

    act = _DT[x.dtype]
    hact = torch.empty(P, inter, dtype=x.dtype, device=dev)
    g = _C.MoeGemmAnyArgs()
    g.x, g.weights, g.out, g.expert_offsets = _p(x), _p(w13), _p(hact), _p(offsets)
    g.a_rows, g.a_rows_div, g.max_rows, g.K, g.N, g.num_experts, g.gated, g.act_dtype = _p(sorted_pair), top, P, H, inter, E, 1, act
    g.x_stride_m, g.out_stride_m, g.w_stride_e = x.stride(0), hact.stride(0), w13.stride(0)
    _C.check(lib.hymeta_moe_gemm_any(C.byref(g), st), "hymeta_moe_gemm_any (w13)")
    y = torch.empty(P, H, dtype=x.dtype, device=dev)
    d = _C.MoeGemmAnyArgs()
    d.x, d.weights, d.out, d.expert_offsets = _p(hact), _p(w2), _p(y), _p(offsets)
    d.scale_rows, d.row_scale = _p(sorted_pair), _p(wts)
    d.a_rows_div, d.max_rows, d.K, d.N, d.num_experts, d.gated, d.act_dtype = 1, P, inter, H, E, 0, act
    d.x_stride_m, d.out_stride_m, d.w_stride_e = hact.stride(0), y.stride(0), w2.stride(0)
    _C.check(lib.hymeta_moe_gemm_any(C.byref(d), st), "hymeta_moe_gemm_any (w2)")
    c = _C.MoeCombineAnyArgs()
    c.y, c.out, c.pair_pos = _p(y), _p(out), _p(pair_pos)
    c.num_tokens, c.width, c.top_k, c.act_dtype = T, H, top, act
    c.y_stride_m, c.out_stride_m = y.stride(0), out.stride(0)
    _C.check(lib.hymeta_moe_combine_any(C.byref(c), st), "hymeta_moe_combine_any")
    return out


# ---------------------------------------------------------------------------
# Building blocks of post-norm designs with latent and linear attention.
# ---------------------------------------------------------------------------
def token_shift(x: torch.Tensor, mix: torch.Tensor, state: Optional[torch.Tensor], out_dtype: torch.dtype,
                query_start_loc: torch.Tensor, context_lens: torch.Tensor, slot_idx: Optional[torch.Tensor]) -> torch.Tensor:
    """``x[t] + (x[t - 1] - x[t]) * mix`` over each sequence's rows of the fp32 stream ``x [T, W]`` (zeros before a
    sequence's first token); ``state`` fp32 ``[slots, W]`` carries a sequence's last row between steps, in place."""
    _dev(x, mix, state, query_start_loc, context_lens, slot_idx)
    _require(x.dim() == 2 and x.dtype == torch.float32 and x.stride(1) == 1, "x must be row-contiguous fp32 [T, W]")
    T, W = x.shape
    _f32vec(mix, W, "mix")
    _require(out_dtype in _DT, "out_dtype must be bf16 or fp32")
    S = query_start_loc.numel() - 1
    _i32vec(query_start_loc, S + 1, "query_start_loc")
    _i32vec(context_lens, S, "context_lens")
    out = torch.empty(T, W, dtype=out_dtype, device=x.device)
    a = _C.TokenShiftArgs()
    a.x, a.mix, a.out, a.query_start_loc, a.context_lens = _p(x), _p(mix), _p(out), _p(query_start_loc), _p(context_lens)
    if state is not None:
        _require(slot_idx is not None, "state needs slot_idx")
        _i32vec(slot_idx, S, "slot_idx")
        _require(state.dtype == torch.float32 and state.is_contiguous() and state.dim() == 2 and state.shape[1] == W,
                 "state must be contiguous fp32 [slots, W]")
        a.state, a.slot_idx = _p(state), _p(slot_idx)
    a.num_tokens, a.num_seqs, a.width, a.act_dtype, a.x_stride_t = T, S, W, _DT[out_dtype], x.stride(0)
    _C.check(_C.load().hymeta_token_shift(C.byref(a), _stream(x)), "hymeta_token_shift")
    return out


def add_group_norm(x: torch.Tensor, y: Optional[torch.Tensor], weight: torch.Tensor, groups: int, eps: float, alpha: float = 1.0,
                   y2: Optional[torch.Tensor] = None, in_place: bool = True, out_dtype: Optional[torch.dtype] = None):
    """``norm(alpha x + y (+ y2))`` with the RMS taken over each of ``groups`` equal consecutive parts of a row, times
    ``weight``.  ``in_place``: written back into the fp32 stream ``x [T, W]``; ``out_dtype``: (also) returned as a new tensor
    of that type (the rounded copy the next projections read).  Returns that tensor, or ``x``."""
    _dev(x, y, y2, weight)
    _require(x.dim() == 2 and x.dtype == torch.float32 and x.stride(1) == 1, "x must be row-contiguous fp32 [T, W]")
    T, W = x.shape
    _require(groups >= 1 and W % groups == 0, "the width must split into equal groups")
    _require(in_place or out_dtype is not None, "the result must go somewhere")
    _f32vec(weight, W, "weight")
    act = None
    for t, name in ((y, "y"), (y2, "y2")):
        if t is not None:
            _require(t.shape == (T, W) and t.stride(1) == 1 and t.dtype in _DT, f"{name} must be row-contiguous [T, W], bf16 or fp32")
            _require(act is None or act == t.dtype, "y and y2 must share a type")
            act = t.dtype
    if out_dtype is not None:
        _require(out_dtype in _DT and (act is None or act == out_dtype), "out_dtype must be the activations' type")
        act = out_dtype
    out = None if out_dtype is None else torch.empty(T, W, dtype=out_dtype, device=x.device)
    a = _C.AddGroupNormArgs()
    a.x, a.y, a.y2, a.weight, a.out = _p(x), _p(y), _p(y2), _p(weight), _p(out)
    a.num_tokens, a.width, a.groups, a.act_dtype, a.in_place = T, W, groups, _DT[act or torch.float32], int(in_place)
    a.eps, a.alpha, a.x_stride_t = eps, alpha, x.stride(0)
    a.y_stride_t, a.y2_stride_t = (0 if y is None else y.stride(0)), (0 if y2 is None else y2.stride(0))
    _C.check(_C.load().hymeta_add_group_norm(C.byref(a), _stream(x)), "hymeta_add_group_norm")
    return x if out is None else out


def latent_kv_prep_(proj: torch.Tensor, q_col: int, q_rank: int, kv_col: int, kv_rank: int, rot_dim: int, rot_dims: int,
                    q_norm_weight: torch.Tensor, kv_norm_weight: torch.Tensor, eps: float, rot_freqs: torch.Tensor, rot_mag: float,
                    kv_cache: Optional[torch.Tensor], slot_mapping: Optional[torch.Tensor], query_start_loc: torch.Tensor,
                    seq_lens: torch.Tensor) -> None:
    """On the rows ``proj [T, ...]`` of the fused down projections: RMS norm of the query latent (columns ``q_col ..``) in
    place; RMS norm of the key/value latent (columns ``kv_col ..``) and rotation of the ``rot_dim`` columns behind it,
    both written to ``kv_cache [blocks, block_size, 1, kv_rank + rot_dim]`` at ``slot_mapping``."""
    _dev(proj, q_norm_weight, kv_norm_weight, rot_freqs, kv_cache, slot_mapping, query_start_loc, seq_lens)
    _require(proj.dim() == 2 and proj.stride(1) == 1, "proj must be row-contiguous")
    T = proj.shape[0]
    _require(q_col + q_rank <= proj.shape[1] and kv_col + kv_rank + rot_dim <= proj.shape[1], "the latents' columns must lie inside proj")
    _f32vec(q_norm_weight, q_rank, "q_norm_weight")
    _f32vec(kv_norm_weight, kv_rank, "kv_norm_weight")
    _require(rot_freqs.dtype == torch.float64 and rot_freqs.is_contiguous() and rot_freqs.numel() * 2 >= rot_dims, "rot_freqs must be float64 [rot_dims / 2]")
    S = query_start_loc.numel() - 1
    _i32vec(query_start_loc, S + 1, "query_start_loc")
    _i32vec(seq_lens, S, "seq_lens")
    a = _C.LatentKvPrepArgs()
    a.proj, a.q_norm_weight, a.kv_norm_weight, a.rot_freqs = _p(proj), _p(q_norm_weight), _p(kv_norm_weight), _p(rot_freqs)
    a.query_start_loc, a.seq_lens = _p(query_start_loc), _p(seq_lens)
    a.num_tokens, a.num_seqs, a.q_rank, a.kv_rank, a.rot_dim, a.rot_dims, a.q_col, a.kv_col = T, S, q_rank, kv_rank, rot_dim, rot_dims, q_col, kv_col
    a.block_size, a.act_dtype, a.eps, a.rot_mag, a.proj_stride_t = 1, _act(proj), eps, rot_mag, proj.stride(0)
    if kv_cache is not None and kv_cache.numel() > 0 and slot_mapping is not None:
        _require(kv_cache.dtype == proj.dtype and kv_cache.is_contiguous() and kv_cache.dim() == 4 and kv_cache.shape[2:] == (1, kv_rank + rot_dim),
                 "kv_cache must be contiguous [blocks, block_size, 1, kv_rank + rot_dim]")
        _require(slot_mapping.dtype == torch.int64 and slot_mapping.is_contiguous() and slot_mapping.numel() == T, "slot_mapping must be int64 [T]")
        a.kv_cache, a.slot_mapping, a.num_blocks, a.block_size = _p(kv_cache), _p(slot_mapping), kv_cache.shape[0], kv_cache.shape[1]
    _C.check(_C.load().hymeta_latent_kv_prep(C.byref(a), _stream(proj)), "hymeta_latent_kv_prep")


def latent_q_assemble(q: torch.Tensor, q_abs: torch.Tensor, dim: int, rot_dim: int, rot_dims: int, rot_freqs: torch.Tensor,
                      rot_mag: float, query_start_loc: torch.Tensor, seq_lens: torch.Tensor) -> torch.Tensor:
    """``q [T, H, dim + rot_dim]`` and ``q_abs [H, T, C]`` -> ``[T, H, C + rot_dim]``: the absorbed part followed by the
    rotated part of every head's query."""
    _dev(q, q_abs, rot_freqs, query_start_loc, seq_lens)
    _require(q.dim() == 3 and q.stride(2) == 1 and q.stride(1) == dim + rot_dim and q.shape[2] == dim + rot_dim, "q must be [T, H, dim + rot_dim]")
    T, H, _ = q.shape
    _require(q_abs.dim() == 3 and q_abs.is_contiguous() and q_abs.shape[:2] == (H, T) and q_abs.dtype == q.dtype, "q_abs must be contiguous [H, T, C]")
    Ck = q_abs.shape[2]
    _require(rot_freqs.dtype == torch.float64 and rot_freqs.is_contiguous() and rot_freqs.numel() * 2 >= rot_dims, "rot_freqs must be float64 [rot_dims / 2]")
    S = query_start_loc.numel() - 1
    _i32vec(query_start_loc, S + 1, "query_start_loc")
    _i32vec(seq_lens, S, "seq_lens")
    out = torch.empty(T, H, Ck + rot_dim, dtype=q.dtype, device=q.device)
    a = _C.LatentQAssembleArgs()
    a.q, a.q_abs, a.out, a.rot_freqs, a.query_start_loc, a.seq_lens = _p(q), _p(q_abs), _p(out), _p(rot_freqs), _p(query_start_loc), _p(seq_lens)
    a.num_tokens, a.num_seqs, a.num_heads, a.dim, a.rot_dim, a.rot_dims, a.kv_rank, a.act_dtype = T, S, H, dim, rot_dim, rot_dims, Ck, _act(q)
    a.rot_mag, a.q_stride_t = rot_mag, q.stride(0)
    _C.check(_C.load().hymeta_latent_q_assemble(C.byref(a), _stream(q)), "hymeta_latent_q_assemble")
    return out


def lightning_attention(qkv: torch.Tensor, state: torch.Tensor, decay: torch.Tensor, num_heads: int, head_dim: int, v_dim: int,
                        query_start_loc: torch.Tensor, context_lens: torch.Tensor, slot_idx: torch.Tensor, max_query_len: int) -> torch.Tensor:
    """Linear attention with a decay per head over a step's rows: ``qkv [T, 2 H D + H Dv]`` (before their silu), ``state``
    fp32 ``[slots, H, D, Dv]`` read where ``context_lens > 0`` and written.  Returns fp32 ``[T, H Dv]``."""
    _dev(qkv, state, decay, query_start_loc, context_lens, slot_idx)
    H, D, Dv = num_heads, head_dim, v_dim
    _require(qkv.dim() == 2 and qkv.stride(1) == 1 and qkv.shape[1] >= H * (2 * D + Dv), "qkv must be row-contiguous [T, 2 H D + H Dv]")
    _require(state.dtype == torch.float32 and state.is_contiguous() and state.dim() == 4 and state.shape[1:] == (H, D, Dv),
             "state must be contiguous fp32 [slots, H, D, Dv]")
    _f32vec(decay, H, "decay")
    T = qkv.shape[0]
    S = query_start_loc.numel() - 1
    _i32vec(query_start_loc, S + 1, "query_start_loc")
    _i32vec(context_lens, S, "context_lens")
    _i32vec(slot_idx, S, "slot_idx")
    out = torch.empty(T, H * Dv, dtype=torch.float32, device=qkv.device)
    a = _C.LightningAttentionArgs()
    a.qkv, a.state, a.decay, a.out = _p(qkv), _p(state), _p(decay), _p(out)
    a.query_start_loc, a.context_lens, a.slot_idx = _p(query_start_loc), _p(context_lens), _p(slot_idx)
    a.num_tokens, a.num_seqs, a.num_heads, a.head_dim, a.v_dim, a.act_dtype, a.max_query_len = T, S, H, D, Dv, _act(qkv), max_query_len
    a.qkv_stride_t = qkv.stride(0)
    lib = _C.load()
    nbytes = int(lib.hymeta_lightning_attention_workspace_bytes(S, H, D, Dv, max_query_len))
    if nbytes:
        ws = _workspace(qkv.device, nbytes, "lightning")
        a.workspace, a.workspace_bytes = _p(ws), ws.numel()
    _C.check(lib.hymeta_lightning_attention(C.byref(a), _stream(qkv)), "hymeta_lightning_attention")
    return out


def gated_rms_norm(x: torch.Tensor, gate: torch.Tensor, weight: Optional[torch.Tensor], eps: float, groups: int = 1,
                   gate_act: str = "sigmoid", gate_first: bool = False) -> torch.Tensor:
    """``rmsnorm(x) * weight * sigmoid(gate)``: fp32 rows ``x [T, W]``, ``gate [T, W]`` in the activations' type, which
    is also the result's.  ``groups``: the root mean square is taken over each of that many equal consecutive parts of a row
    (per head, for instance).  ``gate_act``: ``"sigmoid"`` or ``"silu"``.  ``gate_first``: the gate multiplies ``x`` before
    the norm, ``rmsnorm(x * act(gate)) * weight``.  ``weight`` None: ones."""
    _require(gate_act in ("sigmoid", "silu"), "gate_act is sigmoid or silu")
    _require(groups >= 1 and x.shape[1] % groups == 0, "the width must split into equal groups")
    _dev(x, gate, weight)
    _require(x.dim() == 2 and x.dtype == torch.float32 and x.is_contiguous(), "x must be contiguous fp32 [T, W]")
    T, W = x.shape
    _require(gate.shape == (T, W) and gate.stride(1) == 1, "gate must be row-contiguous [T, W]")
    _f32vec(weight, W, "weight")
    out = torch.empty(T, W, dtype=gate.dtype, device=x.device)
    a = _C.GatedRmsNormArgs()
    a.x, a.gate, a.weight, a.out = _p(x), _p(gate), _p(weight), _p(out)
    a.num_tokens, a.width, a.act_dtype, a.eps, a.gate_stride_t = T, W, _act(gate), eps, gate.stride(0)
    a.groups, a.gate_act, a.gate_first = groups, (_C.GATE_SILU if gate_act == "silu" else _C.GATE_SIGMOID), int(bool(gate_first))
    _C.check(_C.load().hymeta_gated_rms_norm(C.byref(a), _stream(x)), "hymeta_gated_rms_norm")
    return out


def _activation(kind: int, x: torch.Tensor, n: int, p0: float, p1: float, gate: Optional[torch.Tensor] = None,
                out: Optional[torch.Tensor] = None, num_rows_dev: Optional[torch.Tensor] = None) -> torch.Tensor:
    _dev(x, gate, out, num_rows_dev)
    _require(x.dim() == 2 and x.stride(1) == 1, "x must be row-contiguous")
    rows = x.shape[0]
    if out is None:
        out = torch.empty(rows, n, dtype=x.dtype, device=x.device)
    _require(out.shape == (rows, n) and out.stride(1) == 1 and out.dtype == x.dtype, "out must be row-contiguous [rows, n] of x's type")
    a = _C.ActivationArgs()
    a.x, a.gate, a.out, a.num_rows_dev = _p(x), _p(gate), _p(out), _p(num_rows_dev)
    a.kind, a.num_rows, a.n, a.act_dtype, a.p0, a.p1 = kind, rows, n, _act(x), p0, p1
    a.x_stride, a.gate_stride, a.out_stride = x.stride(0), (0 if gate is None else gate.stride(0)), out.stride(0)
    _C.check(_C.load().hymeta_activation(C.byref(a), _stream(x)), "hymeta_activation")
    return out


def clamped_glu(x: torch.Tensor, limit: float, alpha: float = 1.702, out: Optional[torch.Tensor] = None,
                num_rows_dev: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``x [rows, 2 n]`` (gate columns, then up columns) -> ``g sigmoid(alpha g) (u + 1)`` with ``g = min(gate, limit)``,
    ``u = clamp(up, -limit, limit)``."""
    _require(x.shape[1] % 2 == 0, "x must hold the gate and the up columns")
    return _activation(_C.ACT_CLAMPED_GLU, x, x.shape[1] // 2, limit, alpha, out=out, num_rows_dev=num_rows_dev)


def xielu(x: torch.Tensor, a_pos: float, a_neg: float) -> torch.Tensor:
    """``z > 0: a_pos z^2 + z / 2``; ``z <= 0: a_neg (exp(z) - 1 - z) + z / 2``."""
    return _activation(_C.ACT_XIELU, x, x.shape[1], a_pos, a_neg)


def sigmoid_gate_mul(x: torch.Tensor, gate: torch.Tensor) -> torch.Tensor:
    """``x * sigmoid(gate)``, both ``[rows, n]``."""
    _require(gate.shape == x.shape and gate.stride(1) == 1 and gate.dtype == x.dtype, "gate must be row-contiguous, of x's shape and type")
    return _activation(_C.ACT_SIGMOID_MUL, x, x.shape[1], 0.0, 0.0, gate=gate)


ROUTE_SIGMOID_SUM, ROUTE_SOFTMAX_CHOSEN, ROUTE_SOFTMAX_GROUPED = _C.ROUTE_SIGMOID_SUM, _C.ROUTE_SOFTMAX_CHOSEN, _C.ROUTE_SOFTMAX_GROUPED


class GroupedChoice(NamedTuple):
    """What ``ROUTE_SOFTMAX_GROUPED`` needs beside the router's matrix: ``correction [outputs]`` added to the scores for the
    choice alone (None: nothing), ``groups`` equal runs of neighbouring outputs of which the ``keep`` best can be chosen
    from, the last ``identity`` outputs being identity experts, and ``extra_rows`` (0 or 1) more rows behind the router's
    whose sigmoid comes back as a gate of one number per token."""
    correction: Optional[torch.Tensor]
    groups: int = 1
    keep: int = 1
    identity: int = 0
    extra_rows: int = 0


def moe_sigmoid_forward(x: torch.Tensor, router_weight: torch.Tensor, w13: torch.Tensor, w2: torch.Tensor, top_k: int,
                        route_scale: float, limit: float, alpha: float = 1.702) -> torch.Tensor:
    """Experts chosen by the ``top_k`` largest ``sigmoid(x router_weight^T)`` (fp32), weighing their scores over the
    chosen's sum times ``route_scale``; every expert is a clamped gated unit (``clamped_glu``) between ``w13 [E, 2I, H]``
    (gate rows, then up rows) and ``w2 [E, H, I]``, all bf16 or all fp32.  bf16 experts in the MFMA tiles' shapes run the
    routed block's grouped GEMMs, everything else the generic grouped GEMM with the activation in its epilogue."""
    return moe_routed_forward(x, router_weight, None, w13, w2, top_k, _C.ROUTE_SIGMOID_SUM, route_scale, "clamped_glu", limit, alpha)


def moe_routed_forward(x: torch.Tensor, router_weight: torch.Tensor, router_bias: Optional[torch.Tensor], w1: torch.Tensor,
                       w2: torch.Tensor, top_k: int, score_mode: int, route_scale: float, expert_act: str, limit: float = 0.0,
                       alpha: float = 1.702, choice: Optional[GroupedChoice] = None):
    """Experts chosen by the ``top_k`` largest router logits ``x router_weight^T (+ router_bias)`` (fp32; the lower expert
    on a tie).  ``score_mode``: ``ROUTE_SIGMOID_SUM`` (weights = sigmoid scores over the chosen's sum),
    ``ROUTE_SOFTMAX_CHOSEN`` (softmax over the chosen logits alone) or ``ROUTE_SOFTMAX_GROUPED`` (softmax over all outputs,
    the choice by corrected scores within the best groups, identity experts: ``choice``), times ``route_scale``.
    ``expert_act``: ``"clamped_glu"``: ``w1 [E, 2I, H]`` (gate rows, then up rows), ``g sigmoid(alpha g) (u + 1)`` clamped at
    ``limit``; ``"silu_glu"``: the same rows, ``silu(g) u``; ``"relu2"``: ``w1 [E, I, H]``, ``max(z, 0)^2``.  ``w2 [E, H, I]``;
    all bf16 or all fp32.  bf16 experts in the MFMA tiles' shapes run the routed block's grouped GEMMs, everything else the
    generic grouped GEMM with the activation in its epilogue.  With ``choice`` the result is ``(out, identity_weight [T] or
    None, gate [T] or None)``: ``out`` holds the real experts' sum; the caller adds ``identity_weight[t] * x[t]``."""
    _dev(x, router_weight, router_bias, w1, w2)
    _require(expert_act in ("clamped_glu", "silu_glu", "relu2"), "expert_act is clamped_glu, silu_glu or relu2")
    _require((score_mode == _C.ROUTE_SOFTMAX_GROUPED) == (choice is not None), "the grouped choice comes with its constants")
    gated = expert_act != "relu2"
    T, H = x.shape
    E, n1, _ = w1.shape
    outputs = E if choice is None else E + choice.identity           # the router's outputs that enter the softmax
    rows = outputs if choice is None else outputs + choice.extra_rows
    inter = n1 // 2 if gated else n1
    _require(x.dtype in _DT and x.stride(1) == 1 and w1.dtype == x.dtype and w2.dtype == x.dtype, "x, w1 and w2 must share bf16 or fp32")
    _require(w1.is_contiguous() and w1.shape == (E, (2 if gated else 1) * inter, H) and w2.is_contiguous() and w2.shape == (E, H, inter),
             "w1 must be contiguous [E, 2I or I, H] and w2 [E, H, I]")
    _require(router_weight.dtype == torch.float32 and router_weight.is_contiguous() and router_weight.shape == (rows, H),
             "router_weight must be contiguous fp32 [router outputs (+ extra rows), H]")
    _f32vec(router_bias, E, "router_bias")
    dev = x.device
    out = torch.empty(T, H, dtype=x.dtype, device=dev)
    identity_weight = gate = None
    if choice is not None:
        _dev(x, choice.correction)
        _f32vec(choice.correction, outputs, "correction")
        _require(choice.groups >= 1 and outputs % choice.groups == 0 and 1 <= choice.keep <= choice.groups, "the outputs must split into equal groups")
        _require(choice.keep == choice.groups or choice.keep * (outputs // choice.groups) >= top_k, "the kept groups hold fewer outputs than top_k")
        _require(choice.extra_rows in (0, 1) and 0 <= choice.identity and top_k <= outputs, "extra_rows is 0 or 1")
        identity_weight = torch.empty(T, dtype=torch.float32, device=dev) if choice.identity else None
        gate = torch.empty(T, dtype=torch.float32, device=dev) if choice.extra_rows else None
    if T == 0:
        return out if choice is None else (out, identity_weight, gate)
    P = T * top_k
    ids = torch.empty(T, top_k, dtype=torch.int32, device=dev)
    wts = torch.empty(T, top_k, dtype=torch.float32, device=dev)
    offsets = torch.empty(E + 1, dtype=torch.int32, device=dev)
    sorted_pair = torch.empty(P, dtype=torch.int32, device=dev)
    pair_pos = torch.empty(P, dtype=torch.int32, device=dev)
    lib, st = _C.load(), _stream(x)
    r = _C.MoeRouteSigmoidArgs()
    r.x, r.router_weight, r.topk_ids, r.topk_weights = _p(x), _p(router_weight), _p(ids), _p(wts)
    r.expert_offsets, r.sorted_pair, r.pair_pos = _p(offsets), _p(sorted_pair), _p(pair_pos)
    r.num_tokens, r.num_experts, r.top_k, r.hidden, r.act_dtype, r.scale, r.x_stride_t = T, outputs, top_k, H, _act(x), route_scale, x.stride(0)
    r.router_bias, r.score_mode = _p(router_bias), score_mode
    if choice is not None:
        r.num_groups, r.keep_groups, r.first_identity, r.extra_rows = choice.groups, choice.keep, (E if choice.identity else 0), choice.extra_rows
        r.correction, r.identity_weight, r.extra_out = _p(choice.correction), _p(identity_weight), _p(gate)
    _C.check(lib.hymeta_moe_route_sigmoid(C.byref(r), st), "hymeta_moe_route_sigmoid")

    def result(o):
        return o if choice is None else (o, identity_weight, gate)

    if (x.dtype == torch.bfloat16 and moe_mfma_shapes(H, inter) and n1 % 64 == 0 and E <= 64 and x.stride(0) % 8 == 0 and x.data_ptr() % 16 == 0):
        h1 = torch.empty(P, n1, dtype=torch.bfloat16, device=dev)
        g = _C.MoeGemmArgs()
        g.x, g.weights, g.out, g.expert_offsets = _p(x), _p(w1), _p(h1), _p(offsets)
        g.a_rows, g.a_rows_div, g.max_rows, g.K, g.N = _p(sorted_pair), top_k, P, H, n1
        g.local_expert_begin, g.local_expert_end = 0, E
        g.x_stride_m, g.out_stride_m, g.w_stride_e = x.stride(0), h1.stride(0), w1.stride(0)
        _C.check(lib.hymeta_moe_gemm(C.byref(g), st), "hymeta_moe_gemm (w1)")
        hact = clamped_glu(h1, limit, alpha) if expert_act == "clamped_glu" else silu_mul(h1) if gated else relu_squared(h1, out=h1)
        y = torch.empty(P, H, dtype=torch.bfloat16, device=dev)
        d = _C.MoeGemmArgs()
        d.x, d.x_stride_m, d.weights, d.out, d.expert_offsets = _p(hact), hact.stride(0), _p(w2), _p(y), _p(offsets)
        d.scale_rows, d.row_scale = _p(sorted_pair), _p(wts)
        d.a_rows_div, d.max_rows, d.K, d.N = 1, P, inter, H
        d.local_expert_begin, d.local_expert_end = 0, E
        d.out_stride_m, d.w_stride_e = y.stride(0), w2.stride(0)
        _C.check(lib.hymeta_moe_gemm(C.byref(d), st), "hymeta_moe_gemm (w2)")
        c = _C.MoeCombineArgs()
        c.y, c.out, c.pair_pos, c.topk_weights = _p(y), _p(out), _p(pair_pos), _p(wts)
        c.num_tokens, c.hidden, c.top_k = T, H, top_k
        c.y_stride_m, c.out_stride_m = y.stride(0), out.stride(0)
        _C.check(lib.hymeta_moe_combine(C.byref(c), st), "hymeta_moe_combine")
        return result(out)

    act = _DT[x.dtype]
    hact = torch.empty(P, inter, dtype=x.dtype, device=dev)
    g = _C.MoeGemmAnyArgs()
    g.x, g.weights, g.out, g.expert_offsets = _p(x), _p(w1), _p(hact), _p(offsets)
    g.a_rows, g.a_rows_div, g.max_rows, g.K, g.N, g.num_experts, g.act_dtype = _p(sorted_pair), top_k, P, H, inter, E, act
    g.gated = _C.GLU_CLAMPED if expert_act == "clamped_glu" else _C.GLU_SILU if gated else _C.GLU_RELU2
    g.act_limit, g.act_alpha = limit, alpha
    g.x_stride_m, g.out_stride_m, g.w_stride_e = x.stride(0), hact.stride(0), w1.stride(0)
    _C.check(lib.hymeta_moe_gemm_any(C.byref(g), st), "hymeta_moe_gemm_any (w1)")
    y = torch.empty(P, H, dtype=x.dtype, device=dev)
    d = _C.MoeGemmAnyArgs()
    d.x, d.weights, d.out, d.expert_offsets = _p(hact), _p(w2), _p(y), _p(offsets)
    d.scale_rows, d.row_scale = _p(sorted_pair), _p(wts)
    d.a_rows_div, d.max_rows, d.K, d.N, d.num_experts, d.gated, d.act_dtype = 1, P, inter, H, E, _C.GLU_NONE, act
    d.x_stride_m, d.out_stride_m, d.w_stride_e = hact.stride(0), y.stride(0), w2.stride(0)
    _C.check(lib.hymeta_moe_gemm_any(C.byref(d), st), "hymeta_moe_gemm_any (w2)")
    c = _C.MoeCombineAnyArgs()
    c.y, c.out, c.pair_pos = _p(y), _p(out), _p(pair_pos)
    c.num_tokens, c.width, c.top_k, c.act_dtype = T, H, top_k, act
    c.y_stride_m, c.out_stride_m = y.stride(0), out.stride(0)
    _C.check(lib.hymeta_moe_combine_any(C.byref(c), st), "hymeta_moe_combine_any")
    return result(out)


def silu_mul(x: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``x [rows, 2 n]`` (gate columns, then up columns) -> ``gate sigmoid(gate) up``, bf16 or fp32 (``silu_and_mul`` is the
    bf16-only form of the quantised linears' path)."""
    _require(x.shape[1] % 2 == 0, "x must hold the gate and the up columns")
    return _activation(_C.ACT_SILU_MUL, x, x.shape[1] // 2, 0.0, 0.0, out=out)


def relu_squared(x: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``max(x, 0)^2`` (``out`` may be ``x``)."""
    return _activation(_C.ACT_RELU2, x, x.shape[1], 0.0, 0.0, out=out)


# ---------------------------------------------------------------------------
# Building blocks of pre-norm designs with several residual streams and head-mixed attention scores.
# ---------------------------------------------------------------------------
def embed_pair(token_ids: torch.Tensor, table: torch.Tensor, pair_table: Optional[torch.Tensor], norm_weight: Optional[torch.Tensor],
               eps: float, copies: int, buckets: int = 0, mul_prev: int = 0, mul_cur: int = 0, prev_token: Optional[torch.Tensor] = None,
               query_start_loc: Optional[torch.Tensor] = None, context_lens: Optional[torch.Tensor] = None,
               slot_idx: Optional[torch.Tensor] = None) -> torch.Tensor:
    """fp32 ``[T, copies, W]``: ``layer_norm(table[token] + pair_table[row]) * norm_weight`` in every copy, with ``row =
    (previous token * mul_prev + token * mul_cur) mod buckets`` and row ``buckets`` for a sequence's first token.
    ``prev_token`` int32 ``[slots]`` carries every sequence's last token between steps and is updated in place."""
    _dev(token_ids, table, pair_table, norm_weight, prev_token, query_start_loc, context_lens, slot_idx)
    _require(token_ids.dtype == torch.int64 and token_ids.dim() == 1 and token_ids.is_contiguous(), "token_ids must be contiguous int64 [T]")
    _require(table.dim() == 2 and table.is_contiguous(), "table must be contiguous [vocab, width]")
    V, W = table.shape
    T = token_ids.shape[0]
    _f32vec(norm_weight, W, "norm_weight")
    out = torch.empty(T, copies, W, dtype=torch.float32, device=table.device)
    a = _C.EmbedPairArgs()
    a.token_ids, a.table, a.norm_weight, a.out = _p(token_ids), _p(table), _p(norm_weight), _p(out)
    a.num_tokens, a.width, a.vocab, a.copies, a.act_dtype, a.eps = T, W, V, copies, _act(table), eps
    if pair_table is not None:
        _require(pair_table.dtype == table.dtype and pair_table.is_contiguous() and pair_table.shape == (buckets + 1, W),
                 "pair_table must be contiguous [buckets + 1, width] of the table's type")
        S = query_start_loc.numel() - 1
        _i32vec(query_start_loc, S + 1, "query_start_loc")
        _i32vec(context_lens, S, "context_lens")
        _i32vec(slot_idx, S, "slot_idx")
        _require(prev_token is not None and prev_token.dtype == torch.int32 and prev_token.is_contiguous(), "prev_token must be contiguous int32 [slots]")
        first_rows = torch.empty(max(S, 1), dtype=torch.int32, device=table.device)
        a.pair_table, a.prev_token, a.first_rows = _p(pair_table), _p(prev_token), _p(first_rows)
        a.query_start_loc, a.context_lens, a.slot_idx, a.num_seqs = _p(query_start_loc), _p(context_lens), _p(slot_idx), S
        a.buckets, a.mul_prev, a.mul_cur = buckets, mul_prev, mul_cur
    _C.check(_C.load().hymeta_embed_pair(C.byref(a), _stream(table)), "hymeta_embed_pair")
    return out


def hyper_stream_(x: torch.Tensor, y: Optional[torch.Tensor], mix: Optional[torch.Tensor], out_w: Optional[torch.Tensor],
                  in_w: Optional[torch.Tensor], norm_weight: Optional[torch.Tensor], eps: float,
                  h_dtype: Optional[torch.dtype]) -> Optional[torch.Tensor]:
    """One step of the residual streams ``x [T, S, W]`` fp32, in place: with ``y [T, W]``, ``x_t <- sum_s mix[s, t] x_s +
    out_w[t] y``; with ``h_dtype``, returns ``layer_norm(sum_s in_w[s] x_s) * norm_weight`` of the new streams in that
    type (``norm_weight`` None: the weighted sum itself)."""
    _dev(x, y, mix, out_w, in_w, norm_weight)
    _require(x.dtype == torch.float32 and x.dim() == 3 and x.is_contiguous(), "x must be contiguous fp32 [T, S, W]")
    T, S, W = x.shape
    _require(y is not None or h_dtype is not None, "nothing to do")
    a = _C.HyperStreamArgs()
    a.x, a.num_tokens, a.streams, a.width, a.eps = _p(x), T, S, W, eps
    act = h_dtype
    if y is not None:
        _require(y.dim() == 2 and y.shape == (T, W) and y.stride(1) == 1 and y.dtype in _DT, "y must be row-contiguous [T, W]")
        _f32vec(mix, S * S, "mix")
        _f32vec(out_w, S, "out_w")
        _require(h_dtype is None or h_dtype == y.dtype, "the sublayer's output and the next input share a type")
        a.y, a.mix, a.out_w, a.y_stride_t = _p(y), _p(mix), _p(out_w), y.stride(0)
        act = y.dtype
    h = None
    if h_dtype is not None:
        _f32vec(in_w, S, "in_w")
        _f32vec(norm_weight, W, "norm_weight")
        h = torch.empty(T, W, dtype=h_dtype, device=x.device)
        a.in_w, a.norm_weight, a.h_out = _p(in_w), _p(norm_weight), _p(h)
    a.act_dtype = _DT[act]
    _C.check(_C.load().hymeta_hyper_stream(C.byref(a), _stream(x)), "hymeta_hyper_stream")
    return h


def talk_qkv_prep(qkv: torch.Tensor, num_heads: int, num_kv_heads: int, head_dim: int, v_dim: int, q_weight: torch.Tensor,
                  k_weight: torch.Tensor, talk: torch.Tensor, eps: float, rot_dims: int, rot_freqs: Optional[torch.Tensor],
                  kv_cache: torch.Tensor, slot_mapping: torch.Tensor, query_start_loc: torch.Tensor, seq_lens: torch.Tensor,
                  v_other: Optional[torch.Tensor] = None, v_blend: float = 0.0, positions: Optional[torch.Tensor] = None) -> torch.Tensor:
    """From ``qkv [T, H D + G D + G Dv]``: RMS norms over the whole query and key projections, rotation of the first
    ``rot_dims`` dimensions of every head in interleaved pairs, values blended with ``v_other`` (``(1 - v_blend) v + v_blend
    v_other``), the paged write of ``(keys of all G heads, values of all G heads)`` into ``kv_cache [blocks, block_size, 1,
    G D + G Dv]``; returns the queries mixed across heads, ``[T, H, G D]``: ``out[h, g D + d] = sum_j talk[h, j] q[j, d]``
    over the query heads ``j`` of group ``g``.  ``positions`` int64 ``[T]``: the rows' positions where the caller has them
    (otherwise they follow from ``query_start_loc`` and ``seq_lens``)."""
    _dev(qkv, q_weight, k_weight, talk, rot_freqs, kv_cache, slot_mapping, query_start_loc, seq_lens, v_other, positions)
    T = qkv.shape[0]
    H, G, D, Dv = num_heads, num_kv_heads, head_dim, v_dim
    _require(qkv.dim() == 2 and qkv.stride(1) == 1 and qkv.shape[1] == (H + G) * D + G * Dv and qkv.dtype in _DT,
             "qkv must be row-contiguous [T, H D + G D + G Dv]")
    _f32vec(q_weight, H * D, "q_weight")
    _f32vec(k_weight, G * D, "k_weight")
    _f32vec(talk, H * H, "talk")
    _require(rot_dims == 0 or (rot_freqs is not None and rot_freqs.dtype == torch.float64 and rot_freqs.is_contiguous()
                               and rot_freqs.numel() == rot_dims // 2), "rot_freqs must be contiguous float64 [rot_dims / 2]")
    _require(kv_cache.dtype == qkv.dtype and kv_cache.is_contiguous() and kv_cache.dim() == 4 and kv_cache.shape[2:] == (1, G * (D + Dv)),
             "kv_cache must be contiguous [blocks, block_size, 1, G D + G Dv]")
    _require(slot_mapping.dtype == torch.int64 and slot_mapping.is_contiguous() and slot_mapping.numel() == T, "slot_mapping must be int64 [T]")
    S = query_start_loc.numel() - 1
    _i32vec(query_start_loc, S + 1, "query_start_loc")
    _i32vec(seq_lens, S, "seq_lens")
    q_out = torch.empty(T, H, G * D, dtype=qkv.dtype, device=qkv.device)
    a = _C.TalkQkvPrepArgs()
    a.qkv, a.q_weight, a.k_weight, a.talk, a.rot_freqs, a.q_out = _p(qkv), _p(q_weight), _p(k_weight), _p(talk), _p(rot_freqs), _p(q_out)
    a.kv_cache, a.slot_mapping, a.query_start_loc, a.seq_lens = _p(kv_cache), _p(slot_mapping), _p(query_start_loc), _p(seq_lens)
    a.num_tokens, a.num_seqs, a.num_heads, a.num_kv_heads, a.head_dim, a.v_dim, a.rot_dims = T, S, H, G, D, Dv, rot_dims
    a.block_size, a.num_blocks, a.act_dtype, a.eps, a.qkv_stride_t = kv_cache.shape[1], kv_cache.shape[0], _act(qkv), eps, qkv.stride(0)
    if v_other is not None:
        _require(v_other.dim() == 2 and v_other.shape == (T, G * Dv) and v_other.stride(1) == 1 and v_other.dtype == qkv.dtype,
                 "v_other must be row-contiguous [T, G Dv] of qkv's type")
        a.v_other, a.v_other_stride_t, a.v_blend = _p(v_other), v_other.stride(0), v_blend
    if positions is not None:
        _require(positions.dtype == torch.int64 and positions.is_contiguous() and positions.numel() == T, "positions must be contiguous int64 [T]")
        a.positions = _p(positions)
    _C.check(_C.load().hymeta_talk_qkv_prep(C.byref(a), _stream(qkv)), "hymeta_talk_qkv_prep")
    return q_out


# ---------------------------------------------------------------------------
# Building blocks of parallel-layer designs (one norm, mixer and feed-forward side by side) with rotate-half rotary
# attention, retention and state-space mixers.
# ---------------------------------------------------------------------------
def stream_add_norm_(x: torch.Tensor, terms: Sequence[Tuple[torch.Tensor, float, Optional[torch.Tensor]]], norm_scale: Optional[float],
                     eps: float, out_dtype: Optional[torch.dtype] = None, norm_weight: Optional[torch.Tensor] = None) -> Optional[torch.Tensor]:
    """``x += sum_i coef_i * (row_scale_i[t] or 1) * y_i`` on the fp32 rows ``x [T, W]``, in place; ``terms`` lists ``(y_i [T, W]
    activations, coef_i, row_scale_i fp32 [T] or None)``.  With ``norm_scale`` also returns ``x / sqrt(mean(x^2) + eps) *
    norm_scale (* norm_weight)`` of the new rows in ``out_dtype``: a parallel layer's sum and the next norm, one launch."""
    _require(x.dim() == 2 and x.dtype == torch.float32 and x.stride(1) == 1, "x must be row-contiguous fp32 [T, W]")
    _require(len(terms) <= _C.STREAM_MAX_TERMS, f"at most {_C.STREAM_MAX_TERMS} terms")
    _require(terms or norm_scale is not None, "nothing to do")
    T, W = x.shape
    act = out_dtype
    a = _C.StreamAddNormArgs()
    for i, (y, coef, row_scale) in enumerate(terms):
        _dev(x, y, row_scale)
        _require(y.shape == (T, W) and y.stride(1) == 1 and y.dtype in _DT and (act is None or act == y.dtype), "terms must be row-contiguous [T, W] of one type")
        _f32vec(row_scale, T, "row_scale")
        act = y.dtype
        a.y[i], a.row_scale[i], a.coef[i], a.y_stride_t[i] = _p(y), _p(row_scale), float(coef), y.stride(0)
    _require(act in _DT, "out_dtype must be bf16 or fp32")
    _f32vec(norm_weight, W, "norm_weight")
    h = torch.empty(T, W, dtype=act, device=x.device) if norm_scale is not None else None
    a.x, a.norm_weight, a.h_out = _p(x), _p(norm_weight), _p(h)
    a.num_tokens, a.width, a.num_terms, a.act_dtype = T, W, len(terms), _DT[act]
    a.eps, a.norm_scale, a.x_stride_t = eps, float(norm_scale or 0.0), x.stride(0)
    _C.check(_C.load().hymeta_stream_add_norm(C.byref(a), _stream(x)), "hymeta_stream_add_norm")
    return h


def rotary_cache_(qkv: torch.Tensor, num_heads: int, num_kv_heads: int, head_dim: int, v_dim: int, rot_dims: int,
                  rot_freqs: Optional[torch.Tensor], k_scale: float = 1.0, kv_cache: Optional[torch.Tensor] = None,
                  slot_mapping: Optional[torch.Tensor] = None, positions: Optional[torch.Tensor] = None,
                  query_start_loc: Optional[torch.Tensor] = None, seq_lens: Optional[torch.Tensor] = None) -> None:
    """On the rows ``qkv [T, H D + G D + G Dv (+ ...)]`` of a fused projection, in place: dimensions ``i`` and ``i + rot_dims / 2``
    of every query and key head turn by ``position * rot_freqs[i]`` (``rot_freqs`` float64 ``[rot_dims / 2]``), keys are
    multiplied by ``k_scale``, and with ``kv_cache [blocks, block_size, G, D + Dv]`` the keys and values are written at
    ``slot_mapping``.  Positions: ``positions`` (int64) or the rows' places in their sequences (``query_start_loc``, ``seq_lens``)."""
    _dev(qkv, rot_freqs, kv_cache, slot_mapping, positions, query_start_loc, seq_lens)
    H, G, D, Dv = num_heads, num_kv_heads, head_dim, v_dim
    T = qkv.shape[0]
    _require(qkv.dim() == 2 and qkv.stride(1) == 1 and qkv.shape[1] >= (H + G) * D + (G * Dv if kv_cache is not None else 0),
             "qkv must be row-contiguous [T, H D + G D + G Dv (+ ...)]")
    _require(rot_dims % 2 == 0 and 0 <= rot_dims <= D, "rot_dims must be even and fit a head")
    a = _C.RotaryCacheArgs()
    if rot_dims:
        _require(rot_freqs is not None and rot_freqs.dtype == torch.float64 and rot_freqs.is_contiguous() and rot_freqs.numel() == rot_dims // 2,
                 "rot_freqs must be contiguous float64 [rot_dims / 2]")
        if positions is not None:
            _require(positions.dtype == torch.int64 and positions.is_contiguous() and positions.numel() == T, "positions must be int64 [T]")
        else:
            _require(query_start_loc is not None and seq_lens is not None, "positions or the step's sequence layout")
    if positions is None and query_start_loc is not None:
        S = query_start_loc.numel() - 1
        _i32vec(query_start_loc, S + 1, "query_start_loc")
        _i32vec(seq_lens, S, "seq_lens")
        a.query_start_loc, a.seq_lens, a.num_seqs = _p(query_start_loc), _p(seq_lens), S
    a.qkv, a.rot_freqs, a.positions = _p(qkv), _p(rot_freqs), _p(positions)
    a.num_tokens, a.num_heads, a.num_kv_heads, a.head_dim, a.v_dim, a.rot_dims = T, H, G, D, Dv, rot_dims
    a.act_dtype, a.k_scale, a.qkv_stride_t, a.block_size = _act(qkv), float(k_scale), qkv.stride(0), 1
    if kv_cache is not None:
        _require(kv_cache.dtype == qkv.dtype and kv_cache.is_contiguous() and kv_cache.dim() == 4 and kv_cache.shape[2:] == (G, D + Dv),
                 "kv_cache must be contiguous [blocks, block_size, G, D + Dv]")
        _require(slot_mapping is not None and slot_mapping.dtype == torch.int64 and slot_mapping.is_contiguous() and slot_mapping.numel() == T,
                 "slot_mapping must be int64 [T]")
        a.kv_cache, a.slot_mapping, a.num_blocks, a.block_size = _p(kv_cache), _p(slot_mapping), kv_cache.shape[0], kv_cache.shape[1]
    _C.check(_C.load().hymeta_rotary_cache(C.byref(a), _stream(qkv)), "hymeta_rotary_cache")


def causal_conv_silu(x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor], conv_state: Optional[torch.Tensor],
                     query_start_loc: torch.Tensor, context_lens: torch.Tensor, slot_idx: Optional[torch.Tensor],
                     dt_in: Optional[torch.Tensor] = None, dt_bias: Optional[torch.Tensor] = None, a_log: Optional[torch.Tensor] = None,
                     max_query_len: Optional[int] = None):
    """``silu(bias + sum_j weight[:, j] x[t - taps + 1 + j])`` per channel over each sequence's rows of ``x [T, C]`` (a view
    with any row stride); ``weight`` fp32 ``[C, taps]``; ``conv_state [slots, taps - 1, C]`` (x's type) carries a sequence's
    last input rows between steps, in place.  With ``dt_in [T, heads]`` also returns fp32 ``softplus(dt_in + dt_bias)`` and
    ``-exp(a_log) dt log2(e)``, both ``[T, heads]``: a state-space layer's step sizes and log2 decays.  ``max_query_len`` 1
    (every sequence brings one row): the state moves on in the same launch.  Returns ``out`` or ``(out, dt, log2_decay)``."""
    _dev(x, weight, bias, conv_state, query_start_loc, context_lens, slot_idx, dt_in, dt_bias, a_log)
    _require(x.dim() == 2 and x.stride(1) == 1 and x.dtype in _DT, "x must be row-contiguous [T, C], bf16 or fp32")
    T, Cn = x.shape
    taps = weight.shape[1]
    _require(weight.dtype == torch.float32 and weight.is_contiguous() and weight.shape == (Cn, taps) and 1 <= taps <= _C.CONV_MAX_TAPS,
             f"weight must be contiguous fp32 [C, taps <= {_C.CONV_MAX_TAPS}]")
    _f32vec(bias, Cn, "bias")
    S = query_start_loc.numel() - 1
    _i32vec(query_start_loc, S + 1, "query_start_loc")
    _i32vec(context_lens, S, "context_lens")
    out = torch.empty(T, Cn, dtype=x.dtype, device=x.device)
    a = _C.CausalConvArgs()
    a.x, a.weight, a.bias, a.out = _p(x), _p(weight), _p(bias), _p(out)
    a.query_start_loc, a.context_lens = _p(query_start_loc), _p(context_lens)
    a.num_tokens, a.num_seqs, a.channels, a.taps, a.act_dtype, a.x_stride_t = T, S, Cn, taps, _act(x), x.stride(0)
    a.single_rows = int(max_query_len == 1 and T == S)
    if conv_state is not None and taps > 1:
        _require(slot_idx is not None, "conv_state needs slot_idx")
        _i32vec(slot_idx, S, "slot_idx")
        _require(conv_state.dtype == x.dtype and conv_state.is_contiguous() and conv_state.dim() == 3 and conv_state.shape[1:] == (taps - 1, Cn),
                 "conv_state must be contiguous [slots, taps - 1, C] of x's type")
        a.conv_state, a.slot_idx = _p(conv_state), _p(slot_idx)
    dt = ld = None
    if dt_in is not None:
        Hh = dt_in.shape[1]
        _require(dt_in.dim() == 2 and dt_in.shape[0] == T and dt_in.stride(1) == 1 and dt_in.dtype == x.dtype, "dt_in must be [T, heads] of x's type")
        _f32vec(dt_bias, Hh, "dt_bias")
        _f32vec(a_log, Hh, "a_log")
        _require(dt_bias is not None and a_log is not None, "dt_in comes with dt_bias and a_log")
        dt = torch.empty(T, Hh, dtype=torch.float32, device=x.device)
        ld = torch.empty(T, Hh, dtype=torch.float32, device=x.device)
        a.dt_in, a.dt_bias, a.a_log, a.dt_out, a.log2_decay_out, a.dt_heads, a.dt_stride_t = _p(dt_in), _p(dt_bias), _p(a_log), _p(dt), _p(ld), Hh, dt_in.stride(0)
    _C.check(_C.load().hymeta_causal_conv(C.byref(a), _stream(x)), "hymeta_causal_conv")
    return out if dt_in is None else (out, dt, ld)


def decay_scan(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, state: torch.Tensor, query_start_loc: torch.Tensor,
               context_lens: torch.Tensor, slot_idx: torch.Tensor, max_query_len: int, decay: Optional[torch.Tensor] = None,
               log2_decay: Optional[torch.Tensor] = None, v_scale: Optional[torch.Tensor] = None, skip: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``S_t = a_t S_{t-1} + b_t k_t v_t^T``, ``out_t = S_t^T q_t + skip[h] v_t`` over a step's rows: ``q, k [T, Hqk, D]`` and
    ``v [T, H, Dv]`` (views with any row stride; head ``h`` reads query / key head ``h // (H / Hqk)``), ``state`` fp32
    ``[slots, H, D, Dv]`` read where ``context_lens > 0`` and written.  ``a_t``: ``decay [H]`` for every token, or
    ``2 ** log2_decay[t, h]``; ``b_t``: ``v_scale [T, H]`` or 1.  Returns fp32 ``[T, H Dv]``."""
    _dev(q, k, v, state, query_start_loc, context_lens, slot_idx, decay, log2_decay, v_scale, skip)
    _require(q.dim() == 3 and k.shape == q.shape and v.dim() == 3 and q.dtype == k.dtype == v.dtype and q.dtype in _DT, "q, k [T, Hqk, D] and v [T, H, Dv] of one type")
    T, Hqk, D = q.shape
    H, Dv = v.shape[1], v.shape[2]
    for t_, n_ in ((q, D), (k, D), (v, Dv)):
        _require(t_.shape[0] == T and t_.stride(2) == 1 and t_.stride(1) == n_, "heads must be contiguous in a row")
    _require(H % Hqk == 0, "the heads must split over the query / key heads")
    _require(state.dtype == torch.float32 and state.is_contiguous() and state.dim() == 4 and state.shape[1:] == (H, D, Dv),
             "state must be contiguous fp32 [slots, H, D, Dv]")
    _require((decay is None) != (log2_decay is None), "decay [H] or log2_decay [T, H]")
    _f32vec(decay, H, "decay")
    _f32vec(log2_decay, T * H, "log2_decay")
    _f32vec(v_scale, T * H, "v_scale")
    _f32vec(skip, H, "skip")
    S = query_start_loc.numel() - 1
    _i32vec(query_start_loc, S + 1, "query_start_loc")
    _i32vec(context_lens, S, "context_lens")
    _i32vec(slot_idx, S, "slot_idx")
    out = torch.empty(T, H * Dv, dtype=torch.float32, device=q.device)
    a = _C.DecayScanArgs()
    a.q, a.k, a.v, a.state, a.out = _p(q), _p(k), _p(v), _p(state), _p(out)
    a.decay, a.log2_decay, a.v_scale, a.skip = _p(decay), _p(log2_decay), _p(v_scale), _p(skip)
    a.query_start_loc, a.context_lens, a.slot_idx = _p(query_start_loc), _p(context_lens), _p(slot_idx)
    a.num_tokens, a.num_seqs, a.num_heads, a.num_qk_heads, a.head_dim, a.v_dim = T, S, H, Hqk, D, Dv
    a.act_dtype, a.max_query_len = _act(q), max_query_len
    a.q_stride_t, a.k_stride_t, a.v_stride_t = q.stride(0), k.stride(0), v.stride(0)
    lib = _C.load()
    nbytes = int(lib.hymeta_decay_scan_workspace_bytes(S, H, D, Dv, max_query_len))
    if nbytes:
        ws = _workspace(q.device, nbytes, "decay_scan")
        a.workspace, a.workspace_bytes = _p(ws), ws.numel()
    _C.check(lib.hymeta_decay_scan(C.byref(a), _stream(q)), "hymeta_decay_scan")
    return out
