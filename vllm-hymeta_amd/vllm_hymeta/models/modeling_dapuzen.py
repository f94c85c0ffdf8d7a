"""The Dapuzen decoder: a scaled token embedding into an fp32 residual stream; parallel layers (``h = norm(x)`` with a
one-number RMS norm, ``x <- x + mixer(h) + ff(h)``) whose mixer is a windowed rotary softmax attention with a sigmoid gate
per head, a retention, or a windowed tanh-capped attention beside a Mamba-2 state-space layer; the feed-forward is dense
(xIELU) or a mixture of silu-gated experts with a softmax router, a corrected group-limited choice, identity experts and a
gated shared expert.  A layer may run with an earlier layer's weights and a cache and state of its own.  The output
projection has a matrix of its own.

The class has the surface of the package's other model classes (``GLAswaForCausalLM``, ``SonuzenForCausalLM``,
``GeponexForCausalLM``, ``LidizenForCausalLM``): ``forward(input_ids, positions, attn_metadata=..., request_ids_to_seq_ids=...,
finished_requests_ids=...)`` returns the final hidden states of the step's rows, ``compute_logits`` the fp32 logits of the
rows asked for, ``load_weights`` takes the checkpoint as a stream of named tensors; the attention layers are found by name
and bound to paged caches by whoever drives the model, the recurrent and convolution states live in a slot-indexed cache
that follows the requests' ids.
"""

from __future__ import annotations

from typing import Dict, Iterable, List, Optional, Set, Tuple

import torch

from .. import hip_ops
from .._compat import HasInnerState, IsHybrid
from ..linear import HymetaLinear
from ..lm_head import lm_head_logits
from ..state_cache import ConstantSizeStateCache
from .attention import bind_kv_cache, current_attn_metadata, standalone_prefix
from .configuration_dapuzen import DapuzenConfig, DenseMlpSpec, GroupedMoeSpec, RetentionSpec, SideBySideSpec, WindowAttentionSpec
from .feed_forward import GroupedSoftmaxMoE, SiluGluMLP, XieluMLP
from .parallel_block import ParallelBlock, SideBySideMixer
from .retention import RetentionMixer
from .rotary_window_attention import PagedWindowAttention, WindowAttentionMixer
from .state_space import StateSpaceMixer
from .stream_block import StepLayout


class DapuzenStateCache(ConstantSizeStateCache):
    """Per layer with a recurrence, fp32 ``[1, slots, heads, D, Dv]`` (a retention's or a state-space layer's matrix state),
    and per state-space layer ``[1, slots, taps - 1, channels]`` in the activations' type (its convolution's last inputs).  A
    slot needs no clearing when it changes hands: a sequence's first step does not read it."""

    def __init__(self, recurrent_shapes: List[Tuple[int, int, int]], conv_shapes: List[Tuple[int, int]], act_dtype: torch.dtype,
                 max_batch_size: int, device):
        super().__init__(max_batch_size, device)
        self.recurrent = [torch.zeros(1, max_batch_size, *s, dtype=torch.float32, device=self.device) for s in recurrent_shapes]
        self.conv = [torch.zeros(1, max_batch_size, *s, dtype=act_dtype, device=self.device) for s in conv_shapes]

    @property
    def cache(self):
        return (self.recurrent, self.conv)

    def _slot_tensors(self):
        return tuple(self.recurrent) + tuple(self.conv)


def _paged(spec: WindowAttentionSpec, name: str, dtype: torch.dtype) -> PagedWindowAttention:
    return PagedWindowAttention(spec.heads, spec.kv_heads, spec.dim, spec.vdim, spec.scale, name, sliding_window=spec.window,
                                softcap=spec.softcap, dtype=dtype)


class DapuzenModel(torch.nn.Module):
    def __init__(self, config: DapuzenConfig, max_num_seqs: int = 256, dtype: torch.dtype = torch.bfloat16, device="cuda",
                 prefix: Optional[str] = None):
        super().__init__()
        if dtype not in (torch.bfloat16, torch.float32):
            raise ValueError("Dapuzen runs in bfloat16 or float32")
        self.config, self.dtype, self.device = config, dtype, torch.device(device)
        self.prefix = standalone_prefix("model") if prefix is None else prefix
        # the cache-owning attention layers exist from construction on (an engine sizes its pages from them); a layer that
        # runs with another's weights still has a cache and states of its own
        self.attn_layers = torch.nn.ModuleDict()
        self._recurrent_index: Dict[int, int] = {}
        self._conv_index: Dict[int, int] = {}
        recurrent: List[Tuple[int, int, int]] = []
        conv: List[Tuple[int, int]] = []
        for i, spec in enumerate(config.layers):
            m = spec.mixer
            if isinstance(m, WindowAttentionSpec):
                self.attn_layers[str(i)] = _paged(m, f"{self.prefix}.layers.{i}.attn", dtype)
            elif isinstance(m, RetentionSpec):
                self._recurrent_index[i] = len(recurrent)
                recurrent.append((m.heads, m.dim, m.vdim))
            else:
                self.attn_layers[str(i)] = _paged(m.left, f"{self.prefix}.layers.{i}.attn", dtype)
                self._recurrent_index[i] = len(recurrent)
                recurrent.append((m.right.heads, m.right.state, m.right.vdim))
                self._conv_index[i] = len(conv)
                conv.append((max(m.right.conv - 1, 1), m.right.conv_channels))
        self.state_cache = DapuzenStateCache(recurrent, conv, dtype, max_num_seqs, self.device)
        self.embed: Optional[torch.Tensor] = None
        self.head: Optional[torch.Tensor] = None
        self.final_norm_scale = 1.0
        self.blocks = torch.nn.ModuleDict()          # by the index of the layer that owns the tensors

    def layout_of(self, attn_metadata, slot_idx: torch.Tensor, token_ids: torch.Tensor, positions: Optional[torch.Tensor]) -> StepLayout:
        md = attn_metadata
        max_seq = max(md.seq_lens) if md.seq_lens else max(md.max_prefill_seq_len, md.max_decode_seq_len)
        return StepLayout(query_start_loc=md.query_start_loc, context_lens=md.context_lens_tensor, seq_lens=md.seq_lens_tensor,
                          slot_idx=slot_idx, block_tables=md.block_tables, slot_mapping=md.slot_mapping,
                          max_query_len=int(md.max_query_len or 1), max_seq_len=int(max_seq), token_ids=token_ids, positions=positions)

    def _mixer_state(self, i: int, recurrent, conv):
        spec = self.config.layers[i].mixer
        if isinstance(spec, WindowAttentionSpec):
            return self.attn_layers[str(i)]
        if isinstance(spec, RetentionSpec):
            return recurrent[self._recurrent_index[i]][0]
        return (self.attn_layers[str(i)], (recurrent[self._recurrent_index[i]][0], conv[self._conv_index[i]][0]))

    def forward(self, input_ids: torch.Tensor, positions: Optional[torch.Tensor] = None, attn_metadata=None,
                kv_caches: Optional[List[torch.Tensor]] = None, residual_out: Optional[List[torch.Tensor]] = None,
                **kwargs) -> torch.Tensor:
        """``positions`` (int64, one per row) spare the rotation a lookup of the row's sequence; without them a row's position
        is its sequence's length minus the rows behind it, which is also what the attention's mask goes by.  ``kv_caches``:
        one page tensor per attention layer, in layer order, bound before the step (callers without an engine).
        ``residual_out``: a list that receives a copy of the stream after every layer (debugging)."""
        if kv_caches is not None:
            for layer, kv in zip(self.attn_layers.values(), kv_caches):
                bind_kv_cache(layer, kv)
        md = attn_metadata if attn_metadata is not None else current_attn_metadata()
        if md is None:
            raise RuntimeError("DapuzenModel.forward needs the step's attention metadata")
        kwargs.setdefault("request_ids_to_seq_ids", {})
        kwargs.setdefault("finished_requests_ids", [])
        (recurrent, conv), slot_idx = self.state_cache.current_run_tensors(**kwargs)
        input_ids = input_ids.to(torch.int64).contiguous()
        if positions is not None:
            positions = positions.to(torch.int64).contiguous()
        layout = self.layout_of(md, slot_idx, input_ids, positions)
        cfg = self.config
        x = hip_ops.embed_rows(input_ids, self.embed, scale=cfg.embedding_scale)
        n = len(cfg.layers)
        h = self.blocks[str(cfg.layers[0].weights_of)].read(x, self.dtype) if n else None
        for i, spec in enumerate(cfg.layers):
            block = self.blocks[str(spec.weights_of)]
            nxt = self.blocks[str(cfg.layers[i + 1].weights_of)].norm_scale if i + 1 < n else self.final_norm_scale
            h = block(x, h, layout, self._mixer_state(i, recurrent, conv), nxt)
            if residual_out is not None:
                residual_out.append(x.clone())
        if h is None:
            h = hip_ops.stream_add_norm_(x, [], self.final_norm_scale, cfg.norm_eps, self.dtype)
        return h


class DapuzenForCausalLM(torch.nn.Module, HasInnerState, IsHybrid):
    # csrc/*.hip sources whose kernels this class calls (a first run in a fresh checkout builds these, see _C.build_library)
    kernel_sources = ("api_misc", "norm_conv", "parallel_ops", "decay_scan", "lightning", "sink_attn", "gated_ops", "moe_sigmoid",
                      "moe_table", "moe", "glue", "dense_gemm", "stream_gemm", "tall_gemm")

    def __init__(self, config: Optional[DapuzenConfig] = None, max_num_seqs: int = 256, dtype: torch.dtype = torch.bfloat16,
                 device="cuda", *, vllm_config=None, prefix: Optional[str] = None):
        super().__init__()
        if vllm_config is not None:
            mc = vllm_config.model_config
            config = mc.hf_config if isinstance(mc.hf_config, DapuzenConfig) else DapuzenConfig(mc.hf_config.to_dict())
            max_num_seqs = int(vllm_config.scheduler_config.max_num_seqs)
            dtype = getattr(mc, "dtype", dtype)
            device = getattr(getattr(vllm_config, "device_config", None), "device", None) or device
            prefix = f"{prefix}.model" if prefix else "model"
        if config is None:
            raise TypeError("DapuzenForCausalLM needs vllm_config= or a DapuzenConfig")
        self.config = config
        self.model = DapuzenModel(config, max_num_seqs=max_num_seqs, dtype=dtype, device=device, prefix=prefix)

    # what an engine asks a model with states of its own (the package's other model classes answer the same calls)
    def copy_inputs_before_cuda_graphs(self, input_buffers, **kwargs):
        return self.model.state_cache.copy_inputs_before_cuda_graphs(input_buffers, **kwargs)

    def get_seqlen_agnostic_capture_inputs(self, batch_size: int):
        return self.model.state_cache.get_seqlen_agnostic_capture_inputs(batch_size)

    def forward(self, input_ids, positions=None, intermediate_tensors=None, inputs_embeds=None, **kwargs):
        return self.model(input_ids, positions, **kwargs)

    def compute_logits(self, hidden_states: torch.Tensor, sampling_metadata=None) -> torch.Tensor:
        idx = getattr(sampling_metadata, "selected_token_indices", None)
        if idx is not None:
            hidden_states = hidden_states.index_select(0, idx)
        return lm_head_logits(hidden_states, self.model.head)

    # ------------------------------------------------------------------ weights
    def load_weights(self, weights: Iterable[Tuple[str, torch.Tensor]]) -> Set[str]:
        """Checkpoint names: ``embed``, ``head``, ``final.norm``, and per layer with tensors of its own ``l<i>.norm1`` (one
        number); ``l<i>.mix.<q|k|v|g|o>`` (attention: ``g`` one row per head), ``l<i>.mix.<q|k|v|g|o>`` (retention),
        ``l<i>.mix.left.<q|k|v|o>`` with ``.b`` biases and ``l<i>.mix.right.<in|conv|conv.b|dt_bias|A_log|D|norm|o>`` (parallel);
        ``l<i>.mlp.<up|down|act>`` (dense) or ``l<i>.mlp.<router|correction|e<j>.gate|e<j>.up|e<j>.down|shared.gate|shared.up|
        shared.down|shared.sg>``.  Linear weights ``[out, in]``."""
        cfg, m = self.config, self.model
        dev, dt = m.device, m.dtype
        got: Dict[str, torch.Tensor] = dict(weights)
        loaded: Set[str] = set()

        def take(name: str, shape: Optional[Tuple[int, ...]] = None) -> torch.Tensor:
            if name not in got:
                raise KeyError(f"checkpoint has no tensor {name!r}")
            loaded.add(name)
            t = got[name]
            if shape is not None and tuple(t.shape) != tuple(shape):
                raise ValueError(f"{name} is {tuple(t.shape)}, the configuration says {tuple(shape)}")
            return t

        def act(name: str, shape=None) -> torch.Tensor:
            return take(name, shape).to(device=dev, dtype=dt).contiguous()

        def f32(name: str, shape=None) -> torch.Tensor:
            return take(name, shape).to(device=dev, dtype=torch.float32).contiguous()

        def number(name: str) -> float:
            t = take(name)
            if t.numel() != 1:
                raise ValueError(f"{name} is {tuple(t.shape)}, one number is expected")
            return float(t.float().reshape(-1)[0])

        def linear(parts: List[torch.Tensor], bias: Optional[List[torch.Tensor]] = None) -> HymetaLinear:
            return HymetaLinear.from_weight(parts[0] if len(parts) == 1 else torch.cat(parts, 0).contiguous(),
                                            None if bias is None else (bias[0] if len(bias) == 1 else torch.cat(bias, 0).contiguous()))

        def freqs(spec) -> Optional[torch.Tensor]:
            return torch.tensor(spec.frequencies(), dtype=torch.float64, device=dev) if spec.rot_dims else None

        W = cfg.hidden_size

        def attention(p: str, a: WindowAttentionSpec, layer: int) -> WindowAttentionMixer:
            H, G, D, Dv = a.heads, a.kv_heads, a.dim, a.vdim
            rows = [act(p + "q", (H * D, W)), act(p + "k", (G * D, W)), act(p + "v", (G * Dv, W))]
            bias = [act(p + "q.b", (H * D,)), act(p + "k.b", (G * D,)), act(p + "v.b", (G * Dv,))] if a.bias else None
            if a.gate:
                # the gates' rows ride behind the values'; zero rows keep the projection's row a whole number of 16 bytes,
                # which the matrix-core attention kernels ask of the queries' stride
                pad = -(sum(r.shape[0] for r in rows) + H) % 8
                rows.append(torch.cat([act(p + "g", (H, W)), torch.zeros(pad, W, dtype=dt, device=dev)], 0))
                if bias is not None:
                    bias.append(torch.zeros(H + pad, dtype=dt, device=dev))
            o = linear([act(p + "o", (W, H * Dv))], [act(p + "o.b", (W,))] if a.bias else None)
            return WindowAttentionMixer(linear(rows, bias), o, m.attn_layers[str(layer)], a.rot_dims, freqs(a), a.gate)

        m.embed = act("embed", (cfg.vocab_size, W))
        m.head = act("head", (cfg.vocab_size, W))
        m.final_norm_scale = number("final.norm")
        m.blocks = torch.nn.ModuleDict()
        for i, spec in enumerate(cfg.layers):
            if spec.weights_of != i:
                continue
            p, a = f"l{i}.", spec.mixer
            if isinstance(a, WindowAttentionSpec):
                mixer = attention(p + "mix.", a, i)
            elif isinstance(a, RetentionSpec):
                H, D, Dv = a.heads, a.dim, a.vdim
                parts = [act(p + "mix.q", (H * D, W)), act(p + "mix.k", (H * D, W)), act(p + "mix.v", (H * Dv, W)), act(p + "mix.g", (H * Dv, W))]
                mixer = RetentionMixer(linear(parts), linear([act(p + "mix.o", (W, H * Dv))]), H, D, Dv,
                                       torch.tensor(a.decay, dtype=torch.float32, device=dev), a.rot_dims, freqs(a), cfg.norm_eps)
            else:
                assert isinstance(a, SideBySideSpec)
                r, q = a.right, p + "mix.right."
                right = StateSpaceMixer(linear([act(q + "in", (2 * r.inner + 2 * r.groups * r.state + r.heads, W))]), linear([act(q + "o", (W, r.inner))]),
                                        r.heads, r.vdim, r.state, r.groups, r.norm_groups, f32(q + "conv", (r.conv_channels, r.conv)),
                                        f32(q + "conv.b", (r.conv_channels,)), f32(q + "dt_bias", (r.heads,)), f32(q + "A_log", (r.heads,)),
                                        f32(q + "D", (r.heads,)), f32(q + "norm", (r.inner,)), cfg.norm_eps)
                mixer = SideBySideMixer(attention(p + "mix.left.", a.left, i), right, a.left_scale, a.right_scale)
            mlp = None
            e = spec.mlp
            if isinstance(e, DenseMlpSpec):
                pq = take(p + "mlp.act", (2,)).float().tolist()
                mlp = XieluMLP(linear([act(p + "mlp.up", (e.ff, W))]), linear([act(p + "mlp.down", (W, e.ff))]), pq[0], pq[1])
            elif isinstance(e, GroupedMoeSpec):
                F = e.ff
                w13 = torch.stack([torch.cat([act(f"{p}mlp.e{j}.gate", (F, W)), act(f"{p}mlp.e{j}.up", (F, W))], 0) for j in range(e.experts)])
                w2 = torch.stack([act(f"{p}mlp.e{j}.down", (W, F)) for j in range(e.experts)])
                shared = gate = None
                if e.shared_ff:
                    Fs = e.shared_ff
                    shared = SiluGluMLP(linear([act(p + "mlp.shared.gate", (Fs, W)), act(p + "mlp.shared.up", (Fs, W))]),
                                        linear([act(p + "mlp.shared.down", (W, Fs))]))
                    gate = f32(p + "mlp.shared.sg", (1, W))
                outputs = e.experts + e.identity
                mlp = GroupedSoftmaxMoE(f32(p + "mlp.router", (outputs, W)), f32(p + "mlp.correction", (outputs,)), w13, w2, e.top, e.groups,
                                        e.keep, e.identity, shared, gate)
            m.blocks[str(i)] = ParallelBlock(number(p + "norm1"), mixer, mlp, cfg.norm_eps)
        return loaded

