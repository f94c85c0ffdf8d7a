"""The Lidizen decoder: token embedding plus a hashed embedding of the (previous, current) token pair, layer-normed, into
one or several fp32 residual streams (hyper-connections); pre-norm layers whose mixer is a softmax attention with grouped
key/value heads, whole-projection query / key norms, interleaved rotary pairs, scores mixed across heads before the
softmax, a sliding window that keeps a sequence's first tokens, and values blended with the first such layer's; the
feed-forward is a biased silu-gated unit or a mixture of squared-relu experts weighed by the softmax over the chosen
router logits.  The output projection is the embedding table.

The class has the surface of the package's other model classes (``GLAswaForCausalLM``, ``SonuzenForCausalLM``,
``GeponexForCausalLM``): ``forward(input_ids, positions, attn_metadata=..., request_ids_to_seq_ids=...,
finished_requests_ids=...)`` returns the final hidden states of the step's rows, ``compute_logits`` the fp32 logits of
the rows asked for, ``load_weights`` takes the checkpoint as a stream of named tensors; the attention layers are found by
name and bound to paged caches by whoever drives the model; the previous token of every sequence lives in a slot-indexed
state cache that follows the requests' ids.
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
from .configuration_lidizen import LidizenConfig, Relu2MoeSpec, SiluMlpSpec
from .feed_forward import Relu2RoutedMoE, SiluGluMLP
from .hyper_block import HyperConnection, HyperStreamBlock, StreamNormRead, flush_pending
from .stream_block import StepLayout
from .talking_attention import PagedSharedKeyAttention, TalkingHeadsAttentionMixer


class LidizenStateCache(ConstantSizeStateCache):
    """``prev_token [1, slots]`` int32: the last token every sequence has run (the pair embedding of the next one reads
    it).  A slot needs no clearing when it changes hands: a sequence's first token does not read it."""

    def __init__(self, max_batch_size: int, device):
        super().__init__(max_batch_size, device)
        self.prev_token = torch.zeros(1, max_batch_size, dtype=torch.int32, device=self.device)

    @property
    def cache(self):
        return (self.prev_token,)


class LidizenModel(torch.nn.Module):
    def __init__(self, config: LidizenConfig, max_num_seqs: int = 256, dtype: torch.dtype = torch.bfloat16, device="cuda",
                 prefix: Optional[str] = None):
        super().__init__()
        if dtype not in (torch.bfloat16, torch.float32):
            raise ValueError("Lidizen runs in bfloat16 or float32")
        self.config, self.dtype, self.device = config, dtype, torch.device(device)
        self.prefix = standalone_prefix("model") if prefix is None else prefix
        # the cache-owning attention layers exist from construction on (an engine sizes its pages from them)
        self.attn_layers = torch.nn.ModuleDict()
        for i, spec in enumerate(config.layers):
            m = spec.mixer
            self.attn_layers[str(i)] = PagedSharedKeyAttention(m.heads, m.kv_heads, m.dim, m.vdim, m.scale, f"{self.prefix}.layers.{i}.attn",
                                                               sliding_window=m.window, keep_first=m.keep_first, dtype=dtype)
        self.state_cache = LidizenStateCache(max_num_seqs, self.device)
        self.streams = max(config.streams, 1)
        self.embed: Optional[torch.Tensor] = None
        self.pair_table: Optional[torch.Tensor] = None
        self.embed_norm: Optional[torch.Tensor] = None
        self.blocks = torch.nn.ModuleList()
        self.final_read: Optional[StreamNormRead] = None

    def layout_of(self, attn_metadata, slot_idx: torch.Tensor, token_ids: torch.Tensor, positions: Optional[torch.Tensor] = None) -> StepLayout:
        md = attn_metadata
        max_seq = max(md.seq_lens) if md.seq_lens else max(md.max_prefill_seq_len, md.max_decode_seq_len)
        return StepLayout(query_start_loc=md.query_start_loc, context_lens=md.context_lens_tensor, seq_lens=md.seq_lens_tensor,
                          slot_idx=slot_idx, block_tables=md.block_tables, slot_mapping=md.slot_mapping,
                          max_query_len=int(md.max_query_len or 1), max_seq_len=int(max_seq), token_ids=token_ids, positions=positions)

    def forward(self, input_ids: torch.Tensor, positions: Optional[torch.Tensor] = None, attn_metadata=None,
                kv_caches: Optional[List[torch.Tensor]] = None, residual_out: Optional[List[torch.Tensor]] = None,
                **kwargs) -> torch.Tensor:
        """``positions`` (int64, one per row) spare the rotation a lookup of the row's sequence; without them a row's
        position is its sequence's length minus the rows behind it, which is also what the attention's mask goes by.  ``kv_caches``:
        one page tensor per attention layer, in layer order, bound before the step (callers without an engine).
        ``residual_out``: a list that receives the sum of the streams after every layer (debugging; it splits the fused
        write-and-read launches)."""
        if kv_caches is not None:
            for layer, kv in zip(self.attn_layers.values(), kv_caches):
                bind_kv_cache(layer, kv)
        md = attn_metadata if attn_metadata is not None else current_attn_metadata()
        if md is None:
            raise RuntimeError("LidizenModel.forward needs the step's attention metadata")
        kwargs.setdefault("request_ids_to_seq_ids", {})
        kwargs.setdefault("finished_requests_ids", [])
        (prev_token,), slot_idx = self.state_cache.current_run_tensors(**kwargs)
        input_ids = input_ids.to(torch.int64).contiguous()
        if positions is not None:
            positions = positions.to(torch.int64).contiguous()
        layout = self.layout_of(md, slot_idx, input_ids, positions)
        big = self.config.bigram
        x = hip_ops.embed_pair(input_ids, self.embed, self.pair_table, self.embed_norm, self.config.norm_eps, self.streams,
                               buckets=big.buckets if big else 0, mul_prev=big.mul_prev if big else 0, mul_cur=big.mul_cur if big else 0,
                               prev_token=prev_token[0], query_start_loc=layout.query_start_loc, context_lens=layout.context_lens,
                               slot_idx=layout.slot_idx)
        pending, v_first = None, None
        for i, block in enumerate(self.blocks):
            pending, v_first = block(x, pending, self.dtype, layout, self.attn_layers[str(i)], v_first)
            if residual_out is not None:
                flush_pending(x, pending)
                pending = None
                residual_out.append(x.sum(1))
        return self.final_read(x, pending, self.dtype)


class LidizenForCausalLM(torch.nn.Module, HasInnerState, IsHybrid):
    # csrc/*.hip sources whose kernels this class calls (a first run in a fresh checkout builds these, see _C.build_library)
    kernel_sources = ("api_misc", "hyper_stream", "talk_attn", "sink_attn", "gated_ops", "moe_sigmoid", "moe_table", "moe", "glue",
                      "dense_gemm", "stream_gemm", "tall_gemm")

    def __init__(self, config: Optional[LidizenConfig] = None, max_num_seqs: int = 256, dtype: torch.dtype = torch.bfloat16,
                 device="cuda", *, vllm_config=None, prefix: Optional[str] = None):
        super().__init__()
        if vllm_config is not None:
            mc = vllm_config.model_config
            config = mc.hf_config if isinstance(mc.hf_config, LidizenConfig) else LidizenConfig(mc.hf_config.to_dict())
            max_num_seqs = int(vllm_config.scheduler_config.max_num_seqs)
            dtype = getattr(mc, "dtype", dtype)
            device = getattr(getattr(vllm_config, "device_config", None), "device", None) or device
            prefix = f"{prefix}.model" if prefix else "model"
        if config is None:
            raise TypeError("LidizenForCausalLM needs vllm_config= or a LidizenConfig")
        self.config = config
        self.model = LidizenModel(config, max_num_seqs=max_num_seqs, dtype=dtype, device=device, prefix=prefix)

    # what an engine asks a model with states of its own (the package's other model classes answer the same calls)
    def copy_inputs_before_cuda_graphs(self, input_buffers, **kwargs):
        return self.model.state_cache.copy_inputs_before_cuda_graphs(input_buffers, **kwargs)

    def get_seqlen_agnostic_capture_inputs(self, batch_size: int):
        return self.model.state_cache.get_seqlen_agnostic_capture_inputs(batch_size)

    def forward(self, input_ids, positions=None, intermediate_tensors=None, inputs_embeds=None, **kwargs):
        return self.model(input_ids, positions, **kwargs)

    def compute_logits(self, hidden_states: torch.Tensor, sampling_metadata=None) -> torch.Tensor:
        """The output projection is the embedding table."""
        idx = getattr(sampling_metadata, "selected_token_indices", None)
        if idx is not None:
            hidden_states = hidden_states.index_select(0, idx)
        return lm_head_logits(hidden_states, self.model.embed)

    # ------------------------------------------------------------------ weights
    def load_weights(self, weights: Iterable[Tuple[str, torch.Tensor]]) -> Set[str]:
        """Checkpoint names: ``embed``, ``bigram``, ``embed.norm``, ``final.norm``, and per layer ``l<i>.norm1|norm2``,
        ``l<i>.mix.<q|k|v>`` with ``.b`` biases, ``l<i>.mix.<q.norm|k.norm|talk|vmix|o>``, ``l<i>.mlp.<gate|up|down>`` with
        ``.b`` biases (dense) or ``l<i>.mlp.<router|router.b|e<j>.up|e<j>.down>``, and with several streams
        ``l<i>.hc<1|2>.<in|out|mix>``.  Linear weights ``[out, in]``."""
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

        def linear(parts: List[torch.Tensor], bias: Optional[List[torch.Tensor]] = None) -> HymetaLinear:
            return HymetaLinear.from_weight(parts[0] if len(parts) == 1 else torch.cat(parts, 0).contiguous(),
                                            None if bias is None else (bias[0] if len(bias) == 1 else torch.cat(bias, 0).contiguous()))

        W, S = cfg.hidden_size, cfg.streams
        m.embed = act("embed", (cfg.vocab_size, W))
        m.pair_table = act("bigram", (cfg.bigram.buckets + 1, W)) if cfg.bigram else None
        m.embed_norm = f32("embed.norm", (W,))

        def connection(name: str) -> HyperConnection:
            if not S:
                return HyperConnection.plain(dev)
            return HyperConnection(f32(name + ".in", (S,)), f32(name + ".out", (S,)), f32(name + ".mix", (S, S)))

        m.final_read = StreamNormRead(HyperConnection.summing(m.streams, dev), f32("final.norm", (W,)), cfg.norm_eps)
        m.blocks = torch.nn.ModuleList()
        blending_seen = False
        for i, spec in enumerate(cfg.layers):
            p, a = f"l{i}.", spec.mixer
            H, G, D, Dv = a.heads, a.kv_heads, a.dim, a.vdim
            qkv = linear([act(p + "mix.q", (H * D, W)), act(p + "mix.k", (G * D, W)), act(p + "mix.v", (G * Dv, W))],
                         [act(p + "mix.q.b", (H * D,)), act(p + "mix.k.b", (G * D,)), act(p + "mix.v.b", (G * Dv,))])
            blend = None
            if a.v_mix:
                lam = float(take(p + "mix.vmix").float().reshape(-1)[0])       # (the first blending layer's is not used)
                blend = lam if blending_seen else 0.0
                blending_seen = True
            freqs = torch.tensor(a.frequencies(), dtype=torch.float64, device=dev) if a.rot_dims else None
            mixer = TalkingHeadsAttentionMixer(qkv, linear([act(p + "mix.o", (W, H * Dv))]), m.attn_layers[str(i)],
                                               f32(p + "mix.q.norm", (H * D,)), f32(p + "mix.k.norm", (G * D,)),
                                               f32(p + "mix.talk", (H, H)), cfg.norm_eps, a.rot_dims, freqs, blend)
            mixer_in = StreamNormRead(connection(p + "hc1"), f32(p + "norm1", (W,)), cfg.norm_eps)
            mlp = mlp_in = None
            e = spec.mlp
            if isinstance(e, SiluMlpSpec):
                mlp = SiluGluMLP(linear([act(p + "mlp.gate", (e.ff, W)), act(p + "mlp.up", (e.ff, W))],
                                        [act(p + "mlp.gate.b", (e.ff,)), act(p + "mlp.up.b", (e.ff,))]),
                                 linear([act(p + "mlp.down", (W, e.ff))], [act(p + "mlp.down.b", (W,))]))
            elif isinstance(e, Relu2MoeSpec):
                w1 = torch.stack([act(f"{p}mlp.e{j}.up", (e.ff, W)) for j in range(e.experts)])
                w2 = torch.stack([act(f"{p}mlp.e{j}.down", (W, e.ff)) for j in range(e.experts)])
                mlp = Relu2RoutedMoE(f32(p + "mlp.router", (e.experts, W)), f32(p + "mlp.router.b", (e.experts,)), w1, w2, e.top)
            if mlp is not None:
                mlp_in = StreamNormRead(connection(p + "hc2"), f32(p + "norm2", (W,)), cfg.norm_eps)
            m.blocks.append(HyperStreamBlock(mixer_in, mixer, mlp_in, mlp))
        return loaded
