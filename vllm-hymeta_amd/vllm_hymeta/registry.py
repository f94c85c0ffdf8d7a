"""Which model class and configuration class serve which ``config.json``: the table behind the vLLM registration hooks
(``register_model``) and behind the package's own engine, which has no vLLM to ask."""

from __future__ import annotations

import importlib
import json
import os
from typing import Any, Callable, Dict, Tuple

# architecture name (``architectures[0]`` or ``architecture`` of config.json) -> (module:class of the model, loader of its config)
_MODELS: Dict[str, Tuple[str, Callable[[str], Any]]] = {}


def register(architecture: str, model_path: str, config_loader: Callable[[str], Any]) -> None:
    _MODELS[architecture] = (model_path, config_loader)


def _sonuzen_config(model_dir: str):
    from .models.configuration_sonuzen import SonuzenConfig
    return SonuzenConfig.from_pretrained(model_dir)


def _geponex_config(model_dir: str):
    from .models.configuration_geponex import GeponexConfig
    return GeponexConfig.from_pretrained(model_dir)


def _lidizen_config(model_dir: str):
    from .models.configuration_lidizen import LidizenConfig
    return LidizenConfig.from_pretrained(model_dir)


def _dapuzen_config(model_dir: str):
    from .models.configuration_dapuzen import DapuzenConfig
    return DapuzenConfig.from_pretrained(model_dir)


def _gla_swa_config(model_dir: str):
    from .model_for_7B.configuration_gla_swa import GLAswaConfig
    with open(os.path.join(model_dir, "config.json")) as f:
        raw = json.load(f)
    raw.pop("architectures", None), raw.pop("model_type", None)
    return GLAswaConfig(**raw)


register("Sonuzen", "vllm_hymeta.models.modeling_sonuzen:SonuzenForCausalLM", _sonuzen_config)
register("SonuzenForCausalLM", "vllm_hymeta.models.modeling_sonuzen:SonuzenForCausalLM", _sonuzen_config)
register("Geponex", "vllm_hymeta.models.modeling_geponex:GeponexForCausalLM", _geponex_config)
register("GeponexForCausalLM", "vllm_hymeta.models.modeling_geponex:GeponexForCausalLM", _geponex_config)
register("Lidizen", "vllm_hymeta.models.modeling_lidizen:LidizenForCausalLM", _lidizen_config)
register("LidizenForCausalLM", "vllm_hymeta.models.modeling_lidizen:LidizenForCausalLM", _lidizen_config)
register("Dapuzen", "vllm_hymeta.models.modeling_dapuzen:DapuzenForCausalLM", _dapuzen_config)
register("DapuzenForCausalLM", "vllm_hymeta.models.modeling_dapuzen:DapuzenForCausalLM", _dapuzen_config)
register("GLAswaForCausalLM", "vllm_hymeta.model_for_7B.modeling_gla_swa:GLAswaForCausalLM", _gla_swa_config)


def architecture_of(model_dir: str) -> str:
    with open(os.path.join(model_dir, "config.json")) as f:
        raw = json.load(f)
    arch = raw.get("architecture") or (raw.get("architectures") or [None])[0]
    if arch not in _MODELS:
        raise ValueError(f"{model_dir}: architecture {arch!r} is not served by this package (known: {sorted(_MODELS)})")
    return arch


def resolve(model_dir: str):
    """``(model class, config)`` for a checkpoint folder."""
    path, load_config = _MODELS[architecture_of(model_dir)]
    module, _, name = path.partition(":")
    return getattr(importlib.import_module(module), name), load_config(model_dir)


def kernel_sources(model_dir: str):
    """The kernel sources the checkpoint's model class names (None: the whole library), read without importing torch."""
    path, _ = _MODELS[architecture_of(model_dir)]
    return _KERNEL_SOURCES.get(path.partition(":")[2])


# (kept beside the table so that asking does not import the model module, which imports torch and the library binding)
_KERNEL_SOURCES = {
    "SonuzenForCausalLM": ("api_misc", "norm_conv", "mingru", "sink_attn", "moe_table", "moe", "glue", "dense_gemm", "stream_gemm",
                           "tall_gemm"),
    "GeponexForCausalLM": ("api_misc", "norm_conv", "post_norm", "latent_attn", "sink_attn", "lightning", "gated_ops", "moe_sigmoid",
                           "moe_table", "moe", "glue", "dense_gemm", "stream_gemm", "tall_gemm"),
    "LidizenForCausalLM": ("api_misc", "hyper_stream", "talk_attn", "sink_attn", "gated_ops", "moe_sigmoid", "moe_table", "moe", "glue",
                           "dense_gemm", "stream_gemm", "tall_gemm"),
    "DapuzenForCausalLM": ("api_misc", "norm_conv", "parallel_ops", "decay_scan", "lightning", "sink_attn", "gated_ops", "moe_sigmoid",
                           "moe_table", "moe", "glue", "dense_gemm", "stream_gemm", "tall_gemm"),
}


def known_architectures():
    return sorted(_MODELS)
