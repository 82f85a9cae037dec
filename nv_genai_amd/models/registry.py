"""Model registry: which class serves a model folder, chosen by its config.json.

A model folder holds ``config.json`` and ``*.safetensors``. ``config.json`` names the design
under ``architecture`` (this framework's layer-list designs) or ``architectures`` / ``model_type``
(HF decoder checkpoints of the Llama-layout families). ``load_model`` builds the config, reads
the weights (safetensors only) and returns the model on the device, ready for
:class:`~nv_genai_amd.engine.llm_engine.LLMEngine` (``EngineConfig.model`` may be such a folder).
"""
from __future__ import annotations

import json
import os
from typing import Callable, Dict, Optional, Tuple

import torch

from .config import LLAMA_PRESETS, BidasunConfig, BiruvikConfig, LizezenConfig, LlamaConfig, LumepelConfig

# design name (lower case) -> (config builder from the config.json dict, model class loader)
_REGISTRY: Dict[str, Tuple[Callable[[dict], object], Callable[[], type]]] = {}


def register(name: str, make_config: Callable[[dict], object], model_class: Callable[[], type]) -> None:
    _REGISTRY[name.lower()] = (make_config, model_class)


def _bidasun_class():
    from .bidasun import BidasunModel

    return BidasunModel


def _biruvik_class():
    from .biruvik import BiruvikModel

    return BiruvikModel


def _lumepel_class():
    from .lumepel import LumepelModel

    return LumepelModel


def _lizezen_class():
    from .lizezen import LizezenModel

    return LizezenModel


def _llama_class():
    from .llama import LlamaModel

    return LlamaModel


_HF_ARCH = {"llama": "llama", "mistral": "mistral", "mixtral": "mixtral", "gemma": "gemma", "starcoder2": "starcoder2"}


def _hf_decoder_config(d: dict) -> LlamaConfig:
    """LlamaConfig of an HF decoder config.json (the Llama-layout families)."""
    arch = _HF_ARCH[d["model_type"]]
    heads = int(d["num_attention_heads"])
    kw = dict(name=d.get("_name_or_path") or arch, arch=arch, vocab_size=int(d["vocab_size"]),
              hidden=int(d["hidden_size"]), layers=int(d["num_hidden_layers"]), heads=heads,
              kv_heads=int(d.get("num_key_value_heads", heads)),
              head_dim=int(d.get("head_dim") or d["hidden_size"] // heads), ffn=int(d["intermediate_size"]),
              rope_theta=float(d.get("rope_theta", 10000.0)), rope_scaling=d.get("rope_scaling"),
              eps=float(d.get("rms_norm_eps", d.get("norm_epsilon", 1e-5))),
              max_position=int(d.get("max_position_embeddings", 8192)),
              tie_embeddings=bool(d.get("tie_word_embeddings", False)),
              sliding_window=int(d.get("sliding_window") or 0))
    base = next((c for c in LLAMA_PRESETS.values() if c.arch == arch), LlamaConfig())
    for f in ("norm", "act", "gated_mlp", "attn_bias", "mlp_bias", "chat_format"):
        kw[f] = getattr(base, f)
    if arch == "gemma":
        kw["embed_scale"] = kw["hidden"] ** 0.5
    if arch == "mixtral":
        kw["num_experts"], kw["experts_per_tok"] = int(d["num_local_experts"]), int(d["num_experts_per_tok"])
    eos = d.get("eos_token_id", 2)
    kw["eos_ids"] = tuple(eos) if isinstance(eos, (list, tuple)) else (int(eos),)
    kw["bos_id"] = int(d.get("bos_token_id", 1) or 0)
    return LlamaConfig(**kw)


register("bidasun", BidasunConfig.from_dict, _bidasun_class)
register("biruvik", BiruvikConfig.from_dict, _biruvik_class)
register("lumepel", LumepelConfig.from_dict, _lumepel_class)
register("lizezen", LizezenConfig.from_dict, _lizezen_class)
for _t in _HF_ARCH:
    register(_t, _hf_decoder_config, _llama_class)


def model_class_for(cfg) -> type:
    """Model class of a config object."""
    if isinstance(cfg, BidasunConfig):
        return _bidasun_class()
    if isinstance(cfg, BiruvikConfig):
        return _biruvik_class()
    if isinstance(cfg, LumepelConfig):
        return _lumepel_class()
    if isinstance(cfg, LizezenConfig):
        return _lizezen_class()
    if isinstance(cfg, LlamaConfig):
        return _llama_class()
    raise ValueError(f"no model class for {type(cfg).__name__}")


def architecture_of(d: dict) -> str:
    """Registry key of a config.json dict."""
    if "architecture" in d:
        return str(d["architecture"]).lower()
    if "model_type" in d:
        return str(d["model_type"]).lower()
    raise ValueError("config.json names no architecture")


def read_config(model_dir: str):
    """(config object, model class) of a model folder."""
    with open(os.path.join(model_dir, "config.json")) as f:
        d = json.load(f)
    key = architecture_of(d)
    if key not in _REGISTRY:
        raise ValueError(f"no model class registered for architecture {key!r} (known: {sorted(_REGISTRY)})")
    make, cls = _REGISTRY[key]
    return make(d), cls()


def is_model_dir(path) -> bool:
    return isinstance(path, str) and os.path.isfile(os.path.join(path, "config.json"))


def load_model(model_dir: str, device="cuda", dtype=torch.bfloat16, pctx=None, cfg_overrides: Optional[dict] = None):
    """The model of a folder (config.json + safetensors) on ``device`` in ``dtype``."""
    from ..utils.checkpoint import load_weights

    cfg, cls = read_config(model_dir)
    if cfg_overrides:
        from dataclasses import replace

        cfg = replace(cfg, **cfg_overrides)
    weights = load_weights(model_dir)
    return cls(cfg, device=device, dtype=dtype, pctx=pctx, weights=weights)
