"""Registers the Llama-3 family (HF ``config.json``) with the architecture registry."""
from __future__ import annotations

from . import config as C
from .registry import Architecture, register


def _build(cfg, device, dtype, comm, max_model_len, quantization):
    from .llama import LlamaModel

    return LlamaModel(cfg, device, dtype, comm, max_model_len, quantization=quantization)


register(Architecture(
    name="llama",
    matches=lambda c: "hidden_size" in c and "num_attention_heads" in c,
    parse=lambda c, name: C.llama_from_dict(c, name),
    build=_build,
    presets=C.MODELS,
))
