"""Model registry: config.json's architecture name -> model class.

The engine builds its model here, so a checkpoint directory selects its class
by what its config.json says.  A class takes (cfg, device, dtype, tp) and
offers forward / compute_logits / random_init / load_safetensors; classes with
`unified_rows` also lay out their own paged caches (alloc_kv_caches).
"""
from __future__ import annotations

import torch

DTYPES = {"bfloat16": torch.bfloat16, "bf16": torch.bfloat16, "float32": torch.float32, "fp32": torch.float32}


def _llama():
    from .llama import LlamaForCausalLM

    return LlamaForCausalLM


def _bekulix():
    from .bekulix import BekulixForCausalLM

    return BekulixForCausalLM


def _bolinex():
    from .bolinex import BolinexForCausalLM

    return BolinexForCausalLM


def _nefivik():
    from .nefivik import NefivikForCausalLM

    return NefivikForCausalLM


def _sobivik():
    from .sobivik import SobivikForCausalLM

    return SobivikForCausalLM


# architecture -> (class loader, activation dtypes the class has kernels for)
MODEL_REGISTRY = {
    "LlamaForCausalLM": (_llama, ("bfloat16",)),
    "LlavaForConditionalGeneration": (_llama, ("bfloat16",)),
    "Bekulix": (_bekulix, ("bfloat16", "float32")),
    "Bolinex": (_bolinex, ("bfloat16", "float32")),
    "Nefivik": (_nefivik, ("bfloat16", "float32")),
    "Sobivik": (_sobivik, ("bfloat16", "float32")),
}


def supports_dtype(architecture: str, dtype: str) -> bool:
    ent = MODEL_REGISTRY.get(architecture)
    return ent is not None and str(DTYPES.get(dtype)).replace("torch.", "") in ent[1]


def build_model(cfg, device, tp=None, dtype: str | torch.dtype = "bfloat16"):
    ent = MODEL_REGISTRY.get(cfg.architecture)
    if ent is None:
        raise ValueError(f"unknown architecture {cfg.architecture!r}; registered: {sorted(MODEL_REGISTRY)}")
    dt = DTYPES[dtype] if isinstance(dtype, str) else dtype
    name = str(dt).replace("torch.", "")
    if name not in ent[1]:
        raise ValueError(f"{cfg.architecture} has no {name} kernels (supported: {', '.join(ent[1])})")
    return ent[0]()(cfg, device=device, dtype=dt, tp=tp)
