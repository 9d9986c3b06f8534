"""
Model registry: config.json names an architecture, the registry maps it to the class that loads and runs it.

    load_model(directory, device, dtype)  ->  a model with  .vocab, .new_cache(slots), .step(StepBatch, cache) -> float32 logits

Registered: the unquantized mixer families (Vofanex, Zagilorn, Fimunex, Dikopel) with the step interface above, and the EXL3-quantized Llama of llama_path.py, which
keeps its own decode_step / prefill_chunk pipelines (`load_model` returns it for `LlamaForCausalLM` checkpoints; the token-level
generator drives step-interface models only).
"""
from __future__ import annotations
import json
import os
import torch

_REGISTRY: dict[str, callable] = {}
_LIBRARIES: dict[str, tuple] = {}


def register(architecture: str, libraries: tuple = ("hip",)):
    """libraries: the native libraries the architecture's kernels live in ("mix": libexl3_mix.so, "hip": libexl3_hip.so) -- what a fresh checkout compiles
    before the model is loaded."""
    def deco(fn):
        _REGISTRY[architecture] = fn
        _LIBRARIES[architecture] = tuple(libraries)
        return fn
    return deco


def native_libraries(architecture: str) -> tuple:
    return _LIBRARIES.get(architecture, ("hip",))


def architectures() -> list[str]:
    return sorted(_REGISTRY)


def architecture_of(config: dict) -> str:
    a = config.get("architecture")
    if a is None:
        archs = config.get("architectures") or []
        a = archs[0] if archs else None
    if a is None:
        raise RuntimeError("config.json names no architecture")
    return a


def load_model(directory: str, device="cuda:0", dtype: torch.dtype | None = None):
    with open(os.path.join(directory, "config.json")) as f:
        config = json.load(f)
    a = architecture_of(config)
    if a not in _REGISTRY:
        raise RuntimeError(f"architecture {a!r} is not registered (known: {', '.join(architectures())})")
    return _REGISTRY[a](directory, config, device, dtype)


@register("Vofanex", libraries=("mix",))
def _load_vofanex(directory, config, device, dtype):
    from .vofanex import VofanexModel
    return VofanexModel.from_directory(directory, device=device, dtype=dtype or torch.bfloat16)


@register("Zagilorn", libraries=("mix",))
def _load_zagilorn(directory, config, device, dtype):
    from .zagilorn import ZagilornModel
    return ZagilornModel.from_directory(directory, device=device, dtype=dtype or torch.bfloat16)


@register("Fimunex", libraries=("mix",))
def _load_fimunex(directory, config, device, dtype):
    from .fimunex import FimunexModel
    return FimunexModel.from_directory(directory, device=device, dtype=dtype or torch.bfloat16)


@register("Dikopel", libraries=("mix",))
def _load_dikopel(directory, config, device, dtype):
    from .dikopel import DikopelModel
    return DikopelModel.from_directory(directory, device=device, dtype=dtype or torch.bfloat16)


@register("LlamaForCausalLM")
def _load_llama(directory, config, device, dtype):
    if dtype not in (None, torch.float16):
        raise RuntimeError("the EXL3 Llama path computes in float16")
    from .llama_path import SyntheticEXL3Llama
    return SyntheticEXL3Llama.from_checkpoint(directory, device=device)
