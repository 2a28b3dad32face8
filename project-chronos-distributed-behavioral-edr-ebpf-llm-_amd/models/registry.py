"""Model registry: which model class serves a checkpoint directory or a preset name.

The engine builds its model through :func:`build_model` only.  A family registers a detector for checkpoint
directories, its preset names and a builder; the builder returns an object with what the engine uses:

  cfg.vocab_size, cfg.num_layers        sizes
  recurrent                             True = per-sequence state beyond pages (no prefix sharing between sequences)
  hq, hkv                               head counts for the decode-split heuristics
  make_cache(num_blocks, block_size, slots, kv_dtype)      the paged cache / state-slot store
  cache_bytes_per_block(block_size, kv_dtype)
  prefill_batch(chunks, starts, block_tables, slots, max_blocks, nqt, split, want)   host builder of a prefill step
  forward(step_batch, cache)            logits of the step batch's wanted tokens
"""
from __future__ import annotations

import os
from dataclasses import dataclass
from typing import Callable, Optional

import torch

from ..parallel.tp import TPContext

DTYPES = {"bf16": torch.bfloat16, "bfloat16": torch.bfloat16, "fp32": torch.float32, "float32": torch.float32}


@dataclass
class Family:
    name: str
    presets: Callable[[], list]
    is_checkpoint: Callable[[str], bool]
    build: Callable  # (name_or_path, device, tp, seed, is_path, max_position, weight_dtype, dtype) -> model
    dtypes: tuple = ("bf16",)


_FAMILIES: list[Family] = []


def register(fam: Family) -> None:
    _FAMILIES.append(fam)


def families() -> list[Family]:
    return list(_FAMILIES)


def family_of(model: str, checkpoint: Optional[str] = None) -> Family:
    path = checkpoint or (model if os.path.isdir(model) else None)
    if path:
        for f in _FAMILIES:
            if f.is_checkpoint(path):
                return f
        raise FileNotFoundError(f"{path}: no registered model family reads this directory")
    for f in _FAMILIES:
        if model in f.presets():
            return f
    raise KeyError(f"unknown model {model!r}; presets: {sorted(p for f in _FAMILIES for p in f.presets())}")


def build_model(model: str = "tiny", device="cpu", tp: TPContext | None = None, seed: int = 0,
                checkpoint: str | None = None, max_position: int | None = None, weight_dtype: str = "bf16",
                dtype: str = "bf16"):
    if not isinstance(model, str):  # a ready configuration object of the Llama family (tests)
        from . import llama

        return llama.build_model(model, device, tp, seed, checkpoint, max_position, weight_dtype)
    fam = family_of(model, checkpoint)
    dt = {"bfloat16": "bf16", "float32": "fp32"}.get(dtype, dtype)
    if dt not in fam.dtypes:
        raise NotImplementedError(f"the {fam.name} family does not run in {dtype}")
    path = checkpoint or (model if os.path.isdir(model) else None)
    return fam.build(path or model, device, tp or TPContext.single(), seed, path is not None, max_position,
                     weight_dtype, dt)


# ---- the families ------------------------------------------------------------------------------------------------


def _llama_build(name, device, tp, seed, is_path, max_position, weight_dtype, dtype):
    from . import llama

    return llama.build_model(name if not is_path else "tiny", device, tp, seed, name if is_path else None,
                             max_position, weight_dtype)


def _llama_is_checkpoint(path: str) -> bool:
    import json

    if os.path.exists(os.path.join(path, "params.json")):
        return True
    cj = os.path.join(path, "config.json")
    if not os.path.exists(cj):
        return False
    with open(cj) as fh:
        c = json.load(fh)
    return c.get("model_type") == "llama" or "LlamaForCausalLM" in (c.get("architectures") or []) or (
        "num_hidden_layers" in c and "architecture" not in c)


def _llama_presets():
    from . import llama

    return list(llama.PRESETS)


def _zokunex_build(name, device, tp, seed, is_path, max_position, weight_dtype, dtype):
    from . import zokunex

    if tp.world > 1:
        raise NotImplementedError("Zokunex runs on full-weight ranks (data-parallel replicas)")
    if weight_dtype != "bf16":
        raise NotImplementedError("Zokunex weights are served in the activation dtype (no fp8 projections)")
    return zokunex.build(name, device, seed, DTYPES[dtype], max_position)


def _zokunex_is_checkpoint(path: str) -> bool:
    from . import zokunex

    return zokunex.is_checkpoint(path)


def _zokunex_presets():
    from . import zokunex

    return list(zokunex.PRESETS)


def _kalesun_build(name, device, tp, seed, is_path, max_position, weight_dtype, dtype):
    from . import kalesun

    if tp.world > 1:
        raise NotImplementedError("Kalesun runs on full-weight ranks (data-parallel replicas)")
    if weight_dtype != "bf16":
        raise NotImplementedError("Kalesun weights are served in the activation dtype (no fp8 projections)")
    return kalesun.build(name, device, seed, DTYPES[dtype], max_position)


def _kalesun_is_checkpoint(path: str) -> bool:
    from . import kalesun

    return kalesun.is_checkpoint(path)


def _kalesun_presets():
    from . import kalesun

    return list(kalesun.PRESETS)


def _tugovik_build(name, device, tp, seed, is_path, max_position, weight_dtype, dtype):
    from . import tugovik

    if tp.world > 1:
        raise NotImplementedError("Tugovik runs on full-weight ranks (data-parallel replicas)")
    if weight_dtype != "bf16":
        raise NotImplementedError("Tugovik weights are served in the activation dtype (no fp8 projections)")
    return tugovik.build(name, device, seed, DTYPES[dtype], max_position)


def _tugovik_is_checkpoint(path: str) -> bool:
    from . import tugovik

    return tugovik.is_checkpoint(path)


def _tugovik_presets():
    from . import tugovik

    return list(tugovik.PRESETS)


def _vogerax_build(name, device, tp, seed, is_path, max_position, weight_dtype, dtype):
    from . import vogerax

    if tp.world > 1:
        raise NotImplementedError("Vogerax runs on full-weight ranks (data-parallel replicas)")
    if weight_dtype != "bf16":
        raise NotImplementedError("Vogerax weights are served in the activation dtype (no fp8 projections)")
    return vogerax.build(name, device, seed, DTYPES[dtype], max_position)


def _vogerax_is_checkpoint(path: str) -> bool:
    from . import vogerax

    return vogerax.is_checkpoint(path)


def _vogerax_presets():
    from . import vogerax

    return list(vogerax.PRESETS)


register(Family("vogerax", _vogerax_presets, _vogerax_is_checkpoint, _vogerax_build, ("bf16", "fp32")))
register(Family("tugovik", _tugovik_presets, _tugovik_is_checkpoint, _tugovik_build, ("bf16", "fp32")))
register(Family("kalesun", _kalesun_presets, _kalesun_is_checkpoint, _kalesun_build, ("bf16", "fp32")))
register(Family("zokunex", _zokunex_presets, _zokunex_is_checkpoint, _zokunex_build, ("bf16", "fp32")))
register(Family("llama", _llama_presets, _llama_is_checkpoint, _llama_build, ("bf16",)))
