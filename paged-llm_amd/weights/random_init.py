"""Random weights from a configuration and a seed: in memory, or as a model folder
(config.json + model.safetensors) that the ordinary loader reads back.

Every matrix and table is drawn from normal(0, 0.02) with a seeded CPU generator, tensor by
tensor in sorted name order, in float and then rounded to the stored type, so that a float32
and a bfloat16 folder of the same seed hold the same draw.  Norm weights are 1.0, or 1 + 0.1 *
normal when ``norm_jitter`` is set (tests use that: a norm weight of exactly one hides a
missing multiplication).
"""

from __future__ import annotations

import json
import os

import torch

from ..config.registry import lookup_architecture

_STORED = {"float32": torch.float32, "bfloat16": torch.bfloat16}


def _declared_weights(hf_config: dict) -> dict:
    from ..models.decoder import DecoderModel
    arch = lookup_architecture(hf_config)
    spec = arch.build_spec(arch.read_config(hf_config))
    return DecoderModel(spec, torch.float32, "cpu", max_positions=1).weight_specs()


def draw_weights(weight_specs: dict, seed: int, stored: torch.dtype = torch.float32, std: float = 0.02,
                 norm_jitter: bool = False):
    """Yields (name, tensor) in sorted name order."""
    gen = torch.Generator().manual_seed(seed)
    for name in sorted(weight_specs):
        ws = weight_specs[name]
        if ws.role == "int":
            raise NotImplementedError("random integer tables")
        if ws.init == "ones":
            t = torch.ones(ws.shape, dtype=torch.float32)
            if norm_jitter:
                t = t + 0.1 * torch.randn(ws.shape, generator=gen, dtype=torch.float32)
        else:
            t = torch.randn(ws.shape, generator=gen, dtype=torch.float32) * std
        yield name, t.to(stored)


def write_random_model(folder: str, hf_config: dict, seed: int = 0, dtype: str | None = None, std: float = 0.02,
                       norm_jitter: bool = False) -> str:
    """Write ``folder/config.json`` and ``folder/model.safetensors``; returns the folder."""
    from safetensors.torch import save_file
    cfg = dict(hf_config)                                       # ("architectures" in it names the model, as everywhere)
    dtype = dtype or cfg.get("torch_dtype") or "float32"
    if dtype not in _STORED:
        raise KeyError(f"random weights are stored as float32 or bfloat16, not {dtype!r}")
    cfg["torch_dtype"] = dtype
    os.makedirs(folder, exist_ok=True)
    tensors = dict(draw_weights(_declared_weights(cfg), seed, _STORED[dtype], std, norm_jitter))
    save_file(tensors, os.path.join(folder, "model.safetensors"))
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(cfg, f, indent=1)
    return folder


def fill_random(model, seed: int = 0, std: float = 0.02, norm_jitter: bool = False) -> None:
    """Random weights straight into a built model (no folder), same draw as ``write_random_model``
    with the model's own compute type as the stored type."""
    stored = model.dtype if model.dtype in (torch.float32, torch.bfloat16) else torch.float32
    for name, t in draw_weights(model.weight_specs(), seed, stored, std, norm_jitter):
        model.assign(name, t)
    model.finalize()
