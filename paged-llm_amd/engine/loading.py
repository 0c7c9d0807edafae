"""From a model folder to a built model and the objects a step needs around it."""

from __future__ import annotations

import torch

from ..cache.block_manager import CacheManager, GroupSpec
from ..cache.kv_cache import KVCacheStorage
from ..config.dtypes import resolve_dtype
from ..config.registry import lookup_architecture, read_config_json
from ..models.decoder import DecoderModel
from ..weights.loader import load_weights
from ..weights.random_init import fill_random
from .runner import ModelRunner


def require_gpu(device) -> torch.device:
    device = torch.device(device)
    if device.type != "cuda" or not torch.cuda.is_available():
        raise RuntimeError("this engine runs on an AMD GPU through its HIP kernels; no GPU is visible "
                           "(there is no CPU path)")
    return device


def build_model(hf_config: dict, dtype: str, device, max_model_len: int | None = None) -> DecoderModel:
    """Typed configuration and model class are chosen by config.json's architecture name."""
    arch = lookup_architecture(hf_config)
    cfg = arch.read_config(hf_config)
    spec = arch.build_spec(cfg)
    torch_dtype = resolve_dtype(dtype, spec.stored_dtype)
    return DecoderModel(spec, torch_dtype, device, max_positions=max_model_len)


def load_model(model_dir: str, dtype: str = "auto", device="cuda", max_model_len: int | None = None) -> DecoderModel:
    device = require_gpu(device)
    model = build_model(read_config_json(model_dir), dtype, device, max_model_len)
    load_weights(model, model_dir)
    return model


def random_model(hf_config: dict, seed: int = 0, dtype: str = "auto", device="cuda", max_model_len: int | None = None,
                 norm_jitter: bool = False) -> DecoderModel:
    device = require_gpu(device)
    model = build_model(hf_config, dtype, device, max_model_len)
    fill_random(model, seed, norm_jitter=norm_jitter)
    return model


def build_runtime(model: DecoderModel, block_size: int, num_pages: int | dict, num_state_slots: int,
                  enable_prefix_caching: bool, use_graphs: bool = False, **runner_options):
    """(CacheManager, KVCacheStorage, ModelRunner) for a model: one page pool per cache group,
    one state slot pool when a mixer keeps per-request state."""
    groups = model.cache_groups()
    specs = [GroupSpec(name, g.spec.kind, g.spec.window) for name, g in groups.items()]
    uses_state = bool(model.state_specs())
    manager = CacheManager(specs, num_pages, block_size, enable_prefix_caching,
                           num_state_slots=num_state_slots if uses_state else 0)
    storage = KVCacheStorage(groups, num_pages, block_size, model.dtype, model.device)
    runner = ModelRunner(model, storage, num_state_slots if uses_state else 0, use_graphs=use_graphs, **runner_options)
    return manager, storage, runner
