"""RMS norm: x * rsqrt(mean(x^2) + eps) * w in float, eps inside the root, plain weight
(pagedllm/model/llama.py:74-83)."""

from __future__ import annotations

import torch

from ..csrc import ops
from .base import Norm
from .registry import BuildEnv, register_norm
from .spec import WeightSpec


class RMSNorm(Norm):
    def __init__(self, params: dict, env: BuildEnv):
        self.eps = float(params["eps"])
        self.size = int(params.get("size", env.hidden_size))
        self.device = env.device
        self.weight: torch.Tensor | None = None

    def weight_specs(self):
        return {"weight": WeightSpec((self.size,), role="vector", init="ones")}

    def assign(self, name, tensor):
        if name != "weight":
            raise KeyError(name)
        self.weight = tensor.to(device=self.device, dtype=torch.float32).contiguous()

    def forward(self, x, row_index=None):
        return ops.rmsnorm(x, self.weight, self.eps, None, row_index)

    def add_norm(self, x, delta, row_index=None, write_residual=True):
        return ops.rmsnorm(x, self.weight, self.eps, delta, row_index, write_residual)


register_norm("rmsnorm", RMSNorm)
