"""Token embedding (a row gather, pagedllm/model/llama.py:197) and the output head
(logits = rows * table^T in float, pagedllm/model/llama.py:203-216; tied = the embedding table)."""

from __future__ import annotations

import torch

from ..csrc import ops
from .base import Part
from .linear import Weight, linear
from .registry import BuildEnv, register_embedding, register_head
from .spec import WeightSpec


class TokenEmbedding(Part):
    def __init__(self, params: dict, env: BuildEnv):
        self.vocab = int(params["vocab_size"])
        self.hidden = env.hidden_size
        self.dtype, self.device = env.dtype, env.device
        self.table: torch.Tensor | None = None

    def weight_specs(self):
        return {"weight": WeightSpec((self.vocab, self.hidden), role="table")}

    def assign(self, name, tensor):
        if name != "weight":
            raise KeyError(name)
        self.table = tensor.to(device=self.device, dtype=self.dtype).contiguous()

    def forward(self, ids: torch.Tensor) -> torch.Tensor:
        return ops.embed_gather(ids, self.table)


class LMHead(Part):
    def __init__(self, params: dict, env: BuildEnv):
        self.vocab = int(params["vocab_size"])
        self.hidden = env.hidden_size
        self.tied = bool(params.get("tied", False))
        self.dtype, self.device = env.dtype, env.device
        self.weight: torch.Tensor | None = None
        self._matrix = None

    def weight_specs(self):
        return {} if self.tied else {"weight": WeightSpec((self.vocab, self.hidden))}

    def assign(self, name, tensor):
        if name != "weight" or self.tied:
            raise KeyError(name)
        self.weight = tensor.to(device=self.device, dtype=self.dtype).contiguous()

    def tie(self, table: torch.Tensor) -> None:
        self.weight = table
        self._matrix = None

    def finalize(self) -> None:
        self._matrix = None

    def forward(self, h) -> torch.Tensor:
        if self._matrix is None:                      # (the tiled copy for decode steps, made once the matrix is there)
            self._matrix = Weight(self.weight)
        return linear(h, self._matrix, out_dtype=torch.float32)


register_embedding("token_embedding", TokenEmbedding)
register_head("lm_head", LMHead)
