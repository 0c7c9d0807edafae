"""RMS norm: x * rsqrt(mean(x^2) + eps) * w in float, eps inside the root, plain weight
(pagedllm/model/llama.py:74-83).

A block hands its mixer and feed-forward a ``PendingNorm`` rather than normed rows: the residual
sum and the norm are then done inside the consumer's first matrix product when that product's
kernel can take them in (few rows, decoding), or by the norm kernel when ``rows()`` is asked for.
Either way the consumer sees the same rows, and the block reads the new residual afterwards.
"""

from __future__ import annotations

import torch

from ..csrc import ops
from .base import Norm
from .registry import BuildEnv, register_norm
from .spec import WeightSpec


class PendingNorm:
    """rows = norm(x[row_index] + delta[row_index]), not computed yet.  ``delta``: rows like x, or the float partial sums
    [ranges, rows, hidden] of the product that made them, which the norm kernel adds in order."""

    def __init__(self, weight: torch.Tensor, eps: float, x: torch.Tensor, delta: torch.Tensor | None = None,
                 row_index: torch.Tensor | None = None, write_residual: bool = True):
        self.weight, self.eps = weight, eps
        self.x, self.delta, self.row_index = x, delta, row_index
        self.write_residual = write_residual and delta is not None
        self._rows: torch.Tensor | None = None
        self._summed = delta is None            # True once x holds x + delta

    # what consumers may ask without forcing the computation
    @property
    def num_rows(self) -> int:
        return self.row_index.numel() if self.row_index is not None else self.x.shape[0]

    @property
    def shape(self):
        return (self.num_rows, self.x.shape[1])

    @property
    def dtype(self):
        return self.x.dtype

    @property
    def device(self):
        return self.x.device

    def rows(self) -> torch.Tensor:
        """The normed rows as a tensor (computed once by the norm kernel)."""
        if self._rows is None:
            delta = None if self._summed else self.delta
            self._rows = ops.rmsnorm(self.x, self.weight, self.eps, delta, self.row_index, self.write_residual)
            if delta is not None and self.write_residual:
                self._summed = True
        return self._rows

    def fusable(self) -> bool:
        """Whether a consumer's kernel may still take the sum and the norm in (not once the rows exist, and not when the
        sum comes as float partial sums of a product, which only the norm kernel adds)."""
        return self._rows is None and (self._summed or self.delta is None or self.delta.dim() == 2)

    def fused_arguments(self) -> dict:
        """Arguments for a kernel that takes the sum and the norm in; call ``fused_done`` after it."""
        x_out = None
        if not self._summed and self.write_residual:
            x_out = torch.empty_like(self.x)
        return dict(delta=None if self._summed else self.delta, norm_weight=self.weight, eps=self.eps, x_out=x_out,
                    row_index=self.row_index)

    def fused_done(self, args: dict) -> None:
        if args["x_out"] is not None:
            self.x = args["x_out"]              # the kernel wrote the new residual there
            self._summed = True

    def residual(self) -> torch.Tensor:
        """x + delta, after whoever consumed the rows has run (forces the sum if nobody did)."""
        if not self._summed and self.write_residual:
            self.rows()
        return self.x


def rows_of(h) -> torch.Tensor:
    return h.rows() if isinstance(h, PendingNorm) else h


class RMSNorm(Norm):
    # ``delta`` may be the float partial sums [ranges, rows, hidden] of a product cut along its inner dimension
    accepts_partial_sums = True

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

    def pending(self, x, delta=None, row_index=None, write_residual=True) -> PendingNorm:
        return PendingNorm(self.weight, self.eps, x, delta, row_index, write_residual)


register_norm("rmsnorm", RMSNorm)
