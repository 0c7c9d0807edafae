"""y = x W^T for the parts: picks the matrix-product kernel by element type and row count.

float32 always takes the plain kernel with float operands (the true 32-bit path).  bfloat16 takes
the weight-streaming kernel for a few rows (decoding) and the MFMA tile kernel for many (prompt
portions); shapes neither accepts go to the plain kernel.  The choice depends on the number of
rows only, never on their content.
"""

from __future__ import annotations

import torch

from ..csrc import ops

SKINNY_MAX_ROWS = 64


def linear(x: torch.Tensor, weight: torch.Tensor, out_dtype: torch.dtype | None = None) -> torch.Tensor:
    """x [T, K] (unit inner stride), weight [N, K] contiguous -> [T, N]."""
    if x.dtype == torch.bfloat16:
        fast = ops.gemm_bf16(x, weight, out_dtype)
        if fast is not None:
            return fast
    return ops.gemm_generic(x, weight, out_dtype)
