"""y = x W^T for the parts, with the kernel chosen by element type and number of rows.

* float32: the plain kernel with float operands (the true 32-bit path), always.
* bfloat16, at most 16 rows (decoding): the fused decode kernel, which also takes in a pending
  residual sum + norm in front and an activation or the rotary/cache write behind.
* bfloat16, 17 to 64 rows and a small matrix: the same kernel's form for plain rows (the norm runs first).
* bfloat16, more rows (prompt portions): the vendor's matrix-product library, with bfloat16 or (logits)
  float results.

The choice depends on the number of rows and the sizes only, never on the rows' content.  ``x`` may
be a tensor or a ``PendingNorm``.
"""

from __future__ import annotations

import torch

from ..csrc import ops
from .norm import PendingNorm, rows_of


def _fused(x, weight: torch.Tensor, epi: int, rope: dict | None = None):
    """The fused decode kernel if it takes the operands, else None."""
    if isinstance(x, PendingNorm):
        if x.fusable() and ops.decode_linear_takes(x.num_rows, x.x.shape[1], x.x, weight):
            args = x.fused_arguments()
            out = ops.decode_linear(x.x, weight, epi, rope=rope, **args)
            x.fused_done(args)
            return out
        x = x.rows()
    if (x.dtype == torch.bfloat16 and ops.decode_linear_takes(x.shape[0], x.shape[1], x, weight, staged=False)
            and ops.decode_linear_pays(x.shape[0], weight.shape[0], x.shape[1], epi, staged=False)):
        return ops.decode_linear(x, weight, epi, rope=rope)
    return None


def linear(x, weight: torch.Tensor, out_dtype: torch.dtype | None = None) -> torch.Tensor:
    """x [T, K] (tensor or pending norm), weight [N, K] -> [T, N]."""
    if weight.dtype == torch.bfloat16:
        out = _fused(x, weight, ops.EPI_F32 if out_dtype == torch.float32 else ops.EPI_BF16)
        if out is not None:
            return out
    x = rows_of(x)
    if x.dtype == torch.bfloat16 and weight.dtype == torch.bfloat16:
        return ops.gemm_bf16(x, weight, out_dtype)
    return ops.gemm_generic(x, weight, out_dtype)


def gated_linear(x, w_gate_up: torch.Tensor) -> torch.Tensor:
    """silu(x Wg^T) * (x Wu^T) with [Wg; Wu] stacked in one matrix."""
    if w_gate_up.dtype == torch.bfloat16:
        out = _fused(x, w_gate_up, ops.EPI_GATED)
        if out is not None:
            return out
    return ops.silu_mul(linear(x, w_gate_up))


def qkv_rotary_cache(x, w_qkv: torch.Tensor, positions: torch.Tensor, position_encoding, num_heads: int, num_kv_heads: int,
                     head_dim: int, slot_mapping, k_pages, v_pages, block_size: int) -> torch.Tensor:
    """q, k, v projections, rotation of q and k, and the write of k and v into the cache pages.
    Returns q as rows of a matrix whose first num_heads * head_dim columns hold the rotated heads
    (the row stride may be larger).  With k_pages None only q is projected and rotated.
    ``position_encoding``: a part with ``cos``/``sin`` tables, ``rotary_dim`` and ``interleaved``, or None.
    The fused kernel pairs element i with i + d/2 over the whole head; another rotated width or pairing
    goes through the product and the rotary kernel apart."""
    write = k_pages is not None
    cos = sin = None
    rotary_dim, interleaved = 0, False                      # no position encoding: nothing turns
    if position_encoding is not None:
        cos, sin = position_encoding.cos, position_encoding.sin
        rotary_dim = position_encoding.rotary_dim or head_dim
        interleaved = bool(position_encoding.interleaved)
    whole_head_halves = position_encoding is None or (rotary_dim == head_dim and not interleaved)
    if write and w_qkv.dtype == torch.bfloat16 and head_dim % 16 == 0 and whole_head_halves:
        rope = dict(positions=positions, cos=cos, sin=sin, slots=slot_mapping, k_pages=k_pages, v_pages=v_pages,
                    num_heads=num_heads, num_kv_heads=num_kv_heads, head_dim=head_dim, block_size=block_size)
        q = _fused(x, w_qkv, ops.EPI_ROPE_KV, rope)
        if q is not None:
            return q
    qkv = linear(x, w_qkv)
    ops.rope_scatter(qkv, positions, cos, sin, num_heads, num_kv_heads, head_dim, slot_mapping if write else None,
                     k_pages, v_pages, block_size, rotary_dim, interleaved)
    return qkv
