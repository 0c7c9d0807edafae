"""y = x W^T for the parts, with the kernel chosen by element type and number of rows.

* float32: the plain kernel with float operands (the true 32-bit path), always.
* bfloat16, at most 16 rows (decoding): the fused decode kernel, which also takes in a pending
  residual sum + norm in front and an activation or the rotary/cache write behind.
* bfloat16, 17 to 128 rows (decoding with many requests, short prompt portions): the streaming kernel over the
  weights' tiled copy (``Weight``), with the same epilogues, or with float partial sums of ranges of K that the
  consuming norm adds; where it was measured slower than the library (the gated product beyond 64 rows, the
  output head) the library stays.
* bfloat16, more rows (prompt portions): the vendor's matrix-product library, with bfloat16 or (logits)
  float results.

The choice depends on the number of rows and the sizes only, never on the rows' content.  ``x`` may
be a tensor or a ``PendingNorm``; a weight may be a tensor [N, K] or a ``Weight``.
"""

from __future__ import annotations

import torch

from ..csrc import ops
from .norm import PendingNorm, rows_of


class Weight:
    """A part's matrix [N, K] with, for bfloat16 matrices whose K is a multiple of 32, a second copy in the tiled
    order that the streaming kernel reads (1 KB tiles in the matrix instruction's operand order; see
    ``ops.tile_weight``).  ``pairing``: which rows share a tile, by what the epilogue behind the product needs:
    "plain", "gated" ([gate; up] rows) or "rotary" ([q; k; v] rows of heads of ``head_dim``).  The plain copy serves
    the other kernels and the library; a step reads one of the two."""

    def __init__(self, plain: torch.Tensor, pairing: str = "plain", head_dim: int = 0):
        self.plain = plain
        self.pairing = pairing
        ok = ops.stream_linear_takes(plain) and (pairing != "rotary" or (head_dim > 0 and head_dim % 16 == 0))
        self.tiled = ops.tile_weight(plain, pairing, head_dim) if ok else None

    @property
    def shape(self):
        return self.plain.shape

    @property
    def dtype(self):
        return self.plain.dtype

    def rows(self, count: int) -> torch.Tensor:
        """The first ``count`` rows as a plain matrix (a view)."""
        return self.plain[:count]


STREAM_MIN_ROWS, STREAM_MAX_ROWS = 17, 128      # rows the streaming kernel is chosen for
TILE_MAX_ROWS = 640                             # rows up to which the tiled kernel is chosen for small matrices cut along K
# ... and from so few rows on for matrices of so many elements that fill the GPU in so many ranges of K at most
TILE_PARTIAL_FROM_ROWS, TILE_PARTIAL_MIN_ELEMENTS, TILE_PARTIAL_MOST_RANGES = 65, 1 << 24, 12
STREAM_GATED_MAX_ROWS = 64                      # the gated product: beyond, its rows' traffic costs more than the library's kernel
                                                # (asked only where the tiled kernel does not take the product: _tiles_gated)
STREAM_LONG_K, STREAM_LONG_K_MAX_ROWS = 8192, 64 # from this K on a product in one range takes the streaming kernel up to so many rows


def _plain(weight) -> torch.Tensor:
    return weight.plain if isinstance(weight, Weight) else weight


def _few_weight_rows(weight) -> bool:
    """Matrices with at most 32 weight rows per compute unit: their workgroups fit one round (with more rows, every
    further workgroup reads all input rows again, and the library's larger tiles win: 11264 x 2048, 32000 x 2048)."""
    return weight.shape[0] <= 32 * ops._num_compute_units(weight.plain.device)


def _tiles(x, weight, partial_ok: bool) -> bool:
    """Whether this plain product goes to the tiled kernel (129 to 640 rows): only as partial sums of ranges of K, which
    give a small matrix enough workgroups, when whoever takes the result adds them (2048 x 5632 at 264 rows: 14 us against
    the library's 23; 2048 x 2048: 8.5 against 12.5; in one range, or for 11264 x 2048, the library's kernels are faster).
    Larger matrices take it from 65 rows on, where the streaming kernel is chosen otherwise: a workgroup's tile of 128
    weight rows over a range of K draws the step's rows a quarter as often as the streaming kernel's 32 weight rows over
    all of K (4096 x 14336 at 64 / 96 / 128 rows: 24.3 / 26.6 / 29.6 us against 28.3 / 45.5 / 55.2; 4096 x 4096: 10.7 / 12.0 /
    13.7 against 13.0 / 16.6 / 19.0; 2048 x 5632 the same either way and 2048 x 2048 8.5 against 7.0 at 128 rows: those
    stay).  Inside whole steps the gain shows from 65 rows on and where a dozen ranges fill the GPU (the norm kernel adds
    them): Llama-3.1-8B shapes at 96 / 128 requests 9,361 -> 9,831 and 10,057 -> 10,633 tok/s, a prompt of 128 tokens 6.09 ->
    5.52 ms; 2048 x 8192, which needs 16 ranges, lost 1 to 2 % there although it is faster on its own (12.5 against 15.9 us)."""
    if not (partial_ok and isinstance(weight, Weight) and weight.tiled is not None and weight.pairing == "plain"):
        return False
    rows = x.num_rows if isinstance(x, PendingNorm) else x.shape[0]
    n, k = weight.shape
    if not (x.dtype == torch.bfloat16 and _few_weight_rows(weight)):
        return False
    ranges = ops.tile_linear_plan(rows, n, k, ops._num_compute_units(weight.plain.device))
    if TILE_PARTIAL_FROM_ROWS <= rows <= STREAM_MAX_ROWS:
        return n * k >= TILE_PARTIAL_MIN_ELEMENTS and 1 < ranges <= TILE_PARTIAL_MOST_RANGES
    return STREAM_MAX_ROWS < rows <= TILE_MAX_ROWS and ranges > 1


def _streams(x, weight, epi: int, partial_ok: bool = False) -> bool:
    """Whether this product goes to the streaming kernel: by sizes and row count only (measured on matrices of
    2048 x 2048 to 11264 x 2048 and 2048 x 5632 against the library and the kernels for fewer rows)."""
    if not (isinstance(weight, Weight) and weight.tiled is not None):
        return False
    rows = x.num_rows if isinstance(x, PendingNorm) else x.shape[0]
    if not STREAM_MIN_ROWS <= rows <= STREAM_MAX_ROWS or x.dtype != torch.bfloat16:
        return False
    n, k = weight.shape
    if epi == ops.SL_GATED:
        return rows <= STREAM_GATED_MAX_ROWS
    if epi == ops.SL_F32:
        return False                                            # (the head: 32000 x 2048 was not faster than the library's kernel)
    # (cut into ranges of K the long products stay ahead of the library up to 128 rows: 4096 x 14336 at 96 / 128 rows 45.7 / 55.4 us
    #  against 62.6 / 74.8, 2048 x 8192 16.1 / 18.4 against 20.8)
    return _few_weight_rows(weight) and (k < STREAM_LONG_K or rows <= STREAM_LONG_K_MAX_ROWS or (partial_ok and epi == ops.SL_BF16))


def _stream(x, weight: Weight, epi: int, rope: dict | None = None, partial_ok: bool = False, activation: str = "silu"):
    x = rows_of(x)
    if x.stride(1) != 1 or x.stride(0) % 8 or x.data_ptr() % 16:
        x = x.contiguous()
    n, k = weight.shape
    if epi == ops.SL_GATED:
        return ops.stream_linear(x, weight.tiled, epi, activation=activation)
    if epi == ops.SL_BF16 and partial_ok:
        nt, splits = ops.stream_linear_plan(x.shape[0], n, k, ops._num_compute_units(x.device), partial=True)
        if splits > 1:
            return ops.stream_linear(x, weight.tiled, ops.SL_PARTIAL, nt=nt, splits=splits)
    return ops.stream_linear(x, weight.tiled, epi, rope=rope)


_PAIRING_OF = {ops.EPI_GATED: "gated", ops.EPI_ROPE_KV: "rotary"}


def _fused(x, weight, epi: int, rope: dict | None = None, activation: str = "silu"):
    """The fused decode kernel if it takes the operands, else None.  With a ``Weight`` whose tiled copy has the pairing
    of the epilogue, products of at most 16 rows with the sum and norm in front stream the weights from that copy
    (11264 x 2048: 12.3 against 13.4 us; 2560 x 2048 with the rotary epilogue: 7.4 against 7.9; 32000 x 2048: 29.0 against 30.4)."""
    tiled = None
    if isinstance(weight, Weight):
        if weight.tiled is not None and weight.pairing == _PAIRING_OF.get(epi, "plain"):
            tiled = weight.tiled
        weight = weight.plain
    if isinstance(x, PendingNorm):
        if x.fusable() and ops.decode_linear_takes(x.num_rows, x.x.shape[1], x.x, weight):
            args = x.fused_arguments()
            out = ops.decode_linear(x.x, weight, epi, rope=rope, tiled=tiled, activation=activation, **args)
            x.fused_done(args)
            return out
        x = x.rows()
    if (x.dtype == torch.bfloat16 and ops.decode_linear_takes(x.shape[0], x.shape[1], x, weight, staged=False)
            and ops.decode_linear_pays(x.shape[0], weight.shape[0], x.shape[1], epi, staged=False)):
        # (plain rows keep the row-major matrix: from the tiled copy 4096 x 4096 and 4096 x 14336 took 10.7 and 32.9 us at 8
        #  rows against 9.3 and 27.7, and the smaller matrices the same time either way)
        return ops.decode_linear(x, weight, epi, rope=rope, activation=activation)
    return None


def linear(x, weight, out_dtype: torch.dtype | None = None, partial_ok: bool = False, bias: torch.Tensor | None = None) -> torch.Tensor:
    """x [T, K] (tensor or pending norm), weight [N, K] -> [T, N].  ``partial_ok``: the caller hands the result to a
    norm as its delta and that norm adds partial sums (``StepContext.partial_sums_ok``): the result may then be float
    [ranges, T, N], the sums over ranges of K.  ``bias`` (float32 [N]): added to the product's float sums, the result
    rounded once (a kernel of its own behind the product)."""
    if bias is not None:
        sums = linear(x, weight, torch.float32)
        return ops.add_bias(sums, bias, out_dtype or _plain(weight).dtype)
    if out_dtype != torch.float32 and _tiles(x, weight, partial_ok):
        x = rows_of(x)
        if x.stride(1) != 1 or x.stride(0) % 8 or x.data_ptr() % 16:
            x = x.contiguous()
        return ops.tile_linear(x, weight.tiled, ops.SL_PARTIAL)
    if _streams(x, weight, ops.SL_F32 if out_dtype == torch.float32 else ops.SL_BF16, partial_ok):
        return _stream(x, weight, ops.SL_F32 if out_dtype == torch.float32 else ops.SL_BF16, partial_ok=partial_ok)
    if weight.dtype == torch.bfloat16:
        out = _fused(x, weight, ops.EPI_F32 if out_dtype == torch.float32 else ops.EPI_BF16)
        if out is not None:
            return out
    weight = _plain(weight)
    x = rows_of(x)
    if x.dtype == torch.bfloat16 and weight.dtype == torch.bfloat16:
        return ops.gemm_bf16(x, weight, out_dtype)
    return ops.gemm_generic(x, weight, out_dtype)


TILE_ROTARY_ROWS = (97, 1536)                   # rows for which the q/k/v product takes the tiled kernel with the rotary epilogue,
                                                # as long as its tiles fit the compute units in one round
TILE_ROTARY_FROM_WHEN_LARGE, TILE_ROTARY_LARGE_ELEMENTS = 65, 1 << 23   # ... and from so few rows on for matrices of so many elements
TILE_GATED_ROWS = (161, 320)                    # rows for which the gated product takes the tiled kernel
TILE_GATED_FROM_WHEN_FILLING = 24               # ... and from so few rows on when one block of rows already fills the GPU
TILE_GATED_FROM_WHEN_NARROW = 17                # ... or when the kernel takes tiles of 64 weight rows for it (one block of rows)


_one_round: dict = {}


def _tiles_in_one_round(rows: int, weight) -> bool:
    """Whether the tiled kernel's tiles for a product of ``rows`` rows in one range of K fit the compute units in one round."""
    cus = ops._num_compute_units(weight.plain.device)
    key = (rows, weight.shape[0], cus)
    if key not in _one_round:
        _one_round[key] = ops.tile_linear_shape(rows, weight.shape[0], cus)[2] <= cus
    return _one_round[key]


def _tiles_gated(x, weight, rows: int) -> bool:
    """Whether the gated product goes to the tiled kernel.  With two blocks of input rows it takes as long as the library's
    product (11264 x 2048 at 264 rows: 28 us both) and saves the activation kernel and its pass over the intermediate rows
    (5 us).  A matrix whose tiles of 128 weight rows fill three quarters of the compute units by themselves takes it with
    one block of rows as well, from a few rows on: there every workgroup draws its own weights and the step's few rows,
    where the streaming kernel's workgroups of 32 to 64 weight rows draw the rows four times as often (28672 x 4096 at
    32 / 64 / 128 rows: 46 / 46 / 52 us against 50 / 57 us streaming and 53 / 53 / 59 us in the library with the activation
    kernel; 24576 x 2048 at 64 rows 27 against 33 and 30).  A matrix whose tiles of 128 fill at most half of the compute
    units is cut into tiles of 64 weight rows by the kernel when there is one block of rows, twice the workgroups (11264 x
    2048 at 64 / 96 / 128 / 160 rows: 14.0 / 16.1 / 19.0 / 21.7 us against 18.8 / 20.3 / 21.8 / 27.6 in the library with the
    activation kernel and 14.8 streaming at 64; 16384 x 2048 at 32 / 64 rows: 15.7 / 16.8 against 19.0 / 21.0 streaming; inside
    whole steps of 24 requests 0.5 to 3.6 % faster than the streaming kernel at three sets of shapes)."""
    if not (isinstance(weight, Weight) and weight.tiled is not None and weight.pairing == "gated" and x.dtype == torch.bfloat16):
        return False
    tiles, cus = weight.shape[0] // 128, ops._num_compute_units(weight.plain.device)
    if 4 * tiles >= 3 * cus:
        first = TILE_GATED_FROM_WHEN_FILLING
    elif 2 * tiles <= cus:
        first = TILE_GATED_FROM_WHEN_NARROW
    else:
        first = TILE_GATED_ROWS[0]
    return first <= rows <= TILE_GATED_ROWS[1]


def gated_linear(x, w_gate_up, activation: str = "silu") -> torch.Tensor:
    """act(x Wg^T) * (x Wu^T) with [Wg; Wu] stacked in one matrix (a tensor, or a ``Weight`` with the gated pairing);
    ``activation``: one of ``ops.ACTIVATIONS``."""
    rows = x.num_rows if isinstance(x, PendingNorm) else x.shape[0]
    tiles = _tiles_gated(x, w_gate_up, rows)
    if not tiles and _streams(x, w_gate_up, ops.SL_GATED) and w_gate_up.pairing == "gated":
        return _stream(x, w_gate_up, ops.SL_GATED, activation=activation)
    if tiles:
        x = rows_of(x)
        if x.stride(1) != 1 or x.stride(0) % 8 or x.data_ptr() % 16:
            x = x.contiguous()
        return ops.tile_linear(x, w_gate_up.tiled, ops.SL_GATED, activation=activation)
    if w_gate_up.dtype == torch.bfloat16:
        out = _fused(x, w_gate_up, ops.EPI_GATED, activation=activation)
        if out is not None:
            return out
    w_gate_up = _plain(w_gate_up)
    return ops.gate_mul(linear(x, w_gate_up), activation)


def qkv_rotary_cache(x, w_qkv, positions: torch.Tensor, position_encoding, num_heads: int, num_kv_heads: int,
                     head_dim: int, slot_mapping, k_pages, v_pages, block_size: int, bias: torch.Tensor | None = None) -> torch.Tensor:
    """q, k, v projections, rotation of q and k, and the write of k and v into the cache pages.
    Returns q as rows of a matrix whose first num_heads * head_dim columns hold the rotated heads
    (the row stride may be larger).  With k_pages None only q is projected and rotated.
    ``position_encoding``: a part with ``cos``/``sin`` tables, ``rotary_dim`` and ``interleaved``, or None.
    The fused kernel pairs element i with i + d/2 over the whole head; another rotated width or pairing, and
    projections with a ``bias`` (float32, one value per row of ``w_qkv``), go through the product and the rotary kernel apart."""
    write = k_pages is not None
    cos = sin = None
    rotary_dim, interleaved = 0, False                      # no position encoding: nothing turns
    if position_encoding is not None:
        cos, sin = position_encoding.cos, position_encoding.sin
        rotary_dim = position_encoding.rotary_dim or head_dim
        interleaved = bool(position_encoding.interleaved)
    whole_head_halves = position_encoding is None or (rotary_dim == head_dim and not interleaved)
    if write and w_qkv.dtype == torch.bfloat16 and head_dim % 16 == 0 and whole_head_halves and bias is None:
        rope = dict(positions=positions, cos=cos, sin=sin, slots=slot_mapping, k_pages=k_pages, v_pages=v_pages,
                    num_heads=num_heads, num_kv_heads=num_kv_heads, head_dim=head_dim, block_size=block_size)
        tiled_ok = (isinstance(w_qkv, Weight) and w_qkv.pairing == "rotary" and w_qkv.tiled is not None and x.dtype == torch.bfloat16
                    and _few_weight_rows(w_qkv) and (cos is None or cos.data_ptr() % 16 == 0))
        rows = x.num_rows if isinstance(x, PendingNorm) else x.shape[0]
        large = tiled_ok and w_qkv.shape[0] * w_qkv.shape[1] >= TILE_ROTARY_LARGE_ELEMENTS
        if (tiled_ok and (TILE_ROTARY_FROM_WHEN_LARGE if large else TILE_ROTARY_ROWS[0]) <= rows <= TILE_ROTARY_ROWS[1]
                and _tiles_in_one_round(rows, w_qkv)):
            # A few hundred rows: the tiled kernel in the shape that fills the GPU in one round, with the rotation and the
            # cache write in its epilogue (2560 x 2048 at 264 rows: 11.8 us against 16.9 in the library with the rotary kernel
            # behind it; 6144 x 4096: 28 against 37; at 1024 rows 21.5 against 27.4, but 90.7 against 61.9 for 6144 x 4096,
            # whose tiles need a second round there).  Larger matrices
            # from 65 rows on, ahead of the streaming kernel (6144 x 4096 at 96 / 128 rows: 20.6 / 22.1 us against 25.0 / 28.7;
            # 5120 x 3072: 14.3 / 17.1 against 17.7 / 20.2); smaller ones from 97 rows (2560 x 2048 at 128 rows: 10.0 against 10.7
            # on its own and 13.3 inside a step; decode at 128 requests 47.2 -> 48.5 k tok/s, a prompt of 128 tokens 1.77 -> 1.70 ms).
            x = rows_of(x)
            if x.stride(1) != 1 or x.stride(0) % 8 or x.data_ptr() % 16:
                x = x.contiguous()
            return ops.tile_linear(x, w_qkv.tiled, ops.SL_ROPE_KV, rope=rope)
        if (isinstance(w_qkv, Weight) and w_qkv.pairing == "rotary" and _streams(x, w_qkv, ops.SL_ROPE_KV)
                and (cos is None or cos.data_ptr() % 16 == 0)):
            return _stream(x, w_qkv, ops.SL_ROPE_KV, rope=rope)
        q = _fused(x, w_qkv, ops.EPI_ROPE_KV, rope)
        if q is not None:
            return q
    w_qkv = _plain(w_qkv)
    qkv = linear(x, w_qkv, bias=bias)
    ops.rope_scatter(qkv, positions, cos, sin, num_heads, num_kv_heads, head_dim, slot_mapping if write else None,
                     k_pages, v_pages, block_size, rotary_dim, interleaved)
    return qkv
