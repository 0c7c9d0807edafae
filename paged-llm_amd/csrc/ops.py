"""Python faces of the HIP kernels.

Every function checks on the host that shapes, element types, strides and devices are what the
kernel and its launch grid assume, and only then passes raw device pointers and the current HIP
stream through ctypes.  A kernel that cannot take a size says so here with a clear error; there
is no CPU fallback, and a missing or unbuildable library raises at the first call.
"""

from __future__ import annotations

import ctypes
import logging
from ctypes import c_float, c_int, c_long, c_longlong, c_ulonglong, c_void_p

import numpy as np
import torch

from . import build

log = logging.getLogger("paged_llm_amd")
_warned_plain_attention: list = []       # (said once per process)
F32, BF16 = 0, 1
_DTYPE_CODE = {torch.float32: F32, torch.bfloat16: BF16}
MAX_HEAD_DIM_GENERIC = 256


class KernelError(RuntimeError):
    pass


def dtype_code(dtype: torch.dtype) -> int:
    try:
        return _DTYPE_CODE[dtype]
    except KeyError:
        raise KernelError(f"kernels take float32 or bfloat16, not {dtype}") from None


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)
_raw_device = getattr(torch._C, "_cuda_getDevice", None)


def _stream():
    """The current HIP stream of the current device, as what ctypes passes for a pointer."""
    if _raw_stream is not None and _raw_device is not None:
        return _raw_stream(_raw_device())
    return torch.cuda.current_stream().cuda_stream


def _ptr(t: torch.Tensor | None):
    return None if t is None else t.data_ptr()


def _check(code: int, what: str) -> None:
    if code != 0:
        raise KernelError(f"{what}: kernel launch failed with code {code}")


def _need(cond: bool, msg: str) -> None:
    if not cond:
        raise KernelError(msg)


def _on_gpu(*tensors: torch.Tensor | None) -> None:
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise KernelError("kernel operands must live on the GPU (there is no CPU path)")


_SIGNATURES = {
    "pllm_embed_gather": [c_int, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_void_p],
    "pllm_rmsnorm": [c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_float, c_void_p, c_void_p, c_int, c_int, c_void_p, c_int, c_long,
                     c_void_p],
    "pllm_gate_mul": [c_int, c_int, c_void_p, c_void_p, c_int, c_int, c_void_p],
    "pllm_add_bias": [c_int, c_void_p, c_int, c_void_p, c_void_p, c_int, c_int, c_int, c_void_p],
    "pllm_rope_scatter": [c_int, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                          c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_void_p],
    "pllm_copy_pages": [c_int, c_void_p, c_void_p, c_void_p, c_int, c_long, c_void_p],
    "pllm_gemm_nt": [c_int, c_int, c_void_p, c_int, c_void_p, c_int, c_void_p, c_int, c_int, c_int, c_int, c_void_p],
    "pllm_paged_attention_generic": [c_int, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_int,
                                     c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_float, c_int,
                                     c_float, c_void_p, c_void_p, c_void_p],
    "pllm_sample": [c_void_p, c_int, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_ulonglong, c_void_p,
                    c_void_p, c_void_p],
    "pllm_sample_workspace_bytes": [c_int, c_int],
    "pllm_argmax": [c_void_p, c_int, c_int, c_void_p, c_void_p],
}
_FUNCS: dict = {}


def _fn(source: str, name: str, defines: dict | None = None, signature: list | None = None):
    key = (source, name, tuple(sorted(defines.items()))) if defines else (source, name)
    f = _FUNCS.get(key)
    if f is None:
        lib = build.load_library(source, defines)
        f = getattr(lib, name)
        f.argtypes = signature if signature is not None else _SIGNATURES[name]
        f.restype = c_int
        _FUNCS[key] = f
    return f


# ------------------------------------------------------------------------------------------- rows
def embed_gather(ids: torch.Tensor, table: torch.Tensor, out: torch.Tensor | None = None) -> torch.Tensor:
    """out[t] = table[ids[t]]; ids int32 [T] (range already checked by the caller)."""
    _on_gpu(ids, table)
    _need(ids.dtype == torch.int32 and ids.dim() == 1 and ids.is_contiguous(), "ids must be contiguous int32 [T]")
    _need(table.dim() == 2 and table.is_contiguous(), "embedding table must be contiguous [vocab, hidden]")
    T, (V, H) = ids.numel(), table.shape
    if out is None:
        out = torch.empty((T, H), dtype=table.dtype, device=table.device)
    _need(out.shape == (T, H) and out.dtype == table.dtype and out.is_contiguous(), "bad output for embed_gather")
    _check(_fn("elementwise.hip", "pllm_embed_gather")(dtype_code(table.dtype), _ptr(ids), _ptr(table), _ptr(out),
                                                        T, H, V, _stream()), "embed_gather")
    return out


def rmsnorm(x: torch.Tensor, weight: torch.Tensor, eps: float, delta: torch.Tensor | None = None,
            row_index: torch.Tensor | None = None, write_residual: bool = True) -> torch.Tensor:
    """RMS norm of the rows of x (after adding delta, when given).

    With ``delta`` the sum ``x + delta`` (float add, rounded to the element type) is the new
    residual; it is written back into ``x`` unless ``write_residual`` is False.  ``row_index``
    (int32) selects which rows are normed; the output then has one row per index.
    ``delta`` may also be a float tensor [ranges, rows, hidden]: the partial sums of a product whose inner dimension
    was cut into ranges (``stream_linear`` with SL_PARTIAL); they are added in order, in float, with x.
    """
    _on_gpu(x, weight, delta, row_index)
    _need(x.dim() == 2 and x.is_contiguous(), "x must be contiguous [rows, hidden]")
    H = x.shape[1]
    _need(weight.dtype == torch.float32 and weight.shape == (H,) and weight.is_contiguous(),
          f"norm weight must be float32 [{H}], got {weight.dtype} {tuple(weight.shape)}")
    _need((H + 16) * 4 <= min(_max_lds_bytes(x.device), 160 * 1024),
          f"rmsnorm kernel stages one row in LDS as floats: hidden size {H} is above its limit")
    parts = None
    if delta is not None and delta.dim() == 3:
        parts, delta = delta, None
        _need(parts.dtype == torch.float32 and tuple(parts.shape[1:]) == tuple(x.shape) and parts.is_contiguous(),
              f"partial sums must be contiguous float32 [ranges, {x.shape[0]}, {H}]")
    if delta is not None:
        _need(delta.shape == x.shape and delta.dtype == x.dtype and delta.is_contiguous(), "delta must match x")
    if row_index is not None:
        _need(row_index.dtype == torch.int32 and row_index.dim() == 1 and row_index.is_contiguous(),
              "row_index must be contiguous int32")
        rows = row_index.numel()
    else:
        rows = x.shape[0]
    out = torch.empty((rows, H), dtype=x.dtype, device=x.device)
    x_out = x if ((delta is not None or parts is not None) and write_residual) else None
    _check(_fn("elementwise.hip", "pllm_rmsnorm")(dtype_code(x.dtype), _ptr(x), _ptr(delta), _ptr(row_index), _ptr(weight),
                                                   c_float(eps), _ptr(out), _ptr(x_out), rows, H, _ptr(parts),
                                                   0 if parts is None else parts.shape[0], 0 if parts is None else x.numel(),
                                                   _stream()), "rmsnorm")
    return out


ACTIVATIONS = {"silu": 0, "gelu_tanh": 1}      # the gate's activation in a gated product (PLLM_ACT_* in common.h)


def activation_code(name: str) -> int:
    _need(name in ACTIVATIONS, f"gate activation {name!r}: one of {sorted(ACTIVATIONS)}")
    return ACTIVATIONS[name]


def gate_mul(gate_up: torch.Tensor, activation: str = "silu") -> torch.Tensor:
    """[T, 2I] -> act(first half) * second half, [T, I]."""
    _on_gpu(gate_up)
    _need(gate_up.dim() == 2 and gate_up.is_contiguous() and gate_up.shape[1] % 2 == 0, "gate_up must be contiguous [T, 2I]")
    T, I = gate_up.shape[0], gate_up.shape[1] // 2
    out = torch.empty((T, I), dtype=gate_up.dtype, device=gate_up.device)
    _check(_fn("elementwise.hip", "pllm_gate_mul")(dtype_code(gate_up.dtype), activation_code(activation), _ptr(gate_up), _ptr(out), T, I,
                                                   _stream()), "gate_mul")
    return out


def silu_mul(gate_up: torch.Tensor) -> torch.Tensor:
    return gate_mul(gate_up, "silu")


def add_bias(sums: torch.Tensor, bias: torch.Tensor, dtype: torch.dtype) -> torch.Tensor:
    """float sums [T, N] + float bias [N], rounded once to ``dtype``."""
    _on_gpu(sums, bias)
    _need(sums.dtype == torch.float32 and sums.dim() == 2 and sums.stride(1) == 1, "add_bias: float rows with unit inner stride")
    _need(bias.dtype == torch.float32 and bias.shape == (sums.shape[1],) and bias.is_contiguous(), f"bias: float32 [{sums.shape[1]}]")
    out = torch.empty(sums.shape, dtype=dtype, device=sums.device)
    _check(_fn("elementwise.hip", "pllm_add_bias")(dtype_code(dtype), _ptr(sums), sums.stride(0), _ptr(bias), _ptr(out), out.stride(0),
                                                   sums.shape[0], sums.shape[1], _stream()), "add_bias")
    return out


def rope_scatter(qkv: torch.Tensor, positions: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor,
                 num_heads: int, num_kv_heads: int, head_dim: int, slot_mapping: torch.Tensor | None,
                 k_pages: torch.Tensor | None, v_pages: torch.Tensor | None, block_size: int,
                 rotary_dim: int | None = None, interleaved: bool = False) -> None:
    """Rotate q (in place) and k by the tables' angles at ``positions``; write k and v into pages.

    qkv: [T, >= (num_heads + 2 kv_heads) * d] rows (only q columns are needed when nothing is
    written).  k_pages [P, kv, bs, d], v_pages [P, kv, d, bs].  ``rotary_dim`` (default: the whole
    head) is how many leading elements of a head turn; ``interleaved`` pairs (2i, 2i + 1) instead of
    (i, i + rotary_dim / 2).  The caller guarantees positions < cos.shape[0] and slots < P * bs
    (checked on the host where the batch is built).
    """
    write_kv = k_pages is not None
    _on_gpu(qkv, positions, cos, sin, slot_mapping, k_pages, v_pages)
    T = qkv.shape[0]
    _need(qkv.dim() == 2 and qkv.stride(1) == 1, "qkv must be [T, width] with unit inner stride")
    need_cols = (num_heads + (2 * num_kv_heads if write_kv else 0)) * head_dim
    _need(qkv.shape[1] >= need_cols, f"qkv rows hold {qkv.shape[1]} values, need {need_cols}")
    rotary_dim = head_dim if rotary_dim is None else int(rotary_dim)
    _need(0 <= rotary_dim <= head_dim and rotary_dim % 2 == 0,
          f"rotary pairing needs an even width of at most the head size {head_dim}, got {rotary_dim}")
    _need(positions.dtype == torch.int32 and positions.shape == (T,) and positions.is_contiguous(), "positions: int32 [T]")
    half = rotary_dim // 2
    _need((cos is None) == (sin is None), "cos and sin tables come together")
    for t in (cos, sin):
        if t is None:
            continue
        _need(t.dtype == torch.float32 and t.dim() == 2 and t.shape[1] == half and t.is_contiguous(),
              f"rotary tables must be float32 [positions, {half}]")
    if write_kv:
        _need(slot_mapping is not None and slot_mapping.dtype == torch.int32 and slot_mapping.shape == (T,)
              and slot_mapping.is_contiguous(), "slot_mapping: int32 [T]")
        P = k_pages.shape[0]
        _need(tuple(k_pages.shape) == (P, num_kv_heads, block_size, head_dim) and k_pages.is_contiguous()
              and k_pages.dtype == qkv.dtype, "k_pages must be contiguous [pages, kv_heads, block_size, head_dim]")
        _need(tuple(v_pages.shape) == (P, num_kv_heads, head_dim, block_size) and v_pages.is_contiguous()
              and v_pages.dtype == qkv.dtype, "v_pages must be contiguous [pages, kv_heads, head_dim, block_size]")
    _check(_fn("elementwise.hip", "pllm_rope_scatter")(
        dtype_code(qkv.dtype), _ptr(qkv), qkv.stride(0), _ptr(positions), _ptr(cos), _ptr(sin), _ptr(slot_mapping),
        _ptr(k_pages), _ptr(v_pages), T, num_heads, num_kv_heads, head_dim, block_size, 1 if write_kv else 0,
        rotary_dim, 1 if interleaved else 0, _stream()), "rope_scatter")


def copy_pages(pages: torch.Tensor, src: torch.Tensor, dst: torch.Tensor) -> None:
    """pages[dst[i]] = pages[src[i]] (whole pages of one tensor of a layer's cache, of any element type: the
    bytes are copied in units of two or four)."""
    _on_gpu(pages, src, dst)
    _need(pages.is_contiguous() and pages.dim() >= 2, "pages must be contiguous [pages, ...]")
    _need(src.dtype == torch.int32 and dst.dtype == torch.int32 and src.shape == dst.shape and src.dim() == 1,
          "src and dst must be int32 vectors of one length")
    page_bytes = pages[0].numel() * pages.element_size()
    _need(page_bytes % 2 == 0 and pages.data_ptr() % 4 == 0, "a page must be an even number of bytes")
    unit, code = (4, F32) if page_bytes % 4 == 0 else (2, BF16)
    _check(_fn("elementwise.hip", "pllm_copy_pages")(code, _ptr(pages), _ptr(src), _ptr(dst),
                                                      src.numel(), page_bytes // unit, _stream()), "copy_pages")


# ------------------------------------------------------------------------------------------- products
def gemm_generic(a: torch.Tensor, w: torch.Tensor, out_dtype: torch.dtype | None = None) -> torch.Tensor:
    """a [M, K] times w [N, K] transposed, float accumulation in ascending k, any sizes."""
    _on_gpu(a, w)
    _need(a.dim() == 2 and w.dim() == 2 and a.shape[1] == w.shape[1], f"gemm shapes {tuple(a.shape)} x {tuple(w.shape)}^T")
    _need(a.stride(1) == 1 and w.stride(1) == 1, "gemm operands need unit inner stride")
    _need(a.dtype == w.dtype, "gemm operands must share their element type")
    out_dtype = out_dtype or a.dtype
    M, K = a.shape
    N = w.shape[0]
    out = torch.empty((M, N), dtype=out_dtype, device=a.device)
    _check(_fn("gemm_generic.hip", "pllm_gemm_nt")(dtype_code(a.dtype), dtype_code(out_dtype), _ptr(a), a.stride(0),
                                                    _ptr(w), w.stride(0), _ptr(out), N, M, N, K, _stream()), "gemm_generic")
    return out


# ------------------------------------------------------------------------------------------- attention
def _check_attention_args(q, k_pages, v_pages, block_tables, cu_seqlens_q, seq_lens_k, num_heads, num_kv_heads, head_dim):
    _on_gpu(q, k_pages, v_pages, block_tables, cu_seqlens_q, seq_lens_k)
    _need(q.dim() == 2 and q.stride(1) == 1 and q.shape[1] >= num_heads * head_dim, "q must be [T, >= heads * d]")
    P, kvh, bs, d = k_pages.shape
    _need(kvh == num_kv_heads and d == head_dim and k_pages.is_contiguous(), "k_pages: contiguous [pages, kv_heads, bs, d]")
    _need(tuple(v_pages.shape) == (P, kvh, d, bs) and v_pages.is_contiguous(), "v_pages: contiguous [pages, kv_heads, d, bs]")
    _need(k_pages.dtype == q.dtype and v_pages.dtype == q.dtype, "q, k_pages and v_pages must share their element type")
    _need(num_heads % num_kv_heads == 0, "heads must be a multiple of kv heads")
    _need(block_tables.dtype == torch.int32 and block_tables.dim() == 2 and block_tables.stride(1) == 1, "block_tables: int32 [S, B]")
    S = block_tables.shape[0]
    _need(cu_seqlens_q.dtype == torch.int32 and cu_seqlens_q.numel() >= S + 1 and cu_seqlens_q.is_contiguous(), "cu_seqlens_q: int32 [S+1]")
    _need(seq_lens_k.dtype == torch.int32 and seq_lens_k.numel() >= S and seq_lens_k.is_contiguous(), "seq_lens_k: int32 [S]")
    return S, bs


class ScoreTerms:
    """Further terms of an attention score, for mixers that have them (None everywhere else).  With x the scaled
    product of a query at position i and a key at position n of head h:

        score = cap(x) + slopes[h] * (n - i),     cap(x) = c * tanh(x / c) for ``cap`` = c > 0, x for 0,

    and ``sinks[h]``: a logit that takes part in the softmax's sum and in nothing else.  ``slopes`` and ``sinks``
    are float32 [heads] on the device or None."""

    __slots__ = ("cap", "slopes", "sinks")

    def __init__(self, cap: float = 0.0, slopes: torch.Tensor | None = None, sinks: torch.Tensor | None = None):
        self.cap, self.slopes, self.sinks = float(cap), slopes, sinks

    def any(self) -> bool:
        return self.cap > 0.0 or self.slopes is not None or self.sinks is not None

    def checked(self, num_heads: int, device) -> "ScoreTerms":
        _need(self.cap >= 0.0 and self.cap == self.cap, f"a cap of the scores is positive, or 0 for none; got {self.cap}")
        for name, t in (("slopes", self.slopes), ("sinks", self.sinks)):
            if t is not None:
                _on_gpu(t)
                _need(t.dtype == torch.float32 and t.shape == (num_heads,) and t.is_contiguous() and t.device == device,
                      f"{name}: float32 [{num_heads}] beside the queries, got {tuple(t.shape)} {t.dtype} on {t.device}")
        return self


def _terms_args(terms: "ScoreTerms | None", num_heads: int, device) -> tuple:
    if terms is None:
        return c_float(0.0), None, None
    terms.checked(num_heads, device)
    return c_float(terms.cap), _ptr(terms.slopes), _ptr(terms.sinks)


def paged_attention_generic(q: torch.Tensor, k_pages: torch.Tensor, v_pages: torch.Tensor, block_tables: torch.Tensor,
                            cu_seqlens_q: torch.Tensor, seq_lens_k: torch.Tensor, num_heads: int, num_kv_heads: int,
                            head_dim: int, scale: float, window: int = 0, out: torch.Tensor | None = None,
                            terms: ScoreTerms | None = None) -> torch.Tensor:
    """Causal attention over paged keys and values; one wavefront per (token, head), all in float.

    The caller guarantees (and the step function checks on the host) that every table entry
    below ceil(seq_len / block_size) is a valid page and that cu_seqlens_q ends at q.shape[0].
    """
    S, bs = _check_attention_args(q, k_pages, v_pages, block_tables, cu_seqlens_q, seq_lens_k, num_heads, num_kv_heads, head_dim)
    _need(0 < head_dim <= MAX_HEAD_DIM_GENERIC, f"attention kernel takes head sizes up to {MAX_HEAD_DIM_GENERIC}, got {head_dim}")
    _need(num_heads <= 65535, "too many heads for one launch")
    T = q.shape[0]
    if out is None:
        out = torch.empty((T, num_heads * head_dim), dtype=q.dtype, device=q.device)
    _need(out.shape == (T, num_heads * head_dim) and out.stride(1) == 1 and out.dtype == q.dtype, "bad attention output")
    _check(_fn("attention_generic.hip", "pllm_paged_attention_generic")(
        dtype_code(q.dtype), _ptr(q), q.stride(0), _ptr(k_pages), _ptr(v_pages), _ptr(out), out.stride(0),
        _ptr(block_tables), block_tables.stride(0), _ptr(cu_seqlens_q), _ptr(seq_lens_k), S, T, num_heads, num_kv_heads,
        head_dim, bs, c_float(scale), int(window or 0), *_terms_args(terms, num_heads, q.device), _stream()),
        "paged_attention_generic")
    return out


# ------------------------------------------------------------------------------------------- sampling
def argmax(logits: torch.Tensor) -> torch.Tensor:
    _on_gpu(logits)
    _need(logits.dtype == torch.float32 and logits.dim() == 2 and logits.is_contiguous(), "logits: contiguous float32 [n, vocab]")
    n, V = logits.shape
    out = torch.empty((n,), dtype=torch.int32, device=logits.device)
    _check(_fn("sampling.hip", "pllm_argmax")(_ptr(logits), n, V, _ptr(out), _stream()), "argmax")
    return out


_sample_workspace: dict = {}


SAMPLE_CANDIDATES_TOP_K, SAMPLE_CANDIDATES_MASS_VOCAB = 64, 65536


def sample_candidates_apply(temperature: float, top_k: int, top_p: float, vocab: int) -> bool:
    """Whether a row with these settings may go by its candidates (the kernel's own rule, for callers that know the
    settings on the host and can spare the launch that picks candidates when no row uses them)."""
    if temperature < 1e-5:
        return False
    if 0 < top_k <= SAMPLE_CANDIDATES_TOP_K:
        return top_k < vocab
    return top_p < 1.0 and vocab >= SAMPLE_CANDIDATES_MASS_VOCAB


def rows_sampled_by_candidates(rows: int, vocab: int, device) -> list:
    """For the last ``sample`` call of this shape on the device: which rows went by their candidates (a look into the
    call's workspace, for tests and measurements)."""
    f = _fn("sampling.hip", "pllm_sample_workspace_bytes")
    f.restype = c_long
    need = int(f(rows, vocab))
    workspace = _sample_workspace.get(str(torch.device(device)))
    if not need or workspace is None:
        return [False] * rows
    chunks = need // 4 // (3 + 2 * 192) // rows
    counts = workspace[: rows * chunks * 4].view(torch.int32).view(rows, chunks)
    return (counts >= 0).all(dim=1).tolist()


def sample(logits: torch.Tensor, temperature: torch.Tensor, top_k: torch.Tensor, top_p: torch.Tensor,
           request_key: torch.Tensor, step: torch.Tensor, seed: int, candidates: bool = True) -> torch.Tensor:
    """One token per row: greedy where temperature < 1e-5, else a draw under top-k / top-p.  ``candidates``: few rows
    of a long vocabulary whose top_k is small are first cut into chunks that hand on their largest logits, and the
    search and the draw run over those (a row's token depends on its own settings only either way; False walks every
    row whole)."""
    _on_gpu(logits, temperature, top_k, top_p, request_key, step)
    _need(logits.dtype == torch.float32 and logits.dim() == 2 and logits.is_contiguous(), "logits: contiguous float32 [n, vocab]")
    n, V = logits.shape
    for t, dt, nm in ((temperature, torch.float32, "temperature"), (top_k, torch.int32, "top_k"), (top_p, torch.float32, "top_p"),
                      (request_key, torch.int64, "request_key"), (step, torch.int32, "step")):
        _need(t.dtype == dt and t.shape == (n,) and t.is_contiguous(), f"{nm}: {dt} [{n}]")
    out = torch.empty((n,), dtype=torch.int32, device=logits.device)
    workspace = None
    if candidates:
        f = _fn("sampling.hip", "pllm_sample_workspace_bytes")
        f.restype = c_long
        need = int(f(n, V))
        if need:
            workspace = _sample_workspace.get(str(logits.device))
            if workspace is None or workspace.numel() < need:
                workspace = _sample_workspace[str(logits.device)] = torch.empty(max(need, 1 << 20), dtype=torch.uint8, device=logits.device)
    _check(_fn("sampling.hip", "pllm_sample")(_ptr(logits), n, V, _ptr(temperature), _ptr(top_k), _ptr(top_p),
                                               _ptr(request_key), _ptr(step), c_ulonglong(seed & (2**64 - 1)), _ptr(out),
                                               _ptr(workspace), _stream()), "sample")
    return out


# ------------------------------------------------------------------------------------------- fused decode products
EPI_BF16, EPI_F32, EPI_GATED, EPI_ROPE_KV = 0, 1, 2, 3
DECODE_MAX_ROWS = 16          # rows of the fused form with a sum or norm in front
DECODE_WIDE_MAX_ROWS = 64     # rows of the form for plain rows
_DECODE_SIG = [c_int, c_void_p, c_int, c_void_p, c_int, c_void_p, c_float, c_void_p, c_int, c_void_p, c_void_p, c_int, c_void_p, c_void_p,
               c_int, c_int, c_int, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int,
               c_int, c_void_p]
_lds_limit: dict = {}


def _max_lds_bytes(device) -> int:
    key = str(device)
    if key not in _lds_limit:
        f = _fn("decode_linear.hip", "pllm_max_lds_bytes", signature=[])
        f.restype = c_long
        with torch.cuda.device(device):
            _lds_limit[key] = int(f())
    return _lds_limit[key]


def decode_linear_takes(rows: int, K: int, x: torch.Tensor, w: torch.Tensor, staged: bool = True) -> bool:
    """Whether the fused decode product takes these operands (else the caller runs the parts apart).
    ``staged``: a residual sum or a norm runs in front, so the rows must fit into LDS; plain rows are read
    straight from memory, may be of any length, and there may be up to 64 of them."""
    if not (x.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and 0 < rows <= (DECODE_MAX_ROWS if staged else DECODE_WIDE_MAX_ROWS) and K % 8 == 0):
        return False
    if not (x.stride(1) == 1 and w.stride(1) == 1 and x.stride(0) % 8 == 0 and w.stride(0) % 8 == 0
            and x.data_ptr() % 16 == 0 and w.data_ptr() % 16 == 0):
        return False
    if not staged:
        return True
    f = _fn("decode_linear.hip", "pllm_decode_linear_lds_bytes", signature=[c_int, c_int, c_int])
    f.restype = c_long
    return int(f(rows, K, 8)) <= _max_lds_bytes(x.device)


def decode_linear_pays(rows: int, N: int, K: int, epi: int, staged: bool) -> bool:
    """Whether the fused decode product is the faster choice for plain rows (measured against the library's
    product; by sizes only).  Every unit of 16 weight rows rereads all rows from the cache: beyond 8 rows
    that is as much as it streams of weights, and the library wins for long rows (K = 5632, 14336); beyond
    16 rows it wins for all but small matrices (q/k/v and output projections of 2048-wide models), where
    the fused kernel still fills the chip better; beyond 32 rows only the saved rotary kernel pays, and matrices of
    at most 2048 rows, whose units leave half of the GPU free for a second line of workgroups.  The gate/up
    product of a 2048-wide model is the exception: with K <= 2048 a wavefront keeps its share of the rows in
    registers for all units of its workgroup, and with the SiLU kernel saved the fused form wins up to 48 rows
    (11264 x 2048: 15.3 against 17.2 us at 32 rows, 18.0 against 18.8 at 48, 20.2 against 18.7 at 64)."""
    if staged or rows <= 8:
        return True
    if rows <= 16:
        return K <= 4096
    if epi == EPI_GATED and K <= 2048 and rows <= 48:
        return True
    small = N * K <= (1 << 23)
    if small and N <= 2048:
        return True          # (at most 128 units: two lines of workgroups with half the rows each, 7.9 against 9.0 us at 64 rows)
    return small and (rows <= 32 or epi == EPI_ROPE_KV)


def decode_linear(x: torch.Tensor, w: torch.Tensor, epi: int = EPI_BF16, delta: torch.Tensor | None = None,
                  norm_weight: torch.Tensor | None = None, eps: float = 0.0, x_out: torch.Tensor | None = None,
                  row_index: torch.Tensor | None = None, rope: dict | None = None, tiled=None,
                  activation: str = "silu") -> torch.Tensor:
    """rows = x[row_index] (+ delta) -> optional RMS norm -> rows W^T -> epilogue, in one kernel.
    ``tiled``: the matrix's ``TiledWeight`` with the pairing that goes with ``epi`` (at most 16 rows): the weights are then
    streamed from that copy, in contiguous pieces, wherever the kernel works in units of 16 weight rows.

    epi EPI_BF16 / EPI_F32: [M, N] out.  EPI_GATED: w = [gate; up], out = act(gate) * up [M, N/2] (``activation``).
    EPI_ROPE_KV: w = [q; k; v] rows; q is rotated and returned [M, heads * d]; k (rotated) and v go
    into the cache pages; ``rope`` = dict(positions, cos, sin, slots, k_pages, v_pages, num_heads,
    num_kv_heads, head_dim, block_size).  ``x_out`` receives x + delta (the new residual).
    """
    _on_gpu(x, w, delta, norm_weight, x_out, row_index)
    M = row_index.numel() if row_index is not None else x.shape[0]
    K = x.shape[1]
    _need(x.dim() == 2 and w.dim() == 2 and w.shape[1] == K, f"decode_linear shapes {tuple(x.shape)} x {tuple(w.shape)}^T")
    staged = delta is not None or norm_weight is not None
    _need(decode_linear_takes(M, K, x, w, staged),
          "decode_linear takes bfloat16, K a multiple of 8, 1..64 plain rows, or with a sum or norm in front 1..16 rows that fit LDS")
    if delta is not None:
        _need(delta.shape == x.shape and delta.dtype == x.dtype and delta.stride(1) == 1 and delta.stride(0) % 8 == 0
              and delta.data_ptr() % 16 == 0, "delta must match x")
    if x_out is not None:
        _need(delta is not None and x_out.shape == x.shape and x_out.dtype == x.dtype and x_out.stride(1) == 1
              and x_out.stride(0) % 8 == 0 and x_out.data_ptr() != x.data_ptr(), "x_out must be a separate buffer like x")
    if norm_weight is not None:
        _need(norm_weight.dtype == torch.float32 and norm_weight.shape == (K,) and norm_weight.is_contiguous(), "norm weight: float32 [K]")
    if row_index is not None:
        _need(row_index.dtype == torch.int32 and row_index.dim() == 1 and row_index.is_contiguous(), "row_index: int32")
    N = w.shape[0]
    r = rope or {}
    if tiled is not None:
        _need(M <= DECODE_MAX_ROWS and tiled.in_features == K and tiled.pairing == {EPI_GATED: "gated", EPI_ROPE_KV: "rotary"}.get(epi, "plain")
              and tiled.out_features * (2 if epi == EPI_GATED else 1) == N and tiled.tiles.is_contiguous()
              and (epi != EPI_ROPE_KV or tiled.head_dim == r.get("head_dim")),
              "the tiled copy does not belong to this matrix and epilogue")
    if epi == EPI_GATED:
        _need(N % 2 == 0, "gated product needs [gate; up] rows")
        N //= 2
        out = torch.empty((M, N), dtype=torch.bfloat16, device=x.device)
    elif epi == EPI_ROPE_KV:
        nh, nkv, d, bs = r["num_heads"], r["num_kv_heads"], r["head_dim"], r["block_size"]
        _need(d % 16 == 0 and N == (nh + 2 * nkv) * d, "fused rotary epilogue needs head sizes in multiples of 16 and [q; k; v] rows")
        kp, vp = r["k_pages"], r["v_pages"]
        P = kp.shape[0]
        _need(tuple(kp.shape) == (P, nkv, bs, d) and tuple(vp.shape) == (P, nkv, d, bs) and kp.is_contiguous() and vp.is_contiguous()
              and kp.dtype == torch.bfloat16 and vp.dtype == torch.bfloat16, "bad cache pages")
        for name in ("positions", "slots"):
            t = r[name]
            _need(t.dtype == torch.int32 and t.shape == (M,) and t.is_contiguous(), f"{name}: int32 [{M}]")
        if r.get("cos") is not None:
            for t in (r["cos"], r["sin"]):
                _need(t.dtype == torch.float32 and t.dim() == 2 and t.shape[1] == d // 2 and t.is_contiguous(), "rotary tables")
        out = torch.empty((M, nh * d), dtype=torch.bfloat16, device=x.device)
    else:
        out = torch.empty((M, N), dtype=torch.float32 if epi == EPI_F32 else torch.bfloat16, device=x.device)
    f = _fn("decode_linear.hip", "pllm_decode_linear", signature=_DECODE_SIG)
    _check(f(epi, _ptr(x), x.stride(0), _ptr(delta), delta.stride(0) if delta is not None else 0, _ptr(norm_weight), c_float(eps),
             _ptr(x_out), x_out.stride(0) if x_out is not None else 0, _ptr(row_index), _ptr(w), w.stride(0),
             None if tiled is None else _ptr(tiled.tiles), _ptr(out),
             out.stride(0), M, N, K, _ptr(r.get("positions")), _ptr(r.get("cos")), _ptr(r.get("sin")), _ptr(r.get("slots")),
             _ptr(r.get("k_pages")), _ptr(r.get("v_pages")), int(r.get("num_heads", 0)), int(r.get("num_kv_heads", 0)),
             int(r.get("head_dim", 0)), int(r.get("block_size", 0)), activation_code(activation), _stream()), "decode_linear")
    return out


# ------------------------------------------------------------------------------------------- products of 17 to a few hundred rows
SL_BF16, SL_F32, SL_GATED, SL_PARTIAL, SL_ROPE_KV = 0, 1, 2, 3, 4
STREAM_TILE_ROWS, STREAM_TILE_K = 16, 32
_STREAM_SIG = [c_int, c_void_p, c_int, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_void_p, c_void_p, c_void_p,
               c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_void_p]


class TiledWeight:
    """A weight matrix [N, K] in the order the streaming product kernel reads it: blocks of 16 rows, each block's tiles of
    16 rows x 32 columns one after the other along K, a tile being 1 KB in the order of the matrix instruction's operand
    (lane g * 16 + r: row r, columns 8 g .. 8 g + 7); zero rows pad the blocks to a multiple of 24.  ``pairing`` says
    which rows share a block: "plain" (16 successive rows), "gated" (8 gate rows and the up rows of the same outputs), or
    "rotary" (8 elements of the lower half of a head and their partners in the upper half, ``head_dim`` apart by half)."""

    def __init__(self, tiles: torch.Tensor, out_features: int, in_features: int, pairing: str, head_dim: int = 0):
        self.tiles, self.out_features, self.in_features, self.pairing, self.head_dim = tiles, out_features, in_features, pairing, head_dim

    @property
    def blocks(self) -> int:
        return self.tiles.shape[0]


def stream_linear_takes(w: torch.Tensor) -> bool:
    return w.dtype == torch.bfloat16 and w.dim() == 2 and w.shape[1] % STREAM_TILE_K == 0 and w.is_cuda


def tile_weight(w: torch.Tensor, pairing: str = "plain", head_dim: int = 0) -> TiledWeight:
    """The tiled copy of ``w`` [N, K] (bfloat16, K a multiple of 32).  "gated": w = [gate rows; up rows].  "rotary":
    w = [q; k; v] rows of heads of ``head_dim`` (a multiple of 16) elements."""
    _need(stream_linear_takes(w), "tiled weights: bfloat16 [N, K] on the GPU with K a multiple of 32")
    N, K = w.shape
    out_features = N
    if pairing == "gated":
        _need(N % 2 == 0, "a gated matrix holds gate rows and as many up rows")
        half = N // 2
        units = -(-half // 8)
        j = torch.arange(units * 8, device=w.device).view(units, 8).clamp_(max=half - 1)
        w = w.index_select(0, torch.cat([j, j + half], dim=1).reshape(-1))           # per block: 8 gate rows, their 8 up rows
        out_features = half
    elif pairing == "rotary":
        _need(head_dim > 0 and head_dim % 16 == 0 and N % head_dim == 0, "rotary pairing: whole heads of a multiple of 16 elements")
        heads, half = N // head_dim, head_dim // 2
        lower = (torch.arange(heads, device=w.device).view(heads, 1, 1) * head_dim
                 + torch.arange(half // 8, device=w.device).view(1, half // 8, 1) * 8 + torch.arange(8, device=w.device).view(1, 1, 8))
        w = w.index_select(0, torch.cat([lower, lower + half], dim=2).reshape(-1))    # per block: 8 lower elements, their partners
    else:
        _need(pairing == "plain", f"unknown pairing {pairing!r}")
    blocks = -(-w.shape[0] // 16)
    blocks_padded = -(-blocks // 24) * 24                                 # (whole workgroups of 1, 2, 3, 4 or 8 blocks)
    if blocks_padded * 16 != w.shape[0]:
        w = torch.cat([w, torch.zeros((blocks_padded * 16 - w.shape[0], K), dtype=w.dtype, device=w.device)])
    tiles = w.view(blocks_padded, 16, K // 32, 4, 8).permute(0, 2, 3, 1, 4).contiguous()       # [block, k step, g, r, 8]
    return TiledWeight(tiles, out_features, K, pairing, head_dim)


def _whole_ranges(stages: int, splits: int) -> int:
    """The largest number of ranges up to ``splits`` such that ranges of ceil(stages / ranges) stages leave none empty."""
    while splits > 1 and -(-stages // splits) * (splits - 1) >= stages:
        splits -= 1
    return splits


def stream_linear_plan(M: int, N: int, K: int, compute_units: int, partial: bool = True) -> tuple[int, int]:
    """(blocks of 16 weight rows per workgroup, ranges of K) for a product of M rows with N weight rows: by sizes only.
    What counts is that the workgroups are about as many as the compute units, in one round, and that each reads as few
    input rows as possible (every workgroup reads all rows of its range of K).  With partial sums allowed: two blocks
    and as many ranges of K as give every compute unit a workgroup (2048 x 5632 at 64 rows: 8.6 us in 4 ranges, 11.2 in 2,
    10.9 in 8); four blocks where K is long and the rows few (4096 x 14336 at 64 rows: 28.5 us against 30.6).  In one
    range: a block per workgroup while that fits one round (2048 x 2048: 6.7 us against 9.1 with two), else two."""
    blocks = -(-N // 16)
    row_blocks = -(-M // 128)
    stages = -(-K // 256)
    if not partial:
        return (1 if blocks * row_blocks <= compute_units else 2), 1
    nt = 4 if (K >= 8192 and M <= 64) else 2
    workgroups = -(-blocks // nt) * row_blocks
    splits = 1
    if workgroups < compute_units:
        splits = _whole_ranges(stages, max(1, min(compute_units // workgroups, stages // 2, 8)))
    return nt, splits


def gated_blocks_per_workgroup(out_features: int, compute_units: int) -> int:
    """Blocks of 16 weight rows (8 gate rows and their up rows) a workgroup of the gated product takes: three while
    that gives every block a workgroup in one round (5632 outputs: 235 workgroups, 14.7 us at 64 rows against 16.0
    with four and 19.4 with two), else four (14336 outputs: 56.9 us against 64.9 with three)."""
    units = -(-out_features // 8)
    return 3 if -(-units // 3) <= compute_units else 4


def stream_linear(x: torch.Tensor, w: TiledWeight, epi: int = SL_BF16, nt: int | None = None, splits: int | None = None,
                  rope: dict | None = None, activation: str = "silu") -> torch.Tensor:
    """x [M, K] bfloat16 times the tiled weights.  SL_BF16 / SL_F32: [M, N]; SL_GATED: act(gate) * up [M, N / 2];
    SL_PARTIAL: float [splits, M, N], the sums over ``splits`` ranges of K, to be added in that order; SL_ROPE_KV: q rotated
    [M, heads * d], k (rotated) and v written to their pages (``rope`` as for ``decode_linear``)."""
    _on_gpu(x, w.tiles)
    M, K = x.shape
    _need(x.dtype == torch.bfloat16 and x.dim() == 2 and x.stride(1) == 1 and x.stride(0) % 8 == 0 and x.data_ptr() % 16 == 0,
          "stream_linear: bfloat16 rows that start on 16-byte boundaries")
    _need(K == w.in_features and w.tiles.is_contiguous() and tuple(w.tiles.shape[1:]) == (K // 32, 4, 16, 8) and w.blocks % 24 == 0,
          f"stream_linear: rows of {K} values against tiled weights of {w.in_features}")
    _need({SL_GATED: "gated", SL_ROPE_KV: "rotary"}.get(epi, "plain") == w.pairing,
          f"epilogue {epi} against weights tiled with the {w.pairing} pairing")
    N = w.out_features
    if epi == SL_GATED:
        plan_nt, plan_splits = gated_blocks_per_workgroup(N, _num_compute_units(x.device)), 1
    else:
        plan_nt, plan_splits = stream_linear_plan(M, N, K, _num_compute_units(x.device), partial=epi == SL_PARTIAL)
    nt = nt or plan_nt
    splits = plan_splits if splits is None else splits
    _need(splits == 1 or epi == SL_PARTIAL, "ranges of K give partial sums")
    r = rope or {}
    if epi == SL_PARTIAL:
        out = torch.empty((splits, M, N), dtype=torch.float32, device=x.device)
    elif epi == SL_ROPE_KV:
        nh, nkv, d, bs = r["num_heads"], r["num_kv_heads"], r["head_dim"], r["block_size"]
        _need(d == w.head_dim and N == (nh + 2 * nkv) * d, "the weights were tiled for other heads")
        kp, vp = r["k_pages"], r["v_pages"]
        P = kp.shape[0]
        _need(tuple(kp.shape) == (P, nkv, bs, d) and tuple(vp.shape) == (P, nkv, d, bs) and kp.is_contiguous() and vp.is_contiguous()
              and kp.dtype == torch.bfloat16 and vp.dtype == torch.bfloat16, "bad cache pages")
        for name in ("positions", "slots"):
            t = r[name]
            _need(t.dtype == torch.int32 and t.shape == (M,) and t.is_contiguous(), f"{name}: int32 [{M}]")
        if r.get("cos") is not None:
            for t in (r["cos"], r["sin"]):
                _need(t.dtype == torch.float32 and t.dim() == 2 and t.shape[1] == d // 2 and t.is_contiguous() and t.data_ptr() % 16 == 0,
                      "rotary tables")
        out = torch.empty((M, nh * d), dtype=torch.bfloat16, device=x.device)
    else:
        out = torch.empty((M, N), dtype=torch.float32 if epi == SL_F32 else torch.bfloat16, device=x.device)
    f = _fn("stream_linear.hip", "pllm_stream_linear", signature=_STREAM_SIG)
    _check(f(epi, _ptr(x), x.stride(0), _ptr(w.tiles), _ptr(out), out.stride(-2), M, N, K, w.blocks, nt, splits,
             _ptr(r.get("positions")), _ptr(r.get("cos")), _ptr(r.get("sin")), _ptr(r.get("slots")), _ptr(r.get("k_pages")),
             _ptr(r.get("v_pages")), int(r.get("num_heads", 0)), int(r.get("num_kv_heads", 0)), int(r.get("head_dim", 0)),
             int(r.get("block_size", 0)), activation_code(activation), _stream()), "stream_linear")
    return out


_TILE_SIG = [c_int, c_void_p, c_int, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_void_p, c_void_p, c_void_p,
             c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_void_p]
TILE_BLOCK_ROWS = 160           # input rows of one workgroup of the tiled kernel, at most


def tile_linear_plan(M: int, N: int, K: int, compute_units: int) -> int:
    """Ranges of K for the tiled product of M rows with N weight rows: as many as give every compute unit a workgroup
    (tiles of up to 160 rows x 128 weight rows), each at least four stages of 64 columns long."""
    workgroups = -(-N // 128) * -(-M // TILE_BLOCK_ROWS)
    stages = -(-K // 64)
    if workgroups >= compute_units:
        return 1
    return _whole_ranges(stages, max(1, min(compute_units // workgroups, stages // 4, 16)))


def tile_linear_shape(M: int, weight_rows: int, compute_units: int) -> tuple[int, int, int]:
    """(rows per block of input rows, weight rows per tile, workgroups) that the tiled kernel takes for a product in one
    range of K: the shape with the most workgroups in one round of the compute units (chosen in the library)."""
    f = _fn("stream_linear.hip", "pllm_tile_linear_shape", signature=[c_int, c_int, c_int, c_void_p, c_void_p])
    rows, tile = c_int(0), c_int(0)
    wgs = f(int(M), int(weight_rows), int(compute_units), ctypes.byref(rows), ctypes.byref(tile))
    _need(wgs > 0, f"tile_linear_shape({M}, {weight_rows}, {compute_units})")
    return rows.value, tile.value, wgs


def tile_linear(x: torch.Tensor, w: TiledWeight, epi: int = SL_BF16, splits: int | None = None, rope: dict | None = None,
                activation: str = "silu") -> torch.Tensor:
    """As ``stream_linear``, for a few hundred rows: tiles of up to 160 rows x 128 weight rows per workgroup, both
    operands through LDS."""
    _on_gpu(x, w.tiles)
    M, K = x.shape
    _need(x.dtype == torch.bfloat16 and x.dim() == 2 and x.stride(1) == 1 and x.stride(0) % 8 == 0 and x.data_ptr() % 16 == 0,
          "tile_linear: bfloat16 rows that start on 16-byte boundaries")
    _need(K == w.in_features and w.tiles.is_contiguous() and tuple(w.tiles.shape[1:]) == (K // 32, 4, 16, 8) and w.blocks % 24 == 0,
          f"tile_linear: rows of {K} values against tiled weights of {w.in_features}")
    _need({SL_GATED: "gated", SL_ROPE_KV: "rotary"}.get(epi, "plain") == w.pairing,
          f"epilogue {epi} against weights tiled with the {w.pairing} pairing")
    N = w.out_features
    if splits is None:
        splits = tile_linear_plan(M, N * (2 if epi == SL_GATED else 1), K, _num_compute_units(x.device)) if epi == SL_PARTIAL else 1
    _need(splits == 1 or epi == SL_PARTIAL, "ranges of K give partial sums")
    r = rope or {}
    if epi == SL_PARTIAL:
        out = torch.empty((splits, M, N), dtype=torch.float32, device=x.device)
    elif epi == SL_ROPE_KV:
        nh, nkv, d, bs = r["num_heads"], r["num_kv_heads"], r["head_dim"], r["block_size"]
        _need(d == w.head_dim and N == (nh + 2 * nkv) * d, "the weights were tiled for other heads")
        kp, vp = r["k_pages"], r["v_pages"]
        P = kp.shape[0]
        _need(tuple(kp.shape) == (P, nkv, bs, d) and tuple(vp.shape) == (P, nkv, d, bs) and kp.is_contiguous() and vp.is_contiguous()
              and kp.dtype == torch.bfloat16 and vp.dtype == torch.bfloat16, "bad cache pages")
        for name in ("positions", "slots"):
            t = r[name]
            _need(t.dtype == torch.int32 and t.shape == (M,) and t.is_contiguous(), f"{name}: int32 [{M}]")
        if r.get("cos") is not None:
            for t in (r["cos"], r["sin"]):
                _need(t.dtype == torch.float32 and t.dim() == 2 and t.shape[1] == d // 2 and t.is_contiguous() and t.data_ptr() % 16 == 0,
                      "rotary tables")
        out = torch.empty((M, nh * d), dtype=torch.bfloat16, device=x.device)
    else:
        out = torch.empty((M, N), dtype=torch.float32 if epi == SL_F32 else torch.bfloat16, device=x.device)
    f = _fn("stream_linear.hip", "pllm_tile_linear", signature=_TILE_SIG)
    _check(f(epi, _ptr(x), x.stride(0), _ptr(w.tiles), _ptr(out), out.stride(-2), M, N, K, w.blocks, splits,
             _ptr(r.get("positions")), _ptr(r.get("cos")), _ptr(r.get("sin")), _ptr(r.get("slots")), _ptr(r.get("k_pages")),
             _ptr(r.get("v_pages")), int(r.get("num_heads", 0)), int(r.get("num_kv_heads", 0)), int(r.get("head_dim", 0)),
             int(r.get("block_size", 0)), activation_code(activation), _stream()), "tile_linear")
    return out


# ------------------------------------------------------------------------------------------- choices
def gemm_bf16(a: torch.Tensor, w: torch.Tensor, out_dtype: torch.dtype | None = None) -> torch.Tensor:
    """a [M, K] times w [N, K]^T for more rows than the fused decode kernel takes (prompt portions, large
    decode batches): the vendor's matrix-product library, as the reference's engine uses a library for
    its products (nn.Linear, pagedllm/model/llama.py:141-144).  Float accumulation; the result is bfloat16
    or, for logits, float32 straight from the accumulators."""
    _on_gpu(a, w)
    _need(a.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and a.dim() == 2 and w.dim() == 2 and a.shape[1] == w.shape[1],
          f"gemm_bf16 takes bfloat16 [M, K] x [N, K]^T, got {tuple(a.shape)} {a.dtype} x {tuple(w.shape)} {w.dtype}")
    if out_dtype == torch.float32:
        return torch.mm(a, w.t(), out_dtype=torch.float32)
    _need(out_dtype in (None, torch.bfloat16), "output is bfloat16 or float32")
    return torch.mm(a, w.t())


_ATTN_SIG = [c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_int, c_void_p, c_void_p, c_int, c_int, c_int,
             c_int, c_int, c_int, c_float, c_int, c_int, c_int, c_void_p, c_int, c_int, c_void_p, c_int, c_void_p]
_ATTN_TERMS_SIG = _ATTN_SIG[:-1] + [c_int, c_float, c_void_p, c_void_p, c_void_p]
_attn_scratch: dict = {}
_attn_scratch_retired: list = []      # outgrown buffers stay allocated: captured graphs still hold their addresses
_attn_checked: set = set()


def mfma_attention_takes(dtype: torch.dtype, num_heads: int, num_kv_heads: int, head_dim: int, block_size: int) -> bool:
    return (dtype == torch.bfloat16 and head_dim % 16 == 0 and 16 <= head_dim <= 256 and block_size >= 16
            and block_size & (block_size - 1) == 0 and num_heads % num_kv_heads == 0 and num_heads // num_kv_heads <= 64)


def attention_decode_registers(head_dim: int, waves: int) -> int:
    """Vector registers per lane of the compiled decode attention kernel (16 columns, ``waves`` wavefronts)."""
    return int(_fn("attention_mfma.hip", "pllm_attention_decode_registers", {"HEAD_DIM": head_dim}, [c_int])(waves))


def attention_decode_spill_bytes(head_dim: int, waves: int) -> int:
    """Bytes per lane that the same kernel keeps outside registers; 0 unless registers were spilled."""
    return int(_fn("attention_mfma.hip", "pllm_attention_decode_spill_bytes", {"HEAD_DIM": head_dim}, [c_int])(waves))


def _merge_lds_bytes(column_blocks: int, waves: int, head_dim: int) -> int:
    """LDS of the attention kernel's several-wavefront variant (as merge_lds_bytes in attention_mfma.hip):
    maximum and weight per column and wavefront, and every wavefront's partial output."""
    return (2 * waves * column_blocks * 16 + waves * column_blocks * (head_dim // 16) * 4 * 64) * 4


def attention_plan(num_seqs: int, num_kv_heads: int, max_q_len: int, max_k_len: int, group: int, head_dim: int,
                   lds_limit: int, compute_units: int = 256) -> tuple[int, int, int]:
    """(wavefronts per work item, partition_size, num_partitions) for a step.

    Prompt portions have many query tiles: one wavefront per tile walks all its keys (1, 0, 1).
    Decoding has one tile per (sequence, kv head), far too few to fill the GPU: the keys are cut
    into aligned partitions, one workgroup each (merged by a second kernel), and inside a
    workgroup the wavefronts share the partition's blocks of 64 keys (merged in LDS)."""
    cols = max_q_len * group
    if cols > 64 or max_k_len <= 64:
        return 1, 0, 1
    ncb = 1 if cols <= 16 else (2 if cols <= 32 else 4)
    max_waves = 8
    while max_waves >= 4 and _merge_lds_bytes(ncb, max_waves, head_dim) > lds_limit:
        max_waves //= 2
    if max_waves < 4:
        return 1, 0, 1
    # Partitions only as far as they fill the GPU in one round: a workgroup of eight wavefronts has a compute unit to
    # itself, so work items x partitions stay at or under the number of compute units (48 sequences x 4 kv heads x 2048
    # keys at head size 64: 28.1 us in one piece on 192 compute units, 37.0 us in two partitions, which make 384
    # workgroups and two rounds; 24 sequences: 18.8 us in two partitions against 21.9 in four and 24.5 in one), and
    # fewer, longer work items are faster than many short ones plus a larger merge.
    items = num_seqs * num_kv_heads
    want_parts = max(1, compute_units // items)
    size = 256                                        # at least four blocks of 64 keys per workgroup
    while (max_k_len + size - 1) // size > want_parts:
        size *= 2
    parts = (max_k_len + size - 1) // size
    waves = max_waves
    while waves > 4 and (waves // 2) * 64 >= min(size, max_k_len):
        waves //= 2
    # Small heads (two blocks of keys under way per wavefront) and more work items than compute units: two
    # workgroups of four wavefronts on a compute unit stream faster than eight-wavefront workgroups in two rounds
    # (96 sequences x 4 kv heads x 2048 keys at head size 64: 48.7 against 57.5 us; 64 sequences x 8 kv heads: a decode
    # step of Llama-3.2-1B shapes 2.68 against 2.74 ms).  At head size 128 eight wavefronts stay ahead (40 sequences x 8
    # kv heads: 86.7 against 106.3 us).
    if head_dim <= 64 and parts == 1 and items > compute_units:
        waves = 4
    return (waves, size, parts) if parts > 1 else (waves, 0, 1)


def paged_attention_mfma(q: torch.Tensor, k_pages: torch.Tensor, v_pages: torch.Tensor, block_tables: torch.Tensor,
                         cu_seqlens_q: torch.Tensor, seq_lens_k: torch.Tensor, num_heads: int, num_kv_heads: int,
                         head_dim: int, scale: float, window: int, max_q_len: int, partition_size: int = 0,
                         num_partitions: int = 1, waves: int = 1, column_blocks: int = 0,
                         out: torch.Tensor | None = None, work_list: torch.Tensor | None = None,
                         terms: ScoreTerms | None = None, single_prompt: bool = False) -> torch.Tensor:
    """Causal attention over paged keys/values on the matrix cores (bfloat16).  ``max_q_len`` bounds
    the queries of any sequence of the batch; ``partition_size`` > 0 splits the keys of every
    work item into aligned partitions that a second kernel merges (best a multiple of 128 for prompt portions, whose
    workgroups walk the keys in steps of up to 128); ``waves`` > 1 shares the keys
    of a work item between the wavefronts of one workgroup (few queries per sequence only).  ``work_list``
    (prompt portions): int32 [n, 2] pairs of (sequence, tile of 128 query columns), the order in which the
    kernel's workgroups take them (``prompt_work_list``).  ``terms``: further terms of the scores (``ScoreTerms``);
    with any of them the kernels come from a library of their own, compiled with those terms in the score loop.
    ``single_prompt``: all queries but a few belong to one sequence (a hint for the prompt kernel's form)."""
    S, bs = _check_attention_args(q, k_pages, v_pages, block_tables, cu_seqlens_q, seq_lens_k, num_heads, num_kv_heads, head_dim)
    _need(mfma_attention_takes(q.dtype, num_heads, num_kv_heads, head_dim, bs),
          f"MFMA attention takes bfloat16, head sizes 16..256 in steps of 16, pages of >= 16 positions and groups of <= 64 "
          f"heads; got {q.dtype}, head size {head_dim}, page {bs}, {num_heads}/{num_kv_heads} heads")
    _need(q.stride(0) % 8 == 0 and q.data_ptr() % 16 == 0, "q rows must start on 16-byte boundaries")
    T = q.shape[0]
    if out is None:
        out = torch.empty((T, num_heads * head_dim), dtype=q.dtype, device=q.device)
    _need(out.shape == (T, num_heads * head_dim) and out.stride(1) == 1 and out.dtype == q.dtype and out.stride(0) % 4 == 0,
          "bad attention output")
    _need(max_q_len >= 1 and partition_size % 64 == 0 and waves in (1, 4, 8), "bad launch parameters")
    ncb = min(column_blocks or 4, 1 if max_q_len * (num_heads // num_kv_heads) <= 16 else (2 if max_q_len * (num_heads // num_kv_heads) <= 32 else 4))
    _need(column_blocks in (0, 1, 2, 4), "column_blocks is 0 (automatic), 1, 2 or 4")
    _need(waves == 1 or _merge_lds_bytes(ncb, waves, head_dim) <= _max_lds_bytes(q.device),
          "the merge buffers of that many wavefronts do not fit LDS")
    if work_list is not None:
        _on_gpu(work_list)
        _need(work_list.dtype == torch.int32 and work_list.dim() == 2 and work_list.shape[1] == 2 and work_list.is_contiguous()
              and 0 < work_list.shape[0] <= 65535, "work_list: int32 [n, 2], n in 1..65535")
    ws = None
    if partition_size > 0:
        floats = T * num_heads * num_partitions * (head_dim + 2)
        key = str(q.device)
        ws = _attn_scratch.get(key)
        if ws is None or ws.numel() < floats:
            if ws is not None:
                _attn_scratch_retired.append(ws)
            ws = torch.empty(max(floats, 1 << 22), dtype=torch.float32, device=q.device)
            _attn_scratch[key] = ws
    with_terms = terms is not None and terms.checked(num_heads, q.device).any()
    defines = {"HEAD_DIM": head_dim, "SCORE_TERMS": 1} if with_terms else {"HEAD_DIM": head_dim}
    if (head_dim, with_terms) not in _attn_checked:   # the library on disk is the one compiled for this head size
        built = _fn("attention_mfma.hip", "pllm_attention_mfma_head_dim", defines, [])()
        _need(built == head_dim, f"attention library for head size {head_dim} reports head size {built}")
        has_terms = _fn("attention_mfma.hip", "pllm_attention_mfma_score_terms", defines, [])()
        _need(bool(has_terms) == with_terms, f"attention library for head size {head_dim}: further score terms compiled in: {has_terms}")
        _attn_checked.add((head_dim, with_terms))
    args = (_ptr(q), q.stride(0), _ptr(k_pages), _ptr(v_pages), _ptr(out), out.stride(0), _ptr(block_tables),
            block_tables.stride(0), _ptr(cu_seqlens_q), _ptr(seq_lens_k), S, T, int(max_q_len), num_heads, num_kv_heads, bs,
            c_float(scale), int(window or 0), int(partition_size), int(num_partitions), _ptr(ws), int(waves), int(column_blocks),
            _ptr(work_list), 0 if work_list is None else work_list.shape[0])
    if with_terms or single_prompt:
        f = _fn("attention_mfma.hip", "pllm_paged_attention_mfma_terms", defines, _ATTN_TERMS_SIG)
        _check(f(*args, int(bool(single_prompt)), *_terms_args(terms, num_heads, q.device), _stream()), "paged_attention_mfma")
    else:
        f = _fn("attention_mfma.hip", "pllm_paged_attention_mfma", defines, _ATTN_SIG)
        _check(f(*args, _stream()), "paged_attention_mfma")
    return out


PROMPT_TILE_COLUMNS = 128   # query columns (queries x heads per kv head) of one workgroup of the prompt kernel
_upload_buffers: dict = {}


def _upload_ints(values: np.ndarray, device) -> torch.Tensor:
    """int32 values to the device without stalling the host: through a pinned buffer (allocated once per
    device) and a copy on the current stream.  A copy from pageable memory would hold the host until the
    stream has caught up, and the kernels of the layers before could then no longer be issued ahead."""
    key = str(device)
    pinned, copied = _upload_buffers.get(key, (None, None))
    if pinned is None or pinned.numel() < values.size:
        pinned, copied = torch.empty(max(values.size, 1 << 14), dtype=torch.int32, pin_memory=True), torch.cuda.Event()
        _upload_buffers[key] = (pinned, copied)
    else:
        copied.synchronize()                                   # the last upload has left the buffer
    staged = pinned[:values.size].view(values.shape)
    staged.copy_(torch.from_numpy(np.ascontiguousarray(values, dtype=np.int32)))
    out = torch.empty(values.shape, dtype=torch.int32, device=device)
    out.copy_(staged, non_blocking=True)
    copied.record()
    return out


def prompt_tiles(q_lens: list, k_lens: list, first_seq: int, group: int, capacity: int | None = None) -> np.ndarray | None:
    """Host side of the prompt kernel's work list for the sequences from ``first_seq`` on: int32 [n, 2] pairs
    (sequence counted from ``first_seq``, tile of PROMPT_TILE_COLUMNS query columns), the tiles that see the most
    keys first.  Without ``capacity``: None when the sequences are all alike (the kernel's own grid then does the
    same).  With ``capacity``: always a list, of exactly that many pairs, the unused ones (-1, -1)."""
    counts = [-(-n * group // PROMPT_TILE_COLUMNS) for n in q_lens[first_seq:]]
    if capacity is None and len(set(counts)) == 1 and len(set(k_lens[first_seq:])) == 1:
        return None
    seqs, tiles, keys = [], [], []
    for i, n in enumerate(counts):
        s = first_seq + i
        t = np.arange(n, dtype=np.int64)
        seqs.append(np.full(n, i, dtype=np.int64))
        tiles.append(t)
        keys.append(k_lens[s] - q_lens[s] + (t + 1) * PROMPT_TILE_COLUMNS // group)
    seqs, tiles, keys = np.concatenate(seqs), np.concatenate(tiles), np.concatenate(keys)
    order = np.argsort(-keys, kind="stable")
    pairs = np.stack([seqs[order], tiles[order]], axis=1).astype(np.int32)
    if capacity is not None:
        _need(pairs.shape[0] <= capacity, f"{pairs.shape[0]} prompt tiles for a list of {capacity}")
        pairs = np.concatenate([pairs, np.full((capacity - pairs.shape[0], 2), -1, dtype=np.int32)])
    return pairs


def prompt_tiles_capacity(num_sequences: int, tokens: int, group: int) -> int:
    """Most pairs ``prompt_tiles`` can give for ``num_sequences`` sequences that share ``tokens`` tokens."""
    return -(-tokens * group // PROMPT_TILE_COLUMNS) + num_sequences


def prompt_work_list(ctx, first_seq: int, group: int) -> torch.Tensor | None:
    """The prompt kernel's work for the sequences from ``first_seq`` on (``prompt_tiles``) on the device.
    Workgroups take the pairs in order, so long pieces start first and none is launched for a tile that a shorter
    sequence does not have (with one long and many short sequences most of a rectangular grid is empty, and
    handing out empty workgroups was measured at 80 us for 3,800 of them).  Built from the host lengths once per
    step and kept in the context; None when the sequences are all alike and the kernel's own grid does the same."""
    cache = getattr(ctx, "launch_cache", None)
    key = ("prompt_tiles", first_seq, group)
    if cache is not None and key in cache:
        return cache[key]
    pairs = prompt_tiles(ctx.q_lens, ctx.k_lens, first_seq, group)
    work = None
    if pairs is not None and 0 < pairs.shape[0] <= 65535:
        work = _upload_ints(pairs, ctx.device)
    if cache is not None:
        cache[key] = work
    return work


_compute_units: dict = {}


def _num_compute_units(device) -> int:
    key = str(device)
    if key not in _compute_units:
        _compute_units[key] = torch.cuda.get_device_properties(device).multi_processor_count
    return _compute_units[key]


PROMPT_PARTITION_MIN_KEYS = 512   # a partition of the prompt kernel holds at least this many keys (four steps of 128)


def prompt_partitions(num_tiles: int, num_kv_heads: int, max_k_len: int, compute_units: int) -> tuple[int, int]:
    """(partition_size, num_partitions) for a launch of the prompt kernel with ``num_tiles`` tiles of query columns
    (all sequences together) whose longest context is ``max_k_len``; (0, 1): no partitions.

    A workgroup walks its tile's keys one step of 128 after the other (about 1.9 us a step at head size 64), so a
    prompt portion of a few hundred tokens behind a long context is a few dozen workgroups that run for a long time
    on a GPU of 256 compute units: 256 tokens at context 2048 took 30 us.  The keys are then cut into as many
    aligned partitions as it takes to give every compute unit a workgroup, each at least PROMPT_PARTITION_MIN_KEYS
    long, and a second kernel merges the partitions (about 5 us)."""
    workgroups = max(1, num_tiles * num_kv_heads)
    parts = min(compute_units // workgroups, max_k_len // PROMPT_PARTITION_MIN_KEYS)
    if parts < 2:
        return 0, 1
    size = -(-max_k_len // parts)
    size = (size + 127) // 128 * 128
    return size, -(-max_k_len // size)


FEW_QUERY_COLUMNS = 64      # queries x heads per kv head that one tile of the decode kernel holds
SPLIT_FROM_CONTEXT_TIMES_HEAD = 160_000   # context x head size of a few-query sequence from which two launches pay


def paged_attention(q, k_pages, v_pages, block_tables, cu_seqlens_q, seq_lens_k, num_heads, num_kv_heads, head_dim,
                    scale, window, ctx, terms: ScoreTerms | None = None) -> torch.Tensor:
    """Attention of one step's queries over the paged cache: the MFMA kernels for bfloat16 where they
    take the shape, else the plain kernel.  ``ctx`` gives host-side lengths for launch decisions.

    A step that holds decoded tokens beside prompt portions is one launch of the prompt kernel, in which a decoded
    token is a tile of its own that one workgroup walks through its whole context; when such a context is long
    (13 us per 1024 keys at head size 64, 34 us at 128) the step is launched in two parts instead, if the sequences
    with few queries come first in the batch (the step function orders them so): those go to the kernel that cuts
    their keys into partitions, the portions to the prompt kernel (a portion of 512 tokens beside 7 decoded tokens
    at context 8192: 109 us in one launch, 36 us in two; at context 1024: 19 us and 24 us)."""
    bs = k_pages.shape[2]
    if mfma_attention_takes(q.dtype, num_heads, num_kv_heads, head_dim, bs) and q.stride(0) % 8 == 0:
        group = num_heads // num_kv_heads
        lds = _max_lds_bytes(q.device)
        layout = getattr(ctx, "graph_layout", None)
        if ctx.capturing and layout is not None:
            # A step with prompt portions that is replayed from a graph: the launches depend on the layout's counts
            # and the context bound only.  The single-token rows go to the kernel that cuts their keys into
            # partitions, the portions to the prompt kernel with the work list the step function has put there.
            few = layout.num_single_rows
            work = ctx.launch_cache.get(("prompt_tiles", few, group))
            _need(work is not None, "a replayed step with prompt portions needs the prompt kernel's work list in the context")
            work = work.view(-1, 2)
            out = torch.empty((q.shape[0], num_heads * head_dim), dtype=q.dtype, device=q.device)
            if few:
                waves, size, parts = attention_plan(few, num_kv_heads, 1, ctx.max_k_len, group, head_dim, lds, _num_compute_units(q.device))
                paged_attention_mfma(q[:few], k_pages, v_pages, block_tables[:few], cu_seqlens_q[:few + 1], seq_lens_k[:few],
                                     num_heads, num_kv_heads, head_dim, scale, window, 1, size, parts, waves,
                                     2 if waves == 1 else 0, out=out[:few], terms=terms)
            prompt_q = max(layout.portion_tokens, FEW_QUERY_COLUMNS // group + 1)     # enough columns for the prompt kernel's form
            psize, pparts = prompt_partitions(work.shape[0], num_kv_heads, layout.portion_context, _num_compute_units(q.device))
            paged_attention_mfma(q, k_pages, v_pages, block_tables[few:], cu_seqlens_q[few:], seq_lens_k[few:], num_heads,
                                 num_kv_heads, head_dim, scale, window, prompt_q, psize, pparts, 1, 2, out=out, work_list=work, terms=terms,
                                 single_prompt=layout.num_portions == 2)      # (one portion and the padding sequence)
            return out
        q_lens, k_lens = ctx.q_lens, ctx.k_lens
        few = 0
        while few < len(q_lens) and q_lens[few] * group <= FEW_QUERY_COLUMNS:
            few += 1
        if (0 < few < len(q_lens) and max(k_lens[:few]) * head_dim >= SPLIT_FROM_CONTEXT_TIMES_HEAD and not ctx.capturing
                and all(n * group > FEW_QUERY_COLUMNS for n in q_lens[few:])):
            rows = sum(q_lens[:few])
            out = torch.empty((q.shape[0], num_heads * head_dim), dtype=q.dtype, device=q.device)
            max_q, max_k = max(q_lens[:few]), max(k_lens[:few])
            waves, size, parts = attention_plan(few, num_kv_heads, max_q, max_k, group, head_dim, lds, _num_compute_units(q.device))
            paged_attention_mfma(q[:rows], k_pages, v_pages, block_tables[:few], cu_seqlens_q[:few + 1], seq_lens_k[:few],
                                 num_heads, num_kv_heads, head_dim, scale, window, max_q, size, parts, waves,
                                 2 if waves == 1 else 0, out=out[:rows], terms=terms)
            # the portions: rows, cu_seqlens_q and the output stay absolute, the per-sequence arrays start at `few`
            psize, pparts = prompt_partitions(sum(-(-n * group // PROMPT_TILE_COLUMNS) for n in q_lens[few:]), num_kv_heads,
                                              max(k_lens[few:]), _num_compute_units(q.device))
            paged_attention_mfma(q, k_pages, v_pages, block_tables[few:], cu_seqlens_q[few:], seq_lens_k[few:], num_heads,
                                 num_kv_heads, head_dim, scale, window, max(q_lens[few:]), psize, pparts, 1, 2, out=out,
                                 work_list=prompt_work_list(ctx, few, group), terms=terms)
            return out
        waves, size, parts = attention_plan(ctx.num_seqs, num_kv_heads, ctx.max_q_len, ctx.max_k_len, group, head_dim, lds,
                                            _num_compute_units(q.device))
        # Prompt portions: 32 columns per wavefront leave registers for two wavefronts per SIMD
        # (measured faster than 64 columns at one).
        prompt = waves == 1 and ctx.max_q_len * group > FEW_QUERY_COLUMNS and not ctx.capturing
        if prompt:
            size, parts = prompt_partitions(sum(-(-n * group // PROMPT_TILE_COLUMNS) for n in q_lens), num_kv_heads, ctx.max_k_len,
                                            _num_compute_units(q.device))
        return paged_attention_mfma(q, k_pages, v_pages, block_tables, cu_seqlens_q, seq_lens_k, num_heads, num_kv_heads,
                                    head_dim, scale, window, ctx.max_q_len, size, parts, waves, 2 if waves == 1 else 0,
                                    work_list=prompt_work_list(ctx, 0, group) if prompt else None, terms=terms)
    if q.dtype == torch.bfloat16 and not _warned_plain_attention:
        _warned_plain_attention.append(True)
        log.warning("bfloat16 attention with pages of %d positions, head size %d, %d/%d heads runs on the plain kernel (one "
                    "wavefront per token and head): the matrix-core kernels take pages of at least 16 positions, head sizes "
                    "16..256 in steps of 16 and groups of at most 64 heads", bs, head_dim, num_heads, num_kv_heads)
    return paged_attention_generic(q, k_pages, v_pages, block_tables, cu_seqlens_q, seq_lens_k, num_heads,
                                   num_kv_heads, head_dim, scale, window, terms=terms)
