"""Causal attention over the paged cache with grouped heads.

q/k/v projections -> rotary encoding of q and k -> k and v written to their slots ->
attention over all keys of the request through the block table -> output projection
(pagedllm/model/llama.py:131-160; the reference's Llama has no biases).  Sizes, the score scale, an optional window,
the position encoding and whether the q/k/v projections have a bias (``qkv_bias``: tensors ``q_proj.bias`` ...; such
a layer gives up the fused product-rotary-cache kernels) come in as parameters, and so do further terms of the scores
for layers that have them: ``score_cap`` c > 0 (the scaled product x becomes c tanh(x / c)), ``position_slopes`` (one
number per head; slope * (key position - query position) is added after the cap) and ``sinks`` (True: a tensor
``sinks`` [heads], one logit per head that takes part in the softmax's sum and in nothing else).  The three input
projections are fused into one matrix when the weights arrive, so one product serves them.
"""

from __future__ import annotations

import torch

from ..csrc import ops
from .base import BLOCK, CacheSpec, Mixer, PageTensor
from .linear import Weight, linear, qkv_rotary_cache
from .registry import BuildEnv, register_mixer
from .spec import PartSpec, WeightSpec


class PagedAttention(Mixer):
    graph_capturable = True
    graph_capturable_prompts = True

    def __init__(self, params: dict, env: BuildEnv):
        self.hidden = env.hidden_size
        self.num_heads = int(params["num_heads"])
        self.num_kv_heads = int(params.get("num_kv_heads", self.num_heads))
        self.head_dim = int(params["head_dim"])
        self.scale = float(params.get("scale", self.head_dim ** -0.5))
        self.window = int(params.get("window") or 0)
        # False for a layer that always reads another layer's cache: it then has no k/v weights.
        self.kv_proj = bool(params.get("kv_proj", True))
        self.qkv_bias = bool(params.get("qkv_bias", False))
        self.score_cap = float(params.get("score_cap") or 0.0)
        slopes = params.get("position_slopes")
        self.has_sinks = bool(params.get("sinks", False))
        if self.score_cap < 0.0:
            raise ValueError(f"a cap of the scores is positive (or 0 for none), got {self.score_cap}")
        if slopes is not None and len(slopes) != self.num_heads:
            raise ValueError(f"{len(slopes)} position slopes for {self.num_heads} heads")
        if self.num_heads % self.num_kv_heads:
            raise ValueError(f"{self.num_heads} heads are no multiple of {self.num_kv_heads} kv heads")
        if not 1 <= self.head_dim <= ops.MAX_HEAD_DIM_GENERIC:
            raise ValueError(f"attention kernels take head sizes 1..{ops.MAX_HEAD_DIM_GENERIC} (the matrix-core kernels "
                             f"multiples of 16, the plain kernel the others), got {self.head_dim}")
        pos = params.get("position")
        self.position = env.position_encoding(PartSpec(**pos) if isinstance(pos, dict) else pos) if pos else None
        self.dtype, self.device = env.dtype, env.device
        self.slopes = None if slopes is None else torch.tensor([float(x) for x in slopes], dtype=torch.float32, device=self.device)
        self.terms: ops.ScoreTerms | None = None                 # put together in finalize(), once the sinks are there
        self._w: dict[str, torch.Tensor] = {}
        self.w_qkv: Weight | None = None
        self.w_o: Weight | None = None
        self.b_qkv: torch.Tensor | None = None

    # ---- weights
    def weight_specs(self):
        q, kv = self.num_heads * self.head_dim, self.num_kv_heads * self.head_dim
        specs = {"q_proj.weight": WeightSpec((q, self.hidden)), "o_proj.weight": WeightSpec((self.hidden, q))}
        if self.kv_proj:
            specs["k_proj.weight"] = WeightSpec((kv, self.hidden))
            specs["v_proj.weight"] = WeightSpec((kv, self.hidden))
        if self.qkv_bias:                                        # (kept in float: the bias is added to float sums)
            specs["q_proj.bias"] = WeightSpec((q,), role="vector")
            if self.kv_proj:
                specs["k_proj.bias"] = WeightSpec((kv,), role="vector")
                specs["v_proj.bias"] = WeightSpec((kv,), role="vector")
        if self.has_sinks:
            specs["sinks"] = WeightSpec((self.num_heads,), role="vector")
        return specs

    def assign(self, name, tensor):
        spec = self.weight_specs().get(name)
        if spec is None:
            raise KeyError(name)
        self._w[name] = tensor.to(device=self.device, dtype=torch.float32 if spec.role == "vector" else self.dtype)

    def finalize(self):
        names = ["q_proj.weight"] + (["k_proj.weight", "v_proj.weight"] if self.kv_proj else [])
        # (a layer without k/v projections only ever projects q: its matrix keeps the plain pairing)
        self.w_qkv = Weight(torch.cat([self._w[n] for n in names], dim=0).contiguous(), "rotary" if self.kv_proj else "plain", self.head_dim)
        self.w_o = Weight(self._w["o_proj.weight"].contiguous())
        if self.qkv_bias:
            self.b_qkv = torch.cat([self._w[n.replace(".weight", ".bias")] for n in names]).contiguous()
        terms = ops.ScoreTerms(self.score_cap, self.slopes, self._w["sinks"].contiguous() if self.has_sinks else None)
        self.terms = terms if terms.any() else None
        self._w.clear()

    # ---- what it keeps
    def cache_spec(self):
        """Keys as rows [kv_heads, positions, d]; values transposed inside the page [kv_heads, d, positions], so that
        8 successive positions of one channel are one 16-byte load, the operand shape of the P*V matrix instruction."""
        kind = "window" if self.window > 0 else "full"
        nkv, d = self.num_kv_heads, self.head_dim
        return CacheSpec(kind, (PageTensor("k", (nkv, BLOCK, d)), PageTensor("v", (nkv, d, BLOCK))), self.window)

    def graph_step_arrays(self, layout):
        """The prompt kernel's work list (pairs of sequence and tile, most keys first) for a replayed step."""
        group = self.num_heads // self.num_kv_heads
        first = layout.num_single_rows
        pairs = ops.prompt_tiles_capacity(layout.num_portions, layout.portion_tokens, group)
        return {("prompt_tiles", first, group): (2 * pairs, lambda q_lens, k_lens: ops.prompt_tiles(q_lens, k_lens, first, group, pairs))}

    # ---- compute
    def forward(self, h, ctx, cache, state):
        nh, nkv, d = self.num_heads, self.num_kv_heads, self.head_dim
        view = ctx.groups[cache.group]
        write = cache.writable
        if write and not self.kv_proj:
            raise RuntimeError("this attention layer has no k/v projections and must read another layer's cache")
        only_q = not write and self.kv_proj
        w_in = self.w_qkv.rows(nh * d) if only_q else self.w_qkv
        bias = self.b_qkv[: nh * d] if only_q and self.b_qkv is not None else self.b_qkv
        k_pages, v_pages = cache["k"], cache["v"]
        qkv = qkv_rotary_cache(h, w_in, ctx.positions, self.position, nh, nkv, d, view.slot_mapping if write else None,
                               k_pages if write else None, v_pages if write else None, cache.block_size, bias=bias)
        o = ops.paged_attention(qkv, k_pages, v_pages, view.block_tables, ctx.cu_seqlens_q, ctx.seq_lens_k,
                                nh, nkv, d, self.scale, self.window, ctx, terms=self.terms)
        return linear(o, self.w_o, partial_ok=bool(getattr(ctx, "partial_sums_ok", False)))


register_mixer("paged_attention", PagedAttention)
