"""A decoder put together from a ModelSpec: embedding -> the scheduled layers -> last norm on the
wanted rows -> head.  It knows parts and the run order, not architectures."""

from __future__ import annotations

import torch

from ..cache.kv_cache import CacheGroup
from ..parts import registry
from ..parts.registry import BuildEnv
from ..parts.spec import ModelSpec, WeightSpec


class DecoderModel:
    def __init__(self, spec: ModelSpec, dtype: torch.dtype, device, max_positions: int | None = None):
        self.spec = spec
        self.dtype = dtype
        self.device = torch.device(device)
        self.max_positions = max(spec.max_positions, max_positions or 0)
        env = BuildEnv(spec.hidden_size, dtype, self.device, self.max_positions, shared={})
        self.env = env
        self.embedding = registry.build("embedding", spec.embedding, env)
        self.blocks = []
        for layer in spec.layers:
            block = registry.build("block", layer.block, env)
            block.build_parts(layer.parts, env)
            self.blocks.append(block)
        self.final_norm = registry.build("norm", spec.final_norm, env)
        self.head = registry.build("head", spec.head, env)
        self._ready = False

    # ------------------------------------------------------------------ weights
    def weight_specs(self) -> dict[str, WeightSpec]:
        s = self.spec
        out = {f"{s.embedding_name}.{n}": w for n, w in self.embedding.weight_specs().items()}
        for layer, block in zip(s.layers, self.blocks):
            out.update({f"{layer.name}.{n}": w for n, w in block.weight_specs().items()})
        out.update({f"{s.final_norm_name}.{n}": w for n, w in self.final_norm.weight_specs().items()})
        out.update({f"{s.head_name}.{n}": w for n, w in self.head.weight_specs().items()})
        return out

    def optional_weights(self) -> dict[str, tuple]:
        """Tensors a checkpoint may carry although the model does not need them (a tied head
        stored a second time): name -> shape."""
        if getattr(self.head, "tied", False):
            return {f"{self.spec.head_name}.weight": (self.spec.vocab_size, self.spec.hidden_size)}
        return {}

    def assign(self, name: str, tensor: torch.Tensor) -> None:
        s = self.spec
        for prefix, part in [(s.embedding_name, self.embedding), (s.final_norm_name, self.final_norm), (s.head_name, self.head)]:
            if name.startswith(prefix + "."):
                return part.assign(name[len(prefix) + 1:], tensor)
        for layer, block in zip(s.layers, self.blocks):
            if name.startswith(layer.name + "."):
                return block.assign(name[len(layer.name) + 1:], tensor)
        raise KeyError(name)

    def finalize(self) -> None:
        self.embedding.finalize()
        for b in self.blocks:
            b.finalize()
        self.final_norm.finalize()
        self.head.finalize()
        if getattr(self.head, "tied", False):
            self.head.tie(self.embedding.table)
        self._ready = True

    # ------------------------------------------------------------------ what the cache manager must provide
    def cache_groups(self) -> dict[str, CacheGroup]:
        """Schedule steps that own pages, grouped by what their mixers keep per token."""
        groups: dict[str, CacheGroup] = {}
        for pos, step in enumerate(self.spec.schedule):
            if step.cache_from is not None:
                continue
            cs = self.blocks[step.layer].cache_spec()
            if cs is None:
                continue
            name = cs.group_name()
            groups.setdefault(name, CacheGroup(name, cs, [])).owners.append(pos)
        return groups

    def state_specs(self) -> dict[int, object]:
        """Schedule step -> StateSpec for mixers with per-request state of fixed size."""
        out = {}
        for pos, step in enumerate(self.spec.schedule):
            ss = self.blocks[step.layer].state_spec()
            if ss is not None:
                out[pos] = ss
        return out

    def graph_capturable(self, prompts: bool = False) -> bool:
        """True when every layer's parts only launch kernels (no host reads of device data, no Python-side
        state): a decode step (``prompts``: also a step with prompt portions) can then be captured into a HIP graph."""
        return all(b.graph_capturable(prompts) for b in self.blocks)

    def graph_step_arrays(self, layout) -> dict:
        """Host-made integer arrays the layers' parts need for a replayed step of that layout (equal keys are one array)."""
        out = {}
        for b in self.blocks:
            out.update(b.graph_step_arrays(layout))
        return out

    # ------------------------------------------------------------------ compute
    def forward(self, ctx, kv_storage, states: dict) -> torch.Tensor:
        """Float logits [n, vocab] at ctx.logits_index (empty tensor when nothing is wanted;
        the layers still run to fill the cache)."""
        assert self._ready, "weights not loaded"
        x = self.embedding.forward(ctx.input_ids)
        delta = None
        schedule = self.spec.schedule
        last_takes_partial = bool(getattr(self.final_norm, "accepts_partial_sums", False))
        for pos, step in enumerate(schedule):
            block = self.blocks[step.layer]
            cache = None
            if block.cache_spec() is not None:
                owner = pos if step.cache_from is None else step.cache_from
                cache = kv_storage.for_step(owner, writable=step.cache_from is None)
            # whether the delta this block hands on may be float partial sums: what consumes it next says
            ctx.partial_sums_ok = (self.blocks[schedule[pos + 1].layer].accepts_partial_delta() if pos + 1 < len(schedule)
                                   else last_takes_partial)
            x, delta = block.forward(x, delta, ctx, cache, states.get(pos))
        ctx.partial_sums_ok = False
        n = ctx.logits_index.numel()
        if n == 0:
            return torch.empty((0, self.spec.vocab_size), dtype=torch.float32, device=self.device)
        h = self.final_norm.pending(x, delta, ctx.logits_index, write_residual=False)
        return self.head.forward(h)
