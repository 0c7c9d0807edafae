"""Data that describes a model: which parts each layer is made of, and in which order layers run.

Nothing here computes.  An architecture's ``build_spec`` turns its typed configuration into a
``ModelSpec``; ``models.decoder.DecoderModel`` builds the parts the spec names from the part
registry.  Sizes and constants travel inside the specs, so no part reads a model configuration.
"""

from __future__ import annotations

import json
from dataclasses import dataclass, field
from typing import Any


@dataclass
class PartSpec:
    """A part by the name it is registered under, with its own parameters."""
    kind: str
    params: dict = field(default_factory=dict)

    def key(self) -> str:
        return json.dumps([self.kind, self.params], sort_keys=True, default=str)


@dataclass
class WeightSpec:
    """One tensor a part expects from the checkpoint.

    role "matrix"/"table": kept in the compute type (bfloat16 or float32).
    role "vector": kept in float32 (norm weights are applied in float).
    role "int": an integer table, kept as int32.
    """
    shape: tuple
    role: str = "matrix"
    # For the random-weights mode: "normal" (std 0.02) or "ones".
    init: str = "normal"


@dataclass
class LayerSpec:
    """One decoder layer: the arrangement (``block``) and the parts it arranges, by role.

    Which roles there are, and which family of parts fills each, is the block kind's business: the
    pre-norm block has "mixer_norm", "mixer", "feed_forward_norm" and "feed_forward"; a block with one
    shared norm, with norms behind its branches or without a feed-forward names other roles."""
    name: str                       # prefix of its tensor names, e.g. "model.layers.3"
    block: PartSpec
    parts: dict = field(default_factory=dict)      # role -> PartSpec


@dataclass
class ScheduleStep:
    """One entry of the run order: which layer runs, and whose cache its mixer uses.

    A layer named by several steps shares its weights between them; each step still owns a
    cache and a state of its own, because what it sees differs.  ``cache_from`` names an earlier
    step whose cache this step's mixer reads instead of writing one."""
    layer: int
    cache_from: int | None = None


@dataclass
class ModelSpec:
    hidden_size: int
    vocab_size: int
    embedding: PartSpec
    layers: list[LayerSpec]
    final_norm: PartSpec
    head: PartSpec
    # The order in which layers run; empty = every layer once, in order.
    schedule: list[ScheduleStep] = field(default_factory=list)
    # Prefixes of the tensor names of the parts outside the layers (the architecture says them: "" is no default
    # that fits any family of checkpoints).
    embedding_name: str = ""
    final_norm_name: str = ""
    head_name: str = ""
    # Tensor names that may be present in a checkpoint and are ignored (suffix match).
    ignored_suffixes: tuple = ()
    max_positions: int = 4096
    eos_token_id: Any = None
    stored_dtype: str = "bfloat16"

    def __post_init__(self) -> None:
        for what in ("embedding_name", "final_norm_name", "head_name"):
            if not getattr(self, what):
                raise ValueError(f"a ModelSpec needs {what}: the prefix of that part's tensor names in the checkpoint")
        if not self.schedule:
            self.schedule = [ScheduleStep(i) for i in range(len(self.layers))]
        self.schedule = [s if isinstance(s, ScheduleStep) else ScheduleStep(int(s)) for s in self.schedule]
        for pos, step in enumerate(self.schedule):
            if not 0 <= step.layer < len(self.layers):
                raise ValueError(f"schedule step {pos} names layer {step.layer}, the model has {len(self.layers)}")
            src = step.cache_from
            if src is not None:
                if not 0 <= src < pos:
                    raise ValueError(f"schedule step {pos} reads the cache of step {src}, which has not run before it")
                if self.schedule[src].cache_from is not None:
                    raise ValueError(f"schedule step {pos} reads the cache of step {src}, which owns none")
