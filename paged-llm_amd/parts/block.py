"""Pre-norm residual block: x += mixer(norm1(x)); x += feed_forward(norm2(x))
(pagedllm/model/llama.py:174-185).

The residual stream travels as (x, delta) with delta not yet added, so each norm adds the
previous branch's output in its own kernel; the sum is formed in float and rounded once to the
stream's element type, which is what a plain add in that type gives.
"""

from __future__ import annotations

from .base import Block
from .registry import BuildEnv, build, register_block
from .spec import PartSpec


class PreNormBlock(Block):
    """params: names of the four sub-parts in tensor names (mixer_norm, mixer, feed_forward_norm,
    feed_forward); the parts themselves come from the LayerSpec."""

    def __init__(self, params: dict, env: BuildEnv):
        self.names = {
            "mixer_norm": params.get("mixer_norm", "mixer_norm"),
            "mixer": params.get("mixer", "mixer"),
            "feed_forward_norm": params.get("feed_forward_norm", "feed_forward_norm"),
            "feed_forward": params.get("feed_forward", "feed_forward"),
        }
        self.parts: dict = {}

    def attach(self, mixer_norm, mixer, feed_forward_norm, feed_forward) -> None:
        self.parts = {"mixer_norm": mixer_norm, "mixer": mixer, "feed_forward_norm": feed_forward_norm,
                      "feed_forward": feed_forward}

    @property
    def mixer(self):
        return self.parts["mixer"]

    def weight_specs(self):
        out = {}
        for role, part in self.parts.items():
            for name, spec in part.weight_specs().items():
                out[f"{self.names[role]}.{name}"] = spec
        return out

    def assign(self, name, tensor):
        for role, part in self.parts.items():
            prefix = self.names[role] + "."
            if name.startswith(prefix):
                return part.assign(name[len(prefix):], tensor)
        raise KeyError(name)

    def finalize(self):
        for part in self.parts.values():
            part.finalize()

    def forward(self, x, delta, ctx, cache, state):
        p = self.parts
        h = p["mixer_norm"].pending(x, delta)             # summed and normed by whoever consumes it first
        a = p["mixer"].forward(h, ctx, cache, state)
        x = h.residual()
        h = p["feed_forward_norm"].pending(x, a)
        m = p["feed_forward"].forward(h, ctx)
        return h.residual(), m


register_block("prenorm", PreNormBlock)
