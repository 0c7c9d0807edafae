"""Gated feed-forward: down(act(gate(x)) * up(x)) without bias; the reference's Llama has act = SiLU
(pagedllm/model/llama.py:163-171), the part takes the activation as a parameter (``ops.ACTIVATIONS``).  gate and up
are fused into one matrix [2I, H] when the weights arrive; the activation and the product run in float in one kernel."""

from __future__ import annotations

import torch

from ..csrc import ops
from .base import FeedForward
from .linear import Weight, gated_linear, linear
from .registry import BuildEnv, register_feed_forward
from .spec import WeightSpec


class GatedMLP(FeedForward):
    graph_capturable = True
    graph_capturable_prompts = True

    def __init__(self, params: dict, env: BuildEnv):
        self.hidden = env.hidden_size
        self.inter = int(params["intermediate_size"])
        self.activation = params.get("activation", "silu")
        if self.activation not in ops.ACTIVATIONS:
            raise NotImplementedError(f"gated feed-forward activation {self.activation!r}: one of {sorted(ops.ACTIVATIONS)}")
        self.dtype, self.device = env.dtype, env.device
        self._w: dict[str, torch.Tensor] = {}
        self.w_gate_up: Weight | None = None
        self.w_down: Weight | None = None

    def weight_specs(self):
        return {"gate_proj.weight": WeightSpec((self.inter, self.hidden)),
                "up_proj.weight": WeightSpec((self.inter, self.hidden)),
                "down_proj.weight": WeightSpec((self.hidden, self.inter))}

    def assign(self, name, tensor):
        if name not in self.weight_specs():
            raise KeyError(name)
        self._w[name] = tensor.to(device=self.device, dtype=self.dtype)

    def finalize(self):
        self.w_gate_up = Weight(torch.cat([self._w["gate_proj.weight"], self._w["up_proj.weight"]], dim=0).contiguous(), "gated")
        self.w_down = Weight(self._w["down_proj.weight"].contiguous())
        self._w.clear()

    def forward(self, h, ctx):
        act = gated_linear(h, self.w_gate_up, self.activation)
        return linear(act, self.w_down, partial_ok=bool(getattr(ctx, "partial_sums_ok", False)))


register_feed_forward("gated_mlp", GatedMLP)
