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
        # the three matrices' own names under the part's prefix (``tensor_names``: {"gate": ..., "up": ..., "down": ...})
        names = params.get("tensor_names") or {}
        self.n_gate = names.get("gate", "gate_proj.weight")
        self.n_up = names.get("up", "up_proj.weight")
        self.n_down = names.get("down", "down_proj.weight")
        self._w: dict[str, torch.Tensor] = {}
        self.w_gate_up: Weight | None = None
        self.w_down: Weight | None = None

    def weight_specs(self):
        return {self.n_gate: WeightSpec((self.inter, self.hidden)),
                self.n_up: WeightSpec((self.inter, self.hidden)),
                self.n_down: WeightSpec((self.hidden, self.inter))}

    def assign(self, name, tensor):
        if name not in self.weight_specs():
            raise KeyError(name)
        self._w[name] = tensor.to(device=self.device, dtype=self.dtype)

    def finalize(self):
        self.w_gate_up = Weight(torch.cat([self._w[self.n_gate], self._w[self.n_up]], dim=0).contiguous(), "gated")
        self.w_down = Weight(self._w[self.n_down].contiguous())
        self._w.clear()

    def forward(self, h, ctx):
        act = gated_linear(h, self.w_gate_up, self.activation)
        if getattr(ctx, "float_branch", False):                 # whoever takes the result norms it in float: no rounding in between
            return linear(act, self.w_down, out_dtype=torch.float32)
        return linear(act, self.w_down, partial_ok=bool(getattr(ctx, "partial_sums_ok", False)))


register_feed_forward("gated_mlp", GatedMLP)
