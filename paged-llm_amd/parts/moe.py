"""A feed-forward of routed experts: each token passes through ``top`` of ``experts`` small gated feed-forwards,
down(act(gate h) * (up h)) without biases, and the results are summed with router scores as weights.

Router: z = W_router h in float, scores s = softmax(z) over all router outputs.  The choice looks at s + correction (a
stored vector): the experts are cut into ``groups`` equal groups of neighbours, a group's mark is its largest corrected
score, and only experts of the ``keep`` best groups can be chosen; the ``top`` largest corrected scores among those win.
The weights are the chosen experts' scores s themselves (no renormalisation).  The last ``identity`` router outputs
stand for experts without weights that hand the token's own row back.

On the GPU the (token, choice) pairs are sorted by expert and the experts' products run over tiles of a run of
rows each (``ops.moe_*``): nothing is read back by the host, so the step can be replayed from a graph, and a pair's
result does not depend on what else is in the batch.
"""

from __future__ import annotations

import torch

from ..csrc import ops
from .base import FeedForward, name_under
from .norm import rows_of
from .registry import BuildEnv, register_feed_forward
from .spec import WeightSpec


class RoutedExperts(FeedForward):
    """params: ``experts``, ``identity`` (pass-through experts behind them, default 0), ``top``, ``groups`` and ``keep``
    (defaults 1 and 1), ``intermediate_size`` (of one expert), ``activation`` (default "silu"), ``correction`` (a stored
    vector is added to the scores for the choice; default True).  Tensors: ``e<i>.gate``, ``e<i>.up`` [ff, width],
    ``e<i>.down`` [width, ff], ``router`` [experts + identity, width], ``correction`` [experts + identity]."""
    graph_capturable = True
    graph_capturable_prompts = True

    def __init__(self, params: dict, env: BuildEnv):
        self.hidden = env.hidden_size
        self.experts, self.identity = int(params["experts"]), int(params.get("identity") or 0)
        self.top, self.groups, self.keep = int(params["top"]), int(params.get("groups") or 1), int(params.get("keep") or 1)
        self.inter = int(params["intermediate_size"])
        self.activation = params.get("activation", "silu")
        self.has_correction = bool(params.get("correction", True))
        self.n = self.experts + self.identity
        if self.activation not in ops.ACTIVATIONS:
            raise NotImplementedError(f"expert activation {self.activation!r}: one of {sorted(ops.ACTIVATIONS)}")
        if self.experts <= 0 or self.experts > ops.MOE_MAX_EXPERTS or self.n % self.groups or not 0 < self.keep <= self.groups \
                or not 0 < self.top <= (self.n // self.groups) * self.keep:
            raise ValueError(f"{self.experts} experts + {self.identity} pass-through in {self.groups} groups, {self.keep} kept, {self.top} chosen")
        self.dtype, self.device = env.dtype, env.device
        self._w: dict = {}
        self.w_gate_up = self.w_down = self.router = self.correction = None

    def weight_specs(self):
        specs = {"router": WeightSpec((self.n, self.hidden), role="vector")}
        if self.has_correction:
            specs["correction"] = WeightSpec((self.n,), role="vector")
        for e in range(self.experts):
            specs[f"e{e}.gate"] = WeightSpec((self.inter, self.hidden))
            specs[f"e{e}.up"] = WeightSpec((self.inter, self.hidden))
            specs[f"e{e}.down"] = WeightSpec((self.hidden, self.inter))
        return specs

    def assign(self, name, tensor):
        spec = self.weight_specs().get(name)
        if spec is None:
            raise KeyError(name)
        self._w[name] = tensor.to(device=self.device, dtype=torch.float32 if spec.role == "vector" else self.dtype).contiguous()

    def finalize(self):
        w, E = self._w, self.experts
        self.router = w.pop("router")
        self.correction = w.pop("correction") if self.has_correction else None
        # one tensor per kind of matrix, the experts one behind the other: [experts, 2 ff, width] with [gate; up], [experts, width, ff]
        self.w_gate_up = torch.stack([torch.cat([w.pop(f"e{e}.gate"), w.pop(f"e{e}.up")], dim=0) for e in range(E)]).contiguous()
        self.w_down = torch.stack([w.pop(f"e{e}.down") for e in range(E)]).contiguous()

    def forward(self, h, ctx):
        h = rows_of(h)
        ids, weights = ops.moe_route(h, self.router, self.correction, self.groups, self.keep, self.top)
        rows = ops.moe_tile_rows(ids.numel(), self.experts, h.dtype, self.hidden, self.inter, h.stride(0))
        sorted_pair, row_of_pair, tiles = ops.moe_align(ids, self.experts, rows)
        act = ops.moe_expert_gemm(h, self.w_gate_up, tiles, sorted_pair, self.top, True, self.activation, tile_rows=rows)
        out = ops.moe_expert_gemm(act, self.w_down, tiles, sorted_pair, self.top, False, tile_rows=rows)
        if getattr(ctx, "float_branch", False) and getattr(ctx, "branch_sum_ok", False):
            return ops.ChoiceSum(out, h, row_of_pair, weights)      # whoever norms the branch forms the sum in its kernel
        y = ops.moe_combine(out, h, row_of_pair, weights)
        if getattr(ctx, "float_branch", False):
            return y
        return y if self.dtype == torch.float32 else ops.round_rows(y)


register_feed_forward("routed_experts", RoutedExperts)
