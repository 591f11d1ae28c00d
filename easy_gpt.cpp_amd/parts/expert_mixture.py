"""A mixture of gated experts as a layer's feed-forward.

Every token goes to the `top` experts with the largest router logits z = W_r x + b (float32), weighted by the softmax
over those logits alone; an expert is W_down (silu(W_gate x) * (W_up x)) without biases.  An optional shared
feed-forward runs for every token and is added.  Routing, grouping of the rows by expert and the experts' products
all happen on the device, so a step with experts is launched like any other and replays from a graph.
"""
from __future__ import annotations

import torch

from .. import kernels
from .base import FeedForward, make_part, register_part
from .spec import ParamSpec, PartSpec


class ExpertMixture(FeedForward):
    graph_safe = True

    def __init__(self, prefix: str, hidden_size: int, n_experts: int, top: int, intermediate_size: int,
                 shared: PartSpec | None = None, router_bias: bool = True, names: dict | None = None):
        """names: `expert` (the prefix of expert i's tensors, with {i}), `gate`, `up`, `down`, `router`, `router_bias`
        behind `prefix`.  shared: a feed-forward part that every token runs through as well."""
        if not 0 < int(top) <= int(n_experts):
            raise ValueError(f"top ({top}) must be between 1 and the number of experts ({n_experts})")
        self.prefix, self.hidden_size = prefix, int(hidden_size)
        self.n_experts, self.top, self.intermediate_size = int(n_experts), int(top), int(intermediate_size)
        self.has_router_bias = bool(router_bias)
        self.names = dict(expert="e{i}.", gate="gate", up="up", down="down", router="router", router_bias="router.b")
        self.names.update(names or {})
        self.shared = make_part("feed_forward", shared, hidden_size=hidden_size) if shared is not None else None
        if self.shared is not None and not self.shared.graph_safe:
            self.graph_safe = False
        self.w_router = self.b_router = self.w_gate_up = self.w_down = None

    def _expert(self, i: int, which: str) -> str:
        return self.prefix + self.names["expert"].format(i=i) + self.names[which]

    def param_specs(self):
        h, f = self.hidden_size, self.intermediate_size
        specs = []
        for i in range(self.n_experts):
            specs += [ParamSpec(self._expert(i, "gate"), (f, h)), ParamSpec(self._expert(i, "up"), (f, h)),
                      ParamSpec(self._expert(i, "down"), (h, f))]
        specs.append(ParamSpec(self.prefix + self.names["router"], (self.n_experts, h)))
        if self.has_router_bias:
            specs.append(ParamSpec(self.prefix + self.names["router_bias"], (self.n_experts,), role="bias"))
        if self.shared is not None:
            specs += self.shared.param_specs()
        return specs

    def load(self, get, dtype, device):
        e, h, f = self.n_experts, self.hidden_size, self.intermediate_size
        self.w_gate_up = torch.empty((e, 2 * f, h), dtype=dtype, device=device)      # an expert's gate rows, then its up rows
        self.w_down = torch.empty((e, h, f), dtype=dtype, device=device)
        for i in range(e):
            self.w_gate_up[i, :f].copy_(get(self._expert(i, "gate")).to(dtype))
            self.w_gate_up[i, f:].copy_(get(self._expert(i, "up")).to(dtype))
            self.w_down[i].copy_(get(self._expert(i, "down")).to(dtype))
        self.w_router = self._to(get(self.prefix + self.names["router"]), "compute", dtype, device)
        if self.has_router_bias:
            self.b_router = self._to(get(self.prefix + self.names["router_bias"]), "compute", dtype, device)
        if self.shared is not None:
            self.shared.load(get, dtype, device)

    def forward(self, x, ctx=None):
        out = kernels.backend().expert_mixture(x, self.w_router, self.b_router, self.w_gate_up, self.w_down, self.top)[None]
        if self.shared is None:
            return out
        s = self.shared.forward(x, ctx)
        if s.dim() != 3:
            s = s.float()[None]
        return torch.cat([out, s], dim=0)          # float32 partial sums: whoever adds to the stream adds them up


register_part("feed_forward", "expert_mixture", ExpertMixture)
