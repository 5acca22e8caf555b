"""A feed-forward of routed experts (the spec: :class:`~mini_engine_amd.config.specs.RoutedExpertsSpec`): a router picks
``top_k`` of ``num_experts`` small gated feed-forwards per token by its float32 logits and weights them by the softmax
over the picked logits; the token's result is the weighted sum of what they give.

The experts' weights are stacked at load time (``[experts, 2 ff, hidden]`` gate rows then up rows, ``[experts, hidden,
ff]``); the router's weight is kept in float32. A step routes on the device: the pairs (token, expert) are sorted by
expert and served in tiles of one expert (``csrc/routed_ff.hip``), so a decode step reads the weights of the experts
that its tokens picked and no others. The results wait as float32 partial sums, one per pick of a token, that the
next add of the residual stream sums up in the order of the picks.
"""

from __future__ import annotations

import torch

from ..ops import kernels as K
from ..weights.loader import TensorWant
from .base import FEED_FORWARDS, FeedForward


class RoutedExperts(FeedForward):
    graph_safe = True

    def __init__(self, spec, dtype, device):
        super().__init__(spec, dtype, device)
        if spec.activation not in K.GATE_ACTIVATIONS:
            raise ValueError(f"routed experts know the activations {sorted(K.GATE_ACTIVATIONS)}, got {spec.activation!r}")
        if not 1 <= spec.top_k <= spec.num_experts:
            raise ValueError(f"{spec.top_k} of {spec.num_experts} experts a token")
        names = dict(getattr(spec, "names", ()) or ())
        self._n = {r: names.get(r, d) for r, d in (("router", "router"), ("expert", "experts."), ("gate", "gate_proj.weight"),
                                                    ("up", "up_proj.weight"), ("down", "down_proj.weight"))}
        self.router = self.w_gate_up = self.w_down = None

    def _expert(self, prefix: str, e: int, role: str) -> str:
        return f"{prefix}.{self._n['expert']}{e}.{self._n[role]}"

    def weight_wants(self, prefix: str) -> dict[str, TensorWant]:
        s = self.spec
        wants = {f"{prefix}.{self._n['router']}": TensorWant((s.num_experts, s.hidden_size), "vector")}
        for e in range(s.num_experts):
            wants[self._expert(prefix, e, "gate")] = TensorWant((s.intermediate_size, s.hidden_size))
            wants[self._expert(prefix, e, "up")] = TensorWant((s.intermediate_size, s.hidden_size))
            wants[self._expert(prefix, e, "down")] = TensorWant((s.hidden_size, s.intermediate_size))
        return wants

    def load(self, tensors, prefix: str) -> None:
        s = self.spec
        self.router = tensors[f"{prefix}.{self._n['router']}"]
        self.w_gate_up = torch.stack([torch.cat((tensors[self._expert(prefix, e, "gate")], tensors[self._expert(prefix, e, "up")]), dim=0)
                                      for e in range(s.num_experts)]).contiguous()
        self.w_down = torch.stack([tensors[self._expert(prefix, e, "down")] for e in range(s.num_experts)]).contiguous()

    def forward(self, h, batch=None):
        raise NotImplementedError("routed experts run in the step program only")

    def emit(self, program, h) -> None:
        x = h.value() if hasattr(h, "value") else h
        program.routed_ff(x, router=self.router, gate_up=self.w_gate_up, down=self.w_down, top_k=int(self.spec.top_k),
                          activation=self.spec.activation)


FEED_FORWARDS.register("routed_experts", RoutedExperts)
