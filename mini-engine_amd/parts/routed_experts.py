"""A feed-forward of routed experts (the spec: :class:`~mini_engine_amd.config.specs.RoutedExpertsSpec`): a router picks
``top_k`` of ``num_experts`` small gated feed-forwards per token by its float32 logits and weights them by the softmax
over the picked logits; the token's result is the weighted sum of what they give.

The experts' weights are stacked at load time (``[experts, 2 ff, hidden]`` gate rows then up rows, ``[experts, hidden,
ff]``); the router's weight is kept in float32. A step routes on the device: the pairs (token, expert) are sorted by
expert and served in tiles of one expert (``csrc/routed_ff.hip``), so a decode step reads the weights of the experts
that its tokens picked and no others. The results wait as float32 partial sums, one per pick of a token, that the
next add of the residual stream sums up in the order of the picks.

The spec may also: score by the sigmoid of the logits and weight the picks by their scores over their sum, times a scale;
bound the picks to the experts of the best few of some equal groups of neighbours; give the activation a limit to clamp by;
and add an expert that every token uses, multiplied by the sigmoid of one number per token (one more partial sum).
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
        self.gated = bool(getattr(spec, "gated", True))
        known = sorted(set(K.GATE_ACTIVATIONS) | set(K.LIMITED_GATE_ACTIVATIONS)) if self.gated else sorted(K.UNGATED_ACTIVATIONS)
        if spec.activation not in known:
            raise ValueError(f"routed experts {'with' if self.gated else 'without'} a gate know the activations {known}, got {spec.activation!r}")
        self.identity = int(getattr(spec, "identity_experts", 0))
        self.corrected = bool(getattr(spec, "score_correction", False))
        self.shared_gated = bool(getattr(spec, "shared_gated", True))
        self.scoring = getattr(spec, "scoring", "softmax_picked")
        if self.identity < 0 or ((self.identity or self.corrected) and self.scoring != "softmax_all"):
            raise ValueError("identity experts and a correction of the scores belong to a router that scores by softmax_all")
        if not self.gated and self.shared_gated and int(getattr(spec, "shared_size", 0)):
            raise ValueError("a shared expert without gate rows has no gate of its own either")
        if spec.num_experts < 1 or not 1 <= spec.top_k <= spec.num_experts + self.identity:
            raise ValueError(f"{spec.top_k} of {spec.num_experts + self.identity} experts a token")
        self.groups, self.keep = int(getattr(spec, "num_groups", 1)), int(getattr(spec, "keep_groups", 1))
        if self.scoring != "sigmoid_normalized" and (self.groups, self.keep) != (1, 1):
            raise ValueError("groups of experts bound the picks of a router that scores by sigmoid_normalized")
        if (self.groups < 1 or spec.num_experts % self.groups or not 1 <= self.keep <= self.groups
                or self.keep * (spec.num_experts // self.groups) + self.identity < spec.top_k):
            raise ValueError(f"{spec.num_experts} experts in {self.groups} groups of which {self.keep} are kept, {spec.top_k} picks")
        self.shared_size = int(getattr(spec, "shared_size", 0))
        names = dict(getattr(spec, "names", ()) or ())
        self._n = {r: names.get(r, d) for r, d in (("router", "router"), ("expert", "experts."), ("gate", "gate_proj.weight"),
                                                    ("up", "up_proj.weight"), ("down", "down_proj.weight"), ("shared", "shared"),
                                                    ("shared_gate", "gate"), ("correction", "correction"))}
        self.router = self.w_gate_up = self.w_down = self.w_shared_gate_up = self.w_shared_down = self.correction = None

    def _expert(self, prefix: str, e: int, role: str) -> str:
        return f"{prefix}.{self._n['expert']}{e}.{self._n[role]}"

    def weight_wants(self, prefix: str) -> dict[str, TensorWant]:
        s = self.spec
        wants = {f"{prefix}.{self._n['router']}": TensorWant((s.num_experts + self.identity, s.hidden_size), "vector")}
        if self.corrected:
            wants[f"{prefix}.{self._n['correction']}"] = TensorWant((s.num_experts + self.identity,), "vector")
        for e in range(s.num_experts):
            if self.gated:
                wants[self._expert(prefix, e, "gate")] = TensorWant((s.intermediate_size, s.hidden_size))
            wants[self._expert(prefix, e, "up")] = TensorWant((s.intermediate_size, s.hidden_size))
            wants[self._expert(prefix, e, "down")] = TensorWant((s.hidden_size, s.intermediate_size))
        if self.shared_size:
            sp = f"{prefix}.{self._n['shared']}"
            if self.gated:
                wants[f"{sp}.{self._n['gate']}"] = TensorWant((self.shared_size, s.hidden_size))
            wants[f"{sp}.{self._n['up']}"] = TensorWant((self.shared_size, s.hidden_size))
            wants[f"{sp}.{self._n['down']}"] = TensorWant((s.hidden_size, self.shared_size))
            if self.shared_gated:
                wants[f"{sp}.{self._n['shared_gate']}"] = TensorWant((1, s.hidden_size), "vector")
        return wants

    def load(self, tensors, prefix: str) -> None:
        s = self.spec
        self.router = tensors[f"{prefix}.{self._n['router']}"]
        if self.gated:
            self.w_gate_up = torch.stack([torch.cat((tensors[self._expert(prefix, e, "gate")], tensors[self._expert(prefix, e, "up")]), dim=0)
                                          for e in range(s.num_experts)]).contiguous()
        else:  # (experts without a gate: their up rows alone)
            self.w_gate_up = torch.stack([tensors[self._expert(prefix, e, "up")] for e in range(s.num_experts)]).contiguous()
        if self.corrected:
            self.correction = tensors[f"{prefix}.{self._n['correction']}"].contiguous()
        self.w_down = torch.stack([tensors[self._expert(prefix, e, "down")] for e in range(s.num_experts)]).contiguous()
        if self.shared_size:
            sp = f"{prefix}.{self._n['shared']}"
            up = tensors[f"{sp}.{self._n['up']}"]
            self.w_shared_gate_up = torch.cat((tensors[f"{sp}.{self._n['gate']}"], up), dim=0) if self.gated else up.contiguous()
            self.w_shared_down = tensors[f"{sp}.{self._n['down']}"]
            if self.shared_gated:
                # the shared expert's gate as one more row of the router: the kernel that routes a token computes it on the way
                self.router = torch.cat((self.router, tensors[f"{sp}.{self._n['shared_gate']}"].reshape(1, -1)), dim=0).contiguous()

    def forward(self, h, batch=None):
        raise NotImplementedError("routed experts run in the step program only")

    def emit(self, program, h) -> None:
        x = h.value() if hasattr(h, "value") else h
        s = self.spec
        program.routed_ff(x, router=self.router, gate_up=self.w_gate_up, down=self.w_down, top_k=int(s.top_k), activation=s.activation,
                          activation_limit=float(getattr(s, "activation_limit", 0.0)), scoring=self.scoring, num_groups=self.groups,
                          keep_groups=self.keep, route_scale=float(getattr(s, "route_scale", 1.0)),
                          shared_gate_up=self.w_shared_gate_up, shared_down=self.w_shared_down,
                          shared_limit=float(getattr(s, "shared_limit", 0.0)), identity_experts=self.identity, correction=self.correction,
                          shared_gated=self.shared_gated, gated=self.gated)


FEED_FORWARDS.register("routed_experts", RoutedExperts)
