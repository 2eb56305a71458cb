"""Dense gated feed-forward: ``down(act(gate(x)) * up(x))`` without biases
(reference: ``src/mini_engine/model.py:122-131``). Gate and up weights are stacked at load time so
that one product feeds the activation, which is the epilogue of that product where a kernel of this
package computes it (silu as in the reference, or the tanh form of gelu)."""

from __future__ import annotations

import torch

from ..ops import kernels as K
from ..weights.loader import TensorWant
from .base import FEED_FORWARDS, FeedForward


class GatedMlp(FeedForward):
    graph_safe = True

    def __init__(self, spec, dtype, device):
        super().__init__(spec, dtype, device)
        if spec.activation not in K.GATE_ACTIVATIONS:
            raise ValueError(f"gated_mlp knows the activations {sorted(K.GATE_ACTIVATIONS)}, got {spec.activation!r}")
        self.w_gate_up = self.w_down = None
        names = dict(getattr(spec, "names", ()) or ())
        self._gate, self._up, self._down = (names.get(r, d) for r, d in (("gate", "gate_proj.weight"), ("up", "up_proj.weight"),
                                                                         ("down", "down_proj.weight")))

    def weight_wants(self, prefix: str) -> dict[str, TensorWant]:
        s = self.spec
        return {
            f"{prefix}.{self._gate}": TensorWant((s.intermediate_size, s.hidden_size)),
            f"{prefix}.{self._up}": TensorWant((s.intermediate_size, s.hidden_size)),
            f"{prefix}.{self._down}": TensorWant((s.hidden_size, s.intermediate_size)),
        }

    def load(self, tensors, prefix: str) -> None:
        self.w_gate_up = torch.cat((tensors[f"{prefix}.{self._gate}"], tensors[f"{prefix}.{self._up}"]), dim=0)
        self.w_down = tensors[f"{prefix}.{self._down}"]

    takes_normed_input = True

    def forward(self, h, batch=None) -> torch.Tensor:
        act = K.linear(h, self.w_gate_up, gated=self.spec.activation)
        return K.linear(act, self.w_down, as_delta=True)

    def emit(self, program, h) -> None:
        act = program.linear(h, self.w_gate_up, gated=self.spec.activation)
        program.linear_delta(act, self.w_down)


class ActivatedMlp(FeedForward):
    """Dense feed-forward without a gate, ``down(act(up(x)))``: a product, the activation as a pass of its own, a product."""

    graph_safe = True

    def __init__(self, spec, dtype, device):
        super().__init__(spec, dtype, device)
        if spec.activation not in K.UNGATED_ACTIVATIONS:
            raise ValueError(f"activated_mlp knows the activations {sorted(K.UNGATED_ACTIVATIONS)}, got {spec.activation!r}")
        names = dict(getattr(spec, "names", ()) or ())
        self._up, self._down = names.get("up", "up_proj.weight"), names.get("down", "down_proj.weight")
        self.w_up = self.w_down = None

    def weight_wants(self, prefix: str) -> dict[str, TensorWant]:
        s = self.spec
        return {f"{prefix}.{self._up}": TensorWant((s.intermediate_size, s.hidden_size)),
                f"{prefix}.{self._down}": TensorWant((s.hidden_size, s.intermediate_size))}

    def load(self, tensors, prefix: str) -> None:
        self.w_up, self.w_down = tensors[f"{prefix}.{self._up}"], tensors[f"{prefix}.{self._down}"]

    def forward(self, h, batch=None):
        raise NotImplementedError("the ungated feed-forward runs in the step program only")

    def emit(self, program, h) -> None:
        act = program.activate(program.linear(h, self.w_up), self.spec.activation)
        program.linear_delta(act, self.w_down)


FEED_FORWARDS.register("gated_mlp", GatedMlp)
FEED_FORWARDS.register("activated_mlp", ActivatedMlp)
