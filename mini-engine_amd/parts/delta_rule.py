"""Linear attention by the generalized delta rule, with a matrix of state per request and head.

Per head, with r, k, v of ``head_dim`` elements and the unit key ``u = k / sqrt(sum(k^2) + 1e-6)``::

    S_t = diag(w_t) S_(t-1) - (a_t * u_t) (u_t^T S_(t-1)) + k_t v_t^T,     o_t = S_t^T r_t

where both terms read the old state, ``w_t = exp(-decay_coef * sigmoid(W_2 tanh(W_1 h_t) + w_0))`` is a decay per head and key
channel and ``a_t = sigmoid(W_a h_t + b_a)`` a removal rate. ``S`` starts at zero, is float32, and lives in the request's state
slot between steps. One product gives r, k, v, the gate, a and the decay's inner projection (the six weights are stacked at
load time); the kernel of ``csrc/delta_rule.hip`` does everything behind it in float32: the sigmoids and exponentials, the
unit key, the walk over the new tokens from the state, the norm of each head's output over its root mean square, the weight
over all heads and the sigmoid of the gate. The output projection follows. Sizes, eps and the decay's coefficient come from the
spec.

The mixer can stand beside another one (:mod:`.pair`): it then reads its projections at a column of a wider product and
writes its result, scaled, at a column of a wider value, and the pair does both products.
"""

from __future__ import annotations

import torch

from ..weights.loader import TensorWant
from .base import MIXERS, Mixer, StateBinding, StateNeed

MAX_HEAD_DIM = 256  # csrc/delta_rule.hip: DR_MAX_D
MAX_DECAY_RANK = 1024  # DR_MAX_LORA
INPUT_ROLES = ("r", "k", "v", "g", "a", "w1")  # the order of the stacked input weight's rows


class DeltaRule(Mixer):
    graph_safe = True

    def __init__(self, spec, dtype, device):
        super().__init__(spec, dtype, device)
        s = spec
        if not (1 <= s.head_dim <= MAX_HEAD_DIM and 1 <= s.num_heads <= 65535 and 1 <= s.decay_rank <= MAX_DECAY_RANK):
            raise ValueError(f"delta_rule takes heads of up to {MAX_HEAD_DIM} elements and a decay of inner size up to {MAX_DECAY_RANK}, "
                             f"got {s.num_heads} heads of {s.head_dim}, inner size {s.decay_rank}")
        self.h, self.d, self.rank = int(s.num_heads), int(s.head_dim), int(s.decay_rank)
        names = dict(getattr(s, "names", ()) or ())
        self._n = {r: names.get(r, r) for r in ("r", "k", "v", "g", "a", "a_bias", "w1", "w2", "w0", "norm", "o")}
        self.w_in = self.w_o = self.w2 = self.w0 = self.a_bias = self.norm_w = None

    # ---- weights
    def weight_wants(self, prefix: str) -> dict[str, TensorWant]:
        s, n, hd = self.spec, self._n, self.h * self.d
        wants = {f"{prefix}.{n[r]}": TensorWant((hd, s.hidden_size)) for r in ("r", "k", "v", "g", "a")}
        wants[f"{prefix}.{n['w1']}"] = TensorWant((self.rank, s.hidden_size))
        wants[f"{prefix}.{n['w2']}"] = TensorWant((hd, self.rank))
        wants[f"{prefix}.{n['o']}"] = TensorWant((s.hidden_size, hd))
        for r in ("a_bias", "w0", "norm"):
            wants[f"{prefix}.{n[r]}"] = TensorWant((hd,), "vector")
        return wants

    def load(self, tensors, prefix: str) -> None:
        n = self._n
        self.w_in = torch.cat([tensors[f"{prefix}.{n[r]}"] for r in INPUT_ROLES], dim=0)
        self.w_o = tensors[f"{prefix}.{n['o']}"]
        self.w2 = tensors[f"{prefix}.{n['w2']}"].contiguous()
        self.w0, self.a_bias, self.norm_w = (tensors[f"{prefix}.{n[r]}"] for r in ("w0", "a_bias", "norm"))

    # ---- state
    def cache_need(self):
        return StateNeed((self.h, self.d, self.d), torch.float32)

    # ---- what a pair of mixers asks of each of them
    @property
    def input_cols(self) -> int:
        return 5 * self.h * self.d + self.rank

    @property
    def output_cols(self) -> int:
        return self.h * self.d

    def emit_projected(self, program, proj: int, col: int, out: int, out_col: int, out_scale: float, cache) -> None:
        """The mixer between its two products: the projections lie in the value ``proj`` from column ``col`` on (the rows of
        ``w_in``), the result goes to the value ``out`` at column ``out_col``, times ``out_scale``."""
        if not isinstance(cache, StateBinding):
            raise RuntimeError("delta_rule mixer was given no state")
        hd = self.h * self.d
        cols = {role: col + i * hd for i, role in enumerate(INPUT_ROLES)}
        program.delta_rule(proj, out, cols=cols, out_col=out_col, decay_outer=self.w2, decay_bias=self.w0, rate_bias=self.a_bias,
                           norm_weight=self.norm_w, state=cache.state, heads=self.h, head_dim=self.d, decay_rank=self.rank,
                           eps=float(self.spec.norm_eps), decay_coef=float(self.spec.decay_coef), out_scale=out_scale)

    # ---- step
    def forward(self, h, batch, cache=None):
        raise NotImplementedError("the delta rule runs in the step program only")

    def emit(self, program, h, cache: StateBinding | None = None) -> None:
        proj = program.linear(h, self.w_in)
        out = program.take(self.output_cols)
        self.emit_projected(program, proj, 0, out, 0, 1.0, cache)
        program.linear_delta(out, self.w_o)


MIXERS.register("delta_rule", DeltaRule)
