"""Linear attention with a decay per token, head and key channel and a bonus for the current token (the spec:
:class:`~mini_engine_amd.config.specs.TimeMixSpec`): a ``head_dim x head_dim`` float32 state per request and head,

    o_t = (S_(t-1) + diag(u) k_t v_t^T)^T r_t,        S_t = diag(w_t) S_(t-1) + k_t v_t^T

Each of r, k, v, the gate and the decay reads its own blend of the token's input and the input of the token before it, so the
mixer makes its five products itself, from the sublayer's input (it takes no share of a stacked product of a pair). The state
row of a request holds S and, behind it, the input of its last token.
"""

from __future__ import annotations

import torch

from ..weights.loader import TensorWant
from .base import MIXERS, Mixer, StateBinding, StateNeed

MAX_HEAD_DIM = 256  # csrc/time_mix.hip: the scan's widest instance
MAX_DECAY_RANK = 1024  # TM_MAX_RANK
BLENDS = ("r", "k", "v", "g", "w")  # the order of the rows of mu


class TimeMix(Mixer):
    graph_safe = True
    reads_input = True  # in a pair of mixers: it is handed the sublayer's input beside its (empty) columns of the stacked product

    def __init__(self, spec, dtype, device):
        super().__init__(spec, dtype, device)
        s = spec
        if not (1 <= s.head_dim <= MAX_HEAD_DIM and 1 <= s.num_heads <= 65535 and 1 <= s.decay_rank <= MAX_DECAY_RANK):
            raise ValueError(f"time_mix takes heads of up to {MAX_HEAD_DIM} elements and a decay of inner size up to {MAX_DECAY_RANK}, "
                             f"got {s.num_heads} heads of {s.head_dim}, inner size {s.decay_rank}")
        self.h, self.d, self.rank = int(s.num_heads), int(s.head_dim), int(s.decay_rank)
        names = dict(getattr(s, "names", ()) or ())
        roles = tuple(f"mu_{b}" for b in BLENDS) + ("r", "k", "v", "g", "w1", "w2", "w0", "u", "norm", "o")
        self._n = {r: names.get(r, r) for r in roles}
        self.w_in = self.w_o = self.mu = self.w_rkvg = self.w1 = self.w2 = self.w0 = self.bonus = self.norm_w = self.w_all = None

    # ---- weights
    def weight_wants(self, prefix: str) -> dict[str, TensorWant]:
        s, n, hd = self.spec, self._n, self.h * self.d
        wants = {f"{prefix}.{n[r]}": TensorWant((hd, s.hidden_size)) for r in ("r", "k", "v", "g")}
        for b in BLENDS:
            wants[f"{prefix}.{n['mu_' + b]}"] = TensorWant((s.hidden_size,), "vector")
        wants[f"{prefix}.{n['w1']}"] = TensorWant((self.rank, s.hidden_size))
        wants[f"{prefix}.{n['w2']}"] = TensorWant((hd, self.rank))
        wants[f"{prefix}.{n['o']}"] = TensorWant((s.hidden_size, hd))
        wants[f"{prefix}.{n['u']}"] = TensorWant((self.h, self.d), "vector")
        for r in ("w0", "norm"):
            wants[f"{prefix}.{n[r]}"] = TensorWant((hd,), "vector")
        return wants

    def load(self, tensors, prefix: str) -> None:
        n = self._n
        self.mu = torch.stack([tensors[f"{prefix}.{n['mu_' + b]}"] for b in BLENDS]).contiguous()
        self.w_rkvg = tuple(tensors[f"{prefix}.{n[r]}"].contiguous() for r in ("r", "k", "v", "g"))
        self.w1 = tensors[f"{prefix}.{n['w1']}"].contiguous()
        # the five weights behind each other, for steps of few tokens (one product of five rows a token)
        self.w_all = torch.cat((*self.w_rkvg, self.w1), dim=0).contiguous()
        self.w2 = tensors[f"{prefix}.{n['w2']}"].contiguous()
        self.w_o = tensors[f"{prefix}.{n['o']}"]
        self.w0, self.norm_w = (tensors[f"{prefix}.{n[r]}"] for r in ("w0", "norm"))
        self.bonus = tensors[f"{prefix}.{n['u']}"].reshape(-1).contiguous()
        # (in a pair of mixers: no rows of the stacked input product are this mixer's)
        self.w_in = torch.zeros((0, self.spec.hidden_size), dtype=self.w_o.dtype, device=self.w_o.device)

    # ---- state
    def cache_need(self):
        return StateNeed((self.h * self.d * self.d + int(self.spec.hidden_size),), torch.float32)

    # ---- what a pair of mixers asks of each of them
    @property
    def input_cols(self) -> int:
        return 0

    @property
    def output_cols(self) -> int:
        return self.h * self.d

    def emit_projected(self, program, proj: int, col: int, out: int, out_col: int, out_scale: float, cache, h: int | None = None) -> None:
        """The mixer up to its output product: it reads the sublayer's input ``h`` (a value), the result goes to the value ``out`` at
        column ``out_col``, times ``out_scale``."""
        if not isinstance(cache, StateBinding):
            raise RuntimeError("time_mix mixer was given no state")
        if h is None:
            raise RuntimeError("time_mix reads the sublayer's input")
        program.time_mix(h, out, out_col=out_col, mu=self.mu, w_rkvg=self.w_rkvg, w1=self.w1, w2=self.w2, w0=self.w0, bonus=self.bonus,
                         norm_weight=self.norm_w, state=cache.state, heads=self.h, head_dim=self.d, eps=float(self.spec.norm_eps),
                         out_scale=out_scale, w_all=self.w_all)

    # ---- step
    def forward(self, h, batch, cache=None):
        raise NotImplementedError("time mixing runs in the step program only")

    def emit(self, program, h, cache: StateBinding | None = None) -> None:
        out = program.take(self.output_cols)
        self.emit_projected(program, -1, 0, out, 0, 1.0, cache, h=h.value() if hasattr(h, "value") else h)
        program.linear_delta(out, self.w_o)


MIXERS.register("time_mix", TimeMix)
