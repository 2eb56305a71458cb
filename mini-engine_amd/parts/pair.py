"""Two mixers side by side: both read the same normed input, and the result is ``left_scale * left + right_scale * right``.

Each of the two is a mixer of its own kind with its own spec, tensors (under ``<prefix>.<left_name>`` and
``<prefix>.<right_name>``) and cache or state. The pair stacks their input weights into one product and their output weights,
side by side along k, into another: the two mixers read their projections at their columns of the first product's result and
write their results, each times its scale (in float32, before the rounding to the compute dtype), at their columns of the
second product's input. So the pair costs two products a layer, as one mixer does.

A mixer can stand in a pair when it has ``w_in`` (its stacked input weight), ``w_o``, ``input_cols``, ``output_cols`` and
``emit_projected(program, proj, col, out, out_col, out_scale, cache)``. A mixer whose projections do not all read the sublayer's
input as it is (``reads_input``) has no rows in the stacked product and is handed the input itself, as the keyword ``h``.
"""

from __future__ import annotations

import torch

from .base import MIXERS, Mixer, PairBinding


class PairMixer(Mixer):
    def __init__(self, spec, dtype, device):
        super().__init__(spec, dtype, device)
        self.left = MIXERS.build(spec.left, dtype, device)
        self.right = MIXERS.build(spec.right, dtype, device)
        for m in (self.left, self.right):
            if not callable(getattr(m, "emit_projected", None)):
                raise ValueError(f"a {getattr(m.spec, 'kind', type(m).__name__)!r} mixer cannot stand in a pair: it has no emit_projected")
        self.w_in = self.w_o = None

    @property
    def graph_safe(self):
        return bool(self.left.graph_safe and self.right.graph_safe)

    def _prefixes(self, prefix: str):
        return f"{prefix}.{self.spec.left_name}", f"{prefix}.{self.spec.right_name}"

    def weight_wants(self, prefix: str):
        lp, rp = self._prefixes(prefix)
        wants = dict(self.left.weight_wants(lp))
        wants.update(self.right.weight_wants(rp))
        return wants

    def load(self, tensors, prefix: str) -> None:
        lp, rp = self._prefixes(prefix)
        self.left.load(tensors, lp)
        self.right.load(tensors, rp)
        self.w_in = torch.cat((self.left.w_in, self.right.w_in), dim=0)
        self.w_o = torch.cat((self.left.w_o, self.right.w_o), dim=1).contiguous()
        for m in (self.left, self.right):  # the stacked copies serve both
            m.w_in = m.w_o = None

    def cache_need(self):
        return (self.left.cache_need(), self.right.cache_need())

    def forward(self, h, batch, cache=None):
        raise NotImplementedError("a pair of mixers runs in the step program only")

    def emit(self, program, h, cache: PairBinding | None = None) -> None:
        if not isinstance(cache, PairBinding):
            raise RuntimeError("a pair of mixers was given no pair of bindings")
        s = self.spec
        sides = ((self.left, 0, 0, float(s.left_scale), cache.left),
                 (self.right, self.left.input_cols, self.left.output_cols, float(s.right_scale), cache.right))
        reads = any(getattr(m, "reads_input", False) for m in (self.left, self.right))
        hv = h.value() if reads and hasattr(h, "value") else h  # (the input as a value of its own, where a mixer reads it itself)
        proj = program.linear(h, self.w_in)
        out = program.take(self.left.output_cols + self.right.output_cols)
        for m, col, out_col, scale, binding in sides:
            extra = {"h": hv} if getattr(m, "reads_input", False) else {}
            m.emit_projected(program, proj, col, out, out_col, scale, binding, **extra)
        program.linear_delta(out, self.w_o)


MIXERS.register("pair", PairMixer)
