"""Arrangements of a mixer, a feed-forward and their norms into one residual block.

``pre_norm`` (reference: ``src/mini_engine/model.py:142-151``)::

    x = x + mixer(norm1(x));  x = x + ffn(norm2(x))

``parallel``::

    h = norm1(x);  x = x + scale * (mixer(h) + ffn(h))

one norm that both parts read; ``scale`` is the layer spec's ``residual_scale``; the feed-forward may be absent. With a
norm of its own for the feed-forward (both norms of the same x)::

    x = x + scale * (mixer(norm1(x)) + ffn(norm2(x)))

``result_norm``: the norms sit on the sublayers' results and what a sublayer takes in is the stream as it stands::

    x = x + norm1(mixer(x));  x = x + norm2(ffn(x))

optionally followed by an input from the token itself (``token_input`` of the layer spec): with e a slice of the token's row of a
table, ``y = W_proj (act(W_gate x) * e)`` and ``x = x + norm(y)``.

The residual stream ``x`` is kept in float32 and every sum into it is a float32 sum. A block returns
its feed-forward output unadded; the next norm kernel (of the next block, or the model's final norm)
adds it while it norms, so each residual add costs no pass of its own.
"""

from __future__ import annotations

import torch

from .base import BLOCK_ARRANGEMENTS, FEED_FORWARDS, MIXERS, NORMS


class PreNormBlock:
    def __init__(self, spec, dtype: torch.dtype, device: torch.device):
        self.spec, self.dtype = spec, dtype
        self.mixer = MIXERS.build(spec.mixer, dtype, device)
        self.ffn = FEED_FORWARDS.build(spec.ffn, dtype, device)
        self.mixer_norm = NORMS.build(spec.mixer_norm, dtype, device)
        self.ffn_norm = NORMS.build(spec.ffn_norm, dtype, device)

    def weight_wants(self):
        s = self.spec
        wants = {}
        wants.update(self.mixer_norm.weight_wants(s.mixer_norm_name))
        wants.update(self.mixer.weight_wants(s.mixer_prefix))
        wants.update(self.ffn_norm.weight_wants(s.ffn_norm_name))
        wants.update(self.ffn.weight_wants(s.ffn_prefix))
        return wants

    def load(self, tensors) -> None:
        s = self.spec
        self.mixer_norm.load(tensors, s.mixer_norm_name)
        self.mixer.load(tensors, s.mixer_prefix)
        self.ffn_norm.load(tensors, s.ffn_norm_name)
        self.ffn.load(tensors, s.ffn_prefix)

    # ---- the native step program
    def emit(self, program, cache=None) -> None:
        """Write the block into a step program. A part with ``emit`` writes its own operations; any other part, and
        any norm that is not RMS-shaped, enters as a call of its ``forward``."""
        for part, norm, extra in ((self.mixer, self.mixer_norm, (cache,)), (self.ffn, self.ffn_norm, ())):
            with program.scope():
                h = program.normed(norm) if norm.as_fused() is not None else program.normed_by(norm)
                if callable(getattr(part, "emit", None)):
                    out = part.emit(program, h, *extra)
                else:
                    out = program.call_part(part, h, extra)
                if not h.used:  # the part never looked at its input: the add still has to happen
                    h.value()
                if out is not None:
                    program.delta(out)


class ParallelBlock:
    """One norm; the mixer and the feed-forward both read its output; their sum, times the spec's ``residual_scale``,
    is added to the stream. The mixer's result is set aside while the feed-forward runs (it reads the normed
    activations, not the stream); the next norm adds both results, scaled, while it norms."""

    def __init__(self, spec, dtype: torch.dtype, device: torch.device):
        self.spec, self.dtype = spec, dtype
        self.mixer = MIXERS.build(spec.mixer, dtype, device)
        self.ffn = None if spec.ffn is None else FEED_FORWARDS.build(spec.ffn, dtype, device)
        self.mixer_norm = NORMS.build(spec.mixer_norm, dtype, device)
        # a norm of its own for the feed-forward, of the same stream (None: both parts read the one norm)
        self.ffn_norm = None if self.ffn is None or spec.ffn_norm is None else NORMS.build(spec.ffn_norm, dtype, device)
        if self.ffn_norm is not None and self.ffn_norm.as_fused() is None:
            raise ValueError("the feed-forward's own norm in a parallel block is RMS-shaped")
        self.scale = float(spec.residual_scale)

    def weight_wants(self):
        s = self.spec
        wants = {}
        wants.update(self.mixer_norm.weight_wants(s.mixer_norm_name))
        wants.update(self.mixer.weight_wants(s.mixer_prefix))
        if self.ffn is not None:
            if self.ffn_norm is not None:
                wants.update(self.ffn_norm.weight_wants(s.ffn_norm_name))
            wants.update(self.ffn.weight_wants(s.ffn_prefix))
        return wants

    def load(self, tensors) -> None:
        s = self.spec
        self.mixer_norm.load(tensors, s.mixer_norm_name)
        self.mixer.load(tensors, s.mixer_prefix)
        if self.ffn is not None:
            if self.ffn_norm is not None:
                self.ffn_norm.load(tensors, s.ffn_norm_name)
            self.ffn.load(tensors, s.ffn_prefix)

    def emit(self, program, cache=None) -> None:
        parts = [(self.mixer, (cache,))] + ([(self.ffn, ())] if self.ffn is not None else [])
        norm = self.mixer_norm
        with program.scope():
            h = program.normed(norm) if norm.as_fused() is not None else program.normed_by(norm)
            h.value()  # the normed activations as a value of their own: two parts read them
            before, program.delta_scale = program.delta_scale, self.scale
            stays_before = program.delta_stays
            try:
                for at, (part, extra) in enumerate(parts):
                    # a second norm reads the stream as the first did: the mixer's result may not add itself into it on the way
                    program.delta_stays = stays_before or (at == 0 and self.ffn_norm is not None)
                    if at == 1 and self.ffn_norm is not None:  # the feed-forward's own norm of the same stream
                        h = program.normed_again(self.ffn_norm)
                    if callable(getattr(part, "emit", None)):
                        out = part.emit(program, h, *extra)
                    else:
                        out = program.call_part(part, h, extra)
                    if out is not None:
                        program.delta(out)
                    if at + 1 < len(parts):
                        program.hold()  # set aside: the next norm's kernel adds it together with the last part's result
            finally:
                program.delta_scale = before
                program.delta_stays = stays_before


class HyperConnectionBlock:
    """The pre-norm arrangement over several residual streams (hyper-connections). A part (the mixer, then the feed-forward,
    which may be absent) reads ``u = sum_s in[s] x_s``, gives ``y = part(norm(u))``, and all streams are rewritten at once
    from the old ones: ``x_t = sum_s mix[s, t] x_s + out[t] y``. The coefficients are tensors of the checkpoint (the layer
    spec's ``mixer_streams`` / ``ffn_streams`` name them), kept in float32. The rewrite rides on the kernel that reads and
    norms the next part's input, as the single stream's add rides on its next norm."""

    def __init__(self, spec, dtype: torch.dtype, device: torch.device):
        self.spec, self.dtype = spec, dtype
        self.mixer = MIXERS.build(spec.mixer, dtype, device)
        self.ffn = None if spec.ffn is None else FEED_FORWARDS.build(spec.ffn, dtype, device)
        self.mixer_norm = NORMS.build(spec.mixer_norm, dtype, device)
        self.ffn_norm = None if spec.ffn is None else NORMS.build(spec.ffn_norm, dtype, device)
        if spec.mixer_streams is None or (self.ffn is not None and spec.ffn_streams is None):
            raise ValueError("every part of a hyper-connection block needs its stream coefficients")
        for norm in (self.mixer_norm, self.ffn_norm):
            if norm is not None and (norm.as_fused() is None or getattr(norm, "groups", 1) != 1):
                raise ValueError("the parts of a hyper-connection block are normed by an RMS norm without groups")
        self.reads: dict[str, torch.Tensor] = {}
        self.rewrites: dict[str, torch.Tensor] = {}

    def _ties(self):
        s = self.spec
        return [s.mixer_streams] + ([s.ffn_streams] if self.ffn is not None else [])

    def weight_wants(self):
        from ..weights.loader import TensorWant

        s = self.spec
        wants = {}
        wants.update(self.mixer_norm.weight_wants(s.mixer_norm_name))
        wants.update(self.mixer.weight_wants(s.mixer_prefix))
        if self.ffn is not None:
            wants.update(self.ffn_norm.weight_wants(s.ffn_norm_name))
            wants.update(self.ffn.weight_wants(s.ffn_prefix))
        for tie in self._ties():
            n = int(tie.streams)
            wants[f"{tie.prefix}.in"] = TensorWant((n,), "vector")
            wants[f"{tie.prefix}.out"] = TensorWant((n,), "vector")
            wants[f"{tie.prefix}.mix"] = TensorWant((n, n), "vector")
        return wants

    def load(self, tensors) -> None:
        s = self.spec
        self.mixer_norm.load(tensors, s.mixer_norm_name)
        self.mixer.load(tensors, s.mixer_prefix)
        if self.ffn is not None:
            self.ffn_norm.load(tensors, s.ffn_norm_name)
            self.ffn.load(tensors, s.ffn_prefix)
        for tie in self._ties():
            self.reads[tie.prefix] = tensors[f"{tie.prefix}.in"].contiguous()
            # mix[from, to] row by row, then out[to]: what the kernel that rewrites the streams reads
            self.rewrites[tie.prefix] = torch.cat((tensors[f"{tie.prefix}.mix"].reshape(-1), tensors[f"{tie.prefix}.out"])).contiguous()

    def emit(self, program, cache=None) -> None:
        s = self.spec
        parts = [(self.mixer, self.mixer_norm, s.mixer_streams, (cache,))]
        if self.ffn is not None:
            parts.append((self.ffn, self.ffn_norm, s.ffn_streams, ()))
        for part, norm, tie, extra in parts:
            if int(tie.streams) != program.num_streams:
                raise ValueError(f"a block of {tie.streams} streams in a model of {program.num_streams}")
            with program.scope():
                h = program.stream_normed(norm, self.reads[tie.prefix])
                if callable(getattr(part, "emit", None)):
                    out = part.emit(program, h, *extra)
                else:
                    out = program.call(lambda frame, part=part, extra=extra: frame.write(part.forward(frame.input, frame.batch, *extra)),
                                       in_=h.value(), out_cols=program.hidden)
                if not h.used:  # the part never looked at its input: the streams' rewrite still has to happen
                    h.value()
                if out is not None:
                    program.delta(out)
                program.rewrites_streams(self.rewrites[tie.prefix])


class ResultNormBlock:
    """``x += norm1(mixer(x)); x += norm2(ffn(x))``: RMS norms on the sublayers' results. A sublayer reads the stream in the compute
    dtype; its result waits (a tensor, or float32 partial sums) for one kernel that adds the sums up, norms them, adds the normed row
    to the float32 stream and writes the stream in the compute dtype for the next sublayer: what the add-and-norm kernel is to a
    pre-norm block. The feed-forward may be absent. With a ``token_input`` a third sublayer of the same shape follows: a small product
    of the stream, an activation times a slice of the token's row of a table, a product back, its norm."""

    def __init__(self, spec, dtype: torch.dtype, device: torch.device):
        self.spec, self.dtype = spec, dtype
        self.mixer = MIXERS.build(spec.mixer, dtype, device)
        self.ffn = None if spec.ffn is None else FEED_FORWARDS.build(spec.ffn, dtype, device)
        self.mixer_norm = NORMS.build(spec.mixer_norm, dtype, device)
        self.ffn_norm = None if spec.ffn is None else NORMS.build(spec.ffn_norm, dtype, device)
        for norm in (self.mixer_norm, self.ffn_norm):
            if norm is not None and (norm.as_fused() is None or getattr(norm, "groups", 1) != 1):
                raise ValueError("a sublayer's result is normed by an RMS norm without groups")
        self.token_input = getattr(spec, "token_input", None)
        self.token_norm = None
        if self.token_input is not None:
            from ..config.specs import NormSpec
            from ..ops.kernels import UNGATED_ACTIVATIONS

            ti = self.token_input
            if ti.activation not in UNGATED_ACTIVATIONS:
                raise ValueError(f"a token input knows the activations {sorted(UNGATED_ACTIVATIONS)}, got {ti.activation!r}")
            if ti.dim < 1 or ti.index < 0:
                raise ValueError(f"a token input reads {ti.dim} elements at index {ti.index}")
            self.hidden = int(spec.mixer_norm.dim)
            self.token_norm = NORMS.build(NormSpec(dim=self.hidden, eps=float(ti.eps)), dtype, device)
            names = dict(getattr(ti, "names", ()) or ())
            self._tn = {r: names.get(r, r) for r in ("gate", "proj", "norm")}
        self.token_table = self.token_gate = self.token_proj = None
        self.table_columns = 0

    def weight_wants(self):
        s = self.spec
        wants = {}
        wants.update(self.mixer_norm.weight_wants(s.mixer_norm_name))
        wants.update(self.mixer.weight_wants(s.mixer_prefix))
        if self.ffn is not None:
            wants.update(self.ffn_norm.weight_wants(s.ffn_norm_name))
            wants.update(self.ffn.weight_wants(s.ffn_prefix))
        return wants

    def token_wants(self, vocab: int, table_columns: int):
        """The tensors of the token input; the table is the model's, ``[vocab, table_columns]``, and every layer names it."""
        from ..weights.loader import TensorWant

        ti = self.token_input
        if ti is None:
            return {}
        if (ti.index + 1) * ti.dim > table_columns:
            raise ValueError(f"a token input reads the columns {ti.index * ti.dim} .. {(ti.index + 1) * ti.dim - 1} of a table of {table_columns}")
        wants = {ti.table_name: TensorWant((vocab, table_columns)),
                 f"{ti.prefix}.{self._tn['gate']}": TensorWant((ti.dim, self.hidden)),
                 f"{ti.prefix}.{self._tn['proj']}": TensorWant((self.hidden, ti.dim))}
        wants.update(self.token_norm.weight_wants(f"{ti.prefix}.{self._tn['norm']}"))
        return wants

    def load(self, tensors) -> None:
        s = self.spec
        self.mixer_norm.load(tensors, s.mixer_norm_name)
        self.mixer.load(tensors, s.mixer_prefix)
        if self.ffn is not None:
            self.ffn_norm.load(tensors, s.ffn_norm_name)
            self.ffn.load(tensors, s.ffn_prefix)
        ti = self.token_input
        if ti is not None:
            self.token_table = tensors[ti.table_name]
            self.token_gate = tensors[f"{ti.prefix}.{self._tn['gate']}"]
            self.token_proj = tensors[f"{ti.prefix}.{self._tn['proj']}"]
            self.token_norm.load(tensors, f"{ti.prefix}.{self._tn['norm']}")

    def emit(self, program, cache=None) -> None:
        before, program.delta_stays = program.delta_stays, True  # no product adds itself into the stream: its result is normed first
        try:
            h = program.stream_value if program.stream_value is not None else program.result_normed(None)
            sublayers = [(self.mixer, self.mixer_norm, (cache,))]
            if self.ffn is not None:
                sublayers.append((self.ffn, self.ffn_norm, ()))
            for part, norm, extra in sublayers:
                with program.scope():
                    from ..engine.program import NormedValue

                    if callable(getattr(part, "emit", None)):
                        out = part.emit(program, NormedValue(h), *extra)
                    else:
                        out = program.call_part(part, NormedValue(h), extra)
                    if out is not None:
                        program.delta(out)
                    h = program.result_normed(norm)
            if self.token_input is not None:
                ti = self.token_input
                with program.scope():
                    z = program.linear(h, self.token_gate)
                    g = program.token_gate(z, self.token_table, ti.index * ti.dim, ti.activation)
                    program.linear_delta(g, self.token_proj)
                    h = program.result_normed(self.token_norm)
        finally:
            program.delta_stays = before


BLOCK_ARRANGEMENTS.register("pre_norm", PreNormBlock)
BLOCK_ARRANGEMENTS.register("result_norm", ResultNormBlock)
BLOCK_ARRANGEMENTS.register("parallel", ParallelBlock)
BLOCK_ARRANGEMENTS.register("hyper_connections", HyperConnectionBlock)


def build_block(spec, dtype, device):
    return BLOCK_ARRANGEMENTS.build(spec, dtype, device)
