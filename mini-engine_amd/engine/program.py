"""Python face of the native step program (``csrc/host/program.cpp``, ``csrc/host/runner.cpp``).

When a model is built, every part writes the operations of its forward pass into a
:class:`StepProgram` (a part's ``emit`` method; it says what the part computes, not which kernels
run). A step of the model then is one call into C++, which checks and packs the step that the
host core holds, uploads the indices, picks a kernel per operation for the step's size, launches
them all and draws the next tokens. A part that has no ``emit`` (a part defined outside the package,
with code of its own) enters the program as a *call*: the program hands its ``forward`` the step's
values as tensors when the step reaches it, so such a part, with or without state of its own, runs in
the same one pass as every other.

Values are ``[tokens, columns]`` buffers of a step; parts get them from the program and the program
hands a buffer out again once the scope that took it has ended, so a model of any depth needs the
buffers of one layer.
"""

from __future__ import annotations

import contextlib
import ctypes
import weakref

import numpy as np
import torch

from ..ops.library import lib

_vp, _i64, _i32 = ctypes.c_void_p, ctypes.c_int64, ctypes.c_int
_declared = False

(EMBED, NORM_LINEAR, NORM, LINEAR, LINEAR_DELTA, DELTA, ATTENTION, HEAD, SAMPLE, ADD, CALL, HEAD_ROWS, DECAY_STATE, HOLD, STREAMS,
 STREAM_NORM, STREAM_HEAD, LATENT_ATTENTION, ROUTED_FF, STREAM_NORM_LINEAR, POOLED_ATTENTION, DELTA_RULE, RESULT_NORM, TOKEN_GATE,
 ACTIVATE, TIME_MIX) = range(26)
ROUTER_SCORINGS = {"softmax_picked": 0, "sigmoid_normalized": 1, "softmax_all": 2}  # csrc/routed_ff.hip: RF_SCORE_*
OP_PTRS, OP_INTS, OP_FLOATS = 12, 16, 4  # csrc/host/program.h: kOpPtrs, kOpInts, kOpFloats
MAX_STREAMS = 8  # csrc/streams.hip: ME_MAX_STREAMS
_RAISES = {1: ValueError, 2: RuntimeError, 3: AssertionError}


class _RawFrame(ctypes.Structure):  # csrc/host/program.h: CallFrame
    _fields_ = [("context", _vp), ("in_", _vp), ("out", _vp), ("x", _vp), ("in_cols", _i64), ("out_cols", _i64),
                ("in_elem", _i32), ("out_elem", _i32), ("tokens", _i32), ("rows", _i32), ("stream", _vp)]


_CALL_FN = ctypes.CFUNCTYPE(ctypes.c_int, ctypes.POINTER(_RawFrame))


class Frame:
    """What a called part sees of the step that has reached it: its input and output values and the residual
    stream as tensors (views into the step's memory, valid during the call only) and the step's batch."""

    def __init__(self, program: "StepProgram", raw: _RawFrame):
        self.program, self.tokens, self.rows = program, int(raw.tokens), int(raw.rows)
        dtype_of = {2: torch.bfloat16, 4: torch.float32}
        arena = program.current_arena
        self.input = view_in(arena, raw.in_, (self.tokens, int(raw.in_cols)), dtype_of[raw.in_elem]) if raw.in_ else None
        self.output = view_in(arena, raw.out, (self.tokens, int(raw.out_cols)), dtype_of[raw.out_elem]) if raw.out else None
        self.x = view_in(arena, raw.x, (self.tokens, program.hidden), torch.float32)

    @property
    def batch(self):
        """The step's batch (:class:`~mini_engine_amd.engine.batch.StepBatch`), made once per step."""
        return self.program.current_batch()

    def write(self, result) -> None:
        """A part's result into the output value: a tensor ``[tokens, columns]``, or partial sums over runs of k."""
        from ..ops.kernels import PartialSums

        if isinstance(result, PartialSums):
            result = result.parts.sum(dim=0)
        if tuple(result.shape) != tuple(self.output.shape):
            raise ValueError(f"a part returned {tuple(result.shape)} where the step has {tuple(self.output.shape)}")
        self.output.copy_(result)


def _api():
    global _declared
    L = lib()
    if not _declared:
        L.me_runner_new.restype = _vp
        L.me_runner_new.argtypes = [_i32, _i32, _i32]
        L.me_runner_delete.argtypes = [_vp]
        L.me_runner_delete.restype = None
        L.me_runner_value.argtypes = [_vp, _i64, _i32]
        L.me_runner_op.argtypes = [_vp, _i32, _i32, _i32, _vp, _vp, _vp]
        L.me_runner_arena_need.restype = _i64
        L.me_runner_arena_need.argtypes = [_vp, _i64, _i64, _i64, _i64]
        L.me_runner_index_need.restype = _i64
        L.me_runner_index_need.argtypes = [_vp, _i32, _i32, _i32, _vp, _i32]
        L.me_runner_memory.argtypes = [_vp, _vp, _i64, _vp, _vp, _i64, _vp, _i64, _i32, _i32]
        L.me_runner_step.argtypes = [_vp, _vp, _vp, _vp]
        L.me_runner_static.argtypes = [_vp, _vp, _i64, _vp, _i32, _vp, _i32, _i32, _i32, _vp, _i32, _vp, _vp]
        _declared = True
    return L


def _ok(code: int) -> int:
    if code < 0:
        L = lib()
        raise _RAISES.get(L.me_runner_error_kind(), RuntimeError)(L.me_last_error().decode())
    return code


class Normed:
    """The residual add and the norm that a block owes before a part, not yet written into the
    program. The part's first product takes it as its input (the program then fuses add, norm and
    product where the step is small enough); ``value()`` gives the normed activations as a value of
    their own."""

    def __init__(self, program: "StepProgram", weight: torch.Tensor, eps: float, groups: int = 1):
        self.program, self.weight, self.eps, self.groups = program, weight, float(eps), int(groups)
        self.used = False
        self._value: int | None = None

    def value(self) -> int:
        if self._value is None:
            p = self.program
            self._value = p.take(p.hidden, p.elem)
            p.op(NORM, out=self._value, ptrs=[self.weight], ints=[self.groups], floats=[self.eps])
            p.pending_consumed()
            self.used = True
        return self._value


class CalledNorm:
    """As :class:`Normed`, for a norm that is no RMS norm: the residual add as a kernel of its own, then the norm
    part's ``forward`` on the residual stream. Parts get its value; nothing of it rides on their products."""

    def __init__(self, program: "StepProgram", norm):
        self.program, self.norm = program, norm
        self.used = False
        self._value: int | None = None

    def value(self) -> int:
        if self._value is None:
            p, norm = self.program, self.norm
            p.add()
            self._value = p.call(lambda frame: frame.output.copy_(norm.forward(frame.x)), out_cols=p.hidden)
            self.used = True
        return self._value


class StreamNormed:
    """As :class:`Normed`, over several residual streams: the pending rewrite of the streams, the read of the coming part's
    input and its norm, not yet written into the program. The part's first product takes it as its input (the program then
    puts all of it into that product's kernel where the step is small enough); ``value()`` gives the normed input as a value
    of its own."""

    def __init__(self, program: "StepProgram", weight: torch.Tensor, eps: float, reads: torch.Tensor, rewrite: torch.Tensor | None):
        self.program, self.weight, self.eps, self.reads, self.rewrite = program, weight, float(eps), reads, rewrite
        self.used = False
        self._value: int | None = None

    def value(self) -> int:
        if self._value is None:
            p = self.program
            self._value = p.take(p.hidden, p.elem)
            p.op(STREAM_NORM, out=self._value, ptrs=[self.weight, self.rewrite, self.reads], floats=[self.eps])
            p.pending_consumed()
            self.used = True
        return self._value


class NormedValue:
    """Normed activations that are a value already, with the face of :class:`Normed`."""

    def __init__(self, value: int):
        self._value, self.used = value, True

    def value(self) -> int:
        return self._value


class StepProgram:
    def __init__(self, dtype: torch.dtype, hidden: int, vocab: int, max_positions: int):
        self._L = _api()
        self.dtype, self.hidden, self.vocab, self.max_positions = dtype, int(hidden), int(vocab), int(max_positions)
        self.elem = 4 if dtype is torch.float32 else 2
        handle = self._L.me_runner_new(0 if dtype is torch.float32 else 1, self.hidden, self.vocab)
        if not handle:
            raise RuntimeError(lib().me_last_error().decode())
        self.handle = _vp(handle)
        self._keep: list[torch.Tensor] = []  # every tensor whose address an operation holds
        self._free: dict[tuple[int, int], list[int]] = {}
        self._value_kinds: list[tuple[int, int]] = []
        self._scopes: list[list[int]] = []
        self._pending_value: int | None = None
        self._held_value: int | None = None  # the value of a delta that was set aside (hold)
        self.num_ops = 0
        self.delta_scale = 1.0  # what the block being written multiplies its parts' results by (set by the block)
        # a part's result must wait for the next add whatever the step's size: the block reads the stream once more before it
        # (no product adds itself into the stream)
        self.delta_stays = False
        self.num_streams = 0  # residual streams of a token (0: the one plain stream)
        self._stream_rewrite: torch.Tensor | None = None  # how the pending result rewrites the streams (mix, then out)
        self.draws = False
        # the residual stream in the compute dtype as the last norm of a sublayer's result left it (a value that no scope owns), for
        # blocks whose sublayers take in the stream as it stands
        self.stream_value: int | None = None
        self.last_prefill_columns = 0  # query columns of the prefill attention's blocks in the last eager step (0: none ran)
        # called parts: their C trampolines (kept alive), the memory and the batch of the step that is running,
        # and the exception a call raised (raised again once the step's call into C++ has come back)
        self._calls: list = []
        self.current_arena: torch.Tensor | None = None
        self.current_batch = lambda: None
        self.call_error: BaseException | None = None

    def __del__(self):
        handle, self.handle = getattr(self, "handle", None), None
        if handle:
            self._L.me_runner_delete(handle)

    # ------------------------------------------------------------------ values
    def take(self, cols: int, elem: int | None = None, scoped: bool = True) -> int:
        """A ``[tokens, cols]`` buffer (elements of the compute dtype unless ``elem`` bytes are asked for)
        that stays the caller's until the scope it was taken in ends (``scoped`` false: until the caller hands it back)."""
        key = (int(cols), int(elem or self.elem))
        pool = self._free.setdefault(key, [])
        if pool:
            v = pool.pop()
        else:
            v = _ok(self._L.me_runner_value(self.handle, key[0], key[1]))
            self._value_kinds.append(key)
        if self._scopes and scoped:
            self._scopes[-1].append(v)
        return v

    @contextlib.contextmanager
    def scope(self):
        """Values taken inside are handed out again afterwards; the one that holds the pending delta of
        the residual stream only once the next norm has added it."""
        self._scopes.append([])
        try:
            yield
        finally:
            for v in self._scopes.pop():
                if v != self._pending_value and v != self._held_value:
                    self._give_back(v)

    def _give_back(self, v: int) -> None:
        self._free[self._value_kinds[v]].append(v)

    def pending_consumed(self) -> None:
        for v in (self._pending_value, self._held_value):
            if v is not None and not any(v in s for s in self._scopes):
                self._give_back(v)
        self._pending_value = self._held_value = None

    # -------------------------------------------------------------- operations
    def op(self, kind: int, in_: int = -1, out: int = -1, ptrs=(), ints=(), floats=()) -> None:
        p = (ctypes.c_void_p * OP_PTRS)()
        for i, t in enumerate(ptrs):
            if t is not None:
                if not t.is_contiguous():
                    raise ValueError("a step program holds contiguous tensors only")
                self._keep.append(t)
                p[i] = t.data_ptr()
        iv = (ctypes.c_int64 * OP_INTS)(*[int(v) for v in ints])
        fv = (ctypes.c_float * OP_FLOATS)(*[float(v) for v in floats])
        self.num_ops = _ok(self._L.me_runner_op(self.handle, kind, in_, out, p, iv, fv))

    def embed(self, table: torch.Tensor, multiplier: float = 1.0) -> None:
        """The residual stream starts as the tokens' rows of ``table``, times ``multiplier``."""
        self._want(table, self.dtype, (self.vocab, self.hidden), "embedding table")
        self.op(EMBED, ptrs=[table], floats=[multiplier])

    def normed(self, norm) -> Normed:
        """The add-and-norm before a part, for a norm that is RMS-shaped (``norm.as_fused()`` gives its
        float32 weight and its eps)."""
        weight, eps = norm.as_fused()
        self._want(weight, torch.float32, (self.hidden,), "norm weight")
        return Normed(self, weight, eps, getattr(norm, "groups", 1))

    def linear(self, x, weight: torch.Tensor, gated: "bool | str" = False) -> int:
        """``x @ weight.T`` (``gated``, True or the name of an activation: ``act(gate) * up`` with the weight's
        rows being gate rows, then up rows) for a value or a :class:`Normed`; returns the value that holds
        the result."""
        from ..ops.kernels import gate_code

        gate = gate_code(gated)
        rows, k = weight.shape
        self._want(weight, self.dtype, None, "weight")
        if gated and rows % 2:
            raise ValueError("a gated product needs as many gate rows as up rows")
        out = self.take(rows // 2 if gated else rows)
        if isinstance(x, Normed) and x._value is None:
            if k != self.hidden:
                raise ValueError("a product behind the norm reads the hidden size")
            self.op(NORM_LINEAR, out=out, ptrs=[x.weight, weight], ints=[rows, k, gate, x.groups], floats=[x.eps])
            x.used = True
            self.pending_consumed()
            return out
        if isinstance(x, StreamNormed) and x._value is None:
            if k != self.hidden:
                raise ValueError("a product behind the norm reads the hidden size")
            self.op(STREAM_NORM_LINEAR, out=out, ptrs=[x.weight, weight, x.rewrite, x.reads], ints=[rows, k, gate], floats=[x.eps])
            x.used = True
            self.pending_consumed()
            return out
        src = x.value() if isinstance(x, (Normed, CalledNorm, StreamNormed, NormedValue)) else x
        if self._value_kinds[src][0] != k:
            raise ValueError(f"the weight reads {k} columns, the value has {self._value_kinds[src][0]}")
        self.op(LINEAR, in_=src, out=out, ptrs=[None, weight], ints=[rows, k, gate])
        return out

    def linear_delta(self, x: int, weight: torch.Tensor) -> None:
        """``x @ weight.T`` as the part's result: the delta that the next norm adds to the residual stream."""
        rows, k = weight.shape
        self._want(weight, self.dtype, (self.hidden, self._value_kinds[x][0]), "weight")
        out = self.take(rows)
        self.op(LINEAR_DELTA, in_=x, out=out, ptrs=[None, weight], ints=[rows, k, int(self.delta_stays)], floats=[self.delta_scale])
        self._pending_value = out

    def delta(self, x: int) -> None:
        """A value ``[tokens, hidden]`` in the compute dtype as the part's result."""
        if self._value_kinds[x] != (self.hidden, self.elem):
            raise ValueError("a part's result has the hidden size and the compute dtype")
        self.op(DELTA, in_=x, floats=[self.delta_scale])
        self._pending_value = x

    def attention(self, qkv: int, *, q_norm: torch.Tensor | None, k_norm: torch.Tensor | None, rope: torch.Tensor | None,
                  k_cache: torch.Tensor, v_cache: torch.Tensor, heads: int, kv_heads: int, head_dim: int, block_size: int,
                  window: int, writes: bool, group: int, eps: float, scale: float, value_dim: int | None = None,
                  keep_first: int = 0, pairing: int = 0, value_rope: torch.Tensor | None = None, value_pairing: int = 0,
                  query_temperature: tuple[float, int] | None = None, gated: bool = False) -> int:
        """Per-head q/k norm, rotation, page write and causal attention over the request's pages for a
        value ``[tokens, (heads + 2 kv_heads) head_dim]`` (``writes`` false: ``[tokens, heads head_dim]``,
        the pages are another layer's); returns the value ``[tokens, heads head_dim]``.

        ``value_dim``: the value heads' size where it is not ``head_dim`` (the input then ends in ``kv_heads``
        heads of that size and the result has ``heads * value_dim`` columns); ``keep_first``: the first keys that stay
        visible behind the window; ``pairing``: 0 pairs element j with j + r/2, 1 pairs 2j with 2j + 1;
        ``value_rope`` / ``value_pairing``: the table ``[positions, 2, value_dim / 2]`` that the values are turned by
        before they are cached and the outputs turned back by; ``query_temperature`` ``(coef, every)``: the query at position p
        is multiplied by ``1 + coef * ln(floor((p + 1) / every) + 1)``; ``gated``: the input ends in one more column per head,
        whose sigmoid multiplies the head's output."""
        dv = head_dim if value_dim is None else int(value_dim)
        cols = heads * head_dim + (kv_heads * (head_dim + dv) if writes else 0) + (heads if gated else 0)
        coef, every = (0.0, 0) if query_temperature is None else (float(query_temperature[0]), int(query_temperature[1]))
        if query_temperature is not None and every < 1:
            raise ValueError("a temperature on the queries grows every so many positions, at least every one")
        if self._value_kinds[qkv] != (cols, self.elem):
            raise ValueError(f"the attention's input has {self._value_kinds[qkv][0]} columns, not {cols}")
        rotary_dim = covers = 0
        if rope is not None:
            self._want(rope, torch.float32, None, "rotary table")
            rotary_dim, covers = 2 * rope.shape[2], rope.shape[0]
            if covers < self.max_positions:
                raise ValueError(f"the rotary table covers {covers} positions of {self.max_positions}")
        turned = 0
        if value_rope is not None:
            self._want(value_rope, torch.float32, None, "table of the values' angles")
            if 2 * value_rope.shape[2] != dv or value_rope.shape[0] < self.max_positions:
                raise ValueError(f"the values' table must cover {self.max_positions} positions and {dv} elements")
            turned = 1 + int(value_pairing)
        out = self.take(heads * dv)
        self.op(ATTENTION, in_=qkv, out=out, ptrs=[q_norm, k_norm, rope, k_cache, v_cache, value_rope],
                ints=[heads, kv_heads, head_dim, rotary_dim, block_size, window, int(writes), group, covers,
                      0 if dv == head_dim else dv, keep_first, pairing, turned, every, int(gated)],
                floats=[eps, scale, coef])
        return out

    def latent_attention(self, proj: int, *, latent_norm: torch.Tensor, rope: torch.Tensor, k_cache: torch.Tensor,
                         v_cache: torch.Tensor, key_map: torch.Tensor, value_map: torch.Tensor, sink: torch.Tensor | None,
                         heads: int, head_dim: int, rotary_dim: int, rank: int, value_dim: int, block_size: int, group: int,
                         eps: float, scale: float, writes: bool = True) -> int:
        """Attention over one cached latent per token for a value ``[tokens, heads (head_dim + rotary_dim) | rank + rotary_dim |
        heads]`` (queries; the latent projection and the key part that all heads share; a gate per head). ``key_map`` ``[heads,
        rank, head_dim]`` (the keys' map per head, transposed) and ``value_map`` ``[heads, value_dim, rank]`` in the compute
        dtype; ``sink`` float32 ``[heads]`` or None; pages of one key/value head with keys of ``rank + rotary_dim`` and values
        of ``rank`` elements. Returns the value ``[tokens, heads * value_dim]``, gated."""
        # (``writes`` false: the pages are another layer's; the rows hold no latent projection, ``[tokens, heads (head_dim + rotary_dim) | heads]``)
        cols = heads * (head_dim + rotary_dim) + (rank + rotary_dim if writes else 0) + heads
        if self._value_kinds[proj][0] < cols or self._value_kinds[proj][1] != self.elem:  # (columns of padding may follow)
            raise ValueError(f"the projections have {self._value_kinds[proj][0]} columns, not {cols}")
        self._want(latent_norm, torch.float32, (rank,), "weight of the latent's norm")
        self._want(rope, torch.float32, None, "rotary table")
        if 2 * rope.shape[2] != rotary_dim or rope.shape[0] < self.max_positions:
            raise ValueError(f"the rotary table must cover {self.max_positions} positions and {rotary_dim} elements")
        self._want(key_map, self.dtype, (heads, rank, head_dim), "the keys' map")
        self._want(value_map, self.dtype, (heads, value_dim, rank), "the values' map")
        if sink is not None:
            self._want(sink, torch.float32, (heads,), "sink")
        value_rows = int(v_cache.shape[2])  # the latent's rank, or the whole key's size (what the matrix-core kernels take)
        if (tuple(k_cache.shape[1:]) != (1, block_size, rank + rotary_dim) or tuple(v_cache.shape[1:]) != (1, value_rows, block_size)
                or value_rows not in (rank, rank + rotary_dim)):
            raise ValueError("a latent attention layer keeps pages of one head: keys of rank + rotary_dim, values of rank (or as many) elements")
        out = self.take(heads * value_dim)
        self.op(LATENT_ATTENTION, in_=proj, out=out, ptrs=[latent_norm, rope, k_cache, v_cache, key_map, value_map, sink],
                ints=[heads, head_dim, rotary_dim, rank, value_dim, block_size, group, rope.shape[0], value_rows, int(not writes)],
                floats=[eps, scale])
        return out

    def routed_ff(self, x: int, *, router: torch.Tensor, gate_up: torch.Tensor, down: torch.Tensor, top_k: int, activation: str,
                  activation_limit: float = 0.0, scoring: str = "softmax_picked", num_groups: int = 1, keep_groups: int = 1,
                  route_scale: float = 1.0, shared_gate_up: torch.Tensor | None = None, shared_down: torch.Tensor | None = None,
                  shared_limit: float = 0.0, identity_experts: int = 0, correction: torch.Tensor | None = None,
                  shared_gated: bool = True, gated: bool = True) -> None:
        """A feed-forward of routed experts on the value ``x`` as the part's result. ``router`` float32 ``[experts, hidden]``;
        ``gate_up`` ``[experts, 2 ff, hidden]`` (an expert's gate rows, then its up rows) and ``down`` ``[experts, hidden, ff]``
        in the compute dtype. ``scoring``, ``num_groups``, ``keep_groups``, ``route_scale``: how the picks are bounded and weighted
        (:class:`~mini_engine_amd.config.specs.RoutedExpertsSpec`). ``shared_gate_up`` ``[2 ff_s, hidden]`` and ``shared_down``
        ``[hidden, ff_s]``: an expert that every token uses; the router then has one more row behind the experts', the token's
        product with which, through a sigmoid, multiplies that expert's result."""
        from ..ops.kernels import UNGATED_ACTIVATIONS, gate_code

        # ``gated`` false (an activation of UNGATED_ACTIVATIONS): the experts have no gate, ``gate_up`` is ``[experts, ff, hidden]`` (up rows alone) and
        # ``shared_gate_up`` ``[ff_s, hidden]``. ``identity_experts``: that many router outputs behind the experts' stand for identity
        # experts (the token's input itself, times the weight); ``correction`` float32 ``[experts + identity_experts]`` is added to the
        # scores for the choice alone (scoring "softmax_all"). ``shared_gated`` false: nothing multiplies the shared expert's result.
        ungated = not gated
        if ungated and activation not in UNGATED_ACTIVATIONS:
            raise ValueError(f"experts without a gate know the activations {sorted(UNGATED_ACTIVATIONS)}, got {activation!r}")
        experts, two_ff, hidden = gate_up.shape
        if ungated:
            two_ff *= 2
        if self._value_kinds[x] != (self.hidden, self.elem) or hidden != self.hidden:
            raise ValueError("routed experts read the hidden size in the compute dtype")
        shared_ff = 0
        if shared_gate_up is not None:
            shared_ff = shared_gate_up.shape[0] if ungated else shared_gate_up.shape[0] // 2
            self._want(shared_gate_up, self.dtype, ((1 if ungated else 2) * shared_ff, hidden), "the shared expert's gate and up rows")
            self._want(shared_down, self.dtype, (hidden, shared_ff), "the shared expert's down rows")
            if ungated and shared_gated:
                raise ValueError("a shared expert without gate rows has no gate of its own either")
        if identity_experts < 0 or (identity_experts and scoring != "softmax_all"):
            raise ValueError("identity experts are picked by a router that scores by softmax_all")
        if correction is not None:
            self._want(correction, torch.float32, (experts + identity_experts,), "the scores' correction")
        self._want(router, torch.float32, (experts + identity_experts + (1 if shared_ff and shared_gated else 0), hidden), "router")
        self._want(gate_up, self.dtype, None, "experts' gate and up rows")
        self._want(down, self.dtype, (experts, hidden, two_ff // 2), "experts' down rows")
        if not 1 <= top_k <= experts + identity_experts:
            raise ValueError(f"{top_k} of {experts + identity_experts} experts a token")
        if scoring not in ROUTER_SCORINGS:
            raise ValueError(f"a router scores by one of {sorted(ROUTER_SCORINGS)}, not {scoring!r}")
        if num_groups < 1 or experts % num_groups or not 1 <= keep_groups <= num_groups or keep_groups * (experts // num_groups) + identity_experts < top_k:
            raise ValueError(f"{experts} experts in {num_groups} groups of which {keep_groups} are kept, {top_k} picks")
        code = UNGATED_ACTIVATIONS[activation] if ungated else gate_code(activation, limited=True)
        self.op(ROUTED_FF, in_=x, ptrs=[router, gate_up, down, shared_gate_up, shared_down, correction],
                ints=[experts, top_k, two_ff // 2, code, ROUTER_SCORINGS[scoring], num_groups, keep_groups, shared_ff, identity_experts,
                      int(not shared_gated)],
                floats=[activation_limit, route_scale, shared_limit, self.delta_scale])
        self._pending_value = None

    def normed_again(self, norm) -> NormedValue:
        """A second norm of the residual stream as the norm before left it (an RMS-shaped norm, in groups or not): nothing is
        pending, and a result that was set aside stays aside. Returns the value of the normed activations."""
        weight, eps = norm.as_fused()
        self._want(weight, torch.float32, (self.hidden,), "norm weight")
        if self._pending_value is not None:
            raise ValueError("a result is pending before a second norm of the stream")
        out = self.take(self.hidden, self.elem)
        self.op(NORM, out=out, ptrs=[weight], ints=[getattr(norm, "groups", 1), 1], floats=[eps])
        return NormedValue(out)

    def pooled_attention(self, proj: int, out: int, *, q_col: int, k_col: int, v_col: int, out_col: int, q_norm: torch.Tensor,
                         k_norm: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, k_pool: torch.Tensor | None,
                         v_pool: torch.Tensor | None, heads: int, kv_heads: int, head_dim: int, value_dim: int, block_size: int,
                         window: int, pooled_block: int, group: int, eps: float, scale: float, out_scale: float = 1.0,
                         rope: torch.Tensor | None = None, conv: torch.Tensor | None = None, conv_state: torch.Tensor | None = None,
                         sink: torch.Tensor | None = None, softcap: float = 0.0) -> None:
        """Causal attention without rotation whose q and k are normed over their whole projection, over a window of ``window``
        keys (0: all) and, with ``pooled_block`` P > 0, the means of the whole blocks of P keys and values before the window. The
        value ``proj`` holds the queries at column ``q_col``, the keys at ``k_col`` and the values at ``v_col`` (-1: the values are
        the keys as projected); the result (``heads * value_dim`` columns, times ``out_scale``) goes to the value ``out`` at
        column ``out_col``.

        ``rope`` float32 ``[positions, 2, r/2]``: q and k are turned by the position behind their norm (the first r elements of every
        head, element i with i + r/2). ``conv`` float32 ``[nq + nk + nv, taps]`` with ``conv_state`` float32 ``[slots, (taps - 1) (nq + nk +
        nv)]``: a short causal convolution over time on every channel of q, k and v ahead of the norm. ``sink`` float32 ``[heads]``:
        logits that count once in the softmax's denominator and have no value. ``softcap`` > 0: scores become ``softcap tanh(score /
        softcap)``."""
        row, out_row = self._value_kinds[proj][0], self._value_kinds[out][0]
        if self._value_kinds[proj][1] != self.elem or self._value_kinds[out][1] != self.elem:
            raise ValueError("attention reads and writes values of the compute dtype")
        rotary = covers = taps = 0
        if rope is not None:
            self._want(rope, torch.float32, None, "rotary table")
            rotary, covers = 2 * rope.shape[2], rope.shape[0]
            if covers < self.max_positions or rotary > head_dim:
                raise ValueError(f"the rotary table covers {covers} positions of {self.max_positions} and {rotary} elements of {head_dim}")
        if conv is not None:
            channels = heads * head_dim + kv_heads * (head_dim + value_dim)
            taps = int(conv.shape[1])
            self._want(conv, torch.float32, (channels, taps), "the convolutions' weights")
            if taps > 1:
                self._want(conv_state, torch.float32, (conv_state.shape[0], (taps - 1) * channels), "the convolutions' state rows")
        if (rope is not None or conv is not None) and (pooled_block or v_col < 0):
            raise ValueError("a rotation or a convolution comes with a value projection and without pooled blocks")
        if sink is not None:
            self._want(sink, torch.float32, (heads,), "sink")
        if softcap < 0:
            raise ValueError("scores are bounded by a positive number")
        for col, n in ((q_col, heads * head_dim), (k_col, kv_heads * head_dim)) + (((v_col, kv_heads * value_dim),) if v_col >= 0 else ()):
            if col < 0 or col + n > row:
                raise ValueError(f"columns {col} .. {col + n - 1} of a value of {row}")
        if out_col < 0 or out_col + heads * value_dim > out_row:
            raise ValueError(f"the result at column {out_col} of a value of {out_row}")
        if v_col < 0 and value_dim != head_dim:
            raise ValueError("values that are the keys have the keys' size")
        self._want(q_norm, torch.float32, (heads * head_dim,), "weight of the queries' norm")
        self._want(k_norm, torch.float32, (kv_heads * head_dim,), "weight of the keys' norm")
        pages = int(k_cache.shape[0])
        for t, shape, what in ((k_cache, (pages, kv_heads, block_size, head_dim), "key pages"),
                               (v_cache, (pages, kv_heads, value_dim, block_size), "value pages")):
            self._want(t, self.dtype, shape, what)
        if pooled_block:
            if window <= 0:
                raise ValueError("pooled blocks lie before a window")
            self._want(k_pool, self.dtype, tuple(k_cache.shape), "pooled key pages")
            self._want(v_pool, self.dtype, tuple(v_cache.shape), "pooled value pages")
        self.op(POOLED_ATTENTION, in_=proj, out=out,
                ptrs=[q_norm, k_norm, k_cache, v_cache, k_pool, v_pool, rope, conv, conv_state if taps > 1 else None, sink],
                ints=[heads, kv_heads, head_dim, value_dim, block_size, window, pooled_block, group, q_col, k_col, v_col, out_col,
                      rotary, covers, taps],
                floats=[eps, scale, out_scale, softcap])

    def delta_rule(self, proj: int, out: int, *, cols: dict, out_col: int, decay_outer: torch.Tensor, decay_bias: torch.Tensor,
                   rate_bias: torch.Tensor, norm_weight: torch.Tensor, state: torch.Tensor, heads: int, head_dim: int,
                   decay_rank: int, eps: float, decay_coef: float, out_scale: float = 1.0) -> None:
        """Linear attention by the generalized delta rule over the step's items, from and into their rows of ``state``
        ``[slots, heads, head_dim, head_dim]`` (float32). ``cols`` gives the columns of the value ``proj`` at which r, k, v, the
        gate ``g`` and the removal rate ``a`` (``heads * head_dim`` wide each) and the decay's inner projection ``w1``
        (``decay_rank`` wide) begin; the result (times ``out_scale``) goes to the value ``out`` at column ``out_col``."""
        row, out_row = self._value_kinds[proj][0], self._value_kinds[out][0]
        n = heads * head_dim
        if self._value_kinds[proj][1] != self.elem or self._value_kinds[out][1] != self.elem:
            raise ValueError("the delta rule reads and writes values of the compute dtype")
        for role in ("r", "k", "v", "g", "a", "w1"):
            width = decay_rank if role == "w1" else n
            if cols[role] < 0 or cols[role] + width > row:
                raise ValueError(f"{role}: columns {cols[role]} .. {cols[role] + width - 1} of a value of {row}")
        if out_col < 0 or out_col + n > out_row:
            raise ValueError(f"the result at column {out_col} of a value of {out_row}")
        self._want(decay_outer, self.dtype, (n, decay_rank), "the decay's outer weight")
        for t, what in ((decay_bias, "the decay's bias"), (rate_bias, "the removal rate's bias"), (norm_weight, "weight of the output norm")):
            self._want(t, torch.float32, (n,), what)
        self._want(state, torch.float32, (state.shape[0], heads, head_dim, head_dim), "state")
        self.op(DELTA_RULE, in_=proj, out=out, ptrs=[decay_outer, decay_bias, rate_bias, norm_weight, state],
                ints=[heads, head_dim, decay_rank, cols["r"], cols["k"], cols["v"], cols["g"], cols["a"], cols["w1"], out_col],
                floats=[eps, decay_coef, out_scale])

    # ----------------------------------------------------------- a block that norms its sublayers' results
    def result_normed(self, norm=None, out: bool = True) -> int:
        """``x += rmsnorm(pending result) * weight`` (``norm`` RMS-shaped; None where nothing is pending), then the stream in the compute
        dtype as a value, which the next sublayer reads (-1 with ``out`` false)."""
        weight = eps = None
        if norm is not None:
            fused = norm.as_fused()
            if fused is None or getattr(norm, "groups", 1) != 1:
                raise ValueError("a sublayer's result is normed by an RMS norm without groups")
            weight, eps = fused
            self._want(weight, torch.float32, (self.hidden,), "norm weight")
        value = self.take(self.hidden, self.elem, scoped=False) if out else -1
        self.op(RESULT_NORM, out=value, ptrs=[weight], floats=[eps or 0.0])
        self.pending_consumed()
        if self.stream_value is not None:  # (the sublayer that read the stream as it was is done)
            self._give_back(self.stream_value)
        self.stream_value = value if out else None
        return value

    def token_gate(self, z: int, table: torch.Tensor, col: int, activation: str) -> int:
        """``act(z) * table[token, col : col + n]`` for a value ``z`` ``[tokens, n]``; ``table`` ``[vocab, row]`` in the compute dtype."""
        from ..ops.kernels import UNGATED_ACTIVATIONS

        n = self._value_kinds[z][0]
        self._want(table, self.dtype, (self.vocab, table.shape[1]), "a table of rows per token id")
        if col < 0 or col + n > table.shape[1] or self._value_kinds[z][1] != self.elem:
            raise ValueError(f"columns {col} .. {col + n - 1} of a table of {table.shape[1]}")
        out = self.take(n)
        self.op(TOKEN_GATE, in_=z, out=out, ptrs=[table], ints=[col, table.shape[1], UNGATED_ACTIVATIONS[activation]])
        return out

    def activate(self, x: int, activation: str) -> int:
        """``act(x)`` elementwise, in place; returns ``x``."""
        from ..ops.kernels import UNGATED_ACTIVATIONS

        if activation not in UNGATED_ACTIVATIONS:
            raise ValueError(f"an ungated feed-forward knows the activations {sorted(UNGATED_ACTIVATIONS)}, got {activation!r}")
        self.op(ACTIVATE, in_=x, out=x, ints=[UNGATED_ACTIVATIONS[activation]])
        return x

    def time_mix(self, h: int, out: int, *, out_col: int, mu: torch.Tensor, w_rkvg: tuple, w1: torch.Tensor, w2: torch.Tensor,
                 w0: torch.Tensor, bonus: torch.Tensor, norm_weight: torch.Tensor, state: torch.Tensor, heads: int, head_dim: int,
                 eps: float, out_scale: float = 1.0, w_all: torch.Tensor | None = None) -> None:
        """Linear attention with a decay per token and channel and a bonus for the current token, on the value ``h`` ``[tokens, hidden]``
        (the sublayer's input). ``mu`` float32 ``[5, hidden]`` (the blends of r, k, v, gate, decay with the token before); ``w_rkvg`` four weights ``[n,
        hidden]`` (r, k, v, gate), ``w1`` ``[rank, hidden]``, ``w2`` ``[n, rank]`` in the compute dtype (n = heads * head_dim); ``w0``, ``bonus``, ``norm_weight``
        float32 ``[n]``; ``state`` float32 ``[slots, heads * head_dim^2 + hidden]``. The result (times ``out_scale``) goes to ``out`` at
        ``out_col``."""
        n, rank = heads * head_dim, int(w1.shape[0])
        if self._value_kinds[h] != (self.hidden, self.elem) or self._value_kinds[out][1] != self.elem:
            raise ValueError("time mixing reads the hidden size and writes the compute dtype")
        if out_col < 0 or out_col + n > self._value_kinds[out][0]:
            raise ValueError(f"the result at column {out_col} of a value of {self._value_kinds[out][0]}")
        self._want(mu, torch.float32, (5, self.hidden), "the blends' mu")
        for w in w_rkvg:
            self._want(w, self.dtype, (n, self.hidden), "a weight of r, k, v or the gate")
        self._want(w1, self.dtype, (rank, self.hidden), "the decay's inner weight")
        self._want(w2, self.dtype, (n, rank), "the decay's outer weight")
        for t, what in ((w0, "the decay's bias"), (bonus, "the bonus"), (norm_weight, "weight of the output norm")):
            self._want(t, torch.float32, (n,), what)
        if w_all is not None:  # r, k, v, gate and w1 behind each other: one product serves a step of few tokens
            self._want(w_all, self.dtype, (4 * n + rank, self.hidden), "the stacked weights of time mixing")
        row = heads * head_dim * head_dim + self.hidden
        self._want(state, torch.float32, (state.shape[0], row), "state")
        self.op(TIME_MIX, in_=h, out=out, ptrs=[mu, w_rkvg[0], w1, w2, w0, bonus, norm_weight, state, w_rkvg[1], w_rkvg[2], w_rkvg[3], w_all],
                ints=[heads, head_dim, rank, out_col, row, heads * head_dim * head_dim], floats=[eps, out_scale])

    # ----------------------------------------------------------- several residual streams
    def spread_streams(self, streams: int) -> None:
        """From here on every token has ``streams`` residual streams, each a copy of the stream as it is now."""
        if not 1 <= streams <= MAX_STREAMS:
            raise ValueError(f"1 to {MAX_STREAMS} residual streams are taken, not {streams}")
        if self.num_streams:
            raise ValueError("the streams are spread once")
        self.op(STREAMS, ints=[streams])
        self.num_streams = int(streams)

    def stream_normed(self, norm, reads: torch.Tensor) -> StreamNormed:
        """The input of the coming part, not yet written: the pending result rewrites the streams (by what
        :meth:`rewrites_streams` said of it), ``sum_s reads[s] x_s`` is normed by ``norm`` (RMS-shaped). The part's first product
        takes it (:meth:`linear`), or its ``value()`` does."""
        weight, eps = norm.as_fused()
        if getattr(norm, "groups", 1) != 1:
            raise ValueError("the norm over several streams is not cut into groups")
        self._want(weight, torch.float32, (self.hidden,), "norm weight")
        self._want(reads, torch.float32, (self.num_streams,), "what a part reads of the streams")
        rewrite, self._stream_rewrite = self._stream_rewrite, None
        return StreamNormed(self, weight, eps, reads, rewrite)

    def rewrites_streams(self, mix_out: torch.Tensor) -> None:
        """The result that is pending now rewrites the streams by ``mix_out`` float32 ``[S * S + S]``: ``mix[from, to]``, then
        ``out[to]``."""
        s = self.num_streams
        self._want(mix_out, torch.float32, (s * s + s,), "how a result rewrites the streams")
        self._stream_rewrite = mix_out

    def decay_state(self, proj: int, *, decay: torch.Tensor, rope: torch.Tensor | None, pairing: int, norm_weight: torch.Tensor | None,
                    state: torch.Tensor, heads: int, key_dim: int, value_dim: int, input_act: int, key_scale: float,
                    norm_kind: int, gate_act: int, eps: float) -> int:
        """Linear attention with a decay per head over the step's items, from and into their rows of ``state``
        ``[slots, heads, key_dim, value_dim]`` (float32), for a value ``[tokens, heads (2 key_dim + 2 value_dim)]`` (q, k,
        v and gate projections); returns the value ``[tokens, heads * value_dim]`` that the output projection reads."""
        cols = 2 * heads * (key_dim + value_dim)
        if self._value_kinds[proj] != (cols, self.elem):
            raise ValueError(f"the projections have {self._value_kinds[proj][0]} columns, not {cols}")
        self._want(decay, torch.float32, (2, heads), "decay")
        self._want(state, torch.float32, (state.shape[0], heads, key_dim, value_dim), "state")
        if norm_weight is not None:
            self._want(norm_weight, torch.float32, (heads * value_dim,), "weight of the output norm")
        rotary_dim = covers = 0
        if rope is not None:
            self._want(rope, torch.float32, None, "rotary table")
            rotary_dim, covers = 2 * rope.shape[2], rope.shape[0]
            if covers < self.max_positions:
                raise ValueError(f"the rotary table covers {covers} positions of {self.max_positions}")
        out = self.take(heads * value_dim)
        self.op(DECAY_STATE, in_=proj, out=out, ptrs=[decay, rope, norm_weight, state],
                ints=[heads, key_dim, value_dim, rotary_dim, pairing, input_act, norm_kind, gate_act, covers],
                floats=[key_scale, eps])
        return out

    def add(self) -> None:
        """The pending delta into the residual stream, as a kernel of its own (before a norm that is not RMS-shaped)."""
        self.op(ADD)
        self.pending_consumed()

    def hold(self) -> None:
        """The pending delta is set aside: another part that reads the same normed input follows, and the next add (of
        the next norm, of the head, or a kernel of its own) takes both results at once."""
        self.op(HOLD)
        self._held_value, self._pending_value = self._pending_value, None

    def call(self, fn, in_: int = -1, out_cols: int | None = None, out_elem: int | None = None) -> int:
        """A part with code of its own: when a step reaches this place, ``fn(frame)`` is called with a
        :class:`Frame` (the value ``in_`` as ``frame.input``, a new value of ``out_cols`` columns as
        ``frame.output``, the residual stream as ``frame.x``, the step's batch). It launches what it has to on the
        current stream and returns nothing. Returns the output value (-1 without ``out_cols``)."""
        out = self.take(out_cols, out_elem) if out_cols else -1
        me = weakref.ref(self)  # (the program keeps the trampoline: no cycle through it)

        def trampoline(raw):
            program = me()
            try:
                fn(Frame(program, raw.contents))
                return 0
            except BaseException as e:  # an exception cannot cross the C frames in between: it is raised after the step
                program.call_error = e
                return 1

        c_fn = _CALL_FN(trampoline)
        self._calls.append(c_fn)
        p = (ctypes.c_void_p * OP_PTRS)()
        p[0] = ctypes.cast(c_fn, ctypes.c_void_p).value
        iv, fv = (ctypes.c_int64 * OP_INTS)(), (ctypes.c_float * OP_FLOATS)()
        self.num_ops = _ok(self._L.me_runner_op(self.handle, CALL, in_, out, p, iv, fv))
        return out

    def call_part(self, part, h, extra=()) -> int:
        """A mixer or feed-forward without ``emit``: its ``forward(h, batch, *extra)`` on the normed activations, its
        result as a value ``[tokens, hidden]``."""
        src = h.value()
        return self.call(lambda frame: frame.write(part.forward(frame.input, frame.batch, *extra)), in_=src,
                         out_cols=self.hidden)

    def normed_by(self, norm) -> "CalledNorm":
        """The add-and-norm before a part, for a norm part of any shape (its ``forward`` is called)."""
        return CalledNorm(self, norm)

    def head_by(self, norm, weight: torch.Tensor, logit_scale: float = 1.0) -> None:
        """As :meth:`head`, for a final norm of any shape: the add, the norm part's ``forward`` on the wanted rows,
        the head product."""
        self._want(weight, self.dtype, (self.vocab, self.hidden), "head")
        self.add()

        def run(frame):
            if frame.rows:
                rows = frame.batch.want_rows[:frame.rows].long()
                frame.output[:frame.rows].copy_(norm.forward(frame.x.index_select(0, rows)))

        with self.scope():
            picked = self.call(run, out_cols=self.hidden)
            self.op(HEAD_ROWS, in_=picked, ptrs=[None, weight], floats=[0.0, logit_scale])

    def head(self, norm, weight: torch.Tensor, logit_scale: float = 1.0) -> None:
        """Final norm of the wanted rows, the head product, the logits times ``logit_scale``."""
        norm_weight, eps = norm.as_fused()
        self._want(weight, self.dtype, (self.vocab, self.hidden), "head")
        if self.num_streams:  # the streams' sum, with the pending rewrite applied to the wanted rows
            if getattr(norm, "groups", 1) != 1:
                raise ValueError("the norm over several streams is not cut into groups")
            self.op(STREAM_HEAD, ptrs=[norm_weight, weight, self._stream_rewrite], floats=[eps, logit_scale])
            self._stream_rewrite = None
        else:
            self.op(HEAD, ptrs=[norm_weight, weight], ints=[getattr(norm, "groups", 1)], floats=[eps, logit_scale])
        self.pending_consumed()

    def sample(self) -> None:
        self.op(SAMPLE)
        self.draws = True

    def _want(self, t: torch.Tensor, dtype, shape, what: str) -> None:
        if t.dtype is not dtype or (shape is not None and tuple(t.shape) != tuple(shape)) or not t.is_cuda:
            raise ValueError(f"{what}: expected {dtype} {shape} on the GPU, got {t.dtype} {tuple(t.shape)} on {t.device}")

    # ------------------------------------------------------------------ memory
    def arena_need(self, tokens: int, items: int, rows: int, max_ctx: int) -> int:
        return _ok(self._L.me_runner_arena_need(self.handle, tokens, items, rows, max_ctx))

    def index_need(self, tokens: int, items: int, rows: int, widths: list[int]) -> int:
        w = np.ascontiguousarray(widths, dtype=np.int32)
        return _ok(self._L.me_runner_index_need(self.handle, tokens, items, rows, _vp(w.ctypes.data), len(w)))


class StepMemory:
    """What eager steps of a program run on: an arena for activations and workspaces, two pinned
    staging buffers and the index buffer on the device, sized for the largest step seen so far."""

    def __init__(self, program: StepProgram, device, widths: list[int], spare_page: int, spare_slot: int):
        self.program, self.device, self.widths = program, device, list(widths)
        self.spare_page, self.spare_slot = spare_page, spare_slot
        self.caps = (0, 0, 0, 0)
        self.arena = self.staging = self.index = None

    def ensure(self, tokens: int, items: int, rows: int, max_ctx: int) -> None:
        c = self.caps
        if tokens <= c[0] and items <= c[1] and rows <= c[2] and max_ctx <= c[3]:
            return
        torch.cuda.synchronize()  # nothing of the old memory is in use once the device is idle
        c = self.caps = (max(tokens, c[0]), max(items, c[1]), max(rows, c[2]), max(max_ctx, c[3]))
        p = self.program
        self.arena = torch.empty(p.arena_need(*c), dtype=torch.uint8, device=self.device)
        ints = p.index_need(c[0], c[1], c[2], self.widths)
        self.staging = [torch.empty(ints, dtype=torch.int32, pin_memory=True) for _ in range(2)]
        self.index = torch.empty(ints, dtype=torch.int32, device=self.device)
        _ok(p._L.me_runner_memory(p.handle, _vp(self.arena.data_ptr()), self.arena.numel(), _vp(self.staging[0].data_ptr()),
                                  _vp(self.staging[1].data_ptr()), ints, _vp(self.index.data_ptr()), ints, self.spare_page,
                                  self.spare_slot))


def view_in(arena: torch.Tensor, address: int, shape: tuple[int, ...], dtype: torch.dtype) -> torch.Tensor:
    """The tensor of ``shape`` that lies at ``address`` inside ``arena``."""
    offset = address - arena.data_ptr()
    count = int(np.prod(shape)) * torch.empty((), dtype=dtype).element_size()
    if offset < 0 or offset + count > arena.numel():
        raise RuntimeError("a step's result lies outside its arena")
    return arena[offset:offset + count].view(dtype).view(shape)


def _after_calls(program: StepProgram, code: int) -> None:
    """The step's call into C++ has come back: an exception that a called part raised on the way is raised now."""
    error, program.call_error = program.call_error, None
    if error is not None:
        raise error
    _ok(code)


def run_step(program: StepProgram, memory: StepMemory, core) -> tuple[torch.Tensor | None, torch.Tensor | None, int]:
    """Run the step that ``core`` holds; (logits float32 [rows, vocab], drawn int32 [rows], rows)."""
    out = np.zeros(4, dtype=np.int64)
    stream = _vp(torch.cuda.current_stream().cuda_stream)
    program.current_arena = memory.arena
    _after_calls(program, program._L.me_runner_step(program.handle, core._box, stream, _vp(out.ctypes.data)))
    rows = int(out[1])
    program.last_prefill_columns = int(out[3])
    logits = view_in(memory.arena, int(out[0]), (rows, program.vocab), torch.float32) if out[0] else None
    drawn = view_in(memory.arena, int(out[2]), (rows,), torch.int32) if out[2] else None
    return logits, drawn, rows


def run_static(program: StepProgram, arena: torch.Tensor, index: torch.Tensor, bucket: int, widths: list[int], max_ctx: int,
               least_live: int, drawn: torch.Tensor | None = None, fed: bool = False):
    """Launch a decode step of ``bucket`` one-token items whose indices are in ``index`` on the device
    (what a graph captures); (logits [bucket, vocab], drawn [bucket])."""
    out = np.zeros(4, dtype=np.int64)
    w = np.ascontiguousarray(widths, dtype=np.int32)
    stream = _vp(torch.cuda.current_stream().cuda_stream)
    program.current_arena = arena
    _after_calls(program, program._L.me_runner_static(program.handle, _vp(arena.data_ptr()), arena.numel(), _vp(index.data_ptr()),
                                                      bucket, _vp(w.ctypes.data), len(w), max_ctx, least_live,
                                                      _vp(None if drawn is None else drawn.data_ptr()), int(fed), stream,
                                                      _vp(out.ctypes.data)))
    logits = view_in(arena, int(out[0]), (bucket, program.vocab), torch.float32)
    tokens = drawn if drawn is not None else view_in(arena, int(out[2]), (bucket,), torch.int32)
    return logits, tokens
