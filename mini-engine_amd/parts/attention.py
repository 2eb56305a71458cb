"""Grouped-query attention mixer over a paged key/value cache.

Per step (reference: ``src/mini_engine/model.py:111-119`` and ``attention.py:104-175``):
one product for q, k and v (the three weights are stacked at load time), then one fused kernel for
the per-head q/k RMSNorm, the position encoding and the write of the new keys and values into their
pages, then attention of every new token over the pages of its request (causal, optionally within a
window), then the output projection.

Sizes and constants all come from the spec: head counts, head size, score scale, eps of the q/k
norm (None: no norm), window (0: none), position encoding (None: none), and ``cache_from`` (read
another layer's pages and write none).

Beyond that plain form the spec may give the value heads a size of their own, keep the first keys of a
request visible behind the window, pair neighbouring elements in the rotation, and have the values turned
by their position before they are cached (every output is then turned back by its query's position). A
layer that uses any of these runs the kernels that take every size (``qkv_rotate_scatter``,
``attention_general``), in both dtypes.
"""

from __future__ import annotations

import torch

from ..ops import kernels as K
from ..weights.loader import TensorWant
from .base import MIXERS, POSITION_ENCODINGS, KVBinding, KVCacheNeed, Mixer, PairBinding, StateBinding, StateNeed

MAX_HEAD_DIM = 256


class Attention(Mixer):
    graph_safe = True

    def __init__(self, spec, dtype, device):
        super().__init__(spec, dtype, device)
        s = spec
        if not (float(s.scale) > 0.0 and float(s.scale) < float("inf")):
            raise ValueError(f"the score scale must be positive and finite, got {s.scale}: the matrix-core kernels take a "
                             f"tile's maximum before they scale")
        if s.num_heads % s.num_kv_heads:
            raise ValueError(f"{s.num_heads} query heads are not a multiple of {s.num_kv_heads} key/value heads")
        if s.window < 0:
            raise ValueError(f"window={s.window} must be >= 0")
        self.nh, self.nkv, self.d = s.num_heads, s.num_kv_heads, s.head_dim
        self.dv = int(getattr(s, "v_dim", s.head_dim))
        self.keep_first = int(getattr(s, "keep_first", 0))
        if self.keep_first < 0 or (self.keep_first and not s.window):
            raise ValueError(f"keep_first={self.keep_first} must be >= 0 and needs a window")
        self.position = None if s.position is None else POSITION_ENCODINGS.build(s.position, dtype, device)
        vp = getattr(s, "value_position", None)
        self.value_position = None if vp is None else POSITION_ENCODINGS.build(vp, dtype, device)
        if self.value_position is not None and self.value_position.rotary_dim != self.dv:
            raise ValueError(f"values of size {self.dv} are turned over all of their elements, not {self.value_position.rotary_dim}")
        self.pairing = 0 if self.position is None else int(getattr(self.position, "pairing_code", 0))
        self.q_temp = getattr(s, "query_temperature", None)
        if self.q_temp is not None and int(self.q_temp[1]) < 1:
            raise ValueError(f"a temperature on the queries grows every {self.q_temp[1]} positions: at least every one")
        self.gated = bool(getattr(s, "output_gate", False))
        self.norm_weighted = bool(getattr(s, "qk_norm_weight", True))
        # q and k normed over their whole projection (no rotation): a form of its own, which may take its values from the keys
        # as projected and see the means of whole blocks of keys before its window
        self.whole = getattr(s, "qk_norm_over", "head") == "projection"
        self.values_from_keys = bool(getattr(s, "values_from_keys", False))
        self.pooled_block = int(getattr(s, "pooled_block", 0))
        if getattr(s, "qk_norm_over", "head") not in ("head", "projection"):
            raise ValueError(f"q and k are normed over 'head' or 'projection', not {s.qk_norm_over!r}")
        if (self.values_from_keys or self.pooled_block) and not self.whole:
            raise ValueError("values taken from the keys and pooled blocks are built for q and k normed over their whole projection")
        # (forms of the attention normed over the whole projection: a short convolution ahead of the norm, a rotation behind it,
        # bounded scores, a sink of score 0)
        self.conv_taps = int(getattr(s, "conv_taps", 0))
        self.softcap = float(getattr(s, "softcap", 0.0) or 0.0)
        self.unit_sink = bool(getattr(s, "unit_sink", False))
        if (self.conv_taps or self.softcap or self.unit_sink) and not self.whole:
            raise ValueError("a short convolution, bounded scores and a sink of score 0 are built for q and k normed over their whole projection")
        if self.conv_taps < 0 or self.conv_taps > 16 or self.softcap < 0:
            raise ValueError(f"conv_taps={self.conv_taps} must be in 0..16 and softcap={self.softcap} positive")
        if self.whole:
            if (s.qk_norm_eps is None or self.keep_first or self.value_position is not None
                    or self.q_temp is not None or self.gated or s.cache_from is not None or not self.norm_weighted):
                raise ValueError("attention normed over the whole projection has a weighted norm, no kept first keys, "
                                 "no gate, no temperature, and pages of its own")
            if self.position is not None and (self.pairing != 0 or self.pooled_block or self.values_from_keys):
                raise ValueError("attention normed over the whole projection is turned in pairs of halves, with a value projection and "
                                 "without pooled blocks")
            if self.conv_taps and (self.pooled_block or self.values_from_keys):
                raise ValueError("a short convolution comes with a value projection and without pooled blocks")
            if self.values_from_keys and self.dv != self.d:
                raise ValueError(f"values that are the keys have the keys' size {self.d}, not {self.dv}")
            if self.pooled_block < 0 or (self.pooled_block and not s.window):
                raise ValueError(f"pooled_block={self.pooled_block} must be >= 0 and needs a window")
        # the plain form: what the matrix-core kernels and the fused decode prologue are written for
        self.plain = (self.dv == self.d and not self.keep_first and self.pairing == 0 and self.value_position is None
                      and self.q_temp is None and not self.gated and not self.whole)
        if self.plain and (s.head_dim % 16 or not 16 <= s.head_dim <= MAX_HEAD_DIM):
            raise ValueError(f"head_dim={s.head_dim} is not supported: the attention kernels take head sizes "
                             f"from 16 to {MAX_HEAD_DIM} in steps of 16")
        if not self.plain:
            if not (1 <= self.d <= MAX_HEAD_DIM and 1 <= self.dv <= MAX_HEAD_DIM):
                raise ValueError(f"head sizes {self.d} and {self.dv} must be in 1..{MAX_HEAD_DIM}")
            if s.cache_from is not None:
                raise ValueError("an attention layer beyond the plain form owns its pages")
        names = dict(getattr(s, "names", ()) or ())
        self._n = {r: names.get(r, d) for r, d in (("q", "q_proj.weight"), ("k", "k_proj.weight"), ("v", "v_proj.weight"),
                                                    ("o", "o_proj.weight"), ("q_norm", "q_norm.weight"),
                                                    ("k_norm", "k_norm.weight"), ("g", "g_proj.weight"))}
        self._n.update({r: names.get(r, d) for r, d in (("q_conv", "q_conv.weight"), ("k_conv", "k_conv.weight"), ("v_conv", "v_conv.weight"))})
        self.q_norm_w = self.k_norm_w = None
        self.w_qkv = self.w_o = None
        self.conv_w = self.sink = None

    # ---- weights
    def weight_wants(self, prefix: str) -> dict[str, TensorWant]:
        s = self.spec
        n = self._n
        wants = {
            f"{prefix}.{n['q']}": TensorWant((s.num_heads * s.head_dim, s.hidden_size)),
            f"{prefix}.{n['o']}": TensorWant((s.hidden_size, s.num_heads * self.dv)),
        }
        if s.cache_from is None:
            wants[f"{prefix}.{n['k']}"] = TensorWant((s.num_kv_heads * s.head_dim, s.hidden_size))
            if not self.values_from_keys:
                wants[f"{prefix}.{n['v']}"] = TensorWant((s.num_kv_heads * self.dv, s.hidden_size))
        if self.whole:
            wants[f"{prefix}.{n['q_norm']}"] = TensorWant((s.num_heads * s.head_dim,), "vector")
            wants[f"{prefix}.{n['k_norm']}"] = TensorWant((s.num_kv_heads * s.head_dim,), "vector")
        elif s.qk_norm_eps is not None and self.norm_weighted:
            wants[f"{prefix}.{n['q_norm']}"] = TensorWant((s.head_dim,), "vector")
            if s.cache_from is None:
                wants[f"{prefix}.{n['k_norm']}"] = TensorWant((s.head_dim,), "vector")
        if self.gated:
            wants[f"{prefix}.{n['g']}"] = TensorWant((s.num_heads, s.hidden_size))
        if self.conv_taps:
            for role, channels in (("q_conv", s.num_heads * s.head_dim), ("k_conv", s.num_kv_heads * s.head_dim), ("v_conv", s.num_kv_heads * self.dv)):
                wants[f"{prefix}.{n[role]}"] = TensorWant((channels, self.conv_taps), "vector")
        return wants

    def load(self, tensors, prefix: str) -> None:
        s = self.spec
        n = self._n
        q = tensors[f"{prefix}.{n['q']}"]
        if self.values_from_keys:
            rows = [q, tensors[f"{prefix}.{n['k']}"]]
        else:
            rows = [q] if s.cache_from is not None else [q, tensors[f"{prefix}.{n['k']}"], tensors[f"{prefix}.{n['v']}"]]
        if self.gated:  # the gates' rows ride behind q, k and v: one product for all
            rows.append(tensors[f"{prefix}.{n['g']}"])
        self.w_qkv = torch.cat(rows, dim=0) if len(rows) > 1 else q.contiguous()
        self.w_o = tensors[f"{prefix}.{n['o']}"]
        if s.qk_norm_eps is not None and self.norm_weighted:
            self.q_norm_w = tensors[f"{prefix}.{n['q_norm']}"]
            self.k_norm_w = tensors.get(f"{prefix}.{n['k_norm']}")
        elif s.qk_norm_eps is not None:  # the norm has no weight: the kernels multiply by ones
            self.q_norm_w = self.k_norm_w = torch.ones(s.head_dim, dtype=torch.float32, device=q.device)
        if self.conv_taps:  # the three convolutions' weights behind each other, as the channels of [q | k | v] lie
            self.conv_w = torch.cat([tensors[f"{prefix}.{n[r]}"] for r in ("q_conv", "k_conv", "v_conv")], dim=0).contiguous()
        if self.unit_sink:  # a logit of 0 per head in the softmax's denominator
            self.sink = torch.zeros(s.num_heads, dtype=torch.float32, device=q.device)

    # ---- cache
    def cache_need(self):
        if self.spec.cache_from is not None:
            return None
        if self.whole:
            pages = KVCacheNeed(self.nkv, self.d, self.spec.window, value_dim=self.dv, pooled_block=self.pooled_block)
            if self.conv_taps > 1:  # the last taps - 1 projections of a sequence, every channel of q, k and v
                return (pages, StateNeed(((self.conv_taps - 1) * self.input_cols,), torch.float32))
            return pages
        if self.plain:
            return KVCacheNeed(self.nkv, self.d, self.spec.window)
        return KVCacheNeed(self.nkv, self.d, self.spec.window, value_dim=self.dv, keep_first=self.keep_first)

    def cache_source(self):
        return self.spec.cache_from

    # ---- step
    takes_normed_input = True

    def forward(self, h, batch, cache: KVBinding | None = None) -> torch.Tensor:
        s, b = self.spec, cache
        if b is None:
            raise RuntimeError("attention mixer was given no cache")
        owns = s.cache_from is None
        if self.q_temp is not None or self.gated or self.whole:
            raise NotImplementedError("a temperature on the queries, an output gate and the norm over the whole projection run in "
                                      "the step program only")
        proj = K.linear(h, self.w_qkv)  # [T, (nh + 2 nkv) d] or [T, nh d]
        table = batch.block_table(b.group)
        rope = None if self.position is None else self.position.tables(batch.max_ctx)
        eps = 0.0 if s.qk_norm_eps is None else float(s.qk_norm_eps)
        if not self.plain:
            vt = None if self.value_position is None else self.value_position.tables(batch.max_ctx)
            v_pairing = 0 if self.value_position is None else self.value_position.pairing_code
            q = K.qkv_rotate_scatter(proj, self.q_norm_w, self.k_norm_w, rope, self.pairing, vt, v_pairing, batch.positions,
                                     batch.token_item, table, b.k_cache, b.v_cache, self.nh, self.nkv, self.d, self.dv, eps)
            tiled = (self.dtype is torch.bfloat16 and self.dv == self.d
                     and K.attention_mfma_supported(self.d, b.block_size, self.nh // self.nkv))
            if tiled and batch.decode_only:  # one new token per item: the split-context matrix-core kernel
                out = K.attention_decode_bf16(q, b.k_cache, b.v_cache, batch.item_ctx, table, float(s.scale), int(s.window),
                                              batch.max_ctx, live=(batch.live_items, batch.least_live),
                                              keep_first=self.keep_first)
                if vt is not None:
                    K.unturn_rows(out, vt, v_pairing, batch.positions, self.nh)
                return K.linear(out, self.w_o, as_delta=True)
            if tiled:
                # prompts and portions: the tiled matrix-core kernel, then the outputs turned back in a pass of their own
                key = ("prefill_plan", self.nh, self.nkv, self.d, int(s.window), self.keep_first)
                plan = batch.derived.get(key)
                if plan is None:
                    plan = K.prefill_plan(batch.starts, batch.qlens, self.nh, self.nkv, self.d, int(s.window), q.device,
                                          keep_first=self.keep_first)
                    batch.derived[key] = plan
                out = K.attention_prefill_bf16(q, b.k_cache, b.v_cache, batch.positions, batch.item_start, batch.qlens, table,
                                               float(s.scale), int(s.window), plan=plan, keep_first=self.keep_first)
                if vt is not None:
                    K.unturn_rows(out, vt, v_pairing, batch.positions, self.nh)
                return K.linear(out, self.w_o, as_delta=True)
            out = K.attention_general(q, b.k_cache, b.v_cache, batch.positions, batch.token_item, table, float(s.scale),
                                      int(s.window), keep_first=self.keep_first, unturn=vt, un_pairing=v_pairing)
            return K.linear(out, self.w_o, as_delta=True)
        if (self.dtype is torch.bfloat16 and batch.decode_only and K.attention_decode_fused_supported(
                self.d, b.block_size, 0 if rope is None else 2 * rope.shape[2], self.nh // self.nkv)):
            # one new token per item: norm, rotary, page write and attention in one launch
            out = K.attention_decode_fused_bf16(
                proj, self.q_norm_w, self.k_norm_w if owns else None, rope, eps, owns, b.k_cache, b.v_cache,
                batch.item_ctx, table, self.nh, float(s.scale), int(s.window), batch.max_ctx,
                live=(batch.live_items, batch.least_live))
            return K.linear(out, self.w_o, as_delta=True)
        q = K.qk_norm_rope_scatter(
            proj, self.q_norm_w, self.k_norm_w if owns else None, rope, batch.positions, batch.token_item,
            table, b.k_cache, b.v_cache, self.nh, self.nkv, self.d, eps, write_kv=owns,
            item_start=batch.item_start, starts=batch.starts, qlens=batch.qlens)
        out = self.attend(q, batch, table, b)
        return K.linear(out, self.w_o, as_delta=True)

    # ---- what a pair of mixers asks of each of them (the form normed over the whole projection)
    @property
    def w_in(self):
        return self.w_qkv

    @w_in.setter
    def w_in(self, value):
        self.w_qkv = value

    @property
    def input_cols(self) -> int:
        return self.nh * self.d + self.nkv * self.d + (0 if self.values_from_keys else self.nkv * self.dv)

    @property
    def output_cols(self) -> int:
        return self.nh * self.dv

    def emit_projected(self, program, proj: int, col: int, out: int, out_col: int, out_scale: float, cache) -> None:
        """The mixer between its two products: the projections lie in the value ``proj`` from column ``col`` on (the rows of
        ``w_in``), the result goes to the value ``out`` at column ``out_col``, times ``out_scale``."""
        if not self.whole:
            raise NotImplementedError("only attention normed over its whole projection reads and writes at columns of wider values")
        conv_state = None
        if isinstance(cache, PairBinding) and isinstance(cache.left, KVBinding) and isinstance(cache.right, StateBinding):
            cache, conv_state = cache.left, cache.right.state  # pages, and the state rows of the short convolutions
        if not isinstance(cache, KVBinding):
            raise RuntimeError("attention mixer was given no cache")
        if self.conv_taps > 1 and conv_state is None:
            raise RuntimeError("attention with a short convolution was given no state rows (it stands alone, not in a pair of mixers)")
        s, b = self.spec, cache
        k_col = col + self.nh * self.d
        program.pooled_attention(
            proj, out, q_col=col, k_col=k_col, v_col=-1 if self.values_from_keys else k_col + self.nkv * self.d, out_col=out_col,
            q_norm=self.q_norm_w, k_norm=self.k_norm_w, k_cache=b.k_cache, v_cache=b.v_cache, k_pool=b.k_pool, v_pool=b.v_pool,
            heads=self.nh, kv_heads=self.nkv, head_dim=self.d, value_dim=self.dv, block_size=b.block_size, window=int(s.window),
            pooled_block=self.pooled_block, group=b.group, eps=float(s.qk_norm_eps), scale=float(s.scale), out_scale=out_scale,
            rope=None if self.position is None else self.position.tables(program.max_positions), conv=self.conv_w,
            conv_state=conv_state, sink=self.sink, softcap=self.softcap)

    def emit(self, program, h, cache: KVBinding | None = None) -> None:
        s, b = self.spec, cache
        if b is None:
            raise RuntimeError("attention mixer was given no cache")
        if self.whole:
            proj = program.linear(h, self.w_qkv)
            out = program.take(self.output_cols)
            self.emit_projected(program, proj, 0, out, 0, 1.0, cache)
            program.linear_delta(out, self.w_o)
            return
        owns = s.cache_from is None
        qkv = program.linear(h, self.w_qkv)
        out = program.attention(
            qkv, q_norm=self.q_norm_w, k_norm=self.k_norm_w if owns else None,
            rope=None if self.position is None else self.position.tables(program.max_positions),
            k_cache=b.k_cache, v_cache=b.v_cache, heads=self.nh, kv_heads=self.nkv, head_dim=self.d,
            block_size=b.block_size, window=int(s.window), writes=owns, group=b.group,
            eps=0.0 if s.qk_norm_eps is None else float(s.qk_norm_eps), scale=float(s.scale),
            value_dim=self.dv, keep_first=self.keep_first, pairing=self.pairing,
            value_rope=None if self.value_position is None else self.value_position.tables(program.max_positions),
            value_pairing=0 if self.value_position is None else self.value_position.pairing_code,
            query_temperature=self.q_temp, gated=self.gated)
        program.linear_delta(out, self.w_o)

    def attend(self, q: torch.Tensor, batch, table: torch.Tensor, b: KVBinding) -> torch.Tensor:
        """bfloat16 with sizes the matrix-core kernels take: the split-context kernel when every item
        brings one token, else the tiled prefill kernel. Everything else (float32, other head or page
        sizes): the general kernel."""
        s = self.spec
        scale, window = float(s.scale), int(s.window)
        if self.dtype is torch.bfloat16 and K.attention_mfma_supported(self.d, b.block_size, self.nh // self.nkv):
            if batch.decode_only:
                return K.attention_decode_bf16(q, b.k_cache, b.v_cache, batch.item_ctx, table, scale, window,
                                               batch.max_ctx, live=(batch.live_items, batch.least_live))
            key = ("prefill_plan", self.nh, self.nkv, self.d, window)
            plan = batch.derived.get(key)
            if plan is None:  # the same for every layer of this shape: made once per step
                plan = K.prefill_plan(batch.starts, batch.qlens, self.nh, self.nkv, self.d, window, q.device)
                batch.derived[key] = plan
            return K.attention_prefill_bf16(q, b.k_cache, b.v_cache, batch.positions, batch.item_start, batch.qlens,
                                            table, scale, window, plan=plan)
        return K.attention_general(q, b.k_cache, b.v_cache, batch.positions, batch.token_item, table, scale, window)


MIXERS.register("attention", Attention)
