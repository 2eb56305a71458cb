"""Attention whose keys and values are linear maps of one latent per token (the spec:
:class:`~mini_engine_amd.config.specs.LatentAttentionSpec`).

The layer never expands the latents. With c the normed latent and k_r the rotated key part that all heads share,

    score_h(i, j) = q_h[:d] . (W_uk_h c_j) + rot(q_h[d:]) . k_r_j = (W_uk_h^T q_h[:d]) . c_j + rot(q_h[d:]) . k_r_j
    out_h(i)      = W_uv_h (sum_j p_h(i, j) c_j)

so a token keeps one key ``[c | k_r]`` for all heads, whose first ``rank`` elements are also its value: the pages of a
layer are those of one key/value head. Per step: one product for the queries, the latent projection and the gates (the
three weights are stacked at load time); the latent's norm, the rotation and the page write; the keys' map folded into
the queries, head by head; attention over the pages (with the sink in the softmax's denominator); the values' map on the
weighted latents, head by head, times the sigmoid of the head's gate; the output projection.

A position encoding that pairs neighbouring elements (2j with 2j + 1) is served by the kernels that pair halves: the rows of the
weights that give the turned parts (of the queries, head by head, and of the shared key part) are put into the order ``0, 2, 4, ..,
1, 3, 5, ..`` when they are loaded. The turned parts only ever meet each other in a score, which no order of their elements changes.
A layer with ``cache_from`` reads the pages of the layer it names (which orders its shared key part alike) and has no latent
projection of its own.
"""

from __future__ import annotations

import torch

from ..weights.loader import TensorWant
from .base import MIXERS, POSITION_ENCODINGS, KVBinding, KVCacheNeed, Mixer

MAX_KEY_DIM = 512  # what the attention kernel that takes every size allows for rank + rotary_dim
MATRIX_CORE_KEY_DIMS = (32, 64, 96, 128, 192, 256)  # csrc/attention_mfma.hip: me_attention_mfma_supported


class LatentAttention(Mixer):
    graph_safe = True

    def __init__(self, spec, dtype, device):
        super().__init__(spec, dtype, device)
        s = spec
        if not (float(s.scale) > 0.0 and float(s.scale) < float("inf")):
            raise ValueError(f"the score scale must be positive and finite, got {s.scale}")
        self.nh, self.d, self.r, self.dv, self.rank = s.num_heads, s.head_dim, s.rotary_dim, s.value_dim, s.latent_rank
        if min(self.nh, self.d, self.r, self.dv, self.rank) < 1 or self.r % 2:
            raise ValueError("heads, sizes and rank must be positive and rotary_dim even")
        if self.rank + self.r > MAX_KEY_DIM:
            raise ValueError(f"latent_rank + rotary_dim = {self.rank + self.r} is not supported: at most {MAX_KEY_DIM}")
        if not s.output_gate:
            raise ValueError("a latent attention layer has an output gate per head (the ungated form is not built)")
        self.position = POSITION_ENCODINGS.build(s.position, dtype, device)
        if int(self.position.rotary_dim) != self.r:
            raise ValueError("the shared key part is turned over all of its elements")
        self.neighbours = int(getattr(self.position, "pairing_code", 0)) == 1
        self.cache_from = getattr(s, "cache_from", None)
        names = dict(getattr(s, "names", ()) or ())
        self._n = {r: names.get(r, r) for r in ("q", "dkv", "dkv_norm", "uk", "uv", "sink", "g", "o")}
        self.w_in = self.w_o = self.key_map = self.value_map = self.latent_norm = self.sink = None

    # ---- weights
    def weight_wants(self, prefix: str) -> dict[str, TensorWant]:
        s, n = self.spec, self._n
        wants = {f"{prefix}.{n['q']}": TensorWant((self.nh * (self.d + self.r), s.hidden_size))}
        if self.cache_from is None:  # (a layer that reads another layer's pages has no latent projection of its own)
            wants[f"{prefix}.{n['dkv']}"] = TensorWant((self.rank + self.r, s.hidden_size))
            wants[f"{prefix}.{n['dkv_norm']}"] = TensorWant((self.rank,), "vector")
        wants[f"{prefix}.{n['uk']}"] = TensorWant((self.nh * self.d, self.rank))
        wants[f"{prefix}.{n['uv']}"] = TensorWant((self.nh * self.dv, self.rank))
        wants[f"{prefix}.{n['o']}"] = TensorWant((s.hidden_size, self.nh * self.dv))
        if s.sink:
            wants[f"{prefix}.{n['sink']}"] = TensorWant((self.nh,), "vector")
        if s.output_gate:
            wants[f"{prefix}.{n['g']}"] = TensorWant((self.nh, s.hidden_size))
        return wants

    def load(self, tensors, prefix: str) -> None:
        s, n = self.spec, self._n
        q = tensors[f"{prefix}.{n['q']}"]
        owns = self.cache_from is None
        dkv = tensors[f"{prefix}.{n['dkv']}"] if owns else None
        if self.neighbours:  # the turned parts' rows: evens, then odds (what pairs of neighbours are to the kernels' pairs of halves)
            order = torch.cat((torch.arange(0, self.r, 2), torch.arange(1, self.r, 2))).to(q.device)
            q = q.view(self.nh, self.d + self.r, -1)
            q = torch.cat((q[:, : self.d], q[:, self.d:].index_select(1, order)), dim=1).reshape(self.nh * (self.d + self.r), -1).contiguous()
            if owns:
                dkv = torch.cat((dkv[: self.rank], dkv[self.rank:].index_select(0, order)), dim=0).contiguous()
        rows = [q] + ([dkv] if owns else []) + [tensors[f"{prefix}.{n['g']}"]]
        pad = -sum(t.shape[0] for t in rows) % 8  # rows of zeros: every token's projections then start at a multiple of 16 bytes
        if pad:
            rows.append(torch.zeros((pad, q.shape[1]), dtype=q.dtype, device=q.device))
        self.w_in = torch.cat(rows, dim=0)
        self.w_o = tensors[f"{prefix}.{n['o']}"]
        # the keys' map per head, transposed: [heads, rank, d] reads a head's query part and gives its image in the latent space
        self.key_map = tensors[f"{prefix}.{n['uk']}"].view(self.nh, self.d, self.rank).transpose(1, 2).contiguous()
        self.value_map = tensors[f"{prefix}.{n['uv']}"].view(self.nh, self.dv, self.rank).contiguous()
        self.latent_norm = tensors[f"{prefix}.{n['dkv_norm']}"] if owns else torch.ones(self.rank, dtype=torch.float32, device=q.device)
        self.sink = tensors[f"{prefix}.{n['sink']}"] if s.sink else None

    # ---- cache
    def cache_source(self):
        return self.cache_from

    def cache_need(self):
        if self.cache_from is not None:
            return None
        # bfloat16 with a key size that the matrix-core attention kernels take and at most 16 heads: those kernels read keys and
        # values of one size, so the value pages hold the whole key (its first `rank` rows are the values that count)
        dk = self.rank + self.r
        whole = self.dtype is torch.bfloat16 and dk in MATRIX_CORE_KEY_DIMS and self.nh <= 16
        return KVCacheNeed(1, dk, 0, value_dim=dk if whole else self.rank)

    # ---- step
    def forward(self, h, batch, cache=None):
        raise NotImplementedError("latent attention runs in the step program only")

    def emit(self, program, h, cache: KVBinding | None = None) -> None:
        s, b = self.spec, cache
        if b is None:
            raise RuntimeError("latent attention mixer was given no cache")
        proj = program.linear(h, self.w_in)
        out = program.latent_attention(
            proj, latent_norm=self.latent_norm, rope=self.position.tables(program.max_positions), k_cache=b.k_cache,
            v_cache=b.v_cache, key_map=self.key_map, value_map=self.value_map, sink=self.sink, heads=self.nh, head_dim=self.d,
            rotary_dim=self.r, rank=self.rank, value_dim=self.dv, block_size=b.block_size, group=b.group,
            eps=float(s.norm_eps), scale=float(s.scale), writes=self.cache_from is None)
        program.linear_delta(out, self.w_o)


MIXERS.register("latent_attention", LatentAttention)
