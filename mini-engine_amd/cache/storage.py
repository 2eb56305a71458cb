"""Device storage behind the page tables: for every run of a layer (a position in the model's
order) that owns a cache, one tensor of key pages and one of value pages, or one tensor of state
rows for a mixer with per-request state.

Runs whose mixers state the same need (heads, head size, window) form one group and share one
block table per request. A page id indexes every run of its group at once. Each group has one page
more than the manager hands out: rows that pad a replayed graph write there.

Layout of a layer's pages: keys ``[pages, kv_heads, block_size, head_dim]`` and values transposed,
``[pages, kv_heads, value_dim, block_size]``, so that the matrix cores read both along the
contiguous direction (keys along head_dim for q.k, values along the keys for p.v).
"""

from __future__ import annotations

from dataclasses import dataclass

import torch

from ..parts.base import KVBinding, KVCacheNeed, PairBinding, StateBinding, StateNeed
from .block_manager import GroupSpec


@dataclass
class CacheLayout:
    groups: list[GroupSpec]
    group_needs: list[KVCacheNeed]
    layer_group: dict[int, int]  # run (position in the order) -> group index, for runs that own pages
    state_layers: dict[int, StateNeed]  # run -> its state need

    @property
    def has_state(self) -> bool:
        return bool(self.state_layers)


def plan_layout(decoder) -> CacheLayout:
    """Group the runs of a decoder by what their mixers need."""
    needs: list[KVCacheNeed] = []
    layer_group: dict[int, int] = {}
    state_layers: dict[int, StateNeed] = {}
    for i, layer in enumerate(decoder.plan.order):
        if decoder.cache_owner[i] != i:
            continue
        need = decoder.blocks[layer].mixer.cache_need()
        for one in (need if isinstance(need, tuple) else (need,)):  # (a mixer made of two mixers states a pair of needs)
            if isinstance(one, KVCacheNeed):
                if i in layer_group:
                    raise TypeError(f"layer {i}: one run keeps one set of pages")
                if one not in needs:
                    needs.append(one)
                layer_group[i] = needs.index(one)
            elif isinstance(one, StateNeed):
                if i in state_layers:
                    raise TypeError(f"layer {i}: one run keeps one state")
                state_layers[i] = one
            elif one is not None:
                raise TypeError(f"layer {i}: unknown cache need {one!r}")
    # (a group with pooled blocks keeps every page: the pooled entries of a request lie in its first pages)
    groups = [GroupSpec(window=0 if n.pooled_block else n.window, keep_first=0 if n.pooled_block else n.keep_first) for n in needs] or [GroupSpec()]
    return CacheLayout(groups, needs, layer_group, state_layers)


class CacheStorage:
    def __init__(self, decoder, layout: CacheLayout, num_blocks: int, block_size: int, num_state_slots: int,
                 dtype: torch.dtype, device: torch.device):
        self.layout, self.block_size, self.dtype = layout, block_size, dtype
        self.spare_block = num_blocks  # never handed out by the manager
        self.spare_slot = num_state_slots
        self.kv: dict[int, tuple[torch.Tensor, torch.Tensor]] = {}
        self.state: dict[int, torch.Tensor] = {}
        self.pooled: dict[int, tuple[torch.Tensor, torch.Tensor]] = {}
        for i, g in layout.layer_group.items():
            need = layout.group_needs[g]
            k = torch.zeros((num_blocks + 1, need.num_kv_heads, block_size, need.head_dim), dtype=dtype, device=device)
            v = torch.zeros((num_blocks + 1, need.num_kv_heads, need.v_dim, block_size), dtype=dtype, device=device)
            self.kv[i] = (k, v)
            if need.pooled_block:
                self.pooled[i] = (torch.zeros_like(k), torch.zeros_like(v))
        for i, need in layout.state_layers.items():
            self.state[i] = torch.zeros((num_state_slots + 1, *need.shape), dtype=need.dtype, device=device)
        for r, owner in enumerate(decoder.cache_owner):
            pages = state = None
            if owner in self.kv:
                k, v = self.kv[owner]
                kp, vp = self.pooled.get(owner, (None, None))
                pages = KVBinding(layout.layer_group[owner], k, v, block_size, kp, vp)
            if r in self.state:
                state = StateBinding(self.state[r])
            need = decoder.blocks[decoder.plan.order[r]].mixer.cache_need()
            if isinstance(need, tuple):  # a mixer made of two mixers: each one's binding, in the order of its needs
                decoder.bindings[r] = PairBinding(*(pages if isinstance(one, KVCacheNeed) else state if isinstance(one, StateNeed) else None
                                                    for one in need))
            elif pages is not None or state is not None:
                decoder.bindings[r] = pages if pages is not None else state

    def kv_bytes_per_token(self) -> int:
        """Bytes of keys and values one token occupies over all runs that own pages."""
        elem = torch.empty((), dtype=self.dtype).element_size()
        return sum(self.layout.group_needs[g].num_kv_heads * (self.layout.group_needs[g].head_dim + self.layout.group_needs[g].v_dim) * elem
                   * (2 if self.layout.group_needs[g].pooled_block else 1) for g in self.layout.layer_group.values())

    def zero_state(self, slots: list[int]) -> None:
        if self.state and slots:
            idx = torch.tensor(slots, dtype=torch.long, device=next(iter(self.state.values())).device)
            for s in self.state.values():
                s.index_fill_(0, idx, 0)
