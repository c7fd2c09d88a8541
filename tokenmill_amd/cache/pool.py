"""The cache memory on the device.

Per group two tensors in the model's storage type: keys [cache layers of the group, pages,
page_size, kv_heads, head_dim], the reference's layout (reference
src/infer/kv/paged_cache.py:1-6,28-34), and values [cache layers, pages, kv_heads, head_dim,
page_size]: inside a page the values lie key-contiguous for each (head, d), which is the operand
layout of the MFMA attention kernels (no transposition through LDS). Per state-holding layer one
tensor [slots, *shape].
"""
from __future__ import annotations

import torch

from tokenmill_amd.parts.base import KVCacheSpec, KVCacheView, StateSpec, StateView


def group_specs(cache_specs: list) -> tuple[list[KVCacheSpec], list[int | None]]:
    """Distinct KV specs in order of first use, and for each run call its group (or None)."""
    groups: list[KVCacheSpec] = []
    of_call: list[int | None] = []
    for spec in cache_specs:
        if isinstance(spec, KVCacheSpec):
            if spec not in groups:
                groups.append(spec)
            of_call.append(groups.index(spec))
        else:
            of_call.append(None)
    return groups, of_call


class CachePools:
    def __init__(self, model, num_pages: int | list[int], page_size: int, num_state_slots: int, dtype, device):
        specs = model.cache_specs()
        self.groups, group_of_call = group_specs(specs)
        counts = [num_pages] * len(self.groups) if isinstance(num_pages, int) else list(num_pages)
        self.page_size, self.num_pages, self.num_state_slots = page_size, counts, num_state_slots
        members: list[list[int]] = [[] for _ in self.groups]
        for j, g in enumerate(group_of_call):
            if g is not None:
                members[g].append(j)
        self.k = [torch.zeros((len(members[g]), counts[g], page_size, s.kv_heads, s.head_dim), dtype=dtype,
                              device=device) for g, s in enumerate(self.groups)]
        self.v = [torch.zeros((len(members[g]), counts[g], s.kv_heads, s.head_dim, page_size), dtype=dtype,
                              device=device) for g, s in enumerate(self.groups)]
        self.states: dict[int, torch.Tensor] = {}
        views: list = [None] * len(specs)
        for g, calls in enumerate(members):
            for idx, j in enumerate(calls):
                views[j] = KVCacheView(self.k[g][idx], self.v[g][idx], g, True)
        for j, spec in enumerate(specs):
            if isinstance(spec, StateSpec):
                # one row more than there are slots: where the padding rows of a replayed step put their state
                self.states[j] = torch.zeros((num_state_slots + 1, *spec.shape), dtype=spec.dtype, device=device)
                views[j] = StateView(self.states[j])
        for j, call in enumerate(model.run):
            if call.cache_of is not None:
                src = views[call.cache_of]
                views[j] = KVCacheView(src.k, src.v, src.group, False) if isinstance(src, KVCacheView) else src
        self.views = views

    @property
    def padding_state_slot(self) -> int:
        """The state row that belongs to no request."""
        return self.num_state_slots

    @property
    def windows(self) -> list[int | None]:
        return [s.window for s in self.groups]

    def reset_state_slot(self, slot: int) -> None:
        for t in self.states.values():
            t[slot].zero_()

    @property
    def nbytes(self) -> int:
        return sum(t.numel() * t.element_size() for t in self.k + self.v) + \
            sum(t.numel() * t.element_size() for t in self.states.values())

    @staticmethod
    def bytes_per_token(model, dtype) -> int:
        """Cache bytes one token takes over all layers (reference src/infer/config.py:37-39)."""
        size = torch.empty((), dtype=dtype).element_size()
        return sum(2 * s.kv_heads * s.head_dim * size for s in model.cache_specs() if isinstance(s, KVCacheSpec))
