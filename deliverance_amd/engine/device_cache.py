"""The device side of the cache: the tensors that pages and state slots index, built from
what the model's mixers say they need, plus the host-side manager that hands pages out.

Layout of one cache slot (one caching layer call): ``[n_pages, 2 (K, V), n_kv_heads,
page_size, head_dim]`` in the compute dtype, so that the rows of one page and head lie next
to each other for the attention kernels.  All slots of a group live in one allocation,
``[n_slots, n_pages, ...]``, and share page ids.  The reference's page is
``[layersPerPage, 2, rowsPerPage, kvLength]`` per request
(core/src/main/java/io/teknek/deliverance/tensor/KvBufferCache.java:588-592,609-623).
"""
from __future__ import annotations

from typing import Dict, List

import torch

from ..cache.manager import CacheManager, KVGroupSpec, StateSpec
from ..config.engine_config import check_page_size
from ..parts.base import KVNeed, StateNeed


class DeviceCache:
    def __init__(self, needs: Dict[int, object], dtype: torch.dtype, device, page_size: int,
                 max_cached_tokens: int, n_state_slots: int, poison_freed: bool = False):
        self.dtype = dtype
        self.device = torch.device(device)
        self.page_size = check_page_size(page_size)
        by_shape: Dict[tuple, List[int]] = {}
        state_specs: List[StateSpec] = []
        state_needs: Dict[int, StateNeed] = {}
        for slot in sorted(needs):
            need = needs[slot]
            if isinstance(need, KVNeed):
                by_shape.setdefault((need.n_kv_heads, need.head_dim, need.window), []).append(slot)
            elif isinstance(need, StateNeed):
                state_specs.append(StateSpec(slot, need.elems))
                state_needs[slot] = need
            else:
                raise TypeError(f"cache slot {slot}: unknown kind of need {need!r}")
        self.groups: List[KVGroupSpec] = [KVGroupSpec(tuple(slots), h, d, w) for (h, d, w), slots in by_shape.items()]
        self.n_pages = -(-max_cached_tokens // page_size)
        self.group_of_slot: Dict[int, int] = {}
        self.kv: Dict[int, torch.Tensor] = {}
        self._group_tensors: List[torch.Tensor] = []
        for g, spec in enumerate(self.groups):
            t = torch.empty((len(spec.slots), self.n_pages, 2, spec.n_kv_heads, page_size, spec.head_dim),
                            dtype=dtype, device=self.device)
            # Pages are never cleared when they change hands (what a request may see is decided
            # by its length); the pool starts as NaN so that a read of a row nobody wrote shows.
            t.fill_(float("nan"))
            self._group_tensors.append(t)
            for i, slot in enumerate(spec.slots):
                self.kv[slot] = t[i]
                self.group_of_slot[slot] = g
        self.state: Dict[int, torch.Tensor] = {}
        n_slots = n_state_slots if state_specs else 0
        for s in state_specs:          # [state slots, *shape] in the dtype the mixer asked for
            need = state_needs[s.slot]
            self.state[s.slot] = torch.zeros((n_slots, *need.row_shape), dtype=need.dtype, device=self.device)
        self.manager = CacheManager(self.groups, page_size, [self.n_pages] * len(self.groups),
                                    state_specs, n_slots)
        if poison_freed:
            # debug runs: a page that goes back is filled with NaN again (after the steps that were
            # launched before, in stream order), so that a row read before its new owner wrote it shows
            self.manager.on_release = self._poison

    def _poison(self, group: int, pages) -> None:
        idx = torch.tensor(list(pages), dtype=torch.long, device=self.device)
        self._group_tensors[group].index_fill_(1, idx, float("nan"))

    def reset_state(self, state_slot: int) -> None:
        """A request that starts gets a zeroed state row in every state tensor."""
        if state_slot >= 0:
            for t in self.state.values():
                t[state_slot].zero_()

    def bytes_per_token(self) -> int:
        el = torch.empty((), dtype=self.dtype).element_size()
        return sum(len(g.slots) * 2 * g.n_kv_heads * g.head_dim * el for g in self.groups)

    def state_bytes(self) -> int:
        return sum(t.numel() * t.element_size() for t in self.state.values())

    @staticmethod
    def state_bytes_for(needs: Dict[int, object], n_state_slots: int) -> int:
        """What the fixed-size state of ``n_state_slots`` requests takes."""
        return n_state_slots * sum(n.nbytes for n in needs.values() if isinstance(n, StateNeed))

    @staticmethod
    def tokens_for_budget(needs: Dict[int, object], dtype: torch.dtype, budget_bytes: int, n_state_slots: int = 0) -> int:
        """How many tokens' keys and values fit into ``budget_bytes`` once the state slots are paid for."""
        el = torch.empty((), dtype=dtype).element_size()
        per_token = sum(2 * n.n_kv_heads * n.head_dim * el for n in needs.values() if isinstance(n, KVNeed))
        left = budget_bytes - DeviceCache.state_bytes_for(needs, n_state_slots)
        return max(0, left // max(per_token, 1))
