"""Device tensors behind the cache manager's page ids and slots.

Per group: keys ``[entries, pages, nkv, P, d]`` and values
``[entries, pages, nkv, d, P]`` (values transposed inside a page, so that both
the key rows of a page and the value columns of a page are contiguous for the
attention kernels).  The reference keeps ``[pages, P, nkv, d]`` per layer for both
(tokasaurus/model/kv_cache.py:27-54).  Per run entry with fixed-size state:
``[slots, *shape]``.
"""

from __future__ import annotations

import torch

from tokasaurus_amd.cache.manager import CacheGroup
from tokasaurus_amd.parts.base import StateNeed


class CacheStorage:
    def __init__(
        self,
        groups: list[CacheGroup],
        num_pages: list[int],
        page_size: int,
        state_needs: list[StateNeed | None],
        max_slots: int,
        dtype: torch.dtype,
        device: torch.device,
    ):
        self.page_size = page_size
        self.keys: list[torch.Tensor] = []
        self.values: list[torch.Tensor] = []
        for grp, n in zip(groups, num_pages):
            nkv, d = grp.need.num_kv_heads, grp.need.head_dim
            self.keys.append(torch.zeros((len(grp.entries), n, nkv, page_size, d), dtype=dtype, device=device))
            self.values.append(torch.zeros((len(grp.entries), n, nkv, d, page_size), dtype=dtype, device=device))
        self.states: list[torch.Tensor | None] = [
            torch.zeros((max_slots, *need.shape), dtype=need.dtype, device=device) if need is not None else None
            for need in state_needs
        ]
        self.last_token = torch.zeros((max_slots,), dtype=torch.int32, device=device)

    def bytes(self) -> int:
        return sum(t.numel() * t.element_size() for t in self.keys + self.values)
