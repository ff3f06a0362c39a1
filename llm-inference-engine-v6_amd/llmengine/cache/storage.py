"""Device memory of the caches: for every cache a model's schedule names, the
paged tensors (one row per page of its group's pool) and the state tensors (one
row per request slot). The reference keeps one host pool indexed
[block][K|V][layer][token][kv head][dim] (src/paged_kv.cpp:49-66); here every
layer has tensors of its own, in the layout its mixer asks for, and layers of one
group are indexed by the same page ids."""
from __future__ import annotations

import torch

from ..parts.base import PAGE, CacheSpec, LayerCache
from .manager import GroupSpec


def group_name(spec: CacheSpec) -> str:
    kind, window = spec.group_key
    return "full" if kind == "full" else f"window{window}"


def plan_groups(specs: dict[int, CacheSpec | None], num_pages: int | dict[str, int]) -> list[GroupSpec]:
    """The page groups that a model's cache specs ask for. `num_pages`: pages of every
    group's pool, or a number per group name."""
    groups: dict[str, GroupSpec] = {}
    for spec in specs.values():
        if spec is None or not spec.paged:
            continue
        name = group_name(spec)
        if name not in groups:
            n = num_pages[name] if isinstance(num_pages, dict) else num_pages
            groups[name] = GroupSpec(name=name, kind=spec.kind, window=spec.window, num_pages=int(n))
    return list(groups.values())


class CacheStorage:
    def __init__(self, specs: dict[int, CacheSpec | None], groups: list[GroupSpec], page_size: int,
                 num_slots: int, dtype: torch.dtype, device: torch.device):
        self.page_size = page_size
        pages = {g.name: g.num_pages for g in groups}
        self.layers: dict[int, LayerCache | None] = {}
        self.bytes = 0
        for cache_id, spec in specs.items():
            if spec is None:
                self.layers[cache_id] = None
                continue
            group = group_name(spec) if spec.paged else None
            paged = {}
            for name, (shape, page_dtype) in spec.paged_tensors(dtype).items():
                full = (pages[group],) + tuple(page_size if d == PAGE else d for d in shape)
                paged[name] = torch.zeros(full, dtype=page_dtype, device=device)
                self.bytes += paged[name].numel() * paged[name].element_size()
            state = {}
            for name, (shape, sdtype) in spec.state.items():
                state[name] = torch.zeros((num_slots,) + tuple(shape), dtype=sdtype, device=device)
                self.bytes += state[name].numel() * state[name].element_size()
            self.layers[cache_id] = LayerCache(paged=paged, state=state, page_size=page_size, group=group)

    def clear_slot(self, slot: int) -> None:
        """A request is admitted into this slot: its fixed-size state starts at zero."""
        for layer in self.layers.values():
            if layer is not None:
                for t in layer.state.values():
                    t[slot].zero_()
