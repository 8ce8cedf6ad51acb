"""Device memory behind the cache manager, and the grouping of runs.

The reference allocates per layer [2, num_blocks, P, nkv, hd]
(engine/generation/model_runner.py:420-437).  Here each group of runs has one
pair of tensors: keys [runs, num_pages, nkv, P, hd] and values, transposed inside a
page, [runs, num_pages, nkv, hd, P].  One key/value head's part of a page is contiguous
in both; keys are contiguous along the head size (the reduction of q.k) and values along
the positions (the reduction of p.v), which is what the matrix-core kernels read without
a transpose.  A run's view is `LayerCache`.
A group of latent runs (one vector per token that all heads share) has one tensor
[runs, num_pages, P, dim] and no second one.
Per-request state of fixed size lives in [num_slots + 1, *shape] tensors, one per run
and name that asks for it (a run may keep pages and several states); the last row (`idle_slot`) belongs to no request: the idle lanes of a
captured decode batch point there, so whatever a part writes for them lands nowhere.
"""

from __future__ import annotations

from dataclasses import dataclass, field

import torch

from tokensprint_amd.cache.pages import GroupLayout
from tokensprint_amd.parts.base import PagedKVNeed, PagedLatentNeed, SlotStateNeed, flat_needs


def group_runs(needs) -> tuple[list[GroupLayout], dict[int, int]]:
    """Group the runs that own a paged cache by (kv heads, head size, window, kind)."""
    keyed: dict[tuple, list[int]] = {}
    for r, need in enumerate(needs):
        paged = [n for n in flat_needs(need) if isinstance(n, (PagedKVNeed, PagedLatentNeed))]
        if len(paged) > 1:
            raise ValueError(f"run {r} asks for {len(paged)} paged caches; a run owns one")
        for n in paged:
            if isinstance(n, PagedKVNeed):
                keyed.setdefault((n.num_kv_heads, n.head_dim, n.window, "kv"), []).append(r)
            else:
                keyed.setdefault((1, n.dim, n.window, "latent"), []).append(r)
    groups, group_of_run = [], {}
    for g, (key, runs) in enumerate(keyed.items()):
        groups.append(GroupLayout(key[0], key[1], key[2], tuple(runs), key[3]))
        for r in runs:
            group_of_run[r] = g
    return groups, group_of_run


def page_bytes(groups: list[GroupLayout], page_size: int, dtype: torch.dtype) -> int:
    """Bytes one page id costs summed over all groups (each group has its own pool)."""
    item = torch.empty((), dtype=dtype).element_size()
    return sum(len(g.runs) * (1 if g.kind == "latent" else 2) * g.num_kv_heads * page_size
               * g.head_dim * item for g in groups)


def state_bytes(needs, num_slots: int) -> int:
    """Bytes the fixed-size per-request states of all runs take for `num_slots` slots (and
    the spare one)."""
    total = 0
    for need in needs:
        for n in flat_needs(need):
            if isinstance(n, SlotStateNeed):
                count = 1
                for d in n.shape:
                    count *= d
                total += (num_slots + 1) * count * torch.empty((), dtype=n.dtype).element_size()
    return total


@dataclass
class LayerCache:
    """The cache of one run, as a mixer sees it."""

    group: int                     # index into the batch's block tables
    page_size: int
    num_pages: int
    k_pages: torch.Tensor | None   # [num_pages, nkv, P, hd]; a latent run's [num_pages, P, dim]
    v_pages: torch.Tensor | None   # [num_pages, nkv, hd, P]; None for a latent run
    state: torch.Tensor | None = None   # [num_slots + 1, *shape]: the first fixed-size state
    states: dict = field(default_factory=dict)   # every fixed-size state of the run, by name


class CacheStorage:
    def __init__(self, needs, page_size: int, num_pages, num_slots: int,
                 dtype: torch.dtype, device) -> None:
        self.groups, group_of_run = group_runs(needs)
        counts = [num_pages] * len(self.groups) if isinstance(num_pages, int) else list(num_pages)
        self.page_size, self.num_pages, self.num_slots = page_size, counts, num_slots
        self.k_tensors, self.v_tensors = [], []
        for g, n in zip(self.groups, counts):
            if g.kind == "latent":
                self.k_tensors.append(torch.zeros(
                    len(g.runs), n, page_size, g.head_dim, dtype=dtype, device=device))
                self.v_tensors.append(None)
                continue
            self.k_tensors.append(torch.zeros(
                len(g.runs), n, g.num_kv_heads, page_size, g.head_dim, dtype=dtype, device=device))
            self.v_tensors.append(torch.zeros(
                len(g.runs), n, g.num_kv_heads, g.head_dim, page_size, dtype=dtype, device=device))
        self.idle_slot = num_slots
        self.state_runs = tuple(r for r, need in enumerate(needs)
                                if any(isinstance(n, SlotStateNeed) for n in flat_needs(need)))
        self.views: list[LayerCache | None] = []
        for r, need in enumerate(needs):
            parts = flat_needs(need)
            if not parts:
                self.views.append(None)
                continue
            view = LayerCache(-1, page_size, 0, None, None)
            if r in group_of_run:
                g = group_of_run[r]
                i = self.groups[g].runs.index(r)
                v = self.v_tensors[g]
                view = LayerCache(g, page_size, counts[g], self.k_tensors[g][i],
                                  None if v is None else v[i])
            for n in parts:
                if isinstance(n, SlotStateNeed):
                    if n.name in view.states:
                        raise ValueError(f"run {r} asks for two states named '{n.name}'")
                    view.states[n.name] = torch.zeros(num_slots + 1, *n.shape, dtype=n.dtype,
                                                      device=device)
                    if view.state is None:
                        view.state = view.states[n.name]
            self.views.append(view)
