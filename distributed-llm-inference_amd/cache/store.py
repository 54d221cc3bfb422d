"""Device memory of the cache: page pools per group and state arrays per stateful layer.

Layers are grouped by what their mixers declare (:class:`PagedKVSpec`): equal specs share one
group, one block table per request and one pool tensor
``[layers of the group, 2 (keys, values), pages, kv_heads * page_size * head_dim]``
(where a value's size differs from a key's: one tensor ``[layers, 1, pages, ...]`` for the keys
and one for the values, or none if the mixer keeps no values).
Inside a page, keys lie as ``[kv_heads][page_size][head_dim]`` and values as
``[kv_heads][value_dim][page_size]`` (the order in which the attention kernels consume them).
A mixer that declares a :class:`StateSpec` gets an array ``[state slots + 1, *shape]`` instead: one
row per slot that a request can hold, and a last row (``scratch_slot``) that no request holds, for
the padding rows of a replayed graph to write to. A mixer made of several such mixers declares a
:class:`CompositeCacheSpec`; its cache holds one cache per member, each made as if the member were
a layer of its own.
Everything is allocated once and zero-filled (reference: src/dli/kv/paged_store.py:50-52).
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Optional, Sequence

import torch

from ..parts.base import CompositeCacheSpec, PagedKVSpec, Runtime, StateSpec
from .manager import CopyOp, GroupSpec


@dataclass
class LayerCache:
    """What one schedule entry's mixer gets: its pages (with the group whose block tables index
    them) or its state array. ``writable`` is False for an entry that reads another's cache."""

    kind: str  # "paged", "state" or "composite"
    group: int = -1
    k_pages: Optional[torch.Tensor] = None  # [pages, kv_heads, page_size, head_dim]
    v_pages: Optional[torch.Tensor] = None  # [pages, kv_heads, value_dim, page_size]; None: keys only
    state: Optional[torch.Tensor] = None    # [slots, *shape]
    writable: bool = True
    window: int = 0
    members: Optional[dict] = None          # composite: member name -> LayerCache

    def reader(self) -> "LayerCache":
        members = None if self.members is None else {n: c.reader() for n, c in self.members.items()}
        return LayerCache(self.kind, self.group, self.k_pages, self.v_pages, self.state, False, self.window, members)

    def leaves(self) -> list["LayerCache"]:
        """This cache, or the caches of a composite's members."""
        return [self] if self.members is None else [leaf for c in self.members.values() for leaf in c.leaves()]


def flatten_specs(specs: Sequence[Optional[PagedKVSpec | StateSpec | CompositeCacheSpec]]) -> list:
    """Every paged or state spec in order, a composite's members in its place."""
    flat: list = []
    for s in specs:
        if isinstance(s, CompositeCacheSpec):
            flat.extend(m for _, m in s.members)
        else:
            flat.append(s)
    return flat


def plan_groups(specs: Sequence[Optional[PagedKVSpec | StateSpec]]) -> tuple[list[PagedKVSpec], list[int]]:
    """Distinct paged specs in order of first appearance, and the group of each layer (or member
    of a composite, counted as a layer in its place; -1: none)."""
    groups: list[PagedKVSpec] = []
    of_layer: list[int] = []
    for s in flatten_specs(specs):
        if isinstance(s, PagedKVSpec):
            if s not in groups:
                groups.append(s)
            of_layer.append(groups.index(s))
        else:
            of_layer.append(-1)
    return groups, of_layer


def group_specs(groups: Sequence[PagedKVSpec]) -> list[GroupSpec]:
    return [GroupSpec("window", g.window) if g.window > 0 else GroupSpec() for g in groups] or [GroupSpec()]


def bytes_per_page(groups: Sequence[PagedKVSpec], layers_per_group: Sequence[int], page_size: int,
                   dtype: torch.dtype) -> int:
    """Bytes that one page id costs across all groups and layers, keys and values."""
    item = torch.empty((), dtype=dtype).element_size()
    return sum(n * page_size * (g.kv_heads * g.head_dim + g.v_heads * g.v_dim) * item for g, n in zip(groups, layers_per_group))


class CacheStore:
    def __init__(self, rt: Runtime, specs: Sequence[Optional[PagedKVSpec | StateSpec]], *,
                 num_pages: int, page_size: int, max_seqs: int) -> None:
        self.rt = rt
        self.page_size = page_size
        self.num_pages = num_pages
        self.scratch_slot = max_seqs
        self.groups, self._group_of = plan_groups(specs)
        self.layers_per_group = [self._group_of.count(g) for g in range(len(self.groups))]
        # per group: the tensors [layers, 1 or 2, pages, elements] that hold its pages
        self.pools: list[list[torch.Tensor]] = []
        for g, n_layers in zip(self.groups, self.layers_per_group):
            sizes = [g.kv_heads * page_size * g.head_dim, g.v_heads * page_size * g.v_dim]
            if sizes[0] == sizes[1]:
                shapes = [(n_layers, 2, num_pages, sizes[0])]
            else:
                shapes = [(n_layers, 1, num_pages, n) for n in sizes if n > 0]
            self.pools.append([torch.zeros(shape, device=rt.device, dtype=rt.dtype) for shape in shapes])
        self.layers: list[Optional[LayerCache]] = []
        seen = [0] * len(self.groups)
        at = 0   # index into the flattened list of specs, which is what the groups were planned from

        def make(spec) -> Optional[LayerCache]:
            nonlocal at
            g = self._group_of[at]
            at += 1
            if isinstance(spec, PagedKVSpec):
                i = seen[g]
                seen[g] += 1
                pools = self.pools[g]
                keys = pools[0][i, 0]
                values = pools[0][i, 1] if pools[0].shape[1] == 2 else (pools[1][i, 0] if len(pools) > 1 else None)
                return LayerCache(
                    "paged", g,
                    keys.view(num_pages, spec.kv_heads, page_size, spec.head_dim),
                    None if values is None else values.view(num_pages, spec.v_heads, spec.v_dim, page_size),
                    window=spec.window)
            if isinstance(spec, StateSpec):
                return LayerCache(
                    "state", state=torch.zeros(max_seqs + 1, *spec.shape, device=rt.device, dtype=spec.dtype))
            return None

        for spec in specs:
            if isinstance(spec, CompositeCacheSpec):
                self.layers.append(LayerCache("composite", members={name: make(m) for name, m in spec.members}))
            else:
                self.layers.append(make(spec))

    @property
    def stateful(self) -> bool:
        return any(leaf.kind == "state" for c in self.layers if c is not None for leaf in c.leaves())

    def bytes_per_page(self) -> int:
        return bytes_per_page(self.groups, self.layers_per_group, self.page_size, self.rt.dtype)

    def copy_pages(self, ops_list: Sequence[CopyOp]) -> None:
        """Do the copy-on-write copies of a step, every layer of each group at once
        (reference: src/dli/kv/paged_store.py:110-118)."""
        if not ops_list:
            return
        from ..kernels import ops

        for g, pools in enumerate(self.pools):
            mine = [o for o in ops_list if o.group == g]
            if not mine:
                continue
            for o in mine:
                if not (0 <= o.src < self.num_pages and 0 <= o.dst < self.num_pages):
                    raise ValueError(f"page copy {o} names a page outside the pool")
            src = torch.tensor([o.src for o in mine], dtype=torch.int32, device=self.rt.device)
            dst = torch.tensor([o.dst for o in mine], dtype=torch.int32, device=self.rt.device)
            for pool in pools:
                ops.copy_pages(pool, src, dst)
