"""Device memory of the caches: paged keys and values per cache-owning layer entry, and state slots.

Layout of the paged tensors: keys ``[pages + 1, kv_heads, block_size, head_dim]``, values transposed
``[pages + 1, kv_heads, head_dim, block_size]`` (the attention kernels read consecutive positions of
one output dim); the last page is a scratch page that is never handed out, which padding tokens of
a captured step write to.  A state
tensor is ``[slots + 1, *shape]``: the last row is the scratch row of those padding entries
(``CacheStorage.scratch_slot``), so that a mixer that keeps state never sees a padding entry in a live
request's row.  ``slot_table`` (int64 ``[slots + 1, 2]``) holds what every request keeps whatever the model: the
state of its sampling generator and the position of its next token (the reference keeps both per turn,
crates/vipera-runtime/src/engine.rs:130-159, crates/vipera-sampler/src/rng.rs:13-38).
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, List, Optional, Sequence, Tuple, Union

import torch

from ..errors import InvalidArgumentError
from .manager import CacheGroupSpec


@dataclass
class PagedKV:
    k: torch.Tensor
    v: torch.Tensor
    group: int
    block_size: int


def group_key(kv) -> Tuple[int, int]:
    """What makes two cache-owning layers share a group: the same window and the same page size asked for."""
    return int(kv.window), int(kv.block_size)


def group_keys(needs) -> List[Tuple[int, int]]:
    """The groups of a run order, in the order in which its entries first need each."""
    keys: List[Tuple[int, int]] = []
    for need in needs:
        if need.kv is not None and group_key(need.kv) not in keys:
            keys.append(group_key(need.kv))
    return keys


def _per_group(value: Union[int, Sequence[int]], count: int, what: str) -> List[int]:
    if isinstance(value, int):
        return [value] * count
    values = [int(v) for v in value]
    if len(values) != count:
        raise InvalidArgumentError(f"{what} lists {len(values)} values for {count} cache groups")
    return values


def plan_groups(needs, block_size: Union[int, Sequence[int]], num_blocks: Union[int, Sequence[int]]) -> List[CacheGroupSpec]:
    """One group per distinct (window, page size asked for) among the run order's attention entries, in the order
    of :func:`group_keys`.  ``block_size`` and ``num_blocks``: one number for every group, or one per group; a
    page size that a mixer asks for itself (``KVCacheSpec.block_size``) stands."""
    keys = group_keys(needs)
    sizes, counts = _per_group(block_size, len(keys), "block_size"), _per_group(num_blocks, len(keys), "num_blocks")
    return [CacheGroupSpec(asked or sizes[g], counts[g], window) for g, (window, asked) in enumerate(keys)]


class CacheStorage:
    def __init__(self, needs, groups: Sequence[CacheGroupSpec], num_slots: int, runtime):
        self.kv: List[Optional[PagedKV]] = [None] * len(needs)
        self.state: List[Optional[torch.Tensor]] = [None] * len(needs)
        self.groups = list(groups)
        self.bytes = 0
        self.scratch_slot = num_slots
        # what every request keeps whatever the model: the state of its sampling generator and the position of
        # its next token, two 64-bit words per slot, written by the sampling kernel
        self.slot_table = torch.zeros((num_slots + 1, 2), dtype=torch.int64, device=runtime.device)
        self.bytes += self.slot_table.numel() * 8
        for index, need in enumerate(needs):
            if need.owner != index:
                continue
            if need.kv is not None:
                keys = group_keys(needs)
                group = keys.index(group_key(need.kv))
                if group >= len(self.groups) or self.groups[group].window != need.kv.window or (
                        need.kv.block_size and self.groups[group].block_size != need.kv.block_size):
                    raise InvalidArgumentError(
                        f"the cache groups do not match the model: entry {index} needs a window of {need.kv.window}"
                        + (f" in pages of {need.kv.block_size}" if need.kv.block_size else ""))
                spec = self.groups[group]
                k = runtime.zeros((spec.num_blocks + 1, need.kv.kv_heads, spec.block_size, need.kv.head_dim))
                v = runtime.zeros((spec.num_blocks + 1, need.kv.kv_heads, need.kv.value_width, spec.block_size))
                self.kv[index] = PagedKV(k, v, group, spec.block_size)
                self.bytes += (k.numel() + v.numel()) * k.element_size()
            if need.state is not None:
                tensor = torch.zeros((num_slots + 1,) + tuple(need.state.shape), dtype=need.state.dtype,
                                     device=runtime.device)
                self.state[index] = tensor
                self.bytes += tensor.numel() * tensor.element_size()
        for index, need in enumerate(needs):
            if need.owner != index:
                self.kv[index] = self.kv[need.owner]
                self.state[index] = self.state[need.owner]

    def bytes_per_token(self) -> int:
        total = 0
        seen = set()
        for entry in self.kv:
            if entry is not None and id(entry) not in seen:
                seen.add(id(entry))
                total += entry.k.shape[1] * (entry.k.shape[3] + entry.v.shape[2]) * entry.k.element_size()
        return total


def group_position_bytes(needs, element: int) -> List[int]:
    """Bytes per cached position of each group (in the order of :func:`group_keys`), over the entries of ``needs``
    that own their storage; ``element`` is the size of a cached key or value."""
    keys = group_keys(needs)
    out = [0] * len(keys)
    for index, need in enumerate(needs):
        if need.owner == index and need.kv is not None:
            out[keys.index(group_key(need.kv))] += need.kv.bytes_per_position(element)
    return out


def cache_bytes(needs, element: int):
    """``(bytes per cached position, bytes per state slot)`` over the entries of ``needs`` that own their
    storage; ``element`` is the size of a cached key or value."""
    per_position = per_slot = 0
    for index, need in enumerate(needs):
        if need.owner != index:
            continue
        if need.kv is not None:
            per_position += need.kv.bytes_per_position(element)
        if need.state is not None:
            per_slot += need.state.bytes_per_slot()
    return per_position, per_slot
