"""The cache manager: pages, block tables and state slots (bookkeeping in the C++ host library).

``CacheGroupSpec`` describes a group of layers with the same needs (page size, keep everything or
a window); each group has a pool of pages of its own and each request a block table per group.
``CacheManager`` wraps the native manager; see ``csrc/host/cache_manager.h`` for the policy and its
sources in the reference (crates/vipera-runtime/src/kv.rs).
"""
from __future__ import annotations

import ctypes
from dataclasses import dataclass
from typing import List, Sequence

from ..errors import InfeasibleError, InternalError, InvalidArgumentError
from ..ops.build import load_module

RESERVE_OK, RESERVE_NO_PAGES, RESERVE_NO_SLOT, RESERVE_NEVER_FITS = 0, 1, 2, 3


@dataclass(frozen=True)
class CacheGroupSpec:
    block_size: int
    num_blocks: int
    window: int = 0  # 0: every position is kept


def _host():
    library = load_module("host")
    if getattr(library, "_vk_typed", False):
        return library
    c = ctypes
    u64, i, p = c.c_ulonglong, c.c_int, c.c_void_p
    ip = c.POINTER(c.c_int)
    up = c.POINTER(c.c_ulonglong)
    table = {
        "vk_cache_create": ([i, ip, ip, ip, i], p),
        "vk_cache_destroy": ([p], None),
        "vk_cache_reserve": ([p, u64, i, i], i),
        "vk_cache_advance": ([p, u64, i], None),
        "vk_cache_release": ([p, u64], i),
        "vk_cache_table": ([p, u64, i, ip, i], i),
        "vk_cache_fill_tables": ([p, c.POINTER(u64), i, i, ip, i, ip, ip], i),
        "vk_cache_allocate_nanos": ([p], u64),
        "vk_cache_slot": ([p, u64], i),
        "vk_cache_knows": ([p, u64], i),
        "vk_cache_free_blocks": ([p, i], i),
        "vk_cache_used_blocks": ([p, i], i),
        "vk_cache_free_slots": ([p], i),
        "vk_cache_live_requests": ([p], i),
        "vk_cache_blocks_needed": ([p, i, i, i], i),
        "vk_cache_check": ([p, c.c_char_p, i], i),
        "vk_sched_create": ([p, i, i, i, i, i], p),
        "vk_sched_destroy": ([p], None),
        "vk_sched_add": ([p, u64, ip, i, i], i),
        "vk_sched_plan": ([p, ip, ip], i),
        "vk_sched_plan_read": ([p, up, ip, ip, ip, ip, up], None),
        "vk_sched_advance": ([p, u64], None),
        "vk_sched_append": ([p, u64, i, i], i),
        "vk_sched_replace_token": ([p, u64, i, i], i),
        "vk_sched_cancel": ([p, u64], i),
        "vk_sched_has_work": ([p], i),
        "vk_sched_num_waiting": ([p], i),
        "vk_sched_num_running": ([p], i),
        "vk_sched_preemptions": ([p], i),
        "vk_sched_generated_of": ([p, u64], i),
        "vk_sched_length_of": ([p, u64], i),
    }
    for name, (argtypes, restype) in table.items():
        fn = getattr(library, name)
        fn.argtypes = argtypes
        fn.restype = restype
    library._vk_typed = True
    return library


class CacheManager:
    """Pages and slots of all live requests. Request ids are non-negative integers."""

    def __init__(self, groups: Sequence[CacheGroupSpec], num_slots: int):
        for index, group in enumerate(groups):
            if group.block_size < 1 or group.num_blocks < 0 or group.window < 0:
                raise InvalidArgumentError(f"cache group {index} has invalid geometry: {group}")
        if num_slots < 1:
            raise InvalidArgumentError(f"the cache needs at least one state slot, got {num_slots}")
        self.groups: List[CacheGroupSpec] = list(groups)
        self.num_slots = num_slots
        self._lib = _host()
        n = len(self.groups)
        arr = ctypes.c_int * max(n, 1)
        self._handle = self._lib.vk_cache_create(
            n, arr(*[g.block_size for g in self.groups]), arr(*[g.num_blocks for g in self.groups]),
            arr(*[g.window for g in self.groups]), num_slots)
        if not self._handle:
            raise InternalError("the native cache manager could not be created")

    def __del__(self):
        handle, self._handle = getattr(self, "_handle", None), None
        if handle:
            self._lib.vk_cache_destroy(handle)

    # --- allocation -------------------------------------------------------------------------
    def try_reserve(self, request: int, start: int, total: int) -> int:
        """Pages (and, for a new request, a slot) for tokens ``[start, total)``; returns a RESERVE_* code."""
        return self._lib.vk_cache_reserve(self._handle, request, start, total)

    def reserve(self, request: int, start: int, total: int) -> None:
        """Like :meth:`try_reserve`, raising when it cannot be done."""
        code = self.try_reserve(request, start, total)
        if code == RESERVE_OK:
            return
        if code == RESERVE_NO_PAGES:
            used = ", ".join(f"{self.used_blocks(g)} of {grp.num_blocks}" for g, grp in enumerate(self.groups))
            raise InfeasibleError(
                f"the cache is full: pages in use per group: {used}; request {request} needs room for "
                f"tokens {start}..{total}")
        if code == RESERVE_NO_SLOT:
            raise InfeasibleError(f"all {self.num_slots} request slots are taken; request {request} cannot start")
        raise InfeasibleError(
            f"request {request} needs more pages for {total} tokens than the cache has in total; "
            "shorten the context or give the cache more pages")

    def advance(self, request: int, processed: int) -> None:
        """Give back the pages that no position at or after ``processed`` can see."""
        self._lib.vk_cache_advance(self._handle, request, processed)

    def release(self, request: int) -> None:
        if self._lib.vk_cache_release(self._handle, request) != 0:
            raise InvalidArgumentError(f"request {request} holds nothing in the cache")

    # --- queries ------------------------------------------------------------------------------
    def knows(self, request: int) -> bool:
        return bool(self._lib.vk_cache_knows(self._handle, request))

    def table(self, request: int, group: int) -> List[int]:
        n = self._lib.vk_cache_table(self._handle, request, group, None, 0)
        if n == 0:
            return []
        buf = (ctypes.c_int * n)()
        self._lib.vk_cache_table(self._handle, request, group, buf, n)
        return list(buf)

    def table_into(self, request: int, group: int, buffer, capacity: int) -> int:
        """Write the table into a ctypes int array; returns its length."""
        return self._lib.vk_cache_table(self._handle, request, group, buffer, capacity)

    def fill_tables(self, requests, group: int, out, need_from, need_to) -> int:
        """Write the block tables of ``requests`` into the rows of ``out`` (a C-contiguous int32 array
        ``[len(requests), width]``, -1 where no page is held) and check that logical blocks
        ``[need_from[k], need_to[k])`` of every request are backed by pages.  Returns -1, or the index
        of the first request that fails the check."""
        count = len(requests)
        ids = (ctypes.c_ulonglong * count)(*requests)
        lo = (ctypes.c_int * count)(*need_from)
        hi = (ctypes.c_int * count)(*need_to)
        return self._lib.vk_cache_fill_tables(self._handle, ids, count, group,
                                              out.ctypes.data_as(ctypes.POINTER(ctypes.c_int)), out.shape[1], lo, hi)

    def slot(self, request: int) -> int:
        return self._lib.vk_cache_slot(self._handle, request)

    def free_blocks(self, group: int) -> int:
        return self._lib.vk_cache_free_blocks(self._handle, group)

    def used_blocks(self, group: int) -> int:
        return self._lib.vk_cache_used_blocks(self._handle, group)

    def free_slots(self) -> int:
        return self._lib.vk_cache_free_slots(self._handle)

    def live_requests(self) -> int:
        return self._lib.vk_cache_live_requests(self._handle)

    def blocks_needed(self, group: int, total: int, portion: int) -> int:
        return self._lib.vk_cache_blocks_needed(self._handle, group, total, portion)

    def allocate_micros(self) -> int:
        """Microseconds spent so far in reserving, advancing and releasing, whoever asked (a scheduler, a replay)."""
        return int(self._lib.vk_cache_allocate_nanos(self._handle) // 1000)

    def check(self) -> str:
        """Empty when every page and slot is free or held exactly once; else what is wrong."""
        buf = ctypes.create_string_buffer(4096)
        self._lib.vk_cache_check(self._handle, buf, 4096)
        return buf.value.decode()
