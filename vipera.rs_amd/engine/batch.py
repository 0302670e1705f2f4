"""The batch of one step as the parts see it: flat tokens with per-token and per-entry metadata.

A step holds *entries*; an entry is a request with its next tokens (a portion of a prompt, or one
decoded token).  All tokens of all entries form one flat batch.  The reference's interface has the
same shape (``BatchEntry`` with ``new_tokens``, ``first_position`` and ``block_table``,
crates/vipera-runtime/src/pipeline.rs:138-152) but its CPU backend runs mixed entries one after
another (crates/vipera-backend-cpu/src/model.rs:796-827); here a mixed batch is the normal case.

Everything is packed into one int32 host buffer and copied to the device once.  The packing has a
fixed order of sections, so a step of single tokens can also be copied into the standing buffer of
a captured graph.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, List, Optional, Sequence

import numpy as np
import torch

from ..errors import InternalError, InvalidArgumentError

TILE_TOKENS = 128  # tokens of one prompt tile of the matrix-core attention kernel


@dataclass
class StepEntry:
    """One request's share of a step: ``tokens`` start at position ``start``; ``want`` lists the
    indices (within ``tokens``) whose logits are asked for."""

    request: int
    start: int
    tokens: Sequence[int]
    want: Sequence[int] = ()
    source: int = -1   # >= 0 (single-token entries only): the token is row ``source`` of the sampler's last output on the device


@dataclass
class StepBatch:
    num_tokens: int
    num_entries: int
    num_logit_rows: int
    tokens: torch.Tensor           # [T] int32
    positions: torch.Tensor        # [T] int32
    entry_of_token: torch.Tensor   # [T] int32
    entry_start: torch.Tensor      # [E + 1] int32, offsets of the entries' tokens
    entry_first_pos: torch.Tensor  # [E] int32
    entry_kv_len: torch.Tensor     # [E] int32, tokens in the cache after this step
    slots: torch.Tensor            # [E] int32, state slot of each entry's request
    logit_rows: torch.Tensor       # [R] int32, flat token indices
    prefill_tiles: torch.Tensor    # [tiles, 2] int32: (entry, first token within it) per 128 tokens of multi-token entries
    decode_entries: torch.Tensor   # [n] int32: entries that hold exactly one token
    block_tables: Dict[int, torch.Tensor]  # group -> [E, width] int32
    token_source: Optional[torch.Tensor] = None    # [T] int32: -1, or the row of `sampled_tokens` that holds the token
    sampled_tokens: Optional[torch.Tensor] = None  # the sampler's output buffer on the device (set by the runner)
    shared: Dict[object, torch.Tensor] = field(default_factory=dict)  # what parts compute once per step for all layers
    # launch decisions that depend on more than the step's shapes (on ``sum_decode_kv_len``), noted by whoever takes
    # them: a captured step is shared between the cases in which they come out the same
    launch_plans: List[tuple] = field(default_factory=list)
    # host copies, for launch decisions
    host_counts: List[int] = field(default_factory=list)
    host_first_pos: List[int] = field(default_factory=list)
    host_slots: List[int] = field(default_factory=list)
    max_count: int = 0
    max_kv_len: int = 0
    all_single: bool = False
    num_prefill_tiles: int = 0
    prefill_tile_tokens: int = TILE_TOKENS   # tokens of one entry of `prefill_tiles`
    num_decode_entries: int = 0
    max_decode_kv_len: int = 0
    sum_decode_kv_len: int = 0     # positions that the single-token entries see, added up (a captured step: assumed)
    max_tile_reach: int = 0        # positions that the last token of the longest prompt tile sees (no window counted)
    sum_tile_reach: int = 0        # the same, added over the prompt tiles


@dataclass
class PackedStep:
    """Host side of a step: the sections in their fixed order, and what the launch decisions need."""

    sections: List[np.ndarray]     # tokens, positions, entry_of, starts, first, kv_len, slots, rows, tiles, singles, sources, tables...
    table_widths: List[int]
    num_tokens: int
    num_entries: int
    num_logit_rows: int
    counts: List[int]
    first: List[int]
    slots: List[int]
    max_kv_len: int
    max_decode_kv_len: int
    max_tile_reach: int = 0
    sum_tile_reach: int = 0
    sum_decode_kv_len: int = 0

    def flat(self) -> np.ndarray:
        return np.concatenate([s.reshape(-1) for s in self.sections]) if self.sections else np.zeros(0, np.int32)


def pack_entries(entries: Sequence[StepEntry], cache, vocab_size: int, min_table_width: int = 1,
                 pad_entries: int = 0, pad_slot: int = 0) -> PackedStep:
    """Check ``entries`` and lay them out for the device.

    The pages of every token must already be reserved in ``cache``.  ``pad_entries`` appends
    single-token dummy entries (token 0 at position 0, every table entry the scratch page of its group, which is
    the page past the pool's last, state slot ``pad_slot``), which a captured graph of a fixed batch size needs; their logits are computed and
    ignored, and what they write goes to the scratch page and the scratch state row, which belong to
    no request.  A step of padding only (no ``entries``) is what a graph is warmed up and captured on.
    """
    if not entries and pad_entries < 1:
        raise InvalidArgumentError("a step needs at least one entry")
    counts = [len(e.tokens) for e in entries]
    if counts and min(counts) < 1:
        raise InvalidArgumentError("every entry of a step needs at least one token")
    seen = set()
    for e in entries:
        if e.request in seen:
            raise InvalidArgumentError(f"request {e.request} appears twice in one step")
        seen.add(e.request)
    real = len(entries)
    T_real = sum(counts)
    flat = np.fromiter((t for e in entries for t in e.tokens), dtype=np.int64, count=T_real)
    if T_real and (flat.min() < 0 or flat.max() >= vocab_size):
        bad = int(flat[(flat < 0) | (flat >= vocab_size)][0])
        raise InvalidArgumentError(f"token {bad} is outside the vocabulary of {vocab_size}")
    first_real = [int(e.start) for e in entries]
    if first_real and min(first_real) < 0:
        raise InvalidArgumentError("an entry starts at a negative position")
    slots_real = [cache.slot(e.request) for e in entries]
    if slots_real and min(slots_real) < 0:
        missing = entries[int(np.argmin(slots_real))].request
        raise InternalError(f"request {missing} has no slot: nothing was reserved for it")

    counts_all = counts + [1] * pad_entries
    E = real + pad_entries
    T = T_real + pad_entries
    tokens = np.zeros(T, dtype=np.int32)
    tokens[:T_real] = flat
    starts = np.zeros(E + 1, dtype=np.int32)
    starts[1:] = np.cumsum(counts_all)
    first = np.array(first_real + [0] * pad_entries, dtype=np.int32)
    kv_len = first + np.array(counts_all, dtype=np.int32)
    entry_of = np.repeat(np.arange(E, dtype=np.int32), counts_all)
    positions = np.arange(T, dtype=np.int32) - starts[entry_of] + first[entry_of]
    slots = np.array(slots_real + [pad_slot] * pad_entries, dtype=np.int32)
    rows: List[int] = []
    for k, e in enumerate(entries):
        for w in e.want:
            if not 0 <= w < counts[k]:
                raise InvalidArgumentError(
                    f"request {e.request}: wanted place {w} is outside its {counts[k]} tokens of this step")
            rows.append(int(starts[k]) + int(w))
    sources = np.full(T, -1, dtype=np.int32)
    for k, e in enumerate(entries):
        if e.source >= 0:
            if counts[k] != 1:
                raise InvalidArgumentError(f"request {e.request}: only a single-token entry can take its token from the device")
            sources[int(starts[k])] = e.source
    tile_list: List[tuple] = []
    singles: List[int] = []
    for k, n in enumerate(counts_all):
        if n == 1:
            singles.append(k)
        else:
            for off in range(0, n, TILE_TOKENS):
                tile_list.append((int(first[k]) + off, k, off))
    # by rising number of visible positions: the attention kernel pairs long tiles with short ones
    tile_list.sort()
    tiles: List[int] = [x for _, k, off in tile_list for x in (k, off)]
    tile_reach = [p + min(TILE_TOKENS, int(counts_all[k]) - off) for p, k, off in tile_list]  # positions a tile's last token sees
    max_decode_kv = max((int(kv_len[k]) for k in singles), default=0)
    sum_decode_kv = sum(int(kv_len[k]) for k in singles)

    tables, widths = [], []
    requests = [e.request for e in entries]
    for g, spec in enumerate(cache.groups):
        width = max(min_table_width, int((int(kv_len.max()) + spec.block_size - 1) // spec.block_size))
        table = np.empty((E, width), dtype=np.int32)
        need_to = [(int(kv_len[k]) + spec.block_size - 1) // spec.block_size for k in range(real)]
        if spec.window > 0:
            need_from = [max(0, e.start + 1 - spec.window) // spec.block_size for e in entries]
        else:
            need_from = [0] * real
        failed = cache.fill_tables(requests, g, table, need_from, need_to) if real else -1
        if failed >= 0:
            e = entries[failed]
            lo = max(0, e.start + 1 - spec.window) if spec.window > 0 else 0
            raise InternalError(
                f"request {e.request}: positions {lo}..{int(kv_len[failed]) - 1} are not all backed by pages "
                f"in cache group {g}; reserve before the step")
        if pad_entries:
            table[real:, :] = spec.num_blocks
        tables.append(table)
        widths.append(width)
    sections = [tokens, positions, entry_of, starts, first, kv_len.astype(np.int32), slots,
                np.array(rows, dtype=np.int32), np.array(tiles, dtype=np.int32), np.array(singles, dtype=np.int32),
                sources]
    sections += tables
    return PackedStep(sections, widths, T, E, len(rows), counts_all, [int(v) for v in first], [int(v) for v in slots],
                      int(kv_len.max()), max_decode_kv, max(tile_reach, default=0), sum(tile_reach), sum_decode_kv)


def batch_from_buffer(packed: PackedStep, dev: torch.Tensor) -> StepBatch:
    """A StepBatch whose tensors are views of ``dev``, which holds ``packed.flat()``."""
    views, at = [], 0
    for section in packed.sections:
        views.append(dev[at:at + section.size])
        at += section.size
    E = packed.num_entries
    fixed = 11
    block_tables = {g: views[fixed + g].view(E, packed.table_widths[g]) for g in range(len(packed.table_widths))}
    return StepBatch(
        num_tokens=packed.num_tokens, num_entries=E, num_logit_rows=packed.num_logit_rows,
        tokens=views[0], positions=views[1], entry_of_token=views[2], entry_start=views[3],
        entry_first_pos=views[4], entry_kv_len=views[5], slots=views[6], logit_rows=views[7],
        prefill_tiles=views[8].view(-1, 2), decode_entries=views[9], block_tables=block_tables,
        token_source=views[10],
        host_counts=packed.counts, host_first_pos=packed.first, host_slots=packed.slots,
        max_count=max(packed.counts), max_kv_len=packed.max_kv_len, all_single=max(packed.counts) == 1,
        num_prefill_tiles=packed.sections[8].size // 2, num_decode_entries=packed.sections[9].size,
        max_decode_kv_len=packed.max_decode_kv_len, max_tile_reach=packed.max_tile_reach,
        sum_tile_reach=packed.sum_tile_reach, sum_decode_kv_len=packed.sum_decode_kv_len,
    )


def build_batch(entries: Sequence[StepEntry], cache, vocab_size: int, device, min_table_width: int = 1) -> StepBatch:
    """Pack ``entries`` and copy them to the device."""
    packed = pack_entries(entries, cache, vocab_size, min_table_width)
    host = torch.from_numpy(packed.flat())
    dev = host.pin_memory().to(device, non_blocking=True) if device.type == "cuda" else host
    return batch_from_buffer(packed, dev)
