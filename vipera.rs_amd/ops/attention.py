"""Attention dispatch: which kernel attends over the paged cache for a step's tokens.

A bfloat16 run whose head width and page size allow 16-byte reads uses the matrix-core kernels: one
launch for the tiles of multi-token entries (prompt portions), one (plus the merge) for the entries
that hold a single token, whose positions are split into chunks.  The 32-bit run has a split kernel for
single tokens too (chunks of 256 positions) and a tiled one for prompt portions (64 tokens of a head a
workgroup); everything of odd sizes uses the general 32-bit kernel, which serves both kinds alike.
"""
from __future__ import annotations

import torch

from . import kernels

DECODE_WAVES_WANTED = 512    # enough waves to keep the memory system busy (each keeps a step of loads in flight)
DECODE_CHUNK_MIN = 128       # below this the merge of the chunks costs more than the waves gain
DECODE_CHUNKS_MAX = 128
DECODE_LONG_CHUNKS = (4096, 2048)   # taken where they still make DECODE_LONG_WAVES waves
DECODE_LONG_WAVES = 2048


def decode_chunking(max_kv_len: int, num_entries: int, kv_heads: int, head_blocks: int, total_kv_len: int = 0):
    """``(chunk, chunks)``: positions per chunk (a multiple of 32) and chunks that cover ``max_kv_len``.

    Chunks of 1,024 positions, or shorter while the waves are fewer than 512; with many requests at long contexts
    chunks of 2,048 or 4,096 where those still make 2,048 waves (a wave then streams longer for every merge: 64
    requests x 4 key heads at 32,768 positions read their 4.3 GB at 6.06 TB/s in chunks of 4,096, at 5.68 in chunks
    of 1,024; with 1,024 waves chunks of 2,048 fall to 4.6 TB/s).

    The waves that count are those with positions to read: the chunks past a request's own length end at once.
    ``total_kv_len``, the lengths of all entries added up, says how many there are: the entries count as
    ``total_kv_len / max_kv_len`` full ones (64 requests of 384 to 8,448 positions, 301,000 together, under a
    longest of 16,384: 147 us a layer in chunks of 1,024, 210 in the chunks of 2,048 that 64 full entries would
    get; 16 such requests 31 us in chunks of 512, 36 in chunks of 1,024).  Zero: every entry counts as full."""
    if total_kv_len > 0 and max_kv_len > 0:
        num_entries = max(1, min(num_entries, -(-total_kv_len // max_kv_len)))
    pairs = num_entries * kv_heads * head_blocks
    for chunk in DECODE_LONG_CHUNKS:
        chunks = (max_kv_len + chunk - 1) // chunk
        if pairs * chunks >= DECODE_LONG_WAVES and chunks <= DECODE_CHUNKS_MAX:
            return chunk, chunks
    chunk = 1024
    while chunk > DECODE_CHUNK_MIN:
        chunks = (max_kv_len + chunk - 1) // chunk
        if pairs * chunks >= DECODE_WAVES_WANTED:
            break
        chunk //= 2
    chunks = max(1, (max_kv_len + chunk - 1) // chunk)
    while chunks > DECODE_CHUNKS_MAX:
        chunk *= 2
        chunks = (max_kv_len + chunk - 1) // chunk
    return chunk, chunks


def joins_decode_chunks(chunks: int, num_entries: int, kv_heads: int, head_blocks: int, cus: int,
                        head_dim: int = 128) -> bool:
    """Whether one workgroup per (entry, key head) takes all chunks, a wave each, and merges them itself instead of
    a workgroup per chunk and a second kernel: where those pairs alone fill the GPU (64 requests x 4 key heads on 256
    CUs), so that the chunks only serve to keep several waves on a CU; the merge kernel and the chunks' round trip
    through memory are saved (4.9 us a layer at the 7B head shape).  Not where the pairs are a few more than the CUs:
    the CUs with two workgroups then set the time (72 requests x 4 key heads at 4,096 positions: 141 us joined, 124
    with a workgroup per chunk; 96 requests: 157 and 155; from 112 on joined is ahead again; a captured step of 96
    entries also serves 65 to 95 requests)."""
    pairs = num_entries * kv_heads * head_blocks
    if cus < pairs < 1.55 * cus:
        return False
    if kernels.attn_bf16_padded_width(head_dim) > 128:
        return False    # eight waves a workgroup are two a SIMD: 256 registers each, which a wider head's sums overflow
    return chunks <= kernels.ATTN_DECODE_JOINED_CHUNKS and pairs >= 0.8 * cus


def halves_prompt_tiles(num_tiles: int, heads: int, longest: int, total: int, cus: int) -> bool:
    """Whether the prompt kernel should give every (tile, head) a workgroup of sixteen waves that halve the
    tile's positions between them: when a CU would otherwise be left with a single workgroup of eight for most of
    the step, which runs at about 0.7 of what two reach together.  That is so when the work items are fewer than
    the CUs, or when all of them are resident at once (two per CU) and differ much in length, as the tiles of one
    long prompt do: the longest then runs on alone (measured at 28 heads: one prompt of 2,048 tokens 70.8 to 60.3 us;
    four portions of 512 tokens at position 1,536, all about equally long, 83.6 to 95.7, so they stay unsplit)."""
    items = num_tiles * heads
    if items <= 0:
        return False
    return items <= cus or (items <= 2 * cus and longest * num_tiles >= 1.25 * total)


PROMPT_CHUNK_MIN_TILES = 8   # a chunk of a prompt tile's positions is at least 512 long


def chunks_prompt_tiles(num_tiles: int, heads: int, longest: int, total: int, cus: int):
    """``(chunk_tiles, max_chunks)`` if the prompt kernel should cut every tile's positions into chunks of
    ``chunk_tiles`` steps of 64, a workgroup each, and merge them with a second kernel, else None.  For a model of
    few heads, whose (tile, head) items are fewer than the CUs (12 heads and four portions of 512 tokens are 192
    items) and as long as their prompts, so that the one deepest in its prompt sets the time.  The chunks are sized
    to give every CU about two workgroups (sizes for one to six measured the same); a tile's partial results (128
    columns x head width in 32-bit per chunk) go through memory, which is why the chunks are no shorter than 512
    positions.  Chosen where an estimate says it pays: a workgroup of sixteen waves that halves a tile takes about
    1.45 us per step of 64 positions, two workgroups of eight on a CU 2.9 us each, the chunked launch measured 1.6
    times its ideal, and the merge costs 9 us (the 1.5B shape: a continuous batch with prompts of up to 8,192
    tokens 2.56 to 2.45 s; one prompt of 2,048 tokens stays with the halved tiles, 47 against 55 us a layer)."""
    items = num_tiles * heads
    if items <= 0 or items > cus:
        return None
    steps = (total + 63) // 64 * heads                       # steps of 64 positions over all items
    chunk_tiles = max(PROMPT_CHUNK_MIN_TILES, -(-steps // (2 * cus)))
    longest_steps = (longest + 63) // 64
    if longest_steps < 2 * chunk_tiles:
        return None
    halved = 1.45 * longest_steps
    chunked = 1.6 * max(2.9 * chunk_tiles, 1.45 * steps / cus) + 9.0
    if halved < 1.25 * chunked:
        return None
    return chunk_tiles, -(-longest_steps // chunk_tiles)


def paged_attention(qkv, k_cache, v_cache, out, batch, table, heads, kv_heads, head_dim, scale, window) -> None:
    if kernels.attn_bf16_supported(qkv, k_cache, head_dim):
        if batch.num_prefill_tiles:
            cus = kernels.compute_units(qkv.device)
            chunked = None
            if kernels.attn_bf16_prefill_loads_directly(k_cache, kv_heads, head_dim):
                chunked = chunks_prompt_tiles(batch.num_prefill_tiles, heads, batch.max_tile_reach, batch.sum_tile_reach, cus)
            split = chunked is None and halves_prompt_tiles(batch.num_prefill_tiles, heads, batch.max_tile_reach,
                                                            batch.sum_tile_reach, cus)
            kernels.attn_bf16_prefill(qkv, k_cache, v_cache, out, batch.prefill_tiles, batch.entry_start,
                                      batch.entry_first_pos, table, heads, kv_heads, head_dim, scale, window, split,
                                      *(chunked or (0, 0)))
        if batch.num_decode_entries:
            group = heads // kv_heads
            visible = batch.max_decode_kv_len
            head_blocks = (group + 15) // 16
            chunk, chunks = decode_chunking(visible, batch.num_decode_entries, kv_heads, head_blocks,
                                            batch.sum_decode_kv_len)
            join = joins_decode_chunks(chunks, batch.num_decode_entries, kv_heads, head_blocks,
                                       kernels.compute_units(qkv.device), head_dim)
            batch.launch_plans.append((chunk, chunks, join))
            partial = None if join else torch.empty(batch.num_decode_entries * heads * chunks * (head_dim + 2),
                                                    dtype=torch.float32, device=qkv.device)
            kernels.attn_bf16_decode(qkv, k_cache, v_cache, out, partial, batch.decode_entries, batch.entry_start,
                                     batch.entry_first_pos, table, heads, kv_heads, head_dim, scale, window, chunk,
                                     chunks, dense=batch.all_single, join=join)
        return
    # the 32-bit run: single tokens on the kernel that splits their positions into chunks and shares the reads among
    # the query heads of a key head, prompt portions on the kernel that walks the positions in LDS tiles; what
    # either does not take (odd widths, pages that are no multiple of 4) is left to the general kernel
    singles = bool(batch.num_decode_entries) and kernels.attn_decode_f32_supported(qkv, k_cache, head_dim)
    portions = bool(batch.num_prefill_tiles) and kernels.attn_prefill_f32_supported(qkv, k_cache, head_dim)
    if singles:
        chunks = (batch.max_decode_kv_len + kernels.ATTN_DECODE_F32_CHUNK - 1) // kernels.ATTN_DECODE_F32_CHUNK
        partial = torch.empty(batch.num_decode_entries * heads * chunks * (head_dim + 2), dtype=torch.float32,
                              device=qkv.device)
        kernels.attn_decode_f32(qkv, k_cache, v_cache, out, partial, batch.decode_entries, batch.entry_start,
                                batch.entry_first_pos, table, heads, kv_heads, head_dim, scale, window, chunks)
    if portions:
        kernels.attn_prefill_f32(qkv, k_cache, v_cache, out, batch.prefill_tiles, batch.prefill_tile_tokens,
                                 batch.entry_start, batch.entry_first_pos, table, heads, kv_heads, head_dim, scale, window)
    if (batch.num_decode_entries and not singles) or (batch.num_prefill_tiles and not portions):
        # the general kernel can leave out the single tokens, not the portions: those it then computes again
        kernels.attn_generic(qkv, k_cache, v_cache, out, batch.positions, batch.entry_of_token, table, heads, kv_heads,
                             head_dim, scale, window, skip_single_of=batch.entry_start if singles else None)
