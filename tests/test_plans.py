"""Which kernel a product or an attention step is given: the decisions of ``ops/linear.py`` and ``ops/attention.py``
at the layer sizes of the 1.5B, 7B and 32B shapes.  Pure functions of the sizes: no GPU is touched."""
from vipera_rs_amd.ops.attention import decode_chunking
from vipera_rs_amd.ops.kernels import follow_stride, follow_sumsq_floats
from vipera_rs_amd.ops.linear import (gated_plan, gated_resident_fits, mid_plan, split_qkv_plan, streams_in_wave_order,
                                      streams_weights)

QKV_7B, O_7B, GATE_UP_7B, DOWN_7B, HEAD_7B = (4608, 3584), (3584, 3584), (37888, 3584), (3584, 18944), (152064, 3584)


def test_few_tokens_stream_the_weights_with_k_split_inside_a_workgroup():
    for n, k in (QKV_7B, O_7B, DOWN_7B, HEAD_7B):
        assert streams_in_wave_order(1, n, k) and streams_in_wave_order(4, n, k)
    assert streams_in_wave_order(16, *QKV_7B) and streams_in_wave_order(16, *O_7B)    # small weights: up to 16 tokens
    assert streams_in_wave_order(16, *QKV_7B, rotates=True) and not streams_in_wave_order(17, *QKV_7B)
    assert streams_in_wave_order(5, *DOWN_7B) and not streams_in_wave_order(6, *DOWN_7B)   # 68 M elements, few rows
    assert streams_in_wave_order(8, 1536, 8960) and not streams_in_wave_order(9, 1536, 8960)   # small, with a long K
    assert streams_in_wave_order(6, 2048, 11008) and not streams_in_wave_order(7, 2048, 11008)     # the 3B down projection
    assert streams_in_wave_order(6, 5120, 5120) and not streams_in_wave_order(7, 5120, 5120)
    assert not streams_in_wave_order(1, 5120, 27648) and not streams_in_wave_order(8, 5120, 27648)   # the 32B down projection
    assert streams_in_wave_order(1, 152064, 5120) and not streams_in_wave_order(8, *HEAD_7B)      # many rows: up to 4
    # 60 M elements and 4,096 rows or more: K goes over workgroups from the first token on
    assert not streams_in_wave_order(1, 5120, 13824) and not streams_in_wave_order(1, 8192, 8192)
    # q/k/v, whose second kernel costs more
    assert streams_in_wave_order(3, 10240, 8192, rotates=True) and not streams_in_wave_order(4, 10240, 8192, rotates=True)
    assert streams_in_wave_order(10, 7168, 5120, rotates=True) and not streams_in_wave_order(11, 7168, 5120, rotates=True)


def test_the_lds_shared_product_splits_k_where_rows_are_few():
    assert mid_plan(8, *DOWN_7B) == (4, 1)                 # 56 row blocks x 4 ranges fill 256 CUs
    assert mid_plan(64, *DOWN_7B) == (9, 2)                # many tokens and a long K: two tiles per wave, 28 row blocks x 9
    assert mid_plan(32, 5120, 27648) == (6, 2) and mid_plan(31, 5120, 27648) == (3, 1)
    assert mid_plan(64, 1536, 8960) == (10, 1)             # few rows: one tile per wave, 24 row blocks x 10
    assert mid_plan(32, 2048, 11008) == (8, 1) and mid_plan(8, 5120, 13824) == (3, 1)     # the 3B and 14B down projections
    assert mid_plan(8, *HEAD_7B) == (1, 1) and mid_plan(64, *HEAD_7B) == (1, 2)
    assert mid_plan(64, *QKV_7B) == (3, 1) and mid_plan(64, *O_7B) == (4, 1)
    ranges, _ = mid_plan(64, 2048, 1536)                   # 1.5B q/k/v: no range shorter than 512
    assert 1536 // ranges >= 512


def test_past_64_tokens_the_weights_are_streamed_where_tiles_would_be_few():
    for n, k in (QKV_7B, O_7B, DOWN_7B, HEAD_7B):
        assert streams_weights(64, n, k) and not streams_weights(129, n, k)
    for m in (65, 96, 128):                                # small weights only: the 7B output projection, the 1.5B widths
        assert streams_weights(m, *O_7B) and streams_weights(m, 2048, 1536) and streams_weights(m, 1536, 8960)
        assert not streams_weights(m, *DOWN_7B) and not streams_weights(m, *QKV_7B) and not streams_weights(m, *HEAD_7B)
        assert not streams_weights(m, 5120, 27648)
    assert mid_plan(65, 1536, 8960) == (8, 1) and mid_plan(96, *O_7B) == (4, 1) and mid_plan(128, 2048, 1536) == (4, 1)
    assert mid_plan(100, 1024, 320) == (1, 1)              # no range shorter than 256
    assert mid_plan(65, 896, 4864) == (8, 1)               # the 0.5B down projection


def test_the_gated_product_goes_resident_tiled_or_lds_shared():
    assert gated_resident_fits(16, *GATE_UP_7B) and not gated_resident_fits(17, *GATE_UP_7B)
    assert not gated_resident_fits(16, 55296, 5120)        # 32B: 16 tokens x 5120 do not fit a CU's LDS
    assert gated_resident_fits(8, 55296, 5120)
    assert not gated_resident_fits(8, 37888, 3584 + 64)    # K in whole chunks of 128 only
    assert gated_resident_fits(8, 9728, 896) and gated_plan(8, 9728, 896) == 0     # the 0.5B width: chunks of 128
    for m in (1, 8, 16):
        assert gated_plan(m, *GATE_UP_7B) == 0             # 18,944 outputs over 256 CUs: 72 or 76 each
    assert gated_plan(8, 17920, 1536) == 0                 # 1.5B: 8,960 outputs are 32 or 36 each, and the norm before it is free
    assert gated_plan(8, 55296, 5120) == 0
    assert gated_plan(17, *GATE_UP_7B) == 3 and gated_plan(64, *GATE_UP_7B) == 3   # past the resident kernel: tiled
    assert gated_plan(32, 59136, 8192) == 2 and gated_plan(33, 59136, 8192) == 3   # 72B: LDS-shared up to 32 tokens
    assert gated_plan(8, 59136, 8192) == 0
    assert gated_plan(24, 55296, 5120) == 3
    assert gated_plan(48, 17920, 1536) in (1, 2) and gated_plan(64, 17920, 1536) == 3
    assert gated_plan(8, *GATE_UP_7B, cus=304) == 0        # over 304 CUs: 60 or 64 outputs each
    assert gated_plan(8, *GATE_UP_7B, cus=500) == 0        # over 500: 36 or 40 each, 6 % above the mean
    assert gated_plan(8, 4096, 1024, cus=256) != 0         # 128 pairs over 256 CUs: half of them would have none


def test_q_k_v_rotates_in_the_kernel_that_adds_its_ranges_where_k_is_split():
    assert split_qkv_plan(64, *QKV_7B) == (3, 1) and split_qkv_plan(17, *QKV_7B) == (3, 1)
    assert split_qkv_plan(16, *QKV_7B) is None and split_qkv_plan(65, *QKV_7B) is None
    assert split_qkv_plan(32, 1024, 512) is None           # K too short to split
    # the widest models split from few tokens on, in two ranges where the rows alone would fill the CUs
    assert split_qkv_plan(8, 10240, 8192) == (2, 1) and split_qkv_plan(3, 10240, 8192) is None
    assert split_qkv_plan(16, 7168, 5120) == (2, 1) and split_qkv_plan(8, 7168, 5120) is None


def test_room_for_the_sums_of_squares():
    assert follow_stride(16) == 16 and follow_stride(17) == 64 and follow_stride(64) == 64
    assert follow_stride(65) == 128 and follow_stride(2048) == 2048
    for n in (16, 64, 1000, 3584, 8192):
        assert follow_sumsq_floats(n, 16) >= ((n + 7) // 8) * 16          # a workgroup per 8 columns, 16 tokens
        assert follow_sumsq_floats(n, 64) >= ((n + 1023) // 1024) * 64    # a workgroup per 1,024 columns, 64 tokens


def test_prompt_tiles_in_chunks_for_models_of_few_heads():
    from vipera_rs_amd.ops.attention import chunks_prompt_tiles
    one_prompt = sum(128 * t for t in range(1, 17))                     # positions that the 16 tiles of 2,048 tokens see
    assert chunks_prompt_tiles(16, 12, 2048, one_prompt, 256) is None   # 12 heads, one short prompt: the halved tiles
    assert chunks_prompt_tiles(16, 28, 2048, one_prompt, 256) is None   # 448 items: more than the CUs
    # four portions of 512 tokens that end at positions 1,000 to 8,000: 192 items, the deepest 125 steps long
    assert chunks_prompt_tiles(16, 12, 8000, 4 * (1000 + 3000 + 5000 + 8000), 256) == (25, 5)
    assert chunks_prompt_tiles(16, 12, 4096, 16 * 3900, 256) is None    # all about equally deep: nothing to balance
    assert chunks_prompt_tiles(0, 12, 0, 0, 256) is None


def test_decode_attention_chunks():
    assert decode_chunking(4096, 8, 4, 1) == (256, 16)     # 8 requests x 4 key heads x 16 chunks = 512 waves
    assert decode_chunking(4096, 64, 4, 1) == (1024, 4)
    assert decode_chunking(4096, 1, 4, 1) == (128, 32)     # never below 128 positions a chunk
    assert decode_chunking(100, 1, 4, 1) == (128, 1)
    # many requests at long contexts: longer chunks while they still make 2,048 waves
    assert decode_chunking(32768, 64, 4, 1) == (4096, 8) and decode_chunking(16384, 64, 4, 1) == (2048, 8)
    assert decode_chunking(8192, 64, 4, 1) == (1024, 8) and decode_chunking(32768, 16, 4, 1) == (1024, 32)
    assert decode_chunking(32768, 64, 2, 1) == (2048, 16)
    chunk, chunks = decode_chunking(1 << 20, 1, 1, 1)      # never more than 128 chunks
    assert chunks <= 128 and chunk * chunks >= 1 << 20 and chunk % 32 == 0


def test_decode_attention_counts_the_entries_by_the_positions_they_hold():
    assert decode_chunking(4096, 8, 4, 1, 8 * 4096) == decode_chunking(4096, 8, 4, 1)      # all full: as without
    assert decode_chunking(16384, 64, 4, 1, 301000) == (1024, 16)      # 64 requests that fill 18 %: no long chunks
    assert decode_chunking(8192, 16, 4, 1, 70000) == (512, 16)         # as 9 full ones
    assert decode_chunking(8192, 8, 4, 1, 8 * 4100) == (256, 32)       # a little past a context bucket's half
    assert decode_chunking(4096, 8, 4, 1, 1) == decode_chunking(4096, 1, 4, 1)             # never fewer than one entry
    assert decode_chunking(4096, 8, 4, 1, 10 ** 9) == decode_chunking(4096, 8, 4, 1)       # nor more than there are


def test_decode_attention_chunks_cover_every_length_for_any_batch():
    import random
    rng = random.Random(5)
    for _ in range(3000):
        longest = rng.choice([1, 31, 32, 33, 100, 1000, 4096, 8191, 40000, rng.randrange(1, 1 << 21)])
        entries = rng.choice([1, 2, 7, 8, 63, 64, 200, 256])
        kv_heads, head_blocks = rng.choice([1, 2, 4, 8]), rng.choice([1, 2])
        total = rng.choice([0, 1, longest, rng.randrange(1, entries * longest + 1), entries * longest, 10 * entries * longest])
        chunk, chunks = decode_chunking(longest, entries, kv_heads, head_blocks, total)
        assert chunk % 32 == 0 and chunk >= 128 and 1 <= chunks <= 128, (longest, entries, total)
        assert chunk * chunks >= longest and chunk * (chunks - 1) < longest, (longest, entries, total)
        # fewer positions in all never make the chunks longer
        if total:
            assert chunk <= decode_chunking(longest, entries, kv_heads, head_blocks)[0]


def test_a_captured_step_is_chosen_by_the_share_of_its_context_bucket_that_is_filled():
    from vipera_rs_amd.engine.graphs import FILL_CLASSES, fill_class
    assert FILL_CLASSES == (1.0, 0.5, 0.25)
    assert fill_class(8 * 4096, 8, 4096) == 0 and fill_class(8 * 3000, 8, 4096) == 0
    assert fill_class(8 * 4100, 8, 8192) == 1              # equal lengths just past a bucket's edge
    assert fill_class(301000, 64, 16384) == 2 and fill_class(8, 8, 256) == 2


def test_one_workgroup_takes_all_chunks_of_a_request_and_key_head_where_those_fill_the_gpu():
    from vipera_rs_amd.ops.attention import joins_decode_chunks
    assert joins_decode_chunks(4, 64, 4, 1, 256) and joins_decode_chunks(4, 128, 4, 1, 256)
    assert not joins_decode_chunks(16, 8, 4, 1, 256)        # 32 pairs for 256 CUs
    assert not joins_decode_chunks(16, 64, 4, 1, 256)       # more chunks than a workgroup has waves
    # a few more pairs than CUs: the CUs with two workgroups would set the time
    assert not joins_decode_chunks(4, 72, 4, 1, 256) and not joins_decode_chunks(4, 40, 8, 1, 256)
    assert not joins_decode_chunks(4, 96, 4, 1, 256) and joins_decode_chunks(4, 112, 4, 1, 256)
    # heads wider than 128 keep a workgroup per chunk: one wave a SIMD, with room for their sums
    assert joins_decode_chunks(4, 64, 4, 1, 256, 128) and joins_decode_chunks(4, 64, 4, 1, 256, 112)
    assert not joins_decode_chunks(4, 64, 4, 1, 256, 160) and not joins_decode_chunks(4, 64, 4, 1, 256, 256)


def test_prompt_tiles_are_halved_between_sixteen_waves_only_where_a_cu_would_be_left_with_one_workgroup():
    from vipera_rs_amd.ops.attention import halves_prompt_tiles
    reach = [128 * (t + 1) for t in range(16)]                       # one prompt of 2,048 tokens
    assert halves_prompt_tiles(16, 28, max(reach), sum(reach), 256)  # 448 items, the longest 1.9 times the mean
    even = [1536 + 128 * (t + 1) for t in range(4)] * 4              # four portions of 512 tokens at position 1,536
    assert not halves_prompt_tiles(16, 28, max(even), sum(even), 256)
    assert halves_prompt_tiles(4, 28, 512, 1280, 256)                # fewer items than CUs
    long = [128 * (t + 1) for t in range(64)]                        # 8,192 tokens: several rounds of workgroups
    assert not halves_prompt_tiles(64, 28, max(long), sum(long), 256)
    assert not halves_prompt_tiles(0, 28, 0, 0, 256)
