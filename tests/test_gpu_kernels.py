"""Each kernel alone against a plain reference of the same operation, at sizes other than the engine's."""
import math

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _rel(got, want):
    want = want.double()
    return float((got.double() - want).abs().max() / want.abs().max().clamp_min(1e-30))


# --- matrix products -----------------------------------------------------------------------------
GEMM_SHAPES = [(1, 48, 64), (7, 300, 96), (8, 3584, 512), (16, 200, 128), (17, 331, 80), (33, 1000, 264),
               (64, 520, 1024), (65, 130, 72), (128, 128, 64), (100, 9000, 72), (200, 257, 136), (515, 384, 200),
               (2050, 4100, 136)]   # the last ones take each tiling of the tiled kernel


@pytest.mark.parametrize("m,n,k", GEMM_SHAPES)
@pytest.mark.parametrize("out_dtype", [torch.float32, torch.bfloat16])
def test_gemm_bf16_against_float64(m, n, k, out_dtype):
    from vipera_rs_amd.ops import kernels
    g = torch.Generator().manual_seed(m * 1000 + n + k)
    a = torch.randn(m, k, generator=g).to(torch.bfloat16).to(DEV)
    w = torch.randn(n, k, generator=g).to(torch.bfloat16).to(DEV)
    bias = torch.randn(n, generator=g).to(DEV)
    want = a.double() @ w.double().T + bias.double()
    out = torch.empty(m, n, dtype=out_dtype, device=DEV)
    kernels.gemm_bf16(a, w, bias, out)
    tol = 1e-5 if out_dtype == torch.float32 else 6e-3
    assert _rel(out, want) < tol
    if out_dtype == torch.float32:  # accumulation into a 32-bit residual, no bias
        base = torch.randn(m, n, generator=g).to(DEV)
        acc = base.clone()
        kernels.gemm_bf16(a, w, None, acc, accumulate=True)
        assert _rel(acc, base.double() + a.double() @ w.double().T) < 1e-5


@pytest.mark.parametrize("tiling", [0, 2, 3, 4, 9, 7, 8, 5])
@pytest.mark.parametrize("ranges", [1, 2, 8])
def test_gemm_bf16_every_tiling_of_the_tiled_kernel(tiling, ranges):
    """Each tiling of both tiled kernels, forced: tails in both directions, one to many K steps (an odd
    number too, so both LDS stages end a run), K split into ranges, and a K that the direct kernel passes on."""
    from vipera_rs_amd.ops import kernels
    shapes = [(257, 520, 1024), (129, 1028, 128), (300, 264, 64), (513, 300, 1600), (65, 2100, 4608), (200, 257, 136)]
    try:
        kernels.gemm_bf16_force_tiling(tiling, ranges)
        for m, n, k in shapes:
            g = torch.Generator().manual_seed(m + n + k)
            a = torch.randn(m, k, generator=g).to(torch.bfloat16).to(DEV)
            w = torch.randn(n, k, generator=g).to(torch.bfloat16).to(DEV)
            bias = torch.randn(n, generator=g).to(DEV)
            product = a.double() @ w.double().T
            for out_dtype, tol in ((torch.float32, 1e-5), (torch.bfloat16, 6e-3)):
                out = torch.full((m, n), 7.0, dtype=out_dtype, device=DEV)
                kernels.gemm_bf16(a, w, bias, out)
                assert _rel(out, product + bias.double()) < tol, (m, n, k, out_dtype)
            base = torch.randn(m, n, generator=g).to(DEV)
            acc = base.clone()
            kernels.gemm_bf16(a, w, None, acc, accumulate=True)
            assert _rel(acc, base.double() + product) < 1e-5, (m, n, k, "accumulate")
    finally:
        kernels.gemm_bf16_force_tiling(-1)


@pytest.mark.parametrize("tiling", [0, 9, 7, 5, 6])
def test_the_tiled_kernel_computes_the_same_in_every_order_of_its_tiles(tiling):
    """The workgroups walk the tiles in blocks of a few rows of tiles (chosen by shape, forced here): every tile is
    computed once whatever the block height, also where the last block has fewer rows and where the launch has
    more workgroups than tiles."""
    from vipera_rs_amd.ops import kernels
    g = torch.Generator().manual_seed(tiling)
    m, n, k = 1100, 1300, 192
    a = torch.randn(m, k, generator=g).to(torch.bfloat16).to(DEV)
    w = torch.randn(n, k, generator=g).to(torch.bfloat16).to(DEV)
    want = a.double() @ w.double().T
    outs = []
    try:
        for ranges in (1, 3):
            kernels.gemm_bf16_force_tiling(tiling, ranges)
            for rows in (0, 1, 2, 4, 5, 7, 50):
                kernels.gemm_bf16_force_tile_group(rows)
                out = torch.full((m, n), 7.0, device=DEV)
                kernels.gemm_bf16(a, w, None, out)
                assert _rel(out, want) < 1e-5, (ranges, rows)
                outs.append(out)
            assert all(torch.equal(outs[0], o) for o in outs[1:]), ranges
            outs.clear()
    finally:
        kernels.gemm_bf16_force_tile_group(0)
        kernels.gemm_bf16_force_tiling(-1)


@pytest.mark.parametrize("tiling", [9, 8])
@pytest.mark.parametrize("ranges", [1, 3])
def test_gemm_bf16_direct_tilings_with_three_lds_stages(tiling, ranges):
    """The 128-token tilings of the kernel that loads straight into LDS, forced to three stages (what up to 128
    tokens take by themselves) at any number of tokens: one, two, three, four and many K steps, so that the run
    ends in each stage, with and without a step whose loads stay in flight."""
    from vipera_rs_amd.ops import kernels
    shapes = [(64, 520, 64), (100, 264, 128), (128, 300, 192), (257, 520, 256), (65, 2100, 4608), (33, 1028, 1600),
              (300, 131, 1024)]
    try:
        kernels.gemm_bf16_force_tiling(tiling, ranges, stages=3)
        for m, n, k in shapes:
            g = torch.Generator().manual_seed(m + n + k)
            a = torch.randn(m, k, generator=g).to(torch.bfloat16).to(DEV)
            w = torch.randn(n, k, generator=g).to(torch.bfloat16).to(DEV)
            bias = torch.randn(n, generator=g).to(DEV)
            product = a.double() @ w.double().T
            for out_dtype, tol in ((torch.float32, 1e-5), (torch.bfloat16, 6e-3)):
                out = torch.full((m, n), 7.0, dtype=out_dtype, device=DEV)
                kernels.gemm_bf16(a, w, bias, out, skinny_limit=0)
                assert _rel(out, product + bias.double()) < tol, (m, n, k, out_dtype)
            base = torch.randn(m, n, generator=g).to(DEV)
            acc = base.clone()
            kernels.gemm_bf16(a, w, None, acc, accumulate=True, skinny_limit=0)
            assert _rel(acc, base.double() + product) < 1e-5, (m, n, k, "accumulate")
    finally:
        kernels.gemm_bf16_force_tiling(-1)


@pytest.mark.parametrize("tiling,stages", [(t, 0) for t in (0, 2, 3, 4, 9, 7, 8, 5, 10, 11, 12)]   # the last three: 128 tokens x 96, 160, 224 rows
                         + [(t, 3) for t in (9, 8, 10, 11, 12)] + [(t, 2) for t in (9, 11)])
def test_gated_product_with_every_tiling(tiling, stages):
    from vipera_rs_amd.ops import kernels
    from vipera_rs_amd.ops.linear import interleave_gate_up
    try:
        kernels.gemm_bf16_force_tiling(tiling, 1, stages)
        for m, inter, k in [(300, 208, 192), (2048, 528, 128), (130, 1008, 640), (70, 48, 72), (64, 304, 3584), (17, 160, 64)]:
            g = torch.Generator().manual_seed(m + inter + k)
            a = torch.randn(m, k, generator=g).to(torch.bfloat16).to(DEV)
            gate = torch.randn(inter, k, generator=g).to(torch.bfloat16).to(DEV)
            up = torch.randn(inter, k, generator=g).to(torch.bfloat16).to(DEV)
            gd, ud = a.double() @ gate.double().T, a.double() @ up.double().T
            out = torch.full((m, inter), 7.0, dtype=torch.bfloat16, device=DEV)
            kernels.gemm_bf16_gated(a, interleave_gate_up(gate, up), out)
            assert _rel(out, ud * (gd / (1 + torch.exp(-gd)))) < 8e-3, (m, inter, k)
    finally:
        kernels.gemm_bf16_force_tiling(-1)


@pytest.mark.parametrize("m,n,k", [(1, 100, 64), (8, 4608, 256), (16, 333, 520), (3, 9, 128), (5, 47, 72)])
def test_skinny_product_with_every_number_of_rows_per_workgroup(m, n, k):
    """A workgroup of the weight-streaming kernel may own 8 to 16 weight rows; the launcher picks the number
    that divides N evenly over the CUs.  Every choice gives the same sums (the order within a row's sum does
    not depend on it), beside bias, accumulation and both output types."""
    from vipera_rs_amd.ops import kernels
    g = torch.Generator().manual_seed(m + n + k)
    a = torch.randn(m, k, generator=g).to(torch.bfloat16).to(DEV)
    w = torch.randn(n, k, generator=g).to(torch.bfloat16).to(DEV)
    bias = torch.randn(n, generator=g).to(DEV)
    base = torch.randn(m, n, generator=g).to(DEV)
    want = a.double() @ w.double().T + bias.double()
    first = {}
    for shape in [0] + list(range(108, 117)):
        out = torch.full((m, n), 7.0, dtype=torch.bfloat16, device=DEV)
        kernels.gemm_bf16(a, w, bias, out, skinny_shape=shape)
        assert _rel(out, want) < 6e-3, shape
        acc = base.clone()
        kernels.gemm_bf16(a, w, bias, acc, accumulate=True, skinny_shape=shape)
        assert _rel(acc, base.double() + want) < 1e-5, shape
        if first:
            assert torch.equal(out, first["out"]) and torch.equal(acc, first["acc"]), shape
        first = first or {"out": out, "acc": acc}



def test_gemm_bf16_tile_and_skinny_kernels_agree():
    from vipera_rs_amd.ops import kernels
    g = torch.Generator().manual_seed(5)
    a = torch.randn(48, 256, generator=g).to(torch.bfloat16).to(DEV)
    w = torch.randn(272, 256, generator=g).to(torch.bfloat16).to(DEV)
    skinny = torch.empty(48, 272, dtype=torch.float32, device=DEV)
    tile = torch.empty_like(skinny)
    kernels.gemm_bf16(a, w, None, skinny, skinny_limit=64)
    kernels.gemm_bf16(a, w, None, tile, skinny_limit=0)
    assert _rel(skinny, tile) < 1e-5


def test_gemm_bf16_strided_views():
    from vipera_rs_amd.ops import kernels
    g = torch.Generator().manual_seed(9)
    wide = torch.randn(20, 96 + 64, generator=g).to(torch.bfloat16).to(DEV)
    a = wide[:, :96]
    w = torch.randn(40, 96, generator=g).to(torch.bfloat16).to(DEV)
    out_wide = torch.zeros(20, 100, dtype=torch.bfloat16, device=DEV)
    out = out_wide[:, 20:60]
    kernels.gemm_bf16(a, w, None, out)
    assert _rel(out, a.double() @ w.double().T) < 6e-3
    assert float(out_wide[:, :20].abs().max()) == 0.0 and float(out_wide[:, 60:].abs().max()) == 0.0


@pytest.mark.parametrize("m,n,k", [(1, 48, 64), (7, 300, 96), (65, 130, 71), (130, 67, 200)])
@pytest.mark.parametrize("dtypes", [(torch.float32,) * 3, (torch.bfloat16, torch.float32, torch.bfloat16),
                                    (torch.bfloat16, torch.bfloat16, torch.float32)])
def test_gemm_generic_against_float64(m, n, k, dtypes):
    from vipera_rs_amd.ops import kernels
    g = torch.Generator().manual_seed(m + n + k)
    a = torch.randn(m, k, generator=g).to(dtypes[0]).to(DEV)
    w = torch.randn(n, k, generator=g).to(dtypes[1]).to(DEV)
    bias = torch.randn(n, generator=g).to(DEV)
    out = torch.empty(m, n, dtype=dtypes[2], device=DEV)
    kernels.gemm_generic(a, w, bias, out)
    want = a.double() @ w.double().T + bias.double()
    assert _rel(out, want) < (2e-6 if dtypes[2] == torch.float32 else 6e-3)


@pytest.mark.parametrize("k", [64, 200, 256, 1100, 2600])
def test_gemm_generic_does_not_depend_on_the_batch(k):
    """Every output element is summed in one fixed order (chains over ranges of 256 k, four ranges to a slab, slabs in
    ascending order), whichever kernel computes it: the weight stream that takes up to 64 tokens gives bit for bit
    the rows of the tiled kernel that takes 70, alone or in any company, with and without a bias, accumulating or not."""
    from vipera_rs_amd.ops import kernels
    g = torch.Generator().manual_seed(k)
    a = torch.randn(70, k, generator=g).to(DEV)
    w = torch.randn(90, k, generator=g).to(DEV)
    bias = torch.randn(90, generator=g).to(DEV)
    base = torch.randn(70, 90, generator=g).to(DEV)
    whole = torch.empty(70, 90, device=DEV)
    kernels.gemm_generic(a, w, None, whole)
    assert _rel(whole, a.double() @ w.double().T) < 2e-6
    for rows in ([37], [0, 1], list(range(5, 12)), list(range(3, 36)), list(range(6, 70))):
        part = torch.empty(len(rows), 90, device=DEV)
        kernels.gemm_generic(a[rows].contiguous(), w, None, part)
        assert torch.equal(part, whole[rows]), f"{len(rows)} rows"      # bit for bit
    with_bias = torch.empty(70, 90, device=DEV)
    kernels.gemm_generic(a, w, bias, with_bias)
    added = base.clone()
    kernels.gemm_generic(a, w, bias, added, accumulate=True)
    few = base[20:28].clone()
    kernels.gemm_generic(a[20:28], w, bias, few, accumulate=True)        # a view with a row stride of its own
    assert torch.equal(few, added[20:28])
    rounded = torch.empty(8, 90, dtype=torch.bfloat16, device=DEV)
    kernels.gemm_generic(a[20:28], w, bias, rounded)
    assert torch.equal(rounded, with_bias[20:28].to(torch.bfloat16))


@pytest.mark.parametrize("m,n,k", [(1024, 1024, 520), (1030, 1100, 1027), (1500, 905, 258), (1153, 1025, 2052)])
def test_the_wide_tiles_of_gemm_generic_sum_in_the_same_order(m, n, k):
    """128 rows and more on enough tiles take 128 x 128 tiles with 8 x 8 outputs a thread: against 64-bit, and bit
    for bit the rows that the 64 x 64 tiles give 70 rows at a time and the weight stream 33 at a time; with a bias,
    accumulating, into bfloat16, from bfloat16 activations, and with rows that start off a 16-byte boundary."""
    from vipera_rs_amd.ops import kernels
    g = torch.Generator().manual_seed(m + n + k)
    a = torch.randn(m, k, generator=g).to(DEV)
    w = torch.randn(n, k, generator=g).to(DEV)
    bias = torch.randn(n, generator=g).to(DEV)
    base = torch.randn(m, n, generator=g).to(DEV)
    whole = torch.full((m, n), float("nan"), device=DEV)
    kernels.gemm_generic(a, w, bias, whole)
    assert _rel(whole, a.double() @ w.double().T + bias.double()) < 2e-6
    for rows in (70, 33):
        for start in (0, 128 * 3 + 5, m - rows):
            part = torch.empty(rows, n, device=DEV)
            kernels.gemm_generic(a[start:start + rows], w, bias, part)
            assert torch.equal(part, whole[start:start + rows]), (rows, start)       # bit for bit
    added = base.clone()
    kernels.gemm_generic(a, w, bias, added, accumulate=True)
    few = base[200:270].clone()
    kernels.gemm_generic(a[200:270], w, bias, few, accumulate=True)
    assert torch.equal(few, added[200:270])
    rounded = torch.empty(m, n, dtype=torch.bfloat16, device=DEV)
    kernels.gemm_generic(a, w, bias, rounded)
    assert torch.equal(rounded, whole.to(torch.bfloat16))
    half = a.to(torch.bfloat16)                                   # bfloat16 activations on a 32-bit weight
    mixed = torch.empty(m, n, device=DEV)
    kernels.gemm_generic(half, w, bias, mixed)
    again = torch.empty(m, n, device=DEV)
    kernels.gemm_generic(half.float(), w, bias, again)
    assert torch.equal(mixed, again)
    shifted = torch.zeros(m, k + 3, device=DEV)                   # rows 4 (k + 3) bytes apart, from a 4-byte offset
    shifted[:, 1:k + 1] = a
    out = torch.zeros(m, n + 8, device=DEV)
    kernels.gemm_generic(shifted[:, 1:k + 1], w, bias, out[:, 4:n + 4])
    assert torch.equal(out[:, 4:n + 4], whole)
    assert float(out[:, :4].abs().max()) == 0.0 and float(out[:, n + 4:].abs().max()) == 0.0


@pytest.mark.parametrize("m,n,k", [(1, 64, 4), (3, 70, 36), (8, 3584, 1536), (9, 129, 1028), (16, 1000, 4096), (40, 200, 520),
                                   (64, 333, 2052)])
def test_gemm_stream_against_float64(m, n, k):
    """The 32-bit weight stream at sizes of its own: K that ends inside a chunk of 32, a range and a slab, rows of
    W that do not fill a workgroup's 64, every count of tokens' class."""
    from vipera_rs_amd.ops import kernels
    g = torch.Generator().manual_seed(m * n + k)
    a = torch.randn(m, k, generator=g).to(DEV)
    w = torch.randn(n, k, generator=g).to(DEV)
    bias = torch.randn(n, generator=g).to(DEV)
    out = torch.full((m, n), float("nan"), device=DEV)
    kernels.gemm_generic(a, w, bias, out)
    assert _rel(out, a.double() @ w.double().T + bias.double()) < 2e-6
    wide = torch.zeros(m, n + 8, device=DEV)                               # an output with a row stride of its own
    kernels.gemm_generic(a, w, None, wide[:, 4:n + 4])
    assert _rel(wide[:, 4:n + 4], a.double() @ w.double().T) < 2e-6
    assert float(wide[:, :4].abs().max()) == 0.0 and float(wide[:, n + 4:].abs().max()) == 0.0


# --- attention -------------------------------------------------------------------------------------
def _plain_attention(q, k, v, first_pos, window, scale):
    """q: [T, heads, hd] at positions first_pos..; k, v: [P, kv_heads, hd] for positions 0..P-1. float64."""
    T, heads, hd = q.shape
    group = heads // k.shape[1]
    out = torch.zeros(T, heads, hd, dtype=torch.float64)
    for t in range(T):
        pos = first_pos + t
        lo = max(0, pos + 1 - window) if window > 0 else 0
        for h in range(heads):
            kk, vv = k[lo:pos + 1, h // group], v[lo:pos + 1, h // group]
            w = torch.softmax((kk @ q[t, h]) * scale, dim=0)
            out[t, h] = w @ vv
    return out


class _Paged:
    """A paged cache filled by hand: shuffled pages, K [page, kvh, slot, hd], V [page, kvh, hd, slot]."""

    def __init__(self, seqs, kv_heads, hd, block_size, dtype, seed, stale_nan=False):
        g = torch.Generator().manual_seed(seed)
        self.block_size = block_size
        need = [(n + block_size - 1) // block_size for n in seqs]
        pages = sum(need) + 3
        order = torch.randperm(pages, generator=g).tolist()
        self.k = (torch.randn(pages, kv_heads, block_size, hd, generator=g) * 7).to(dtype)   # stale values everywhere
        self.v = (torch.randn(pages, kv_heads, hd, block_size, generator=g) * 7).to(dtype)
        if stale_nan:
            # what no live position occupies is not finite, as after a request whose activations overflowed gave its
            # pages back: also the slots of a held page past the request's last position
            self.k.fill_(float("nan"))
            self.v.fill_(float("nan"))
        self.tables, self.keys, self.values = [], [], []
        for n, blocks in zip(seqs, need):
            table = [order.pop() for _ in range(blocks)]
            keys = torch.randn(n, kv_heads, hd, generator=g).to(dtype)
            values = torch.randn(n, kv_heads, hd, generator=g).to(dtype)
            whole, rest = n // block_size, n % block_size       # position p sits in slot p % size of page table[p // size]
            if whole:
                pages_of = torch.tensor(table[:whole])
                self.k[pages_of] = keys[:whole * block_size].view(whole, block_size, kv_heads, hd).permute(0, 2, 1, 3)
                self.v[pages_of] = values[:whole * block_size].view(whole, block_size, kv_heads, hd).permute(0, 2, 3, 1)
            if rest:
                self.k[table[whole], :, :rest, :] = keys[whole * block_size:].permute(1, 0, 2)
                self.v[table[whole], :, :, :rest] = values[whole * block_size:].permute(1, 2, 0)
            self.tables.append(table)
            self.keys.append(keys)
            self.values.append(values)
        width = max(need)
        self.table = torch.full((len(seqs), width), -1, dtype=torch.int32)
        for i, t in enumerate(self.tables):
            self.table[i, :len(t)] = torch.tensor(t, dtype=torch.int32)
        self.spare = order.pop()        # a page that no request holds

    def with_pages_given_back(self, first_visible):
        """The table after a window has passed: the blocks of entry i that lie wholly before position
        ``first_visible[i]`` name a page that nobody holds (in the engine their id is -1, which must not be followed;
        a kernel that reads such a block here reads what the spare page holds, NaN in the tests that say so)."""
        table = self.table.clone()
        for i, first in enumerate(first_visible):
            table[i, :first // self.block_size] = self.spare
        return table


ATTN_CASES = [
    # heads, kv_heads, hd, block_size, window, entries as (kv length after the step, tokens in the step)
    (4, 2, 16, 16, 0, [(37, 37), (70, 1), (5, 2)]),
    (3, 1, 32, 8, 21, [(90, 17), (64, 1), (33, 33), (130, 1)]),
    (6, 3, 48, 16, 0, [(100, 64), (65, 65)]),
    (28, 4, 128, 16, 0, [(300, 1), (257, 130), (31, 1)]),
    (20, 1, 80, 32, 50, [(200, 1), (97, 96)]),
    (2, 2, 256, 64, 0, [(129, 1), (70, 70)]),
    # widths that fill their padded width with pages that divide 64: prompts go through the kernel that loads into LDS directly
    (8, 2, 64, 8, 40, [(200, 150), (64, 64), (300, 1), (391, 130)]),
    (4, 4, 128, 32, 100, [(333, 300), (128, 128), (2, 2)]),
    (5, 5, 64, 64, 0, [(190, 190), (321, 129)]),
    (2, 1, 256, 16, 70, [(260, 200)]),
]


@pytest.mark.parametrize("case", ATTN_CASES, ids=[f"h{c[0]}kv{c[1]}d{c[2]}b{c[3]}w{c[4]}" for c in ATTN_CASES])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("stale", ["finite", "nan"])
def test_attention_kernels_against_plain_softmax(case, dtype, stale):
    """``stale``: what the pool holds wherever no live position lies, the rest of a request's last page included:
    large finite numbers, or NaN (a weight of zero times NaN is NaN on the matrix cores, so such a slot must not
    reach a product at all)."""
    from vipera_rs_amd.ops import kernels
    from vipera_rs_amd.ops.attention import decode_chunking
    heads, kv_heads, hd, bs, window, entries = case
    scale = 1.0 / math.sqrt(hd)
    cache = _Paged([kv for kv, _ in entries], kv_heads, hd, bs, dtype, seed=heads * 100 + hd, stale_nan=stale == "nan")
    g = torch.Generator().manual_seed(hd)
    counts = [n for _, n in entries]
    T = sum(counts)
    width = (heads + 2 * kv_heads) * hd
    qkv = torch.randn(T, width, generator=g).to(dtype)
    starts = [0]
    for n in counts:
        starts.append(starts[-1] + n)
    first = [kv - n for kv, n in entries]
    positions = torch.tensor([first[e] + i for e, n in enumerate(counts) for i in range(n)], dtype=torch.int32)
    entry_of = torch.tensor([e for e, n in enumerate(counts) for _ in range(n)], dtype=torch.int32)
    want = torch.zeros(T, heads, hd, dtype=torch.float64)
    for e, (kv, n) in enumerate(entries):
        q = qkv[starts[e]:starts[e + 1], :heads * hd].double().view(n, heads, hd)
        want[starts[e]:starts[e + 1]] = _plain_attention(q, cache.keys[e].double(), cache.values[e].double(),
                                                         first[e], window, scale)
    want = want.view(T, heads * hd)
    dev = lambda t: t.to(DEV)  # noqa: E731
    # with a window, the pages that the first token of an entry no longer sees have been given back
    table = cache.with_pages_given_back([max(0, first[e] + 1 - window) for e in range(len(entries))]) if window else cache.table
    qkv_d, k_d, v_d, table_d = dev(qkv), dev(cache.k), dev(cache.v), dev(table)
    tol = 2e-6 if dtype == torch.float32 else 1.2e-2

    out = torch.zeros(T, heads * hd, dtype=dtype, device=DEV)
    kernels.attn_generic(qkv_d, k_d, v_d, out, dev(positions), dev(entry_of), table_d, heads, kv_heads, hd, scale, window)
    assert _rel(out.cpu(), want) < tol, "32-bit-arithmetic kernel"

    if dtype == torch.float32 and kernels.attn_decode_f32_supported(qkv_d, k_d, hd):
        # single tokens on the 32-bit kernel that splits their positions, the portions on the general one
        singles = [e for e, n in enumerate(counts) if n == 1]
        es = dev(torch.tensor(starts, dtype=torch.int32))
        fp = dev(torch.tensor(first, dtype=torch.int32))
        out3 = torch.zeros(T, heads * hd, dtype=dtype, device=DEV)
        if singles:
            chunks = (max(entries[e][0] for e in singles) + 255) // 256 + 1      # a chunk that sees nothing, too
            partial = torch.full((len(singles) * heads * chunks * (hd + 2),), float("nan"), device=DEV)
            kernels.attn_decode_f32(qkv_d, k_d, v_d, out3, partial, dev(torch.tensor(singles, dtype=torch.int32)), es, fp,
                                    table_d, heads, kv_heads, hd, scale, window, chunks)
        kernels.attn_generic(qkv_d, k_d, v_d, out3, dev(positions), dev(entry_of), table_d, heads, kv_heads, hd, scale, window,
                             skip_single_of=es)
        assert _rel(out3.cpu(), want) < tol, "32-bit decode kernel beside the general one"
        if kernels.attn_prefill_f32_supported(qkv_d, k_d, hd):
            # the portions on the 32-bit kernel that walks the positions in LDS tiles; tiles of 128 or of 64 tokens
            for tile_tokens in (128, 64):
                tiles = [x for e, n in enumerate(counts) if n > 1 for off in range(0, n, tile_tokens) for x in (e, off)]
                rows = [t for e, n in enumerate(counts) if n > 1 for t in range(starts[e], starts[e + 1])]
                out4 = torch.full((T, heads * hd), float("nan"), dtype=dtype, device=DEV)
                kernels.attn_prefill_f32(qkv_d, k_d, v_d, out4, dev(torch.tensor(tiles, dtype=torch.int32)), tile_tokens, es,
                                         fp, table_d, heads, kv_heads, hd, scale, window)
                assert _rel(out4.cpu()[rows], want[rows]) < tol, f"32-bit prompt kernel, tiles of {tile_tokens}"
                others = [t for t in range(T) if t not in set(rows)]
                assert bool(torch.isnan(out4.cpu()[others]).all()), "the prompt kernel wrote a single token's row"

    if dtype == torch.bfloat16:
        from vipera_rs_amd.engine.batch import TILE_TOKENS
        tiles = [x for e, n in enumerate(counts) if n > 1 for off in range(0, n, TILE_TOKENS) for x in (e, off)]
        singles = [e for e, n in enumerate(counts) if n == 1]
        out2 = torch.zeros(T, heads * hd, dtype=dtype, device=DEV)
        es, fp = dev(torch.tensor(starts, dtype=torch.int32)), dev(torch.tensor(first, dtype=torch.int32))
        if tiles:
            halved = torch.zeros(T, heads * hd, dtype=dtype, device=DEV)   # a tile's positions halved between sixteen waves
            kernels.attn_bf16_prefill(qkv_d, k_d, v_d, halved, dev(torch.tensor(tiles, dtype=torch.int32)), es, fp,
                                      table_d, heads, kv_heads, hd, scale, window, split=True)
            rows = [t for e, n in enumerate(counts) if n > 1 for t in range(starts[e], starts[e + 1])]
            assert _rel(halved.cpu()[rows], want[rows]) < tol, "matrix-core prompt kernel, halved"
            reach = max(kv for kv, n in entries if n > 1)
            for chunk_tiles in (1, 2):          # a tile's positions in chunks of 64 and of 128, merged by a second kernel
                chunked = torch.zeros(T, heads * hd, dtype=dtype, device=DEV)
                kernels.attn_bf16_prefill(qkv_d, k_d, v_d, chunked, dev(torch.tensor(tiles, dtype=torch.int32)), es, fp,
                                          table_d, heads, kv_heads, hd, scale, window, chunk_tiles=chunk_tiles,
                                          max_chunks=-(-((reach + 63) // 64) // chunk_tiles))
                assert _rel(chunked.cpu()[rows], want[rows]) < tol, f"matrix-core prompt kernel, chunks of {chunk_tiles}"
            kernels.attn_bf16_prefill(qkv_d, k_d, v_d, out2, dev(torch.tensor(tiles, dtype=torch.int32)), es, fp,
                                      table_d, heads, kv_heads, hd, scale, window)
        if singles:
            longest = max(entries[e][0] for e in singles)
            for chunk, chunks in {decode_chunking(longest, len(singles), kv_heads, (heads // kv_heads + 15) // 16),
                                  (32, (longest + 31) // 32), (512, (longest + 511) // 512),
                                  (2048, (longest + 2047) // 2048)}:
                partial = torch.empty(len(singles) * heads * chunks * (hd + 2), device=DEV)
                kernels.attn_bf16_decode(qkv_d, k_d, v_d, out2, partial, dev(torch.tensor(singles, dtype=torch.int32)),
                                         es, fp, table_d, heads, kv_heads, hd, scale, window, chunk, chunks)
                assert _rel(out2.cpu(), want) < tol, f"matrix-core kernels, chunk {chunk}"
                if chunks <= kernels.ATTN_DECODE_JOINED_CHUNKS:   # a workgroup that takes all chunks and merges them itself
                    joined = out2.clone()
                    joined[[starts[e] for e in singles]] = 7.0
                    kernels.attn_bf16_decode(qkv_d, k_d, v_d, joined, None, dev(torch.tensor(singles, dtype=torch.int32)),
                                             es, fp, table_d, heads, kv_heads, hd, scale, window, chunk, chunks, join=True)
                    assert _rel(joined.cpu(), want) < tol, f"matrix-core kernels, chunk {chunk}, joined"
        assert _rel(out2.cpu(), want) < tol, "matrix-core kernels"


@pytest.mark.parametrize("window", [0, 1500])
def test_decode_attention_over_thousands_of_positions(window):
    """Single-token entries with long histories: many chunks, chunks that span more pages than a wave
    keeps ids of in a register (the table is then read step by step), chunks cut by a window's edge."""
    from vipera_rs_amd.ops import kernels
    heads, kv_heads, hd, bs = 8, 2, 64, 16
    lengths = [5000, 3333, 1, 4097]
    scale = 1.0 / math.sqrt(hd)
    dtype = torch.bfloat16
    cache = _Paged(lengths, kv_heads, hd, bs, dtype, seed=11)
    g = torch.Generator().manual_seed(5)
    qkv = torch.randn(len(lengths), (heads + 2 * kv_heads) * hd, generator=g).to(dtype)
    first = [n - 1 for n in lengths]
    want = torch.zeros(len(lengths), heads, hd, dtype=torch.float64)
    for e, n in enumerate(lengths):
        q = qkv[e:e + 1, :heads * hd].double().view(1, heads, hd)
        want[e] = _plain_attention(q, cache.keys[e].double(), cache.values[e].double(), first[e], window, scale)[0]
    want = want.view(len(lengths), heads * hd)
    dev = lambda t: t.to(DEV)  # noqa: E731
    qkv_d, k_d, v_d, table_d = dev(qkv), dev(cache.k), dev(cache.v), dev(cache.table)
    es = dev(torch.arange(len(lengths) + 1, dtype=torch.int32))
    fp = dev(torch.tensor(first, dtype=torch.int32))
    singles = dev(torch.arange(len(lengths), dtype=torch.int32))
    longest = max(lengths)
    for chunk in (128, 256, 1024, 4096):
        chunks = (longest + chunk - 1) // chunk
        out = torch.zeros(len(lengths), heads * hd, dtype=dtype, device=DEV)
        partial = torch.empty(len(lengths) * heads * chunks * (hd + 2), device=DEV)
        for dense in (False, True):
            out = torch.zeros(len(lengths), heads * hd, dtype=dtype, device=DEV)
            kernels.attn_bf16_decode(qkv_d, k_d, v_d, out, partial, singles, es, fp, table_d, heads, kv_heads, hd, scale,
                                     window, chunk, chunks, dense=dense)
            assert _rel(out.cpu(), want) < 1.2e-2, f"chunk {chunk}, dense {dense}"
            if chunks <= kernels.ATTN_DECODE_JOINED_CHUNKS:
                out = torch.zeros(len(lengths), heads * hd, dtype=dtype, device=DEV)
                kernels.attn_bf16_decode(qkv_d, k_d, v_d, out, None, singles, es, fp, table_d, heads, kv_heads, hd, scale,
                                         window, chunk, chunks, dense=dense, join=True)
                assert _rel(out.cpu(), want) < 1.2e-2, f"chunk {chunk}, dense {dense}, joined"


def _plain_attention_by_head(q, k, v, first_pos, window, scale):
    """The same as ``_plain_attention`` with one matrix of scores per head, for thousands of positions."""
    T, heads, hd = q.shape
    group = heads // k.shape[1]
    pos = first_pos + torch.arange(T)[:, None]
    key = torch.arange(k.shape[0])[None, :]
    visible = key <= pos
    if window > 0:
        visible &= key > pos - window
    out = torch.zeros(T, heads, hd, dtype=torch.float64)
    for h in range(heads):
        scores = (q[:, h] @ k[:, h // group].T) * scale
        out[:, h] = torch.softmax(scores.masked_fill(~visible, float("-inf")), dim=1) @ v[:, h // group]
    return out


def test_the_two_plain_attentions_agree():
    g = torch.Generator().manual_seed(0)
    q, k, v = (torch.randn(n, h, 16, generator=g, dtype=torch.float64) for n, h in ((5, 6), (40, 2), (40, 2)))
    for window in (0, 7):
        a = _plain_attention(q, k, v, 35, window, 0.25)
        b = _plain_attention_by_head(q, k, v, 35, window, 0.25)
        assert float((a - b).abs().max()) < 1e-12


BENCH_HEADS = [(28, 4, 128), (40, 8, 128), (12, 2, 128)]   # the 7B, 32B and 1.5B head shapes


def _context_bucket(kv_len):
    bucket = 256
    while bucket < kv_len:
        bucket *= 2
    return bucket


@pytest.mark.parametrize("heads,kv_heads,hd", BENCH_HEADS, ids=[f"h{h}kv{k}" for h, k, _ in BENCH_HEADS])
@pytest.mark.parametrize("batch", [8, 64])
def test_decode_attention_at_the_benchmark_head_shapes(heads, kv_heads, hd, batch):
    """Single-token entries at 4,096 and 3,000 positions (and a few short ones) in batches of 8 and 64, with the
    chunking the engine picks for the longest entry and for the context bucket a captured step is built for.
    In every entry one far key is made to stand out for the first head of each group, so that a chunk or a page
    that is dropped shows."""
    from vipera_rs_amd.ops import kernels
    from vipera_rs_amd.ops.attention import decode_chunking, joins_decode_chunks
    bs, scale, dtype = 16, 1.0 / math.sqrt(hd), torch.bfloat16
    lengths = [(4096, 3000, 2049, 4095, 1, 3001, 130, 4096)[e % 8] for e in range(batch)]
    if batch == 64 and heads != 28:
        # the other two head shapes at a quarter of the lengths: the float64 oracle is what the time goes to
        lengths = [(1024, 750, 513, 1023, 1, 751, 130, 1024)[e % 8] for e in range(batch)]
    cache = _Paged(lengths, kv_heads, hd, bs, dtype, seed=heads)
    g = torch.Generator().manual_seed(batch)
    qkv = torch.randn(batch, (heads + 2 * kv_heads) * hd, generator=g).to(dtype)
    group = heads // kv_heads
    for e, n in enumerate(lengths):
        far = (17 * (e + 1)) % n
        page, slot = cache.tables[e][far // bs], far % bs
        for kv in range(kv_heads):
            q = qkv[e, kv * group * hd:(kv * group + 1) * hd].float()
            key = (q / q.norm() * (9.0 / scale / q.norm())).to(dtype)      # a score of about 9 for that head
            cache.keys[e][far, kv] = key
            cache.k[page, kv, slot, :] = key
    first = [n - 1 for n in lengths]
    want = torch.zeros(batch, heads, hd, dtype=torch.float64)
    for e in range(batch):
        q = qkv[e:e + 1, :heads * hd].double().view(1, heads, hd)
        want[e] = _plain_attention_by_head(q, cache.keys[e].double(), cache.values[e].double(), first[e], 0, scale)[0]
    want = want.view(batch, heads * hd)
    dev = lambda t: t.to(DEV)  # noqa: E731
    qkv_d, k_d, v_d = dev(qkv), dev(cache.k), dev(cache.v)
    es = dev(torch.arange(batch + 1, dtype=torch.int32))
    fp = dev(torch.tensor(first, dtype=torch.int32))
    singles = dev(torch.arange(batch, dtype=torch.int32))
    longest = max(lengths)
    for visible in (longest, _context_bucket(longest), 2 * _context_bucket(longest)):
        # a captured step is built for a context bucket: its table is that wide and its chunks cover all of it
        width = (visible + bs - 1) // bs
        table = torch.full((batch, width), -1, dtype=torch.int32)
        table[:, :cache.table.shape[1]] = cache.table
        chunk, chunks = decode_chunking(visible, batch, kv_heads, (group + 15) // 16)
        out = torch.zeros(batch, heads * hd, dtype=dtype, device=DEV)
        partial = torch.full((batch * heads * chunks * (hd + 2),), float("nan"), device=DEV)
        kernels.attn_bf16_decode(qkv_d, k_d, v_d, out, partial, singles, es, fp, dev(table), heads, kv_heads, hd, scale, 0,
                                 chunk, chunks)
        assert _rel(out.cpu(), want) < 1.2e-2, f"visible {visible}: chunk {chunk} x {chunks}"
        # a step of single tokens only: the kernel is told that entry i is slot i and token i and looks neither up
        dense = torch.zeros(batch, heads * hd, dtype=dtype, device=DEV)
        kernels.attn_bf16_decode(qkv_d, k_d, v_d, dense, partial, singles, es, fp, dev(table), heads, kv_heads, hd, scale, 0,
                                 chunk, chunks, dense=True)
        assert torch.equal(dense, out)
        if joins_decode_chunks(chunks, batch, kv_heads, (group + 15) // 16, 256):   # what the engine does at batch 64
            joined = torch.zeros(batch, heads * hd, dtype=dtype, device=DEV)
            kernels.attn_bf16_decode(qkv_d, k_d, v_d, joined, None, singles, es, fp, dev(table), heads, kv_heads, hd, scale,
                                     0, chunk, chunks, dense=True, join=True)
            assert _rel(joined.cpu(), want) < 1.2e-2, f"visible {visible}: chunk {chunk} x {chunks}, joined"
    # the long chunks of many requests at long contexts, over a table as wide as theirs
    visible = 4 * _context_bucket(longest)
    table = torch.full((batch, (visible + bs - 1) // bs), -1, dtype=torch.int32)
    table[:, :cache.table.shape[1]] = cache.table
    for chunk in (2048, 4096):
        chunks = (visible + chunk - 1) // chunk
        out = torch.zeros(batch, heads * hd, dtype=dtype, device=DEV)
        partial = torch.full((batch * heads * chunks * (hd + 2),), float("nan"), device=DEV)
        kernels.attn_bf16_decode(qkv_d, k_d, v_d, out, partial, singles, es, fp, dev(table), heads, kv_heads, hd, scale, 0,
                                 chunk, chunks, dense=True)
        assert _rel(out.cpu(), want) < 1.2e-2, f"visible {visible}: chunk {chunk} x {chunks}"
        joined = torch.zeros(batch, heads * hd, dtype=dtype, device=DEV)
        kernels.attn_bf16_decode(qkv_d, k_d, v_d, joined, None, singles, es, fp, dev(table), heads, kv_heads, hd, scale,
                                 0, chunk, chunks, dense=True, join=True)
        assert _rel(joined.cpu(), want) < 1.2e-2, f"visible {visible}: chunk {chunk} x {chunks}, joined"
    out = torch.zeros(batch, heads * hd, dtype=dtype, device=DEV)
    kernels.attn_generic(qkv_d, k_d, v_d, out, fp, singles, dev(cache.table), heads, kv_heads, hd, scale, 0)
    assert _rel(out.cpu(), want) < 1.2e-2, "32-bit-arithmetic kernel on the bfloat16 cache"


@pytest.mark.parametrize("heads,kv_heads,hd", BENCH_HEADS, ids=[f"h{h}kv{k}" for h, k, _ in BENCH_HEADS])
def test_prompt_attention_at_the_benchmark_head_shapes(heads, kv_heads, hd):
    """One prompt of 2,048 tokens from position 0 and one portion of 512 tokens from position 3,584 in one step."""
    from vipera_rs_amd.engine.batch import TILE_TOKENS
    from vipera_rs_amd.ops import kernels
    bs, scale, dtype = 16, 1.0 / math.sqrt(hd), torch.bfloat16
    entries = [(2048, 2048), (4096, 512)]       # (positions in the cache after the step, tokens of the step)
    cache = _Paged([kv for kv, _ in entries], kv_heads, hd, bs, dtype, seed=hd + heads)
    g = torch.Generator().manual_seed(heads)
    counts = [n for _, n in entries]
    T = sum(counts)
    qkv = torch.randn(T, (heads + 2 * kv_heads) * hd, generator=g).to(dtype)
    starts, first = [0, counts[0], T], [kv - n for kv, n in entries]
    want = torch.zeros(T, heads, hd, dtype=torch.float64)
    for e, (kv, n) in enumerate(entries):
        q = qkv[starts[e]:starts[e + 1], :heads * hd].double().view(n, heads, hd)
        want[starts[e]:starts[e + 1]] = _plain_attention_by_head(q, cache.keys[e].double(), cache.values[e].double(),
                                                                 first[e], 0, scale)
    want = want.view(T, heads * hd)
    dev = lambda t: t.to(DEV)  # noqa: E731
    tiles = [(first[e] + off, e, off) for e, n in enumerate(counts) for off in range(0, n, TILE_TOKENS)]
    tiles = [x for _, e, off in sorted(tiles) for x in (e, off)]                # as the engine orders them
    # whole tiles, tiles in halves, and tiles in chunks of 8 and of 5 steps of 64 positions (the last chunk short)
    for split, chunk_tiles in ((False, 0), (True, 0), (False, 8), (False, 5)):
        out = torch.zeros(T, heads * hd, dtype=dtype, device=DEV)
        max_chunks = -(-(4096 // 64) // chunk_tiles) if chunk_tiles else 0
        kernels.attn_bf16_prefill(dev(qkv), dev(cache.k), dev(cache.v), out, dev(torch.tensor(tiles, dtype=torch.int32)),
                                  dev(torch.tensor(starts, dtype=torch.int32)), dev(torch.tensor(first, dtype=torch.int32)),
                                  dev(cache.table), heads, kv_heads, hd, scale, 0, split=split,
                                  chunk_tiles=chunk_tiles, max_chunks=max_chunks)
        got = out.cpu()
        assert _rel(got, want) < 1.2e-2, (split, chunk_tiles)
        # row by row too: the first tokens of a prompt see few keys, their outputs are large and would hide a fault
        # in a late row of small outputs
        rows = (got.double() - want).abs().amax(dim=1) / want.abs().amax(dim=1)
        assert float(rows.max()) < 3e-2, (split, chunk_tiles, int(rows.argmax()))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_attention_finds_one_far_key_among_hundreds(dtype):
    """One early key is made to dominate: every later token must return (almost exactly) its value.
    An off-by-one in the visible range, a missed page or a wrong tile would lose it."""
    from vipera_rs_amd.ops import kernels
    heads, kv_heads, hd, bs, n = 4, 2, 64, 16, 700
    far = 17
    cache = _Paged([n], kv_heads, hd, bs, dtype, seed=1)
    direction = torch.randn(hd, generator=torch.Generator().manual_seed(3))
    direction = (direction / direction.norm()).to(dtype)
    page, slot = cache.tables[0][far // bs], far % bs
    cache.k[page, :, slot, :] = direction * 40
    q = torch.zeros(2, (heads + 2 * kv_heads) * hd, dtype=dtype)
    q[:, :heads * hd] = (direction * 40).repeat(heads)
    dev = lambda t: t.to(DEV)  # noqa: E731
    out = torch.zeros(2, heads * hd, dtype=dtype, device=DEV)
    positions = torch.tensor([n - 2, n - 1], dtype=torch.int32)
    kernels.attn_generic(dev(q), dev(cache.k), dev(cache.v), out, dev(positions), dev(torch.zeros(2, dtype=torch.int32)),
                         dev(cache.table), heads, kv_heads, hd, 1.0 / math.sqrt(hd), 0)
    want = cache.values[0][far].double().repeat_interleave(heads // kv_heads, dim=0).reshape(-1)
    for row in out.cpu().double():
        assert float((row - want).abs().max()) < (1e-5 if dtype == torch.float32 else 2e-2)
    if dtype == torch.bfloat16:
        out2 = torch.zeros_like(out)
        es, fp = dev(torch.tensor([0, 2], dtype=torch.int32)), dev(torch.tensor([n - 2], dtype=torch.int32))
        kernels.attn_bf16_prefill(dev(q), dev(cache.k), dev(cache.v), out2, dev(torch.tensor([0, 0], dtype=torch.int32)),
                                  es, fp, dev(cache.table), heads, kv_heads, hd, 1.0 / math.sqrt(hd), 0)
        for row in out2.cpu().double():
            assert float((row - want).abs().max()) < 2e-2


@pytest.mark.parametrize("m,n,k", [(1, 48, 64), (7, 300, 96), (8, 3584, 512), (16, 200, 1544), (17, 331, 520), (33, 1000, 264),
                                   (64, 520, 1024), (48, 130, 72), (64, 4608, 3584),
                                   # past 64 tokens K is walked in chunks of 128: K with a rest, K shorter than a chunk
                                   (65, 331, 520), (80, 1000, 264), (97, 200, 1544), (128, 3584, 1024), (113, 130, 72),
                                   # weight rows a multiple of 4 KB apart: the workgroups start at different chunks
                                   (8, 1100, 2048), (40, 2100, 4096), (100, 1100, 2048)])
@pytest.mark.parametrize("ranges,rows_per_wave", [(1, 1), (1, 2), (3, 1), (8, 2), (2, 110), (1, 114), (3, 109)])
def test_gemm_mid_against_float64(m, n, k, ranges, rows_per_wave):
    from vipera_rs_amd.ops import kernels
    g = torch.Generator().manual_seed(m * 1000 + n + k)
    a = torch.randn(m, k, generator=g).to(torch.bfloat16).to(DEV)
    w = torch.randn(n, k, generator=g).to(torch.bfloat16).to(DEV)
    bias = torch.randn(n, generator=g).to(DEV)
    want = a.double() @ w.double().T + bias.double()
    for out_dtype, tol in ((torch.float32, 1e-5), (torch.bfloat16, 6e-3)):
        out = torch.full((m, n), 7.0, dtype=out_dtype, device=DEV)
        kernels.gemm_bf16_mid(a, w, bias, out, ranges=ranges, rows_per_wave=rows_per_wave)
        assert _rel(out, want) < tol
    base = torch.randn(m, n, generator=g).to(DEV)
    acc = base.clone()
    kernels.gemm_bf16_mid(a, w, None, acc, accumulate=True, ranges=ranges, rows_per_wave=rows_per_wave)
    assert _rel(acc, base.double() + a.double() @ w.double().T) < 1e-5


@pytest.mark.parametrize("m,width,k_in,inter", [(8, 3584, 512, 18944), (1, 256, 64, 32), (16, 512, 1024, 16 * 1000),
                                               (5, 768, 264, 16 * 41), (3, 1024, 3584, 16 * 300), (8, 896, 512, 4864)])
def test_the_norm_split_between_the_products_around_it(m, width, k_in, inter):
    """x += a Wo^T, h = rms_norm(x) * g, out = up(h) * silu(gate(h)) as two kernels: the first also leaves
    bfloat16(x * g) and its workgroups' sums of squares, the second adds those and divides gate and up by the
    root mean square.  Against 64-bit, and against residual product, norm kernel and gated product."""
    from vipera_rs_amd.ops import kernels
    from vipera_rs_amd.ops.linear import interleave_gate_up
    g = torch.Generator().manual_seed(m + width + k_in)
    a = torch.randn(m, k_in, generator=g).to(torch.bfloat16).to(DEV)
    w_o = (torch.randn(width, k_in, generator=g) / k_in ** 0.5).to(torch.bfloat16).to(DEV)
    x0 = (torch.randn(m, width, generator=g) * 2).to(DEV)
    x0[0, 0] = 60.0                                          # one row with a far larger mean square
    gain = (1 + 0.2 * torch.randn(width, generator=g)).to(DEV)
    gate = (torch.randn(inter, width, generator=g) / width ** 0.5).to(torch.bfloat16).to(DEV)
    up = (torch.randn(inter, width, generator=g) / width ** 0.5).to(torch.bfloat16).to(DEV)
    fused = interleave_gate_up(gate, up)
    eps = 1e-5
    x = x0.clone()
    scaled = torch.empty(m, width, dtype=torch.bfloat16, device=DEV)
    sumsq = torch.full((kernels.follow_sumsq_floats(width, m),), 7.0, device=DEV)
    groups = kernels.gemm_bf16_follow(a, w_o, None, x, gain, scaled, sumsq)
    want_x = x0.double() + a.double() @ w_o.double().T
    assert _rel(x, want_x) < 1e-5
    assert _rel(scaled, want_x * gain.double()) < 6e-3
    squares = sumsq[: groups * 16].view(groups, 16).double().sum(0)[:m]
    assert _rel(squares, (want_x ** 2).sum(-1)) < 1e-5
    out = torch.full((m, inter), 7.0, dtype=torch.bfloat16, device=DEV)
    kernels.gemm_bf16_gated_scaled(scaled, fused, out, sumsq, groups, eps)
    h = want_x * torch.rsqrt((want_x ** 2).mean(-1, keepdim=True) + eps) * gain.double()
    gd, ud = h @ gate.double().T, h @ up.double().T
    want = ud * (gd / (1 + torch.exp(-gd)))
    assert _rel(out, want) < 1.2e-2
    # the three kernels it replaces
    x3 = x0.clone()
    kernels.gemm_bf16(a, w_o, None, x3, accumulate=True)
    assert torch.equal(x3, x)
    h3 = torch.empty(m, width, dtype=torch.bfloat16, device=DEV)
    kernels.rmsnorm(x3, gain, eps, h3)
    out3 = torch.empty(m, inter, dtype=torch.bfloat16, device=DEV)
    kernels.gemm_bf16_gated(h3, fused, out3, 0)
    assert _rel(out, out3.double()) < 1.2e-2


@pytest.mark.parametrize("tiling", [-1, 0, 2, 3, 4, 9, 7, 8, 5, 10, 11, 12])
@pytest.mark.parametrize("m,width,k_in,inter", [(64, 520, 1024, 16 * 21), (33, 1032, 1536, 16 * 40), (17, 264, 2048, 16 * 9),
                                               (300, 3584, 512, 16 * 64), (5, 200, 0, 16 * 30)])
def test_the_tiled_gated_product_divides_by_the_norm_before_it(tiling, m, width, k_in, inter):
    """17 to 64 tokens: the residual product whose K is split over workgroups leaves bfloat16(x * g) and the sums of
    squares (the kernel that adds its ranges does), and the tiled gated product divides gate and up by the root
    mean square.  Every tiling of both tiled kernels; sums of squares made by hand too (k_in 0), for token counts
    and group counts that no product before the norm produces.  Against 64-bit, as the kernels it replaces."""
    from vipera_rs_amd.ops import kernels
    from vipera_rs_amd.ops.linear import interleave_gate_up
    g = torch.Generator().manual_seed(m + width + k_in)
    gain = (1 + 0.2 * torch.randn(width, generator=g)).to(DEV)
    gate = (torch.randn(inter, width, generator=g) / width ** 0.5).to(torch.bfloat16).to(DEV)
    up = (torch.randn(inter, width, generator=g) / width ** 0.5).to(torch.bfloat16).to(DEV)
    fused = interleave_gate_up(gate, up)
    eps = 1e-5
    stride = kernels.follow_stride(m)
    x0 = (torch.randn(m, width, generator=g) * 2).to(DEV)
    x0[m // 2, 3] = 60.0                                      # one row with a far larger mean square
    if k_in and m <= 64:
        a = torch.randn(m, k_in, generator=g).to(torch.bfloat16).to(DEV)
        w_o = (torch.randn(width, k_in, generator=g) / k_in ** 0.5).to(torch.bfloat16).to(DEV)
        x = x0.clone()
        scaled = torch.full((m, width), 7.0, dtype=torch.bfloat16, device=DEV)
        sumsq = torch.full((kernels.follow_sumsq_floats(width, m),), 7.0, device=DEV)
        groups = kernels.gemm_bf16_mid_follow(a, w_o, None, x, 2, 1, gain, scaled, sumsq)
        want_x = x0.double() + a.double() @ w_o.double().T
        assert _rel(x, want_x) < 1e-5
    else:  # 37 groups of uneven shares of each row's squares
        x, want_x = x0, x0.double()
        scaled = (x0 * gain).to(torch.bfloat16)
        groups = 37
        shares = torch.rand(groups, m, generator=g).to(DEV).double() + 0.1
        shares = shares / shares.sum(0, keepdim=True) * (want_x ** 2).sum(-1)
        sumsq = torch.full((groups * stride,), 7.0, device=DEV)
        sumsq.view(groups, stride)[:, :m] = shares.float()
    try:
        kernels.gemm_bf16_force_tiling(tiling)
        act = torch.full((m, inter), 7.0, dtype=torch.bfloat16, device=DEV)
        kernels.gemm_bf16_gated_tile_scaled(scaled, fused, act, sumsq, groups, eps)
        h = want_x * torch.rsqrt((want_x ** 2).mean(-1, keepdim=True) + eps) * gain.double()
        gd, ud = h @ gate.double().T, h @ up.double().T
        want = ud * (gd / (1 + torch.exp(-gd)))
        assert _rel(act, want) < 1.2e-2
        h3 = torch.empty(m, width, dtype=torch.bfloat16, device=DEV)       # the two kernels it replaces are as far
        kernels.rmsnorm(x, gain, eps, h3)                                  # from the 64-bit result, each on its side
        act3 = torch.empty_like(act)
        kernels.gemm_bf16_gated(h3, fused, act3, 3)
        assert _rel(act3, want) < 1.2e-2 and _rel(act, act3.double()) < 2.4e-2
    finally:
        kernels.gemm_bf16_force_tiling(-1)


@pytest.mark.parametrize("m,inter,k", [(1, 32, 64), (5, 48, 96), (8, 18944, 512), (16, 176, 200), (33, 128, 264), (64, 1024, 256),
                                       (65, 64, 72), (300, 208, 136), (2048, 512, 128), (2048, 8208, 72), (100, 4608, 64),
                                       # the resident kernel: one pair on four waves, fewer units than waves, runs of
                                       # uneven length, a wave's stretch inside one pair, many pairs per workgroup
                                       (1, 16, 256), (3, 48, 256), (16, 16 * 37, 512), (5, 16 * 1000, 1024), (8, 16 * 257, 3584),
                                       (16, 16 * 300, 4352), (2, 16 * 4111, 768), (7, 32, 2048),
                                       # weight rows a multiple of 4 KB apart (the LDS-shared kernel's workgroups
                                       # start at different chunks)
                                       (6, 16 * 70, 2048), (40, 16 * 70, 4096),
                                       # 256 does not divide K: the resident kernel walks chunks of 128
                                       (8, 4864, 896), (3, 48, 128), (16, 16 * 37, 384)])
def test_gated_product_and_interleaved_swiglu(m, inter, k):
    from vipera_rs_amd.ops import kernels
    from vipera_rs_amd.ops.linear import gated_resident_fits, interleave_gate_up, linear_gated
    g = torch.Generator().manual_seed(m + inter + k)
    a = torch.randn(m, k, generator=g).to(torch.bfloat16).to(DEV)
    gate = torch.randn(inter, k, generator=g).to(torch.bfloat16).to(DEV)
    up = torch.randn(inter, k, generator=g).to(torch.bfloat16).to(DEV)
    gd, ud = a.double() @ gate.double().T, a.double() @ up.double().T
    want = ud * (gd / (1 + torch.exp(-gd)))
    fused = interleave_gate_up(gate, up)
    assert torch.equal(fused[:16], gate[:16]) and torch.equal(fused[16:32], up[:16])
    for rows_per_wave in (1, 2, 3):
        out = torch.full((m, inter), 7.0, dtype=torch.bfloat16, device=DEV)
        kernels.gemm_bf16_gated(a, fused, out, rows_per_wave)
        assert _rel(out, want) < 8e-3, f"fused epilogue, plan {rows_per_wave}"
    if gated_resident_fits(m, 2 * inter, k):
        out = torch.full((m, inter), 7.0, dtype=torch.bfloat16, device=DEV)
        kernels.gemm_bf16_gated(a, fused, out, 0)
        assert _rel(out, want) < 8e-3, "resident activations"
    out = torch.empty(m, inter, dtype=torch.bfloat16, device=DEV)
    linear_gated(a, fused, out, True)                       # whichever path the dispatch takes
    assert _rel(out, want) < 1.2e-2
    plain = torch.empty(m, inter, dtype=torch.bfloat16, device=DEV)
    linear_gated(a, torch.cat([gate, up]).contiguous(), plain, False)
    assert _rel(plain, want) < 1.2e-2


@pytest.mark.parametrize("count", [1, 3, 4, 1023, 70_000])
def test_a_steps_words_are_fetched_from_pinned_host_memory(count):
    """The kernel that stands for the host-to-device copy of a step's metadata: the words arrive as they are, in
    stream order, also when the pinned buffer is written again after the stream has been drained."""
    from vipera_rs_amd.errors import InvalidArgumentError
    from vipera_rs_amd.ops import kernels
    g = torch.Generator().manual_seed(count)
    host = torch.randint(-2 ** 31, 2 ** 31 - 1, (count,), generator=g, dtype=torch.int64).to(torch.int32).pin_memory()
    out = torch.full((count,), 7, dtype=torch.int32, device=DEV)
    if not kernels.fetch_words(host, out):
        pytest.skip("this runtime gives pinned host memory no device address")
    assert torch.equal(out.cpu(), host)
    torch.cuda.synchronize()
    host.numpy()[:] = 5
    assert kernels.fetch_words(host, out)
    assert int(out.min()) == 5 and int(out.max()) == 5
    with pytest.raises(InvalidArgumentError):
        kernels.fetch_words(torch.zeros(count, dtype=torch.int32), out)   # pageable memory is refused on the host
