"""Each kernel beside its plain C++ twin: the same parameter list goes to ``vk_*`` with device pointers and to
``plain_*`` with host pointers, and the outputs are compared.  Sizes are not the engine's."""
import ctypes
import math

import numpy as np

import pytest
import torch

from plain import sampler_plain

from helpers import rel_err
from plain_cpp import DT, SIGNATURES, call

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _kernel(module: str, name: str):
    from vipera_rs_amd.ops.build import load_module
    fn = getattr(load_module(module), "vk_" + name)
    fn.argtypes, fn.restype = SIGNATURES["plain_" + name], ctypes.c_int
    return fn


def both(module: str, name: str, args, outputs):
    """Run kernel and twin on copies of ``args``; returns ``[(kernel output, twin output), ...]`` for the argument
    indices in ``outputs``."""
    host = [a.clone() if isinstance(a, torch.Tensor) else a for a in args]
    dev = [a.to(DEV) if isinstance(a, torch.Tensor) else a for a in args]
    call("plain_" + name, *host)
    status = _kernel(module, name)(*[a.data_ptr() if isinstance(a, torch.Tensor) else a for a in dev])
    torch.cuda.synchronize()
    assert status == 0, f"vk_{name} returned {status}"
    return [(dev[i].cpu(), host[i]) for i in outputs]


def i32(values):
    return torch.tensor(values, dtype=torch.int32)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_row_wise_kernels_beside_their_twins(dtype):
    g = torch.Generator().manual_seed(7)
    table = torch.randn(37, 50, generator=g).to(dtype)
    (got, want), = both("elementwise", "embed_gather",
                        [table, DT[dtype], i32([5, 36, 0, 99]), i32([-1, -1, 1, -1]), i32([7, 20]), torch.empty(4, 50), 4, 50,
                         37, None], [5])
    assert torch.equal(got, want) and torch.equal(got[2], table[20].float()) and torch.equal(got[3], table[0].float())
    x, w = torch.randn(6, 1000, generator=g) * 3, 1 + 0.1 * torch.randn(1000, generator=g)
    (got, want), = both("elementwise", "rmsnorm", [x, w, i32([4, 1, 5]), torch.empty(3, 1000, dtype=dtype), DT[dtype], 3, 1000,
                                                   1e-5, None], [3])
    assert rel_err(got.float().numpy(), want.double().numpy()) < (2e-6 if dtype == torch.float32 else 4e-3)
    gate_up = (torch.randn(5, 2 * 208, generator=g) * 4).to(dtype)
    for interleaved in (0, 1):
        (got, want), = both("elementwise", "swiglu", [gate_up, torch.empty(5, 208, dtype=dtype), DT[dtype], 5, 208, interleaved,
                                                      None], [1])
        assert rel_err(got.float().numpy(), want.double().numpy()) < (2e-6 if dtype == torch.float32 else 4e-3)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("hd,rotary_dim", [(48, 48), (128, 128), (64, 32)])
def test_rotation_and_cache_write_beside_its_twin(dtype, hd, rotary_dim):
    heads, kv_heads, bs = 5, 2, 8
    positions, entry_of = [0, 3, 8, 9, 1000, 41], [0, 0, 0, 0, 1, 1]
    g = torch.Generator().manual_seed(hd + rotary_dim)
    qkv = torch.randn(6, (heads + 2 * kv_heads) * hd, generator=g).to(dtype)
    half = rotary_dim // 2
    inv = (1.0 / torch.pow(torch.tensor(1e6), torch.arange(half).float() * 2 / rotary_dim)).float()
    table = torch.full((2, 130), -1, dtype=torch.int32)
    table[0, 0], table[0, 1], table[1, 1000 // bs], table[1, 41 // bs] = 5, 2, 7, 3
    k_cache, v_cache = torch.zeros(9, kv_heads, bs, hd, dtype=dtype), torch.zeros(9, kv_heads, hd, bs, dtype=dtype)
    (angles_d, angles_h), = both("elementwise", "rope_angles", [i32(positions), inv, half, 6, torch.empty(6, half, 2), None], [4])
    assert rel_err(angles_d.numpy(), angles_h.double().numpy()) < 1e-6
    for angles in (None, angles_d):
        outs = both("elementwise", "rope_kvwrite",
                    [qkv, DT[dtype], i32(positions), inv, angles, rotary_dim, k_cache, v_cache, i32(entry_of), table, 130, bs, 6,
                     heads, kv_heads, hd, None], [0, 6, 7])
        tol = 3e-6 if dtype == torch.float32 else 8e-3
        for got, want in outs:
            assert rel_err(got.float().numpy(), want.double().numpy()) < tol
        assert torch.equal(outs[2][0], outs[2][1])                       # values are copied, not computed


@pytest.mark.parametrize("m,heads,kv_heads,hd,k,with_bias,with_cache", [(6, 5, 2, 48, 96, True, True), (1, 4, 4, 128, 256, False, True),
                                                                        (16, 3, 1, 16, 72, True, True), (3, 7, 1, 64, 520, True, False),
                                                                        (8, 28, 4, 128, 256, True, True), (5, 9, 3, 40, 64, True, True),
                                                                        (2, 40, 8, 128, 128, False, True)])
def test_fused_qkv_product_beside_its_twin_and_the_two_kernels(m, heads, kv_heads, hd, k, with_bias, with_cache):
    """Product, rotation and cache write in one kernel: beside its twin, and bit for bit what the product followed
    by the rotation kernel leaves in the q/k/v rows and in both caches (other pages untouched)."""
    bs, n = 8, (heads + 2 * kv_heads) * hd
    g = torch.Generator().manual_seed(m + n + k)
    a = torch.randn(m, k, generator=g).to(torch.bfloat16)
    w = (torch.randn(n, k, generator=g) / math.sqrt(k)).to(torch.bfloat16)
    bias = torch.randn(n, generator=g) if with_bias else None
    positions = [0, 3, 8, 9, 1000, 41, 7, 15, 16, 17, 100, 5, 2, 1, 63, 64][:m]
    entry_of = [0, 0, 0, 0, 1, 1, 2, 2, 2, 2, 3, 3, 3, 3, 3, 3][:m]
    inv = (1.0 / torch.pow(torch.tensor(1e6), torch.arange(hd // 2).float() * 2 / hd)).float()
    table = torch.full((4, 130), -1, dtype=torch.int32)
    pages = iter(torch.randperm(40, generator=g).tolist())
    for e, pos in zip(entry_of, positions):
        if table[e, pos // bs] < 0:
            table[e, pos // bs] = next(pages)
    table[0, 0] = -1                                     # a token without a page writes nothing to the cache
    k_cache = torch.full((40, kv_heads, bs, hd), 9.0, dtype=torch.bfloat16) if with_cache else None
    v_cache = torch.full((40, kv_heads, hd, bs), 9.0, dtype=torch.bfloat16) if with_cache else None
    args = [a, w, bias, torch.empty(m, n, dtype=torch.bfloat16), m, n, k, k, n, i32(positions), inv, k_cache, v_cache,
            i32(entry_of), table, 130, bs, heads, kv_heads, hd, None, 0, 0.0, None]
    outs = both("gemm_bf16", "gemm_bf16_qkv_rope", args, [3, 11, 12] if with_cache else [3])
    for got, want in outs:
        assert rel_err(got.float().numpy(), want.double().numpy()) < 8e-3
    # the same through the two kernels, on the device
    from vipera_rs_amd.ops import kernels
    dev = [x.to(DEV) if isinstance(x, torch.Tensor) else x for x in args]
    qkv = torch.empty(m, n, dtype=torch.bfloat16, device=DEV)
    kernels.gemm_bf16(dev[0], dev[1], dev[2], qkv)
    kernels.rope_kvwrite(qkv, dev[9], dev[10], hd, dev[11], dev[12], dev[13], dev[14] if with_cache else None, heads, kv_heads, hd)
    fused = torch.empty(m, n, dtype=torch.bfloat16, device=DEV)
    kc, vc = (torch.full_like(dev[11], 9.0), torch.full_like(dev[12], 9.0)) if with_cache else (None, None)
    kernels.gemm_bf16_qkv_rope(dev[0], dev[1], dev[2], fused, dev[9], dev[10], kc, vc, dev[13], dev[14] if with_cache else None,
                               heads, kv_heads, hd)
    assert torch.equal(fused, qkv)
    if with_cache:
        assert torch.equal(kc, dev[11]) and torch.equal(vc, dev[12])
        assert torch.equal(kc.cpu(), outs[1][0]) and float((kc == 9.0).float().mean()) > 0.5


@pytest.mark.parametrize("m,width,k_in,heads,kv_heads,hd,split", [(8, 512, 2048, 6, 2, 32, True), (3, 256, 1024, 2, 1, 64, False),
                                                                  (16, 1024, 4096, 12, 4, 16, True), (1, 384, 520, 5, 1, 48, False)])
def test_the_first_norm_of_a_layer_split_between_the_layers(m, width, k_in, heads, kv_heads, hd, split):
    """x += act Wd^T (K split over workgroups or not), h = rms_norm(x) * g, q/k/v = h W^T + b, rotation, cache write
    as two kernels, each beside its twin and together against 64-bit."""
    from vipera_rs_amd.ops import kernels
    n = (heads + 2 * kv_heads) * hd
    g = torch.Generator().manual_seed(m + width + k_in)
    act = torch.randn(m, k_in, generator=g).to(torch.bfloat16)
    w_d = (torch.randn(width, k_in, generator=g) / math.sqrt(k_in)).to(torch.bfloat16)
    x0 = torch.randn(m, width, generator=g) * 2
    gain = 1 + 0.2 * torch.randn(width, generator=g)
    w = (torch.randn(n, width, generator=g) / math.sqrt(width)).to(torch.bfloat16)
    bias = torch.randn(n, generator=g)
    floats = kernels.follow_sumsq_floats(width, m)
    groups_d, groups_h = ctypes.c_int(0), ctypes.c_int(0)
    if split:
        partial = torch.empty(4 * 64 * width)
        name, args = "gemm_bf16_mid_follow", [act, w_d, None, x0, m, width, k_in, k_in, width, 4, 1, partial, partial.numel(), gain,
                                              torch.empty(m, width, dtype=torch.bfloat16), width, torch.zeros(floats), floats, 16]
    else:
        name, args = "gemm_bf16_follow", [act, w_d, None, x0, m, width, k_in, k_in, width, gain,
                                          torch.empty(m, width, dtype=torch.bfloat16), width, torch.zeros(floats), floats]
    x_at, scaled_at, sumsq_at = (3, 14, 16) if split else (3, 10, 12)
    host = [a.clone() if isinstance(a, torch.Tensor) else a for a in args]
    dev = [a.to(DEV) if isinstance(a, torch.Tensor) else a for a in args]
    from plain_cpp import library, ptr
    twin = getattr(library(), "plain_" + name)
    assert twin(*[ptr(a) if isinstance(a, torch.Tensor) else a for a in host], ctypes.byref(groups_h), None) == 0
    fn = _kernel_with_pointer(name)
    assert fn(*[a.data_ptr() if isinstance(a, torch.Tensor) else a for a in dev], ctypes.byref(groups_d), None) == 0
    torch.cuda.synchronize()
    assert rel_err(dev[x_at].cpu().numpy(), host[x_at].double().numpy()) < 1e-5
    assert rel_err(dev[scaled_at].float().cpu().numpy(), host[scaled_at].double().numpy()) < 6e-3
    got = dev[sumsq_at][: groups_d.value * 16].view(groups_d.value, 16).double().sum(0)[:m].cpu()
    assert rel_err(got.numpy(), host[sumsq_at][:m].double().numpy()) < 1e-5
    # the product after the norm, on the device's own output
    positions, entry_of = list(range(40, 40 + m)), list(range(m))
    inv = (1.0 / torch.pow(torch.tensor(1e6), torch.arange(hd // 2).float() * 2 / hd)).float()
    table = torch.arange(m * 4, dtype=torch.int32).view(m, 4)
    bs = 16
    k_cache = torch.zeros(m * 4, kv_heads, bs, hd, dtype=torch.bfloat16)
    v_cache = torch.zeros(m * 4, kv_heads, hd, bs, dtype=torch.bfloat16)
    args = [dev[scaled_at].cpu(), w, bias, torch.empty(m, n, dtype=torch.bfloat16), m, n, width, width, n, i32(positions), inv,
            k_cache, v_cache, i32(entry_of), table, 4, bs, heads, kv_heads, hd, dev[sumsq_at].cpu(), groups_d.value, 1e-5, None]
    for got, want in both("gemm_bf16", "gemm_bf16_qkv_rope", args, [3, 11, 12]):
        assert rel_err(got.float().numpy(), want.double().numpy()) < 8e-3
    # and against 64-bit from the start
    x = x0.double() + act.double() @ w_d.double().T
    h = x * torch.rsqrt((x ** 2).mean(-1, keepdim=True) + 1e-5) * gain.double()
    want_v = (h @ w.double().T + bias.double())[:, (heads + kv_heads) * hd:]
    (got, _), _, _ = both("gemm_bf16", "gemm_bf16_qkv_rope", args, [3, 11, 12])
    assert rel_err(got.float().numpy()[:, (heads + kv_heads) * hd:], want_v.numpy()) < 1e-2


@pytest.mark.parametrize("m,heads,kv_heads,hd,k,scaled", [(17, 5, 2, 48, 1024, False), (64, 4, 4, 128, 2048, True),
                                                          (33, 7, 1, 64, 1536, True), (40, 3, 1, 16, 1024, False),
                                                          (8, 5, 2, 48, 1024, True), (16, 4, 4, 128, 2048, False),
                                                          (3, 7, 1, 64, 1536, True), (1, 3, 1, 32, 1024, False)])
def test_split_qkv_product_that_rotates_while_it_adds_its_ranges(m, heads, kv_heads, hd, k, scaled):
    """Up to 64 tokens (the widest models take this path from few tokens on; the norm's sums then come 16 to a
    group, 64 past 16 tokens): K split over workgroups, and the kernel that adds the ranges divides by the norm (if
    scaled), adds the bias, rotates and writes the cache. Beside its twin; and without the norm bit for bit what the
    split product, its sum and the rotation kernel leave."""
    from vipera_rs_amd.ops import kernels
    bs, n = 8, (heads + 2 * kv_heads) * hd
    g = torch.Generator().manual_seed(m + n + k)
    a = torch.randn(m, k, generator=g).to(torch.bfloat16)
    w = (torch.randn(n, k, generator=g) / math.sqrt(k)).to(torch.bfloat16)
    bias = torch.randn(n, generator=g)
    positions = [(7 * i) % 61 + (i // 9) * 64 for i in range(m)]
    entry_of = [i // 9 for i in range(m)]
    inv = (1.0 / torch.pow(torch.tensor(1e6), torch.arange(hd // 2).float() * 2 / hd)).float()
    entries = max(entry_of) + 1
    table = torch.arange(entries * 70, dtype=torch.int32).view(entries, 70)
    k_cache = torch.full((entries * 70, kv_heads, bs, hd), 9.0, dtype=torch.bfloat16)
    v_cache = torch.full((entries * 70, kv_heads, hd, bs), 9.0, dtype=torch.bfloat16)
    stride = kernels.follow_stride(m)
    sumsq = (torch.rand(3 * stride, generator=g) * k).float() if scaled else None
    partial = torch.empty(2 * 64 * n)
    args = [a, w, bias, torch.empty(m, n, dtype=torch.bfloat16), m, n, k, k, n, 2, 1, partial, partial.numel(), i32(positions), inv,
            k_cache, v_cache, i32(entry_of), table, 70, bs, heads, kv_heads, hd, sumsq, 3 if scaled else 0, stride, 1e-5, None]
    for got, want in both("gemm_bf16", "gemm_bf16_mid_qkv_rope", args, [3, 15, 16]):
        assert rel_err(got.float().numpy(), want.double().numpy()) < 8e-3
    if scaled:
        return
    dev = [x.to(DEV) if isinstance(x, torch.Tensor) else x for x in args]
    qkv = torch.empty(m, n, dtype=torch.bfloat16, device=DEV)
    kernels.gemm_bf16_mid(dev[0], dev[1], dev[2], qkv, ranges=2, rows_per_wave=1)
    kc, vc = torch.full_like(dev[15], 9.0), torch.full_like(dev[16], 9.0)
    kernels.rope_kvwrite(qkv, dev[13], dev[14], hd, kc, vc, dev[17], dev[18], heads, kv_heads, hd)
    fused = torch.empty(m, n, dtype=torch.bfloat16, device=DEV)
    kc2, vc2 = torch.full_like(dev[15], 9.0), torch.full_like(dev[16], 9.0)
    kernels.gemm_bf16_mid_qkv_rope(dev[0], dev[1], dev[2], fused, 2, 1, dev[13], dev[14], kc2, vc2, dev[17], dev[18], heads,
                                   kv_heads, hd)
    assert torch.equal(fused, qkv) and torch.equal(kc2, kc) and torch.equal(vc2, vc)


@pytest.mark.parametrize("m,width,inter,groups", [(70, 264, 16 * 9, 5), (300, 520, 16 * 21, 56), (17, 200, 16 * 6, 1)])
def test_the_tiled_gated_product_on_a_scaled_input_beside_its_twin(m, width, inter, groups):
    from vipera_rs_amd.ops import kernels
    from vipera_rs_amd.ops.linear import interleave_gate_up
    g = torch.Generator().manual_seed(m + width)
    x = torch.randn(m, width, generator=g) * 2
    gain = 1 + 0.2 * torch.randn(width, generator=g)
    scaled = (x * gain).to(torch.bfloat16)
    stride = kernels.follow_stride(m)
    sumsq = torch.full((groups, stride), 3.0)
    shares = torch.rand(groups, m, generator=g) + 0.1
    sumsq[:, :m] = shares / shares.sum(0, keepdim=True) * (x ** 2).sum(-1)
    gate = (torch.randn(inter, width, generator=g) / math.sqrt(width)).to(torch.bfloat16)
    up = (torch.randn(inter, width, generator=g) / math.sqrt(width)).to(torch.bfloat16)
    args = [scaled, interleave_gate_up(gate, up), torch.empty(m, inter, dtype=torch.bfloat16), m, 2 * inter, width, width, inter,
            sumsq, groups, stride, 1e-5, None]
    (got, want), = both("gemm_bf16", "gemm_bf16_gated_tile_scaled", args, [2])
    assert rel_err(got.float().numpy(), want.double().numpy()) < 8e-3
    h = x.double() * torch.rsqrt((x.double() ** 2).mean(-1, keepdim=True) + 1e-5) * gain.double()
    gd, ud = h @ gate.double().T, h @ up.double().T
    assert rel_err(got.float().numpy(), (ud * (gd / (1 + torch.exp(-gd)))).numpy()) < 1.2e-2


def _kernel_with_pointer(name):
    from vipera_rs_amd.ops.build import load_module
    fn = getattr(load_module("gemm_bf16"), "vk_" + name)
    fn.argtypes, fn.restype = SIGNATURES["plain_" + name], ctypes.c_int
    return fn


PRODUCTS = [(1, 48, 64), (7, 300, 96), (33, 1000, 264), (65, 130, 72), (200, 257, 136), (300, 520, 1024), (515, 384, 192)]


@pytest.mark.parametrize("m,n,k", PRODUCTS)
def test_products_beside_their_twins(m, n, k):
    g = torch.Generator().manual_seed(m + n + k)
    a, w, bias = torch.randn(m, k, generator=g), torch.randn(n, k, generator=g), torch.randn(n, generator=g)
    (got, want), = both("gemm_generic", "gemm_generic", [a, 0, w, 0, bias, torch.empty(m, n), 0, m, n, k, k, n, 0, None], [5])
    assert rel_err(got.numpy(), want.double().numpy()) < 2e-6
    if m <= 64 and k % 4 == 0:
        slabs = torch.empty(((k + 1023) // 1024) * m * n)
        (got, want), = both("gemm_generic", "gemm_stream", [a, w, bias, torch.randn(m, n, generator=g), 0, m, n, k, k, n, 1, slabs,
                                                            slabs.numel(), None], [3])
        assert rel_err(got.numpy(), want.double().numpy()) < 2e-6
    ab, wb = a.to(torch.bfloat16), w.to(torch.bfloat16)
    for out_dtype, tol in ((torch.float32, 1e-5), (torch.bfloat16, 6e-3)):
        (got, want), = both("gemm_bf16", "gemm_bf16", [ab, wb, bias, torch.empty(m, n, dtype=out_dtype), DT[out_dtype], m, n, k, k,
                                                       n, 0, 64, 0, None, 0, None], [3])
        assert rel_err(got.float().numpy(), want.double().numpy()) < tol
    base = torch.randn(m, n, generator=g)
    (got, want), = both("gemm_bf16", "gemm_bf16", [ab, wb, None, base, 0, m, n, k, k, n, 1, 64, 0, None, 0, None], [3])
    assert rel_err(got.numpy(), want.double().numpy()) < 1e-5
    if m <= 128:
        partial = torch.empty(3 * m * n)
        (got, want), = both("gemm_bf16", "gemm_bf16_mid", [ab, wb, bias, torch.empty(m, n), 0, m, n, k, k, n, 0, 3, 1, partial,
                                                           partial.numel(), None], [3])
        assert rel_err(got.numpy(), want.double().numpy()) < 1e-5


@pytest.mark.parametrize("m,inter,k,plan", [(5, 48, 96, 1), (33, 128, 264, 1), (64, 1024, 256, 2), (300, 208, 192, 1),
                                            (130, 1008, 640, 1), (6, 16 * 270, 768, 0), (16, 80, 1280, 0)])
def test_gated_product_beside_its_twin(m, inter, k, plan):
    g = torch.Generator().manual_seed(m + inter + k)
    a = torch.randn(m, k, generator=g).to(torch.bfloat16)
    fused = torch.randn(2 * inter, k, generator=g).to(torch.bfloat16)
    (got, want), = both("gemm_bf16", "gemm_bf16_gated", [a, fused, torch.empty(m, inter, dtype=torch.bfloat16), m, 2 * inter, k, k,
                                                         inter, plan, None], [2])
    assert rel_err(got.float().numpy(), want.double().numpy()) < 8e-3


def _paged(T, kv_heads, hd, bs, dtype, seed, entries=1):
    """A cache whose pages are dealt out in a shuffled order, and its table: [entries, pages per entry]."""
    g = torch.Generator().manual_seed(seed)
    per = (T + bs - 1) // bs
    order = torch.randperm(entries * per + 3, generator=g)[: entries * per]
    table = order.view(entries, per).to(torch.int32).contiguous()
    k = torch.randn(entries * per + 3, kv_heads, bs, hd, generator=g).to(dtype)
    v = torch.randn(entries * per + 3, kv_heads, hd, bs, generator=g).to(dtype)
    return k, v, table


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("window", [0, 37])
def test_generic_attention_beside_its_twin(dtype, window):
    heads, kv_heads, hd, bs, T = 6, 3, 48, 8, 301
    k, v, table = _paged(T, kv_heads, hd, bs, dtype, 11)
    g = torch.Generator().manual_seed(12)
    qkv = torch.randn(9, (heads + 2 * kv_heads) * hd, generator=g).to(dtype)
    positions = i32([0, 1, 7, 8, 36, 37, 38, 255, 300])
    (got, want), = both("attn_generic", "attn_generic",
                        [qkv, qkv.shape[1], k, v, torch.empty(9, heads * hd, dtype=dtype), DT[dtype], positions, i32([0] * 9), table,
                         table.shape[1], bs, 9, heads, kv_heads, hd, 1 / math.sqrt(hd), window, None, None], [4])
    assert rel_err(got.float().numpy(), want.double().numpy()) < (3e-6 if dtype == torch.float32 else 8e-3)


@pytest.mark.parametrize("heads,kv_heads,hd,bs", [(6, 3, 48, 8), (7, 1, 128, 16), (12, 1, 64, 4), (5, 5, 256, 32)])
@pytest.mark.parametrize("window", [0, 37])
def test_32_bit_decode_attention_beside_its_twin(heads, kv_heads, hd, bs, window):
    """Single-token entries at positions around the edges of a wave's 64 and a chunk's 256 positions, beside a portion
    of a prompt that the general kernel takes in the same step (and leaves the single tokens alone)."""
    lengths = [1, 2, 64, 65, 256, 257, 300, 777]
    T = max(lengths)
    k, v, table = _paged(T, kv_heads, hd, bs, torch.float32, hd + heads, entries=len(lengths) + 1)
    g = torch.Generator().manual_seed(hd)
    portion = 5                                      # the last entry: tokens 100..104 of a prompt
    tokens = len(lengths) + portion
    qkv = torch.randn(tokens, (heads + 2 * kv_heads) * hd, generator=g)
    entry_start = i32(list(range(len(lengths) + 1)) + [tokens])
    first_pos = i32([n - 1 for n in lengths] + [100])
    chunks = (T + 255) // 256
    partial = torch.full((len(lengths) * heads * chunks * (hd + 2),), float("nan"))
    out = torch.zeros(tokens, heads * hd)
    (got, want), = both("attn_generic", "attn_decode_f32",
                        [qkv, qkv.shape[1], k, v, out, partial, i32(list(range(len(lengths)))), len(lengths), entry_start,
                         first_pos, table, table.shape[1], bs, heads, kv_heads, hd, 1 / math.sqrt(hd), window, chunks, None], [4])
    assert rel_err(got[:len(lengths)].numpy(), want[:len(lengths)].double().numpy()) < 3e-6
    assert float(got[len(lengths):].abs().max()) == 0.0          # the portion's rows are not this kernel's
    positions = i32([n - 1 for n in lengths] + list(range(100, 100 + portion)))
    entry_of = i32(list(range(len(lengths))) + [len(lengths)] * portion)
    (got, want), = both("attn_generic", "attn_generic",
                        [qkv, qkv.shape[1], k, v, torch.zeros(tokens, heads * hd), 0, positions, entry_of, table, table.shape[1], bs,
                         tokens, heads, kv_heads, hd, 1 / math.sqrt(hd), window, entry_start, None], [4])
    assert rel_err(got[len(lengths):].numpy(), want[len(lengths):].double().numpy()) < 3e-6
    assert float(got[:len(lengths)].abs().max()) == 0.0          # and the single tokens not the general kernel's


@pytest.mark.parametrize("heads,kv_heads,hd,bs", [(6, 3, 48, 8), (7, 1, 128, 16), (4, 2, 16, 4), (3, 3, 112, 32)])
@pytest.mark.parametrize("window", [0, 90])
def test_32_bit_prompt_attention_beside_its_twin(heads, kv_heads, hd, bs, window):
    """A portion of 300 tokens after 200 cached ones (its first tile begins inside a tile of positions, its last is
    short) and a second portion of 3 tokens from position 0, beside a single token that is not this kernel's."""
    first, count = 200, 300
    k, v, table = _paged(first + count, kv_heads, hd, bs, torch.float32, hd + heads, entries=3)
    g = torch.Generator().manual_seed(hd + 2)
    T = count + 3 + 1
    qkv = torch.randn(T, (heads + 2 * kv_heads) * hd, generator=g)
    entry_start, first_pos = i32([0, count, count + 3, count + 4]), i32([first, 0, 77])
    tiles = i32([0, 256, 1, 0, 0, 0, 0, 128])     # any order of the tiles
    (got, want), = both("attn_generic", "attn_prefill_f32",
                        [qkv, qkv.shape[1], k, v, torch.zeros(T, heads * hd), tiles, 4, 128, entry_start, first_pos, table,
                         table.shape[1], bs, heads, kv_heads, hd, 1 / math.sqrt(hd), window, None], [4])
    assert rel_err(got[:count + 3].numpy(), want[:count + 3].double().numpy()) < 3e-6
    assert float(got[count + 3:].abs().max()) == 0.0


@pytest.mark.parametrize("hd", [64, 128, 80])
@pytest.mark.parametrize("window", [0, 150])
def test_matrix_core_attention_beside_its_twins(hd, window):
    from vipera_rs_amd.ops import kernels
    heads, kv_heads, bs = 6, 2, 16
    module = f"attn_bf16_hd{kernels.attn_bf16_padded_width(hd)}"
    first, count = 200, 300                       # a portion of 300 tokens after 200 cached ones, and a second entry of one token
    k, v, table = _paged(first + count, kv_heads, hd, bs, torch.bfloat16, hd, entries=2)
    g = torch.Generator().manual_seed(hd + 1)
    T = count + 1
    qkv = torch.randn(T, (heads + 2 * kv_heads) * hd, generator=g).to(torch.bfloat16)
    entry_start, first_pos = i32([0, count, count + 1]), i32([first, 499])
    tiles = i32([0, 256, 0, 0, 0, 128])           # any order of the tiles
    padded = kernels.attn_bf16_padded_width(hd)
    # one workgroup per tile; its positions halved between sixteen waves; or cut into chunks of 128 and of 192
    # positions, a workgroup each, that a second kernel merges (where the width has the kernel for it)
    for split, chunk_tiles in ((0, 0), (1, 0), (0, 2), (0, 3)):
        max_chunks = -(-((first + count + 63) // 64) // chunk_tiles) if chunk_tiles else 0
        partial = torch.full((3 * heads * max_chunks * 128 * (padded + 4),), float("nan")) if chunk_tiles else None
        (got, want), = both(module, "attn_bf16_prefill",
                            [qkv, qkv.shape[1], k, v, torch.zeros(T, heads * hd, dtype=torch.bfloat16), tiles, 3, entry_start,
                             first_pos, table, table.shape[1], bs, heads, kv_heads, hd, 1 / math.sqrt(hd), window, split,
                             partial, partial.numel() if chunk_tiles else 0, chunk_tiles, max_chunks, None], [4])
        assert rel_err(got[:count].float().numpy(), want[:count].double().numpy()) < 8e-3, (split, chunk_tiles)
    chunk, chunks = 128, 4
    partial = torch.empty(1 * heads * chunks * (hd + 2))
    for join in (0, 1):                           # a workgroup per chunk and a merge kernel, or one that merges its waves' chunks
        (got, want), = both(module, "attn_bf16_decode",
                            [qkv, qkv.shape[1], k, v, torch.zeros(T, heads * hd, dtype=torch.bfloat16), None if join else partial,
                             i32([1]), 1, entry_start, first_pos, table, table.shape[1], bs, heads, kv_heads, hd,
                             1 / math.sqrt(hd), window, chunk, chunks, 0, join, None],
                            [4])
        assert rel_err(got[count:].float().numpy(), want[count:].double().numpy()) < 8e-3


def test_sampling_kernels_beside_their_twins():
    g = torch.Generator().manual_seed(5)
    rows, vocab = 40, 3001
    logits = torch.randn(rows, vocab, generator=g) * 3
    logits[3, 17] = float("inf")
    logits[4, :] = float("nan")
    logits[5, 100] = logits[5, 2000] = logits[5].max() + 1
    temperature = torch.where(torch.arange(rows) < 8, torch.zeros(rows), 0.5 + torch.rand(rows, generator=g))
    top_k = torch.where(torch.arange(rows) % 3 == 0, torch.full((rows,), 40), torch.zeros(rows)).to(torch.int32)
    top_p = torch.where(torch.arange(rows) % 2 == 0, torch.full((rows,), 0.9), torch.ones(rows))
    min_p = torch.where(torch.arange(rows) % 5 == 0, torch.full((rows,), 0.02), torch.zeros(rows))
    uniform = torch.rand(rows, generator=g, dtype=torch.float64)
    for slices in (0, 7, 32):     # the rows' best logits searched by one workgroup a row, or by `slices` of them first
        scratch = [torch.empty(rows * slices), torch.empty(rows * slices, dtype=torch.int32)] if slices else [None, None]
        (got, want), = both("sampling", "sample", [logits, rows, vocab, temperature, top_k, top_p, min_p, uniform,
                                                   torch.empty(rows, dtype=torch.int32), *scratch, slices,
                                                   None, None, None, None, None, 0, None], [8])
        assert torch.equal(got[:8], want[:8]) and got[4] == -1 and got[5] == 100
        # a sampled row could differ where u * mass falls within rounding of a boundary between two kept tokens, or where
        # a cut's edge rounds the other way; none of these seeded rows does
        assert torch.equal(got, want)
    # uniforms from the generators in the rows' state slots: two launches, the first seeds every second slot, the
    # others go on from what the table held; greedy rows record their position and leave the state alone
    slots = 64
    table = torch.randint(1, 2 ** 62, (slots, 2), generator=g, dtype=torch.int64)
    slot = torch.randperm(slots, generator=g)[:rows].to(torch.int32)
    for launch in range(2):
        position = torch.randint(0, 4096, (rows,), generator=g, dtype=torch.int32)
        reseed = ((torch.arange(rows) % 2 == 0) & (launch == 0)).to(torch.int32)
        seeds = torch.randint(1, 2 ** 62, (rows,), generator=g, dtype=torch.int64)
        (got, want), (got_table, want_table) = both(
            "sampling", "sample", [logits, rows, vocab, temperature, top_k, top_p, min_p, None,
                                   torch.empty(rows, dtype=torch.int32), None, None, 0,
                                   slot, position, reseed, seeds, table, slots, None], [8, 16])
        assert torch.equal(got_table, want_table), (got_table - want_table).nonzero()
        # the kernel's masses are 2^-40 fixed point, the twin's doubles: where u * mass falls within that rounding of
        # the boundary between two kept tokens they may pick either side, and nowhere else
        for r in (got != want).nonzero().flatten().tolist():
            state = (seeds[r] if reseed[r] else table[slot[r], 0]).item()
            state ^= state >> 12
            state ^= (state << 25) % 2 ** 64
            state ^= state >> 27
            u = ((state * 0x2545F4914F6CDD1D) % 2 ** 64 >> 11) / 2.0 ** 53
            kept = sorted(sampler_plain.kept_set(logits[r].numpy(), temperature[r].item(), top_k[r].item(),
                                                 top_p[r].item(), min_p[r].item()))
            ids = [i for i, _ in kept]
            shares = np.cumsum([float(w) for _, w in kept])
            shares /= shares[-1]
            a, b = sorted((ids.index(got[r].item()), ids.index(want[r].item())))
            assert b == a + 1 and abs(shares[a] - u) < 1e-6, (r, u, shares[a])
        assert torch.equal(got_table[slot.long(), 1], position.long())
        assert torch.equal(got_table[slot.long()[:8], 0], torch.where(reseed[:8].bool(), seeds[:8], table[slot.long()[:8], 0]))
        assert not torch.equal(got_table[slot.long()[8:], 0], table[slot.long()[8:], 0])
        table = got_table
    pen = torch.randn(3, 500, generator=g)
    args = [pen, 500, i32([0, 0, 2]), i32([3, 499, 3]), i32([2, 1, 4]), torch.tensor([1.3, 1.0, 0.7]), torch.tensor([0.2, 0.0, 0.1]),
            torch.tensor([0.1, 0.5, 0.0]), 3, None]
    (got, want), = both("sampling", "penalize", args, [0])
    assert torch.allclose(got, want, rtol=1e-6, atol=1e-6)
    (got, want), = both("sampling", "logit_bias", [pen, 500, i32([1, 2]), i32([4, 499]), torch.tensor([2.5, -1.0]), 2, None], [0])
    assert torch.equal(got, want)
