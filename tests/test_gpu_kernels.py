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
               (64, 520, 1024), (65, 130, 72), (128, 128, 64), (200, 257, 136), (515, 384, 200)]


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


def test_gemm_generic_does_not_depend_on_the_batch():
    from vipera_rs_amd.ops import kernels
    g = torch.Generator().manual_seed(2)
    a = torch.randn(70, 136, generator=g).to(DEV)
    w = torch.randn(90, 136, generator=g).to(DEV)
    whole = torch.empty(70, 90, device=DEV)
    kernels.gemm_generic(a, w, None, whole)
    single = torch.empty(1, 90, device=DEV)
    kernels.gemm_generic(a[37:38].contiguous(), w, None, single)
    assert torch.equal(single[0], whole[37])  # bit for bit: one thread sums each element in k order
