"""Matrix product dispatch: which kernel runs ``out (+)= a @ w.T + bias``.

All-bfloat16 operands whose rows are 16-byte aligned go to the matrix-core kernels; every other
combination (the 32-bit run, or a matrix kept in 32-bit inside a bfloat16 run) goes to the
32-bit FMA kernel.  Among the matrix-core kernels the number of rows of ``a`` (tokens) decides:

* many (prompts): the LDS-tiled kernel;
* up to 64 (decoding), and up to 128 for small weights (:func:`streams_weights`): the
  product is a stream of the weights.  Up to four tokens, or a small weight
  at up to 16 tokens, use the kernel whose waves split K inside a workgroup; otherwise the kernel that
  shares the activations through LDS, with K split over workgroups where the weight has too few rows
  to fill the GPU otherwise.  The thresholds were measured on the seven Qwen2.5 shapes (0.5B to 72B) on an MI355X.  The gated
  product of up to 16 tokens keeps all activations in LDS and gives every CU the same share of rows.
"""
from __future__ import annotations

from typing import Optional, Tuple

import torch

from . import kernels


def streams_weights(m: int, n: int, k: int) -> bool:
    """Whether a bfloat16 product of ``m`` tokens runs on a weight-streaming kernel rather than the tiled one:
    always up to 64 tokens, and up to 128 for a small weight, whose 128-token tiles are too few to fill the GPU
    (at 65 and 112 tokens: the 7B output projection 13.8 and 16.1 us against 16.1 and 17.4 tiled, the 1.5B q/k/v
    9.2 and 10.9 against 17.8 and 13.9; the larger weights are as fast or faster on the tiled kernel with its
    three LDS stages: the 7B down projection 36.3 against 41.8 at 80 tokens)."""
    if m <= 64:
        return True
    return m <= 128 and n * k <= 16_000_000


def mid_plan(m: int, n: int, k: int) -> Tuple[int, int]:
    """``(ranges of K, 16-row tiles per wave)`` for the LDS-shared kernel."""
    if m > 64:  # measured at 65, 96 and 128 tokens: one tile per wave; eight ranges of a long K, else four (the 0.5B
        # down projection, 896 x 4,864, at 65 tokens: 10.7 us with eight ranges, 14.2 with four)
        return max(1, min(8 if k >= 4_096 else 4, k // 256)), 1
    if n >= 100_000:
        return (1, 2) if m > 16 else (1, 1)
    if n >= 16_384:
        return (2, 1) if m > 16 else (1, 1)
    # few weight rows: split K while the workgroups still fit the 256 CUs at once (one more range was
    # measured a third slower), each range at least two chunks long
    # with many tokens, a long K and enough rows, two tiles per wave and twice the ranges measured a tenth faster (the
    # 32B down projection at 32 tokens 54.7 against 60.6 us); with few rows one tile and fewer ranges (the 1.5B down
    # projection at 64 tokens 13.0 against 15.7, the 3B one, 2,048 x 11,008, at 32 tokens 14.6 against 16.6)
    rows_per_wave = 2 if m >= 32 and k >= 8_192 and n >= 3_072 else 1
    row_blocks = (n + 64 * rows_per_wave - 1) // (64 * rows_per_wave)
    return max(1, min(k // 512, 256 // row_blocks)), rows_per_wave


def streams_in_wave_order(m: int, n: int, k: int, rotates: bool = False) -> bool:
    """Whether a bfloat16 product of ``m`` tokens runs on the kernel whose waves split K inside a workgroup (one
    launch; every workgroup of 16 rows reads all activations) and not on the one that shares the activations through
    LDS, splits K over workgroups and adds the ranges with a second kernel.  The first grows with the tokens, the
    second has the second launch to pay, so each weight has a number of tokens up to which the first is chosen
    (times in us of the product with what it fuses, the first kernel against the two, weights rotated so that none
    stays cached):

    * up to 4 tokens for a weight of 16,384 rows or more (the output matrix);
    * never for a weight of fewer rows and more than 100 M elements, whose workgroups would each stream most of a
      megabyte through four waves (the 32B down projection, 5,120 x 27,648: 57.1 against 52.8 at one token, 69.4
      against 52.5 at eight);
    * 60 M elements and more: never with 4,096 rows or more (8,192 x 8,192: 30.2 against 26.7 at one token, 32.4
      against 26.5 at eight; 5,120 x 13,824: 29.6 against 28.5 and 38.1 against 29.1), up to 5 tokens with fewer
      (the 7B down projection, 3,584 x 18,944: 25.9 against 27.7 at one, 28.3 against 27.9 at six, 30.2 against 28.0
      at eight);
    * 20 M elements and more: up to 6 (5,120 x 5,120: 13.5 against 14.0 at one token, 15.1 against 14.6 at six, 16.6
      against 14.4 at eight; 2,048 x 11,008: 14.3 against 13.7 at four, 15.5 against 13.8 at eight);
    * smaller weights: up to 8 with a long K (1,536 x 8,960: 12.7 against 13.1 at eight, 14.3 against 13.0 at
      twelve), up to 16 with a short one (3,584 x 3,584: 11.0 against 12.9 at sixteen).

    ``rotates``: the product is q/k/v, whose second kernel also rotates and writes the cache and costs 2 us more:
    up to 3 tokens from 60 M elements on (10,240 x 8,192: 32.5 against 34.6 at one token, 34.9 against 34.2 at four,
    39.3 against 34.8 at eight), up to 10 from 20 M on (7,168 x 5,120: 19.3 against 20.0 at eight, 24.6 against 20.6
    at sixteen)."""
    if n >= 16_384:
        return m <= 4
    elements = n * k
    if elements > 100_000_000:
        return False
    if elements >= 60_000_000:
        limit = 3 if rotates else 5 if n < 4_096 else 0
    elif elements >= 20_000_000:
        limit = 10 if rotates else 6
    else:
        limit = 8 if k >= 8_192 else 16
    return m <= limit


def linear(a: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor], out: torch.Tensor,
           accumulate: bool = False) -> torch.Tensor:
    if a.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and kernels.gemm_bf16_supported(a, w, out):
        m, k = a.shape
        n = w.shape[0]
        if not streams_weights(m, n, k) or streams_in_wave_order(m, n, k):
            kernels.gemm_bf16(a, w, bias, out, accumulate)
        else:
            ranges, rows_per_wave = mid_plan(m, n, k)
            kernels.gemm_bf16_mid(a, w, bias, out, accumulate, ranges, rows_per_wave)
    else:
        kernels.gemm_generic(a, w, bias, out, accumulate)
    return out


def linear_follow(a: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor], residual: torch.Tensor,
                  gain: torch.Tensor, scaled: torch.Tensor, sumsq: torch.Tensor) -> int:
    """``residual += a @ w.T + bias`` and, where the kernel that :func:`linear` would pick can do it, the first half
    of the RMS norm that follows (``scaled = residual * gain`` in bfloat16 and the sums of squares in groups, see
    :func:`kernels.gemm_bf16_follow`).  Returns the number of groups, or 0 where the product ran without it."""
    m, k = a.shape
    n = w.shape[0]
    bf16 = a.dtype == torch.bfloat16 and w.dtype == torch.bfloat16
    if bf16 and m <= 16 and streams_in_wave_order(m, n, k) and kernels.gemm_bf16_follow_supported(a, w, residual):
        return kernels.gemm_bf16_follow(a, w, bias, residual, gain, scaled, sumsq)
    if (bf16 and m <= 64 and residual.dtype == torch.float32 and residual.is_contiguous()
            and kernels.gemm_bf16_supported(a, w, residual)):
        ranges, rows_per_wave = mid_plan(m, n, k)
        if ranges >= 2 and k // ranges >= 512:
            return kernels.gemm_bf16_mid_follow(a, w, bias, residual, ranges, rows_per_wave, gain, scaled, sumsq)
    linear(a, w, bias, residual, accumulate=True)
    return 0


def split_qkv_plan(m: int, n: int, k: int) -> Optional[Tuple[int, int]]:
    """``(ranges, tiles per wave)`` if a q/k/v product of ``m`` tokens runs with K split over workgroups, so that the
    kernel that adds the ranges can also rotate and write the cache (up to 64 tokens, where the product does not run
    in wave order), else None."""
    if m > 64 or streams_in_wave_order(m, n, k, rotates=True):
        return None
    ranges, rows_per_wave = mid_plan(m, n, k)
    ranges = max(ranges, 2)   # the second kernel is what rotates: two ranges where one would do (10,240 x 8,192)
    return (ranges, rows_per_wave) if k // ranges >= 512 else None


def interleave_gate_up(gate: torch.Tensor, up: torch.Tensor) -> torch.Tensor:
    """The fused weight of a gated feed-forward with rows interleaved in groups of 16: rows ``[32 p, 32 p + 16)``
    are gate rows ``[16 p, 16 p + 16)``, rows ``[32 p + 16, 32 p + 32)`` the up rows of the same outputs."""
    inter, width = gate.shape
    fused = torch.stack([gate.view(inter // 16, 16, width), up.view(inter // 16, 16, width)], dim=1)
    return fused.reshape(2 * inter, width).contiguous()


RESIDENT_LDS_BYTES = 160 * 1024 - (16 * 1024 + 256)   # what the resident kernel may fill with activations


def gated_resident_fits(m: int, n: int, k: int) -> bool:
    """Whether the gated kernel that keeps all activations in LDS takes the shape: up to 16 tokens, K in
    whole chunks of 128, and ``tokens x (K + 8)`` bfloat16 values within a CU's LDS."""
    return m <= 16 and k % 128 == 0 and n % 32 == 0 and m * (k + 8) * 2 <= RESIDENT_LDS_BYTES


def gated_rows_per_wave(m: int, n: int) -> int:
    """One or two 16-row tiles per wave for the LDS-shared gated product (64 or 128 weight rows per workgroup).
    A workgroup reads its weight rows and all of the activations; a CU's time goes with the bytes it pulls,
    so what counts is how many workgroups the busiest CU gets (whole rounds over 256 CUs while they are few;
    with three rounds or more the dispatcher evens them out) times the rows and padded tokens of each.
    Measured at the 1.5B, 7B and 32B widths with 8 to 64 tokens; ties go to one tile."""
    padded = (m + 15) // 16 * 16
    def cost(rows: int) -> float:
        groups = (n + rows - 1) // rows
        rounds = groups / 256 if groups >= 768 else (groups + 255) // 256
        return rounds * (rows + padded)
    return 2 if cost(128) < cost(64) else 1


def gated_plan(m: int, n: int, k: int, cus: int = 256) -> int:
    """What :func:`kernels.gemm_bf16_gated` is asked for at up to 64 tokens: 0, the kernel with resident
    activations and one workgroup per CU, where it takes the shape and the outputs, four at a time, divide evenly
    enough over the ``cus`` workgroups (every CU with a pair of 16-row tiles at least, the busiest within 10 % of the
    mean: at 7B and 32B widths it measured 2 to 7 % faster than the LDS-shared kernel when its runs were still whole
    pairs, and it can divide by the norm before it, which saves that norm's kernel); else the LDS-shared kernel with
    one or two tiles per wave."""
    pairs, quads = n // 32, n // 8
    if gated_resident_fits(m, n, k) and pairs >= cus and -(-quads // cus) * cus <= 1.1 * quads:
        return 0
    if m <= 32 and k % 2048 == 0 and n * k >= 4e8:
        # the largest weights with rows a multiple of 4 KB apart, where the LDS-shared kernel's workgroups start at
        # different chunks: it streams them faster than the tiled one (72B, 59,136 x 8,192, at 17 to 32 tokens: 164
        # to 171 us against 185; at 64 the norm's own kernel, which only the tiled one saves, makes them even)
        return gated_rows_per_wave(m, n)
    if n * k >= 1e8 or m * n * k >= 1.5e9:
        # a large weight, or many tokens on a small one: the tiled kernel (3) with its three LDS stages and tiles
        # of 96 to 224 weight rows that fill the CUs in one round passes the LDS-shared one (7B widths at 17 to 64
        # tokens: 51 to 54 us against 57 to 71; 32B: 102 to 106 against 110 to 120; 1.5B from 64 tokens)
        return 3
    return gated_rows_per_wave(m, n)


def linear_gated(a: torch.Tensor, w_gate_up: torch.Tensor, out: torch.Tensor, interleaved: bool) -> torch.Tensor:
    """``out = up(a) * silu(gate(a))`` with the fused weight ``w_gate_up`` (``interleaved`` or ``[gate; up]``)."""
    m, k = a.shape
    n = w_gate_up.shape[0]
    fusable = (interleaved and a.dtype == torch.bfloat16 and w_gate_up.dtype == torch.bfloat16
               and out.dtype == torch.bfloat16 and kernels.gemm_bf16_supported(a, w_gate_up, out))
    if fusable:
        # the epilogue of the tiled kernel, of the resident kernel, or of the LDS-shared kernel with one K
        # range applies the gate
        plan = gated_plan(m, n, k, kernels.compute_units(a.device)) if m <= 64 else 1
        if m > 4 or plan == 0:
            kernels.gemm_bf16_gated(a, w_gate_up, out, rows_per_wave=plan)
            return out
    gate_up = torch.empty((m, n), dtype=out.dtype, device=out.device)
    linear(a, w_gate_up, None, gate_up)
    kernels.swiglu(gate_up, out, interleaved)
    return out
