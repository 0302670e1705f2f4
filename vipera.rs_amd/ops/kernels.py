"""Python bindings of the HIP kernels: shape checks on the host, then one launch on the current stream.

Every function takes device tensors, checks that their shapes and dtypes are what the kernel
and its grid assume, and launches on ``torch.cuda.current_stream()``.  There is no fallback:
when a library cannot be built or loaded the call raises.
"""
from __future__ import annotations

import ctypes
from typing import Optional

import torch

from ..errors import InternalError, InvalidArgumentError, UnsupportedError
from .build import load_module

_DT = {torch.float32: 0, torch.bfloat16: 1}
_p = ctypes.c_void_p
_i = ctypes.c_int
_ll = ctypes.c_longlong
_f = ctypes.c_float


def _dt(tensor: torch.Tensor, what: str) -> int:
    if tensor.dtype not in _DT:
        raise UnsupportedError(f"{what} has dtype {tensor.dtype}; float32 and bfloat16 are implemented")
    return _DT[tensor.dtype]


def _ptr(tensor: Optional[torch.Tensor]):
    return _p(tensor.data_ptr()) if tensor is not None else _p(0)


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)
_raw_device = getattr(torch._C, "_cuda_getDevice", None)


def _stream():
    """The current stream's handle.  Through torch's raw accessors where it has them: ``torch.cuda.current_stream()``
    builds a Python object on every call, which was a quarter of the host's time for a step launched kernel by kernel."""
    if _raw_stream is not None and _raw_device is not None:
        return _p(_raw_stream(_raw_device()))
    return _p(torch.cuda.current_stream().cuda_stream)


def _need(cond: bool, text: str) -> None:
    if not cond:
        raise InvalidArgumentError(text)


def _dev(*tensors: Optional[torch.Tensor]) -> None:
    for tensor in tensors:
        if tensor is not None and not tensor.is_cuda:
            raise InvalidArgumentError("kernel operands must live on the GPU; got a CPU tensor")


def _status(code: int, name: str) -> None:
    if code == 0:
        return
    if code == -1:
        raise InvalidArgumentError(f"{name}: the launcher refused its arguments")
    if code == -2:
        raise UnsupportedError(f"{name}: a size is outside what this kernel is built for")
    raise InternalError(f"{name}: HIP error {code} at launch")


ATTENTION_MAX_HEAD_DIM = 256    # both attention kernels keep a head's dims in registers or one LDS row
ATTENTION_MAX_HEADS = 65_535    # q, k and v heads of a token are one grid dimension of the rotation kernel
GEMM_BF16_MAX_K = 1 << 23       # the matrix-core products form 32-bit byte offsets inside a tile of rows


def _cache_ok(k_cache, v_cache, kv_heads: int, head_dim: int, dtype) -> bool:
    """K pages ``[pages, kv_heads, block_size, head_dim]``, V pages ``[pages, kv_heads, head_dim, block_size]``."""
    return (k_cache.dim() == 4 and v_cache.dim() == 4 and k_cache.shape[1] == kv_heads
            and k_cache.shape[3] == head_dim and v_cache.shape[1] == kv_heads and v_cache.shape[2] == head_dim
            and v_cache.shape[0] == k_cache.shape[0] and v_cache.shape[3] == k_cache.shape[2]
            and k_cache.dtype == dtype and v_cache.dtype == dtype and k_cache.is_contiguous()
            and v_cache.is_contiguous())


_signatures_done = set()


def _fn(module: str, name: str, argtypes, key: str = None):
    library = load_module(module)
    fn = getattr(library, name)
    key = key or name
    if key not in _signatures_done:
        fn.argtypes = argtypes
        fn.restype = ctypes.c_int
        _signatures_done.add(key)
    return fn


# ----------------------------------------------------------------------------------------------
def fetch_words(pinned: torch.Tensor, out: torch.Tensor) -> bool:
    """``out[:] = pinned[:]`` (int32 words) by a kernel that reads the pinned host tensor directly, in the current
    stream.  Returns False, having done nothing, if the runtime does not give the host memory a device address
    (the caller then copies with ``out.copy_``)."""
    _dev(out)
    _need(not pinned.is_cuda and pinned.is_pinned(), "fetch_words: the source must be pinned host memory")
    _need(pinned.dtype == torch.int32 and out.dtype == torch.int32 and pinned.is_contiguous() and out.is_contiguous()
          and pinned.numel() == out.numel(), "fetch_words: two contiguous int32 tensors of one size")
    fn = _fn("elementwise", "vk_fetch_words", [_p, _p, _ll, _p])
    code = fn(pinned.data_ptr(), _ptr(out), out.numel(), _stream())
    if code == -2:
        return False
    _status(code, "fetch_words")
    return True


# ----------------------------------------------------------------------------------------------
def embed_gather(table: torch.Tensor, tokens: torch.Tensor, out: torch.Tensor,
                 source: Optional[torch.Tensor] = None, sampled: Optional[torch.Tensor] = None) -> None:
    """``out[t, :] = table[tokens[t], :]`` widened to 32-bit.  The caller has checked the ids.

    With ``source`` and ``sampled``: where ``source[t] >= 0`` the id is ``sampled[source[t]]``, which an
    earlier kernel of the stream left on the device."""
    _dev(table, tokens, out, source, sampled)
    num_tokens, width = out.shape
    _need(table.dim() == 2 and table.shape[1] == width and table.is_contiguous(), "embed_gather: table shape")
    _need(tokens.dtype == torch.int32 and tokens.numel() >= num_tokens and tokens.is_contiguous(), "embed_gather: tokens")
    _need(out.dtype == torch.float32 and out.is_contiguous(), "embed_gather: out must be contiguous float32")
    if source is not None:
        _need(sampled is not None and sampled.dtype == torch.int32 and sampled.is_contiguous(),
              "embed_gather: sampled must be contiguous int32")
        _need(source.dtype == torch.int32 and source.numel() >= num_tokens and source.is_contiguous(),
              "embed_gather: source")
    fn = _fn("elementwise", "vk_embed_gather", [_p, _i, _p, _p, _p, _p, _i, _i, _i, _p])
    _status(fn(_ptr(table), _dt(table, "table"), _ptr(tokens), _ptr(source), _ptr(sampled if source is not None else None),
               _ptr(out), num_tokens, width, table.shape[0], _stream()), "embed_gather")


def rmsnorm(x: torch.Tensor, weight: torch.Tensor, eps: float, out: torch.Tensor,
            rows: Optional[torch.Tensor] = None) -> None:
    """``out[r] = x[rows[r]] * rsqrt(mean(x^2) + eps) * weight`` (``rows`` absent: every row in order)."""
    _dev(x, weight, out, rows)
    num_rows, width = out.shape
    _need(x.dtype == torch.float32 and x.dim() == 2 and x.shape[1] == width and x.is_contiguous(), "rmsnorm: x")
    _need(weight.dtype == torch.float32 and weight.numel() == width and weight.is_contiguous(), "rmsnorm: weight")
    _need(out.is_contiguous(), "rmsnorm: out must be contiguous")
    if rows is None:
        _need(x.shape[0] >= num_rows, "rmsnorm: fewer input rows than output rows")
    else:
        _need(rows.dtype == torch.int32 and rows.numel() >= num_rows and rows.is_contiguous(), "rmsnorm: rows")
    fn = _fn("elementwise", "vk_rmsnorm", [_p, _p, _p, _p, _i, _i, _i, _f, _p])
    _status(fn(_ptr(x), _ptr(weight), _ptr(rows), _ptr(out), _dt(out, "out"), num_rows, width, float(eps), _stream()),
            "rmsnorm")


def rope_angles(positions: torch.Tensor, inv_freq: torch.Tensor, num_tokens: int) -> torch.Tensor:
    """``[num_tokens, len(inv_freq), 2]`` floats: sine and cosine of ``float(pos) * inv_freq`` for a step's
    tokens, computed once where many heads and layers would each compute them again."""
    _dev(positions, inv_freq)
    _need(positions.dtype == torch.int32 and positions.numel() >= num_tokens, "rope_angles: positions")
    _need(inv_freq.dtype == torch.float32 and inv_freq.is_contiguous(), "rope_angles: inv_freq must be float32")
    out = torch.empty((num_tokens, inv_freq.numel(), 2), dtype=torch.float32, device=positions.device)
    fn = _fn("elementwise", "vk_rope_angles", [_p, _p, _i, _i, _p, _p])
    _status(fn(_ptr(positions), _ptr(inv_freq), inv_freq.numel(), num_tokens, _ptr(out), _stream()), "rope_angles")
    return out


def rope_kvwrite(qkv: torch.Tensor, positions: torch.Tensor, inv_freq: Optional[torch.Tensor], rotary_dim: int,
                 k_cache: Optional[torch.Tensor], v_cache: Optional[torch.Tensor], entry_of_token: torch.Tensor,
                 block_table: Optional[torch.Tensor], heads: int, kv_heads: int, head_dim: int,
                 angles: Optional[torch.Tensor] = None) -> None:
    """Rotate the q and k heads of ``qkv`` in place, then store the tokens' K and V in their pages.
    ``angles``: the step's table from :func:`rope_angles`, used instead of computing sines and cosines here.

    ``k_cache``: ``[pages, kv_heads, block_size, head_dim]``; ``v_cache`` is transposed,
    ``[pages, kv_heads, head_dim, block_size]``; ``block_table``: ``[entries, width]``.
    The caller guarantees that every token's page exists in its entry's row of the table.
    """
    _dev(qkv, positions, inv_freq, k_cache, v_cache, entry_of_token, block_table)
    num_tokens = qkv.shape[0]
    _need(qkv.dim() == 2 and qkv.shape[1] == (heads + 2 * kv_heads) * head_dim and qkv.is_contiguous(),
          "rope_kvwrite: qkv must be [tokens, (heads + 2 kv_heads) * head_dim]")
    _need(positions.dtype == torch.int32 and positions.numel() >= num_tokens, "rope_kvwrite: positions")
    _need(0 <= rotary_dim <= head_dim and rotary_dim % 2 == 0, "rope_kvwrite: rotary_dim")
    if rotary_dim:
        _need(inv_freq is not None and inv_freq.dtype == torch.float32 and inv_freq.numel() == rotary_dim // 2,
              "rope_kvwrite: inv_freq must hold rotary_dim / 2 floats")
    table_width = block_size = 0
    if k_cache is not None:
        _need(v_cache is not None and block_table is not None, "rope_kvwrite: cache without table")
        _need(_cache_ok(k_cache, v_cache, kv_heads, head_dim, qkv.dtype), "rope_kvwrite: cache shape or dtype")
        _need(block_table.dtype == torch.int32 and block_table.dim() == 2 and block_table.is_contiguous(),
              "rope_kvwrite: block table")
        _need(entry_of_token.dtype == torch.int32 and entry_of_token.numel() >= num_tokens, "rope_kvwrite: entries")
        table_width, block_size = block_table.shape[1], k_cache.shape[2]
    if angles is not None:
        _dev(angles)
        _need(rotary_dim > 0 and angles.dtype == torch.float32 and angles.is_contiguous()
              and angles.shape == (num_tokens, rotary_dim // 2, 2), "rope_kvwrite: angles must be [tokens, rotary_dim / 2, 2]")
    fn = _fn("elementwise", "vk_rope_kvwrite", [_p, _i, _p, _p, _p, _i, _p, _p, _p, _p, _i, _i, _i, _i, _i, _i, _p])
    _status(fn(_ptr(qkv), _dt(qkv, "qkv"), _ptr(positions), _ptr(inv_freq), _ptr(angles), rotary_dim, _ptr(k_cache), _ptr(v_cache),
               _ptr(entry_of_token), _ptr(block_table), table_width, block_size, num_tokens, heads, kv_heads,
               head_dim, _stream()), "rope_kvwrite")


def swiglu(gate_up: torch.Tensor, out: torch.Tensor, interleaved: bool = False) -> None:
    """``out = up * silu(gate)``; a row of ``gate_up`` is ``[gate | up]``, or with ``interleaved`` groups of
    16 gate columns followed by the 16 up columns of the same outputs."""
    _dev(gate_up, out)
    num_tokens, inter = out.shape
    _need(gate_up.shape == (num_tokens, 2 * inter) and gate_up.dtype == out.dtype and gate_up.is_contiguous()
          and out.is_contiguous(), "swiglu: gate_up must be [tokens, 2 * intermediate] of out's dtype")
    _need(not interleaved or inter % 16 == 0, "swiglu: the interleaved layout needs a multiple of 16 outputs")
    fn = _fn("elementwise", "vk_swiglu", [_p, _p, _i, _i, _i, _i, _p])
    _status(fn(_ptr(gate_up), _ptr(out), _dt(out, "out"), num_tokens, inter, 1 if interleaved else 0, _stream()), "swiglu")


def fill_normal(out: torch.Tensor, key: int, std: float, offset: float = 0.0) -> None:
    """Fill with ``offset + std * n_i``, ``n_i`` the counter-based normal stream of ``key``."""
    _dev(out)
    _need(out.is_contiguous(), "fill_normal: out must be contiguous")
    fn = _fn("elementwise", "vk_fill_normal", [_p, _i, _ll, ctypes.c_ulonglong, _f, _f, _p])
    _status(fn(_ptr(out), _dt(out, "out"), out.numel(), key & ((1 << 64) - 1), float(std), float(offset), _stream()),
            "fill_normal")


# ----------------------------------------------------------------------------------------------
def gemm_generic(a: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor], out: torch.Tensor,
                 accumulate: bool = False) -> None:
    """``out (+)= a @ w.T + bias`` in 32-bit FMA; ``a`` and ``out`` may be row-strided views."""
    _dev(a, w, bias, out)
    _need(a.dim() == 2 and w.dim() == 2 and out.dim() == 2, "gemm: operands must be matrices")
    m, k = a.shape
    n = w.shape[0]
    _need(w.shape[1] == k and out.shape == (m, n), f"gemm: shapes {tuple(a.shape)} x {tuple(w.shape)}^T -> {tuple(out.shape)}")
    _need(a.stride(1) == 1 and out.stride(1) == 1 and w.is_contiguous(), "gemm: inner strides must be 1")
    _need(a.stride(0) >= k or m == 1, "gemm: a's row stride")
    _need(out.stride(0) >= n or m == 1, "gemm: out's row stride")
    if bias is not None:
        _need(bias.dtype == torch.float32 and bias.numel() == n and bias.is_contiguous(), "gemm: bias must be float32 [n]")
    if accumulate:
        _need(out.dtype == torch.float32, "gemm: accumulation needs a float32 output")
    lda = a.stride(0) if m > 1 else max(a.stride(0), k)
    ldc = out.stride(0) if m > 1 else max(out.stride(0), n)
    if (m <= 64 and a.dtype == torch.float32 and w.dtype == torch.float32 and k >= 4 and k % 4 == 0 and lda % 4 == 0
            and a.data_ptr() % 16 == 0 and w.data_ptr() % 16 == 0 and k < 65535 * 1024):
        # up to 64 tokens in 32-bit: a stream of the weights (the same sums in the same order as the tiled kernel)
        slabs = _split_k_workspace(a.device, ((k + 1023) // 1024) * m * n, "stream")
        fn = _fn("gemm_generic", "vk_gemm_stream", [_p, _p, _p, _p, _i, _i, _i, _i, _ll, _ll, _i, _p, _ll, _p])
        _status(fn(_ptr(a), _ptr(w), _ptr(bias), _ptr(out), _dt(out, "out"), m, n, k, lda, ldc, 1 if accumulate else 0,
                   _ptr(slabs), slabs.numel(), _stream()), "gemm_stream")
        return
    fn = _fn("gemm_generic", "vk_gemm_generic", [_p, _i, _p, _i, _p, _p, _i, _i, _i, _i, _ll, _ll, _i, _p])
    _status(fn(_ptr(a), _dt(a, "a"), _ptr(w), _dt(w, "w"), _ptr(bias), _ptr(out), _dt(out, "out"), m, n, k, lda, ldc,
               1 if accumulate else 0, _stream()), "gemm_generic")


# ----------------------------------------------------------------------------------------------
def attn_generic(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, out: torch.Tensor,
                 positions: torch.Tensor, entry_of_token: torch.Tensor, block_table: torch.Tensor,
                 heads: int, kv_heads: int, head_dim: int, scale: float, window: int,
                 skip_single_of: Optional[torch.Tensor] = None) -> None:
    """Causal GQA over the paged cache for every token of the step, in 32-bit arithmetic.

    ``q``: a view ``[tokens, >= heads * head_dim]`` whose row holds the query heads first (the fused
    qkv buffer qualifies); ``out``: ``[tokens, heads * head_dim]``.  ``skip_single_of``: the step's
    ``entry_start``; tokens of entries that hold one token are then left alone (for :func:`attn_decode_f32`).
    """
    _dev(q, k_cache, v_cache, out, positions, entry_of_token, block_table, skip_single_of)
    if skip_single_of is not None:
        _need(skip_single_of.dtype == torch.int32 and skip_single_of.numel() == block_table.shape[0] + 1,
              "attention: entry_start must hold one offset per entry and the end")
    num_tokens = out.shape[0]
    _need(q.dim() == 2 and q.shape[0] == num_tokens and q.stride(1) == 1 and q.shape[1] >= heads * head_dim, "attention: q")
    _need(out.shape == (num_tokens, heads * head_dim) and out.is_contiguous() and out.dtype == q.dtype, "attention: out")
    _need(_cache_ok(k_cache, v_cache, kv_heads, head_dim, q.dtype), "attention: cache shape or dtype")
    _need(positions.dtype == torch.int32 and positions.numel() >= num_tokens, "attention: positions")
    _need(entry_of_token.dtype == torch.int32 and entry_of_token.numel() >= num_tokens, "attention: entries")
    _need(block_table.dtype == torch.int32 and block_table.dim() == 2 and block_table.is_contiguous(), "attention: table")
    _need(heads % kv_heads == 0, "attention: heads must be a multiple of kv_heads")
    if head_dim > ATTENTION_MAX_HEAD_DIM:
        raise UnsupportedError(f"attention: head_dim {head_dim} is above the kernels' limit of {ATTENTION_MAX_HEAD_DIM}")
    fn = _fn("attn_generic", "vk_attn_generic",
             [_p, _ll, _p, _p, _p, _i, _p, _p, _p, _i, _i, _i, _i, _i, _i, _f, _i, _p, _p])
    _status(fn(_ptr(q), q.stride(0), _ptr(k_cache), _ptr(v_cache), _ptr(out), _dt(q, "q"), _ptr(positions),
               _ptr(entry_of_token), _ptr(block_table), block_table.shape[1], k_cache.shape[2], num_tokens, heads,
               kv_heads, head_dim, float(scale), int(window), _ptr(skip_single_of), _stream()), "attn_generic")


ATTN_DECODE_F32_CHUNK = 256   # positions of one workgroup of attn_decode_f32 (the kernel's DEC_CHUNK)


def attn_decode_f32_supported(q: torch.Tensor, k_cache: torch.Tensor, head_dim: int) -> bool:
    """Whether :func:`attn_decode_f32` takes the operands: all 32-bit, a head width and pages that are multiples
    of 4, 16-byte rows."""
    return (q.dtype == torch.float32 and k_cache.dtype == torch.float32 and head_dim % 4 == 0
            and head_dim <= ATTENTION_MAX_HEAD_DIM and k_cache.shape[2] % 4 == 0 and q.stride(0) % 4 == 0
            and q.data_ptr() % 16 == 0)


def attn_decode_f32(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, out: torch.Tensor,
                    partial: torch.Tensor, entries: torch.Tensor, entry_start: torch.Tensor,
                    entry_first_pos: torch.Tensor, block_table: torch.Tensor, heads: int, kv_heads: int,
                    head_dim: int, scale: float, window: int, chunks: int) -> None:
    """32-bit attention of the single-token entries listed in ``entries``; their positions are split into
    ``chunks`` of :data:`ATTN_DECODE_F32_CHUNK`, which must cover the longest visible range."""
    _dev(q, k_cache, v_cache, out, partial, entries, entry_start, entry_first_pos, block_table)
    _need(attn_decode_f32_supported(q, k_cache, head_dim), "attn_decode_f32: 32-bit operands, head width and pages "
          "that are multiples of 4")
    _need(q.dim() == 2 and q.stride(1) == 1 and q.shape[1] >= heads * head_dim, "attention: q")
    _need(out.shape == (q.shape[0], heads * head_dim) and out.is_contiguous() and out.dtype == q.dtype, "attention: out")
    _need(_cache_ok(k_cache, v_cache, kv_heads, head_dim, q.dtype), "attention: cache shape or dtype")
    count = entries.numel()
    _need(entries.dtype == torch.int32 and entries.is_contiguous(), "attention: entries")
    _need(partial.dtype == torch.float32 and partial.is_contiguous()
          and partial.numel() >= count * heads * chunks * (head_dim + 2), "attention: workspace too small")
    _need(block_table.dtype == torch.int32 and block_table.dim() == 2 and block_table.is_contiguous(), "attention: table")
    _need(entry_start.dtype == torch.int32 and entry_first_pos.dtype == torch.int32
          and entry_start.numel() == block_table.shape[0] + 1 and entry_first_pos.numel() == block_table.shape[0],
          "attention: entry arrays")
    _need(heads % kv_heads == 0 and chunks >= 1, "attention: heads must be a multiple of kv_heads")
    fn = _fn("attn_generic", "vk_attn_decode_f32",
             [_p, _ll, _p, _p, _p, _p, _p, _i, _p, _p, _p, _i, _i, _i, _i, _i, _f, _i, _i, _p])
    _status(fn(_ptr(q), q.stride(0), _ptr(k_cache), _ptr(v_cache), _ptr(out), _ptr(partial), _ptr(entries), count,
               _ptr(entry_start), _ptr(entry_first_pos), _ptr(block_table), block_table.shape[1], k_cache.shape[2],
               heads, kv_heads, head_dim, float(scale), int(window), int(chunks), _stream()), "attn_decode_f32")


ATTN_PREFILL_F32_MAX_HEAD_DIM = 128   # the K, V and weight tiles of a wider head do not fit a CU's LDS


def attn_prefill_f32_supported(q: torch.Tensor, k_cache: torch.Tensor, head_dim: int) -> bool:
    """Whether :func:`attn_prefill_f32` takes the operands: all 32-bit, a head width that is a multiple of 16 and
    at most 128, pages of a multiple of 4 positions, 16-byte rows."""
    return (q.dtype == torch.float32 and k_cache.dtype == torch.float32 and head_dim % 16 == 0
            and head_dim <= ATTN_PREFILL_F32_MAX_HEAD_DIM and k_cache.shape[2] % 4 == 0 and q.stride(0) % 4 == 0
            and q.data_ptr() % 16 == 0)


def attn_prefill_f32(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, out: torch.Tensor,
                     tiles: torch.Tensor, tile_tokens: int, entry_start: torch.Tensor, entry_first_pos: torch.Tensor,
                     block_table: torch.Tensor, heads: int, kv_heads: int, head_dim: int, scale: float,
                     window: int) -> None:
    """32-bit attention of the entries' tiles listed in ``tiles`` (pairs: entry, first token within it; ``tile_tokens``
    tokens a tile, a multiple of 64): 64 tokens of one head a workgroup, the positions in LDS tiles of 64."""
    _dev(q, k_cache, v_cache, out, tiles, entry_start, entry_first_pos, block_table)
    _need(attn_prefill_f32_supported(q, k_cache, head_dim), "attn_prefill_f32: 32-bit operands, a head width that is a "
          "multiple of 16 up to 128, pages of a multiple of 4 positions")
    _need(q.dim() == 2 and q.stride(1) == 1 and q.shape[1] >= heads * head_dim, "attention: q")
    _need(out.shape == (q.shape[0], heads * head_dim) and out.is_contiguous() and out.dtype == q.dtype, "attention: out")
    _need(_cache_ok(k_cache, v_cache, kv_heads, head_dim, q.dtype), "attention: cache shape or dtype")
    _need(tiles.dtype == torch.int32 and tiles.numel() % 2 == 0 and tiles.is_contiguous(), "attention: tiles")
    _need(tile_tokens >= 64 and tile_tokens % 64 == 0, "attention: tokens of a tile must be a multiple of 64")
    _need(block_table.dtype == torch.int32 and block_table.dim() == 2 and block_table.is_contiguous(), "attention: table")
    _need(entry_start.dtype == torch.int32 and entry_first_pos.dtype == torch.int32
          and entry_start.numel() == block_table.shape[0] + 1 and entry_first_pos.numel() == block_table.shape[0],
          "attention: entry arrays")
    _need(heads % kv_heads == 0, "attention: heads must be a multiple of kv_heads")
    fn = _fn("attn_generic", "vk_attn_prefill_f32",
             [_p, _ll, _p, _p, _p, _p, _i, _i, _p, _p, _p, _i, _i, _i, _i, _i, _f, _i, _p])
    _status(fn(_ptr(q), q.stride(0), _ptr(k_cache), _ptr(v_cache), _ptr(out), _ptr(tiles), tiles.numel() // 2,
               int(tile_tokens), _ptr(entry_start), _ptr(entry_first_pos), _ptr(block_table), block_table.shape[1],
               k_cache.shape[2], heads, kv_heads, head_dim, float(scale), int(window), _stream()), "attn_prefill_f32")


# ----------------------------------------------------------------------------------------------
SAMPLE_SLICES = 32
SAMPLE_SLICES_FROM = 32_768   # columns from which a row's best logit is searched in slices


def sample(logits: torch.Tensor, temperature: torch.Tensor, top_k: torch.Tensor, top_p: torch.Tensor,
           min_p: torch.Tensor, uniform: Optional[torch.Tensor], out: torch.Tensor,
           slot: Optional[torch.Tensor] = None, position: Optional[torch.Tensor] = None,
           reseed: Optional[torch.Tensor] = None, seed_state: Optional[torch.Tensor] = None,
           slot_table: Optional[torch.Tensor] = None) -> None:
    """One token per row: greedy where ``temperature`` is 0, else a draw after the top-k/top-p/min-p cuts.

    ``out[r]`` is -1 when row ``r`` has no finite logit.  The uniform of a row that draws is ``uniform[r]``, or
    with a ``slot_table`` (int64 ``[slots, 2]``: generator state and next position per state slot) the next
    output of the xorshift64* generator in slot ``slot[r]``, which the kernel advances; ``reseed[r]`` puts
    ``seed_state[r]`` there first, and ``position[r]`` is recorded beside it.
    """
    _dev(logits, temperature, top_k, top_p, min_p, uniform, out, slot, position, reseed, seed_state, slot_table)
    rows, vocab = logits.shape
    _need(logits.dtype == torch.float32 and logits.is_contiguous(), "sample: logits must be contiguous float32")
    columns = [("temperature", temperature, torch.float32), ("top_k", top_k, torch.int32),
               ("top_p", top_p, torch.float32), ("min_p", min_p, torch.float32), ("out", out, torch.int32)]
    if slot_table is None:
        _need(uniform is not None, "sample: either uniforms or a table of state slots")
        columns.append(("uniform", uniform, torch.float64))
    else:
        _need(slot_table.dtype == torch.int64 and slot_table.dim() == 2 and slot_table.shape[1] == 2
              and slot_table.is_contiguous(), "sample: the slot table must be contiguous int64 [slots, 2]")
        columns += [("slot", slot, torch.int32), ("position", position, torch.int32), ("reseed", reseed, torch.int32),
                    ("seed_state", seed_state, torch.int64)]
    for name, tensor, dtype in columns:
        _need(tensor is not None and tensor.dtype == dtype and tensor.numel() == rows and tensor.is_contiguous(),
              f"sample: {name} must hold one {dtype} per row")
    # a wide vocabulary: the rows' best logits are found by 32 workgroups a row before the one that draws
    slices = SAMPLE_SLICES if vocab >= SAMPLE_SLICES_FROM else 0
    best = torch.empty(rows * slices, dtype=torch.float32, device=logits.device) if slices else None
    best_id = torch.empty(rows * slices, dtype=torch.int32, device=logits.device) if slices else None
    fn = _fn("sampling", "vk_sample", [_p, _i, _i, _p, _p, _p, _p, _p, _p, _p, _p, _i, _p, _p, _p, _p, _p, _i, _p])
    _status(fn(_ptr(logits), rows, vocab, _ptr(temperature), _ptr(top_k), _ptr(top_p), _ptr(min_p), _ptr(uniform),
               _ptr(out), _ptr(best), _ptr(best_id), slices, _ptr(slot), _ptr(position), _ptr(reseed),
               _ptr(seed_state), _ptr(slot_table), slot_table.shape[0] if slot_table is not None else 0, _stream()),
            "sample")


def penalize(logits: torch.Tensor, rows: torch.Tensor, tokens: torch.Tensor, counts: torch.Tensor,
             repetition: torch.Tensor, presence: torch.Tensor, frequency: torch.Tensor) -> None:
    """Apply the repetition, presence and frequency penalties in place to the listed (row, token) pairs."""
    _dev(logits, rows, tokens, counts, repetition, presence, frequency)
    num_rows, vocab = logits.shape
    n = rows.numel()
    _need(logits.dtype == torch.float32 and logits.is_contiguous(), "penalize: logits must be contiguous float32")
    _need(tokens.numel() == n and counts.numel() == n and all(t.dtype == torch.int32 for t in (rows, tokens, counts)),
          "penalize: rows, tokens and counts must be int32 of one length")
    _need(all(t.dtype == torch.float32 and t.numel() == num_rows for t in (repetition, presence, frequency)),
          "penalize: one float32 factor per row")
    if n:
        _need(int(rows.max()) < num_rows and int(rows.min()) >= 0, "penalize: row index out of range")
    fn = _fn("sampling", "vk_penalize", [_p, _i, _p, _p, _p, _p, _p, _p, _i, _p])
    _status(fn(_ptr(logits), vocab, _ptr(rows), _ptr(tokens), _ptr(counts), _ptr(repetition), _ptr(presence),
               _ptr(frequency), n, _stream()), "penalize")


def logit_bias(logits: torch.Tensor, rows: torch.Tensor, tokens: torch.Tensor, values: torch.Tensor) -> None:
    """``logits[rows[i], tokens[i]] += values[i]`` (pairs are unique)."""
    _dev(logits, rows, tokens, values)
    num_rows, vocab = logits.shape
    n = rows.numel()
    _need(logits.dtype == torch.float32 and logits.is_contiguous(), "logit_bias: logits must be contiguous float32")
    _need(tokens.numel() == n and values.numel() == n and rows.dtype == torch.int32 and tokens.dtype == torch.int32
          and values.dtype == torch.float32, "logit_bias: operand types")
    if n:
        _need(int(rows.max()) < num_rows and int(rows.min()) >= 0, "logit_bias: row index out of range")
    fn = _fn("sampling", "vk_logit_bias", [_p, _i, _p, _p, _p, _i, _p])
    _status(fn(_ptr(logits), vocab, _ptr(rows), _ptr(tokens), _ptr(values), n, _stream()), "logit_bias")


# ----------------------------------------------------------------------------------------------
def gemm_bf16_supported(a: torch.Tensor, w: torch.Tensor, out: torch.Tensor) -> bool:
    """Whether the matrix-core kernels take these operands (16-byte chunks along K, rows short enough for their
    32-bit offsets); what they do not take goes to the 32-bit FMA kernel."""
    k = a.shape[1]
    return (a.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and out.dtype in _DT and k % 8 == 0
            and k < GEMM_BF16_MAX_K and a.stride(0) < GEMM_BF16_MAX_K
            and a.stride(1) == 1 and (a.stride(0) % 8 == 0 or a.shape[0] == 1) and a.data_ptr() % 16 == 0
            and w.is_contiguous() and w.data_ptr() % 16 == 0 and out.stride(1) == 1)


def gemm_bf16(a: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor], out: torch.Tensor,
              accumulate: bool = False, skinny_limit: int = 64, skinny_shape: int = 0) -> None:
    """``out (+)= a @ w.T + bias`` on the matrix cores: bfloat16 products, 32-bit sums."""
    _dev(a, w, bias, out)
    _need(a.dim() == 2 and w.dim() == 2 and out.dim() == 2, "gemm: operands must be matrices")
    m, k = a.shape
    n = w.shape[0]
    _need(w.shape[1] == k and out.shape == (m, n), f"gemm: shapes {tuple(a.shape)} x {tuple(w.shape)}^T -> {tuple(out.shape)}")
    _need(gemm_bf16_supported(a, w, out), "gemm_bf16: operands must be bfloat16, K a multiple of 8, rows 16-byte aligned")
    if bias is not None:
        _need(bias.dtype == torch.float32 and bias.numel() == n and bias.is_contiguous(), "gemm: bias must be float32 [n]")
    if accumulate:
        _need(out.dtype == torch.float32, "gemm: accumulation needs a float32 output")
    lda = a.stride(0) if m > 1 else max(a.stride(0), k)
    lda = lda if lda % 8 == 0 else k
    ldc = out.stride(0) if m > 1 else max(out.stride(0), n)
    _need(ldc >= n, "gemm: out's row stride")
    partial = None
    if m > skinny_limit or m > 64:  # the tiled kernel may split K into a workspace of at most eight ranges
        partial = _split_k_workspace(a.device, min(8 * m * n, _TILE_WORKSPACE_FLOATS), "tile")
    fn = _fn("gemm_bf16", "vk_gemm_bf16", [_p, _p, _p, _p, _i, _i, _i, _i, _ll, _ll, _i, _i, _i, _p, _ll, _p])
    _status(fn(_ptr(a), _ptr(w), _ptr(bias), _ptr(out), _dt(out, "out"), m, n, k, lda, ldc, 1 if accumulate else 0,
               int(skinny_limit), int(skinny_shape), _ptr(partial), partial.numel() if partial is not None else 0,
               _stream()), "gemm_bf16")


def gemm_bf16_qkv_rope_supported(a: torch.Tensor, w: torch.Tensor, qkv: torch.Tensor, head_dim: int) -> bool:
    """Whether :func:`gemm_bf16_qkv_rope` takes the operands: all bfloat16, at most 16 tokens, an even head
    width, a contiguous output, a weight of less than 2 GiB."""
    return (qkv.dtype == torch.bfloat16 and 1 <= a.shape[0] <= 16 and head_dim % 2 == 0 and qkv.is_contiguous()
            and gemm_bf16_supported(a, w, qkv) and w.shape[0] * w.shape[1] * 2 < 2 ** 31)


def gemm_bf16_qkv_rope(a: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor], qkv: torch.Tensor,
                       positions: torch.Tensor, inv_freq: torch.Tensor, k_cache: Optional[torch.Tensor],
                       v_cache: Optional[torch.Tensor], entry_of_token: torch.Tensor, block_table: Optional[torch.Tensor],
                       heads: int, kv_heads: int, head_dim: int, sumsq: Optional[torch.Tensor] = None, groups: int = 0,
                       eps: float = 0.0) -> None:
    """``qkv = a @ w.T + bias`` for up to 16 tokens with the full rotation of its q and k heads and the write of
    the tokens' K and V into their pages in the product's epilogue: what :func:`gemm_bf16` followed by
    :func:`rope_kvwrite` (without a table of angles) leaves, in one launch.  With ``sumsq``, ``a`` is ``x * gain`` as
    :func:`gemm_bf16_follow` left it and the product's sums are divided by the root mean square of ``x`` (from the
    ``groups`` sums of squares and ``eps``) before the bias: the norm in front of the product costs no kernel."""
    _dev(a, w, bias, qkv, positions, inv_freq, k_cache, v_cache, entry_of_token, block_table, sumsq)
    if sumsq is not None:
        _need(sumsq.dtype == torch.float32 and 1 <= groups <= 512 and sumsq.numel() >= groups * 16,
              "gemm_bf16_qkv_rope: sumsq")
    m, k = a.shape
    n = w.shape[0]
    _need(w.shape[1] == k and qkv.shape == (m, n) and n == (heads + 2 * kv_heads) * head_dim, "gemm_bf16_qkv_rope: shapes")
    _need(gemm_bf16_qkv_rope_supported(a, w, qkv, head_dim), "gemm_bf16_qkv_rope: bfloat16 operands, at most 16 tokens, "
          "an even head width")
    if bias is not None:
        _need(bias.dtype == torch.float32 and bias.numel() == n and bias.is_contiguous(), "gemm: bias must be float32 [n]")
    _need(positions.dtype == torch.int32 and positions.numel() >= m, "gemm_bf16_qkv_rope: positions")
    _need(inv_freq.dtype == torch.float32 and inv_freq.numel() == head_dim // 2 and inv_freq.is_contiguous(),
          "gemm_bf16_qkv_rope: inv_freq must hold head_dim / 2 floats")
    table_width = block_size = 0
    if k_cache is not None:
        _need(v_cache is not None and block_table is not None, "gemm_bf16_qkv_rope: cache without table")
        _need(_cache_ok(k_cache, v_cache, kv_heads, head_dim, qkv.dtype), "gemm_bf16_qkv_rope: cache shape or dtype")
        _need(block_table.dtype == torch.int32 and block_table.dim() == 2 and block_table.is_contiguous(),
              "gemm_bf16_qkv_rope: block table")
        _need(entry_of_token.dtype == torch.int32 and entry_of_token.numel() >= m, "gemm_bf16_qkv_rope: entries")
        table_width, block_size = block_table.shape[1], k_cache.shape[2]
    lda = a.stride(0) if m > 1 else max(a.stride(0), k)
    lda = lda if lda % 8 == 0 else k
    fn = _fn("gemm_bf16", "vk_gemm_bf16_qkv_rope",
             [_p, _p, _p, _p, _i, _i, _i, _ll, _ll, _p, _p, _p, _p, _p, _p, _i, _i, _i, _i, _i, _p, _i, _f, _p])
    _status(fn(_ptr(a), _ptr(w), _ptr(bias), _ptr(qkv), m, n, k, lda, n, _ptr(positions), _ptr(inv_freq), _ptr(k_cache),
               _ptr(v_cache), _ptr(entry_of_token), _ptr(block_table), table_width, block_size, heads, kv_heads, head_dim,
               _ptr(sumsq), int(groups), float(eps), _stream()), "gemm_bf16_qkv_rope")


def gemm_bf16_follow_supported(a: torch.Tensor, w: torch.Tensor, out: torch.Tensor) -> bool:
    """Whether :func:`gemm_bf16_follow` takes the operands: bfloat16 product of up to 16 tokens into a float32
    residual whose width is a multiple of four and at most 8,192 (512 workgroups of 16 columns)."""
    return (out.dtype == torch.float32 and 1 <= a.shape[0] <= 16 and out.shape[1] % 4 == 0 and out.shape[1] <= 8192
            and out.is_contiguous() and gemm_bf16_supported(a, w, out))


def follow_stride(tokens: int) -> int:
    """Floats per group of the sums of squares that the first half of a split norm leaves for ``tokens`` rows: 16 for
    up to 16 tokens, else the tokens rounded up to a multiple of 64."""
    return 16 if tokens <= 16 else (tokens + 63) // 64 * 64


def follow_sumsq_floats(n: int, tokens: int) -> int:
    """Floats that the sums of squares of :func:`gemm_bf16_follow` and :func:`gemm_bf16_mid_follow` may take for an
    output of ``n`` columns and ``tokens`` rows (16 per workgroup that owns at least 8 columns, or a
    :func:`follow_stride` per 1,024 columns)."""
    return max(((n + 7) // 8) * 16, ((n + 1023) // 1024) * follow_stride(tokens))


def gemm_bf16_follow(a: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor], out: torch.Tensor,
                     gain: torch.Tensor, scaled: torch.Tensor, sumsq: torch.Tensor) -> int:
    """``out += a @ w.T + bias`` (``out`` float32: the residual) for up to 16 tokens, and the first half of the RMS
    norm that follows: ``scaled = bfloat16(out * gain)`` and per workgroup the sums of squares of its columns
    (``sumsq[groups, 16]``).  Returns ``groups``; :func:`gemm_bf16_gated_scaled` does the other half."""
    _dev(a, w, bias, out, gain, scaled, sumsq)
    m, k = a.shape
    n = w.shape[0]
    _need(w.shape[1] == k and out.shape == (m, n) and scaled.shape == (m, n), "gemm_bf16_follow: shapes")
    _need(gemm_bf16_follow_supported(a, w, out), "gemm_bf16_follow: bfloat16 operands, a float32 output, at most 16 tokens")
    _need(scaled.dtype == torch.bfloat16 and scaled.is_contiguous(), "gemm_bf16_follow: scaled must be bfloat16 [m, n]")
    _need(gain.dtype == torch.float32 and gain.numel() == n and gain.is_contiguous(), "gemm_bf16_follow: gain must be float32 [n]")
    _need(sumsq.dtype == torch.float32 and sumsq.is_contiguous() and sumsq.numel() >= follow_sumsq_floats(n, m),
          "gemm_bf16_follow: sumsq is too small")
    if bias is not None:
        _need(bias.dtype == torch.float32 and bias.numel() == n and bias.is_contiguous(), "gemm: bias must be float32 [n]")
    lda = a.stride(0) if m > 1 else max(a.stride(0), k)
    lda = lda if lda % 8 == 0 else k
    groups = ctypes.c_int(0)
    fn = _fn("gemm_bf16", "vk_gemm_bf16_follow", [_p, _p, _p, _p, _i, _i, _i, _ll, _ll, _p, _p, _ll, _p, _ll,
                                                  ctypes.POINTER(ctypes.c_int), _p])
    _status(fn(_ptr(a), _ptr(w), _ptr(bias), _ptr(out), m, n, k, lda, n, _ptr(gain), _ptr(scaled), n, _ptr(sumsq),
               sumsq.numel(), ctypes.byref(groups), _stream()), "gemm_bf16_follow")
    return int(groups.value)


def gemm_bf16_mid_follow(a: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor], out: torch.Tensor,
                         ranges: int, rows_per_wave: int, gain: torch.Tensor, scaled: torch.Tensor,
                         sumsq: torch.Tensor) -> int:
    """:func:`gemm_bf16_follow` for up to 64 tokens where K is split into ``ranges`` > 1 over workgroups
    (:func:`gemm_bf16_mid` with accumulation): the kernel that adds the ranges leaves ``scaled`` and the sums of
    squares, :func:`follow_stride` floats per group.  Returns the number of groups."""
    _dev(a, w, bias, out, gain, scaled, sumsq)
    m, k = a.shape
    n = w.shape[0]
    _need(m <= 64 and ranges >= 2, "gemm_bf16_mid_follow: at most 64 tokens and at least two ranges")
    _need(w.shape[1] == k and out.shape == (m, n) and scaled.shape == (m, n), "gemm_bf16_mid_follow: shapes")
    _need(out.dtype == torch.float32 and out.is_contiguous() and gemm_bf16_supported(a, w, out),
          "gemm_bf16_mid_follow: bfloat16 operands and a float32 output")
    _need(scaled.dtype == torch.bfloat16 and scaled.is_contiguous(), "gemm_bf16_mid_follow: scaled must be bfloat16 [m, n]")
    _need(gain.dtype == torch.float32 and gain.numel() == n and gain.is_contiguous(), "gemm_bf16_mid_follow: gain")
    _need(sumsq.dtype == torch.float32 and sumsq.is_contiguous() and sumsq.numel() >= follow_sumsq_floats(n, m),
          "gemm_bf16_mid_follow: sumsq is too small")
    if bias is not None:
        _need(bias.dtype == torch.float32 and bias.numel() == n and bias.is_contiguous(), "gemm: bias must be float32 [n]")
    lda = a.stride(0) if m > 1 else max(a.stride(0), k)
    lda = lda if lda % 8 == 0 else k
    partial = _split_k_workspace(a.device, ranges * 64 * n, "mid")
    groups = ctypes.c_int(0)
    fn = _fn("gemm_bf16", "vk_gemm_bf16_mid_follow", [_p, _p, _p, _p, _i, _i, _i, _ll, _ll, _i, _i, _p, _ll, _p, _p, _ll, _p,
                                                      _ll, _i, ctypes.POINTER(ctypes.c_int), _p])
    _status(fn(_ptr(a), _ptr(w), _ptr(bias), _ptr(out), m, n, k, lda, n, int(ranges), int(rows_per_wave), _ptr(partial),
               partial.numel(), _ptr(gain), _ptr(scaled), n, _ptr(sumsq), sumsq.numel(), follow_stride(m),
               ctypes.byref(groups), _stream()), "gemm_bf16_mid_follow")
    return int(groups.value)


def gemm_bf16_mid_qkv_rope(a: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor], qkv: torch.Tensor,
                           ranges: int, rows_per_wave: int, positions: torch.Tensor, inv_freq: torch.Tensor,
                           k_cache: Optional[torch.Tensor], v_cache: Optional[torch.Tensor], entry_of_token: torch.Tensor,
                           block_table: Optional[torch.Tensor], heads: int, kv_heads: int, head_dim: int,
                           sumsq: Optional[torch.Tensor] = None, groups: int = 0, eps: float = 0.0) -> None:
    """:func:`gemm_bf16_qkv_rope` for up to 64 tokens where K is split into ``ranges`` > 1 over workgroups: the
    kernel that adds the ranges also divides by the norm (``sumsq``: ``groups`` groups of :func:`follow_stride`
    floats), adds the bias, rotates and writes the cache."""
    _dev(a, w, bias, qkv, positions, inv_freq, k_cache, v_cache, entry_of_token, block_table, sumsq)
    m, k = a.shape
    n = w.shape[0]
    _need(m <= 64 and ranges >= 2 and head_dim % 8 == 0, "gemm_bf16_mid_qkv_rope: at most 64 tokens, two ranges or more, "
          "a head width that is a multiple of 8")
    _need(w.shape[1] == k and qkv.shape == (m, n) and n == (heads + 2 * kv_heads) * head_dim, "gemm_bf16_mid_qkv_rope: shapes")
    _need(qkv.dtype == torch.bfloat16 and qkv.is_contiguous() and gemm_bf16_supported(a, w, qkv),
          "gemm_bf16_mid_qkv_rope: bfloat16 operands and a contiguous output")
    if bias is not None:
        _need(bias.dtype == torch.float32 and bias.numel() == n and bias.is_contiguous(), "gemm: bias must be float32 [n]")
    _need(positions.dtype == torch.int32 and positions.numel() >= m, "gemm_bf16_mid_qkv_rope: positions")
    _need(inv_freq.dtype == torch.float32 and inv_freq.numel() == head_dim // 2 and inv_freq.is_contiguous(),
          "gemm_bf16_mid_qkv_rope: inv_freq must hold head_dim / 2 floats")
    table_width = block_size = 0
    if k_cache is not None:
        _need(v_cache is not None and block_table is not None, "gemm_bf16_mid_qkv_rope: cache without table")
        _need(_cache_ok(k_cache, v_cache, kv_heads, head_dim, qkv.dtype), "gemm_bf16_mid_qkv_rope: cache shape or dtype")
        _need(block_table.dtype == torch.int32 and block_table.dim() == 2 and block_table.is_contiguous(),
              "gemm_bf16_mid_qkv_rope: block table")
        _need(entry_of_token.dtype == torch.int32 and entry_of_token.numel() >= m, "gemm_bf16_mid_qkv_rope: entries")
        table_width, block_size = block_table.shape[1], k_cache.shape[2]
    if sumsq is not None:
        _need(sumsq.dtype == torch.float32 and groups >= 1 and sumsq.numel() >= groups * follow_stride(m),
              "gemm_bf16_mid_qkv_rope: sumsq")
    lda = a.stride(0) if m > 1 else max(a.stride(0), k)
    lda = lda if lda % 8 == 0 else k
    partial = _split_k_workspace(a.device, ranges * 64 * n, "mid")
    fn = _fn("gemm_bf16", "vk_gemm_bf16_mid_qkv_rope",
             [_p, _p, _p, _p, _i, _i, _i, _ll, _ll, _i, _i, _p, _ll, _p, _p, _p, _p, _p, _p, _i, _i, _i, _i, _i, _p, _i, _i, _f, _p])
    _status(fn(_ptr(a), _ptr(w), _ptr(bias), _ptr(qkv), m, n, k, lda, n, int(ranges), int(rows_per_wave), _ptr(partial),
               partial.numel(), _ptr(positions), _ptr(inv_freq), _ptr(k_cache), _ptr(v_cache), _ptr(entry_of_token),
               _ptr(block_table), table_width, block_size, heads, kv_heads, head_dim, _ptr(sumsq), int(groups),
               follow_stride(m), float(eps), _stream()), "gemm_bf16_mid_qkv_rope")


def gemm_bf16_gated_scaled(scaled: torch.Tensor, w: torch.Tensor, out: torch.Tensor, sumsq: torch.Tensor, groups: int,
                           eps: float) -> None:
    """:func:`gemm_bf16_gated` with resident activations on what :func:`gemm_bf16_follow` left: ``scaled`` is
    ``x * gain`` in bfloat16, and gate and up are divided by the root mean square of ``x`` (from the ``groups``
    sums of squares and ``eps``) before the activation."""
    _dev(scaled, w, out, sumsq)
    m, k = scaled.shape
    n = w.shape[0]
    _need(w.shape[1] == k and out.shape == (m, n // 2) and n % 32 == 0, "gemm_gated: shapes")
    _need(gemm_bf16_supported(scaled, w, out) and out.dtype == torch.bfloat16, "gemm_gated: operands must be bfloat16")
    _need(sumsq.dtype == torch.float32 and sumsq.numel() >= groups * 16 and groups >= 1, "gemm_bf16_gated_scaled: sumsq")
    lda = scaled.stride(0) if m > 1 else max(scaled.stride(0), k)
    lda = lda if lda % 8 == 0 else k
    ldc = out.stride(0) if m > 1 else max(out.stride(0), n // 2)
    fn = _fn("gemm_bf16", "vk_gemm_bf16_gated_scaled", [_p, _p, _p, _i, _i, _i, _ll, _ll, _p, _i, _f, _p])
    _status(fn(_ptr(scaled), _ptr(w), _ptr(out), m, n, k, lda, ldc, _ptr(sumsq), int(groups), float(eps), _stream()),
            "gemm_bf16_gated_scaled")


def gemm_bf16_gated_tile_scaled(scaled: torch.Tensor, w: torch.Tensor, out: torch.Tensor, sumsq: torch.Tensor,
                                groups: int, eps: float) -> None:
    """:func:`gemm_bf16_gated` on the tiled kernel, for any number of tokens, on the first half of a split norm:
    ``scaled`` is ``x * gain`` in bfloat16, and gate and up are divided by the root mean square of ``x`` (from the
    ``groups`` sums of squares, :func:`follow_stride` floats each, and ``eps``) before the activation."""
    _dev(scaled, w, out, sumsq)
    m, k = scaled.shape
    n = w.shape[0]
    _need(w.shape[1] == k and out.shape == (m, n // 2) and n % 32 == 0, "gemm_gated: shapes")
    _need(gemm_bf16_supported(scaled, w, out) and out.dtype == torch.bfloat16, "gemm_gated: operands must be bfloat16")
    stride = follow_stride(m)
    _need(sumsq.dtype == torch.float32 and sumsq.is_contiguous() and groups >= 1 and sumsq.numel() >= groups * stride,
          "gemm_bf16_gated_tile_scaled: sumsq")
    lda = scaled.stride(0) if m > 1 else max(scaled.stride(0), k)
    lda = lda if lda % 8 == 0 else k
    ldc = out.stride(0) if m > 1 else max(out.stride(0), n // 2)
    fn = _fn("gemm_bf16", "vk_gemm_bf16_gated_tile_scaled", [_p, _p, _p, _i, _i, _i, _ll, _ll, _p, _i, _i, _f, _p])
    _status(fn(_ptr(scaled), _ptr(w), _ptr(out), m, n, k, lda, ldc, _ptr(sumsq), int(groups), stride, float(eps), _stream()),
            "gemm_bf16_gated_tile_scaled")


TILE_TILINGS = {0: "128x128 staged", 2: "256x128 staged", 3: "128x256 staged", 4: "256x256 staged",
                9: "128x128 direct", 7: "256x128 direct", 8: "128x256 direct", 5: "256x256 direct", 6: "256x192 direct",
                10: "128x96 direct, gated only", 11: "128x160 direct, gated only", 12: "128x224 direct, gated only"}


def gemm_bf16_force_tiling(tiling: int = -1, ranges: int = 1, stages: int = 0) -> None:
    """For tests and measurements: make the tiled kernel of :func:`gemm_bf16` and :func:`gemm_bf16_gated`
    use one tiling (a key of ``TILE_TILINGS``) and split K into ``ranges``; ``-1`` gives the choice back
    to the launcher.  A "direct" tiling falls back to its staged twin when K is no multiple of 64.  ``stages``:
    2 or 3 LDS stages for the direct 128-token tilings (0: three up to 128 tokens, else two)."""
    if tiling >= 0:
        _need(tiling in TILE_TILINGS and 1 <= ranges <= 8, "gemm_bf16_force_tiling: unknown tiling or ranges")
    _need(stages in (0, 2, 3), "gemm_bf16_force_tiling: stages are 0 (by shape), 2 or 3")
    fn = _fn("gemm_bf16", "vk_gemm_bf16_tile_config", [_i, _i, _i])
    _status(fn(-1 if tiling < 0 else tiling, int(ranges), int(stages)), "gemm_bf16_force_tiling")


def gemm_bf16_force_tile_group(rows: int = 0) -> None:
    """For measurements: the tiled kernel walks its tiles in blocks of ``rows`` rows of tiles (0: chosen by shape)."""
    fn = _fn("gemm_bf16", "vk_gemm_bf16_tile_group", [_i])
    _status(fn(int(rows)), "gemm_bf16_force_tile_group")


# ----------------------------------------------------------------------------------------------
def attn_bf16_padded_width(head_dim: int) -> int:
    """The padded head width a matrix-core attention module is compiled for (a multiple of 32)."""
    return (head_dim + 31) // 32 * 32


def attn_bf16_supported(q: torch.Tensor, k_cache: torch.Tensor, head_dim: int) -> bool:
    return (q.dtype == torch.bfloat16 and head_dim % 8 == 0 and head_dim <= 256 and k_cache.shape[2] % 8 == 0
            and q.stride(0) % 8 == 0 and q.data_ptr() % 16 == 0)


def attn_bf16_prefill_loads_directly(k_cache: torch.Tensor, kv_heads: int, head_dim: int) -> bool:
    """Whether prompt attention runs on the kernel that loads K and V tiles straight into LDS (which alone can cut a
    tile's positions into chunks): a head width of 64, 128 or 256 and pages of 8, 16, 32 or 64 positions."""
    block_size = k_cache.shape[2]
    return (head_dim in (64, 128, 256) and block_size in (8, 16, 32, 64)
            and kv_heads * block_size * head_dim * 2 < 2 ** 32)


ATTN_PREFILL_PARTIAL_ROW_EXTRA = 4   # floats beside the padded head width in a column's partial result


def attn_bf16_prefill(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, out: torch.Tensor,
                      tiles: torch.Tensor, entry_start: torch.Tensor, entry_first_pos: torch.Tensor,
                      block_table: torch.Tensor, heads: int, kv_heads: int, head_dim: int, scale: float,
                      window: int, split: bool = False, chunk_tiles: int = 0, max_chunks: int = 0) -> None:
    """Attention of the entries' 128-token tiles listed in ``tiles`` (pairs: entry, first token within it).
    ``split``: workgroups of sixteen waves that halve a tile's positions between them and merge at the end, where
    the kernel in use has that form (for few tiles of very different lengths); the same result up to rounding.
    ``chunk_tiles`` > 0 (where :func:`attn_bf16_prefill_loads_directly`): a tile's steps of 64 positions are cut into
    chunks of that many, a workgroup each, and a second kernel merges them; no tile may have more than ``max_chunks``."""
    _dev(q, k_cache, v_cache, out, tiles, entry_start, entry_first_pos, block_table)
    _need(attn_bf16_supported(q, k_cache, head_dim), "attn_bf16: operands must be bfloat16 with 16-byte rows")
    _need(q.dim() == 2 and q.stride(1) == 1 and q.shape[1] >= heads * head_dim, "attention: q")
    _need(out.shape == (q.shape[0], heads * head_dim) and out.is_contiguous() and out.dtype == q.dtype, "attention: out")
    _need(_cache_ok(k_cache, v_cache, kv_heads, head_dim, q.dtype), "attention: cache shape or dtype")
    _need(tiles.dtype == torch.int32 and tiles.numel() % 2 == 0 and tiles.is_contiguous(), "attention: tiles")
    _need(block_table.dtype == torch.int32 and block_table.dim() == 2 and block_table.is_contiguous(), "attention: table")
    _need(entry_start.dtype == torch.int32 and entry_first_pos.dtype == torch.int32
          and entry_start.numel() == block_table.shape[0] + 1 and entry_first_pos.numel() == block_table.shape[0],
          "attention: entry arrays")
    num_tiles = tiles.numel() // 2
    partial = None
    if chunk_tiles > 0 and attn_bf16_prefill_loads_directly(k_cache, kv_heads, head_dim):
        _need(max_chunks >= 1, "attention: max_chunks")
        partial = torch.empty(num_tiles * heads * max_chunks * 128 * (head_dim + ATTN_PREFILL_PARTIAL_ROW_EXTRA),
                              dtype=torch.float32, device=q.device)
    else:
        chunk_tiles = max_chunks = 0
    module = f"attn_bf16_hd{attn_bf16_padded_width(head_dim)}"
    fn = _fn(module, "vk_attn_bf16_prefill",
             [_p, _ll, _p, _p, _p, _p, _i, _p, _p, _p, _i, _i, _i, _i, _i, _f, _i, _i, _p, _ll, _i, _i, _p],
             key=module + ".prefill")
    _status(fn(_ptr(q), q.stride(0), _ptr(k_cache), _ptr(v_cache), _ptr(out), _ptr(tiles), num_tiles,
               _ptr(entry_start), _ptr(entry_first_pos), _ptr(block_table), block_table.shape[1], k_cache.shape[2],
               heads, kv_heads, head_dim, float(scale), int(window), 1 if split else 0, _ptr(partial),
               partial.numel() if partial is not None else 0, int(chunk_tiles), int(max_chunks), _stream()),
            "attn_bf16_prefill")


ATTN_DECODE_JOINED_CHUNKS = 8   # waves of a workgroup that merges its chunks itself


def attn_bf16_decode(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, out: torch.Tensor,
                     partial: torch.Tensor, entries: torch.Tensor, entry_start: torch.Tensor,
                     entry_first_pos: torch.Tensor, block_table: torch.Tensor, heads: int, kv_heads: int,
                     head_dim: int, scale: float, window: int, chunk: int, chunks: int, dense: bool = False,
                     join: bool = False) -> None:
    """Attention of the single-token entries listed in ``entries``, positions split into ``chunks`` of ``chunk``.
    ``dense``: the step holds single-token entries only, so entry i is the i-th of them and holds token i; the
    kernel then need not look either up.  ``join``: one workgroup per entry and key head takes all chunks (at most
    ``ATTN_DECODE_JOINED_CHUNKS``), a wave each, and merges them itself; ``partial`` is then not used and may be
    None."""
    _dev(q, k_cache, v_cache, out, partial, entries, entry_start, entry_first_pos, block_table)
    _need(attn_bf16_supported(q, k_cache, head_dim), "attn_bf16: operands must be bfloat16 with 16-byte rows")
    _need(q.dim() == 2 and q.stride(1) == 1 and q.shape[1] >= heads * head_dim, "attention: q")
    _need(out.shape == (q.shape[0], heads * head_dim) and out.is_contiguous() and out.dtype == q.dtype, "attention: out")
    _need(_cache_ok(k_cache, v_cache, kv_heads, head_dim, q.dtype), "attention: cache shape or dtype")
    count = entries.numel()
    _need(entries.dtype == torch.int32 and entries.is_contiguous(), "attention: entries")
    if join:
        _need(chunks <= ATTN_DECODE_JOINED_CHUNKS, "attention: too many chunks for one workgroup")
    else:
        _need(partial is not None and partial.dtype == torch.float32 and partial.is_contiguous()
              and partial.numel() >= count * heads * chunks * (head_dim + 2), "attention: workspace too small")
    _need(chunk >= 32 and chunk % 32 == 0 and chunks >= 1, "attention: chunk must be a multiple of 32")
    _need(block_table.dtype == torch.int32 and block_table.dim() == 2 and block_table.is_contiguous(), "attention: table")
    module = f"attn_bf16_hd{attn_bf16_padded_width(head_dim)}"
    fn = _fn(module, "vk_attn_bf16_decode",
             [_p, _ll, _p, _p, _p, _p, _p, _i, _p, _p, _p, _i, _i, _i, _i, _i, _f, _i, _i, _i, _i, _i, _p], key=module + ".decode")
    _status(fn(_ptr(q), q.stride(0), _ptr(k_cache), _ptr(v_cache), _ptr(out), _ptr(partial), _ptr(entries), count,
               _ptr(entry_start), _ptr(entry_first_pos), _ptr(block_table), block_table.shape[1], k_cache.shape[2],
               heads, kv_heads, head_dim, float(scale), int(window), int(chunk), int(chunks), 1 if dense else 0,
               1 if join else 0, _stream()),
            "attn_bf16_decode")


_workspaces = {}
_retired = []  # outgrown workspaces: kept alive, since a captured graph may still write to them
_TILE_WORKSPACE_FLOATS = 64 * 1024 * 1024   # 256 MB: the most the tiled kernel's K ranges may take


def _split_k_workspace(device: torch.device, floats: int, kind: str) -> torch.Tensor:
    """Partial-sum workspace of a device and a kind of product; grown when a product needs more, never shrunk.

    Every product of the kind on the device shares it, which is safe because products run on one stream.
    """
    key = (device, kind)
    entry = _workspaces.get(key)
    if entry is None or entry.numel() < floats:
        if entry is not None:
            _retired.append(entry)
        entry = torch.empty(floats, dtype=torch.float32, device=device)
        _workspaces[key] = entry
    return entry


def gemm_bf16_mid(a: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor], out: torch.Tensor,
                  accumulate: bool = False, ranges: int = 1, rows_per_wave: int = 2) -> None:
    """``out (+)= a @ w.T + bias`` for at most 128 rows of ``a``: activations shared through LDS, weights
    streamed; ``ranges`` > 1 splits K over workgroups and adds the ranges' partial sums in a second kernel."""
    _dev(a, w, bias, out)
    _need(a.dim() == 2 and w.dim() == 2 and out.dim() == 2, "gemm: operands must be matrices")
    m, k = a.shape
    n = w.shape[0]
    _need(m <= 128, "gemm_bf16_mid takes at most 128 rows")
    _need(w.shape[1] == k and out.shape == (m, n), f"gemm: shapes {tuple(a.shape)} x {tuple(w.shape)}^T -> {tuple(out.shape)}")
    _need(gemm_bf16_supported(a, w, out), "gemm_bf16: operands must be bfloat16, K a multiple of 8, rows 16-byte aligned")
    _need((rows_per_wave in (1, 2) or 108 <= rows_per_wave <= 116) and ranges >= 1,
          "gemm_bf16_mid: rows_per_wave is 1 or 2 (or 108 to 116: one tile with 8 to 16 rows), ranges at least 1")
    if bias is not None:
        _need(bias.dtype == torch.float32 and bias.numel() == n and bias.is_contiguous(), "gemm: bias must be float32 [n]")
    if accumulate:
        _need(out.dtype == torch.float32, "gemm: accumulation needs a float32 output")
    lda = a.stride(0) if m > 1 else max(a.stride(0), k)
    lda = lda if lda % 8 == 0 else k
    ldc = out.stride(0) if m > 1 else max(out.stride(0), n)
    _need(ldc >= n, "gemm: out's row stride")
    partial = None
    if ranges > 1:
        partial = _split_k_workspace(a.device, ranges * (64 if m <= 64 else 128) * n, "mid")
    fn = _fn("gemm_bf16", "vk_gemm_bf16_mid", [_p, _p, _p, _p, _i, _i, _i, _i, _ll, _ll, _i, _i, _i, _p, _ll, _p])
    _status(fn(_ptr(a), _ptr(w), _ptr(bias), _ptr(out), _dt(out, "out"), m, n, k, lda, ldc, 1 if accumulate else 0,
               int(ranges), int(rows_per_wave), _ptr(partial), partial.numel() if partial is not None else 0, _stream()),
            "gemm_bf16_mid")


_COMPUTE_UNITS: dict = {}


def compute_units(device: torch.device) -> int:
    """CUs of the device (cached; what the launchers with one workgroup per CU use as their grid)."""
    index = device.index if device.index is not None else torch.cuda.current_device()
    if index not in _COMPUTE_UNITS:
        _COMPUTE_UNITS[index] = int(torch.cuda.get_device_properties(index).multi_processor_count)
    return _COMPUTE_UNITS[index]


def gemm_bf16_gated(a: torch.Tensor, w: torch.Tensor, out: torch.Tensor, rows_per_wave: int = 1) -> None:
    """``out = up * silu(gate)`` where ``[gate, up] = a @ w.T`` and ``w`` interleaves gate and up rows in
    groups of 16.  ``out``: ``[tokens, w.shape[0] / 2]`` bfloat16.  ``rows_per_wave`` (up to 64 tokens): 1 or
    2 tiles per wave of the LDS-shared kernel, 0 for the kernel with resident activations (up to 16
    tokens, K a multiple of 128, ``tokens x K`` within LDS; refused otherwise), 3 for the tiled kernel that
    more than 64 tokens always take."""
    _dev(a, w, out)
    m, k = a.shape
    n = w.shape[0]
    _need(w.shape[1] == k and out.shape == (m, n // 2) and n % 32 == 0, "gemm_gated: shapes")
    _need(gemm_bf16_supported(a, w, out) and out.dtype == torch.bfloat16, "gemm_gated: operands must be bfloat16")
    lda = a.stride(0) if m > 1 else max(a.stride(0), k)
    lda = lda if lda % 8 == 0 else k
    ldc = out.stride(0) if m > 1 else max(out.stride(0), n // 2)
    fn = _fn("gemm_bf16", "vk_gemm_bf16_gated", [_p, _p, _p, _i, _i, _i, _ll, _ll, _i, _p])
    _status(fn(_ptr(a), _ptr(w), _ptr(out), m, n, k, lda, ldc, int(rows_per_wave), _stream()), "gemm_bf16_gated")
