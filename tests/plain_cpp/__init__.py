"""Plain C++ twins of the engine's kernels (``plain_kernels.cpp``), compiled with the host compiler and called
through ctypes.  A twin takes the parameter list of its ``vk_*`` kernel, with host
pointers and the stream ignored.  Nothing of the engine is used here."""
from __future__ import annotations

import atexit
import ctypes
import hashlib
import os
import shutil
import subprocess
import tempfile

import torch

_lib = None
P, I, LL, F = ctypes.c_void_p, ctypes.c_int, ctypes.c_longlong, ctypes.c_float
DT = {torch.float32: 0, torch.bfloat16: 1}

SIGNATURES = {
    "plain_embed_gather": [P, I, P, P, P, P, I, I, I, P],
    "plain_rmsnorm": [P, P, P, P, I, I, I, F, P],
    "plain_rope_angles": [P, P, I, I, P, P],
    "plain_rope_kvwrite": [P, I, P, P, P, I, P, P, P, P, I, I, I, I, I, I, P],
    "plain_swiglu": [P, P, I, I, I, I, P],
    "plain_gemm_generic": [P, I, P, I, P, P, I, I, I, I, LL, LL, I, P],
    "plain_gemm_stream": [P, P, P, P, I, I, I, I, LL, LL, I, P, LL, P],
    "plain_gemm_bf16": [P, P, P, P, I, I, I, I, LL, LL, I, I, I, P, LL, P],
    "plain_gemm_bf16_mid": [P, P, P, P, I, I, I, I, LL, LL, I, I, I, P, LL, P],
    "plain_gemm_bf16_gated": [P, P, P, I, I, I, LL, LL, I, P],
    "plain_gemm_bf16_follow": [P, P, P, P, I, I, I, LL, LL, P, P, LL, P, LL, P, P],
    "plain_gemm_bf16_gated_scaled": [P, P, P, I, I, I, LL, LL, P, I, F, P],
    "plain_gemm_bf16_gated_tile_scaled": [P, P, P, I, I, I, LL, LL, P, I, I, F, P],
    "plain_gemm_bf16_qkv_rope": [P, P, P, P, I, I, I, LL, LL, P, P, P, P, P, P, I, I, I, I, I, P, I, F, P],
    "plain_gemm_bf16_mid_follow": [P, P, P, P, I, I, I, LL, LL, I, I, P, LL, P, P, LL, P, LL, I, P, P],
    "plain_gemm_bf16_mid_qkv_rope": [P, P, P, P, I, I, I, LL, LL, I, I, P, LL, P, P, P, P, P, P, I, I, I, I, I, P, I, I, F, P],
    "plain_attn_generic": [P, LL, P, P, P, I, P, P, P, I, I, I, I, I, I, F, I, P, P],
    "plain_attn_decode_f32": [P, LL, P, P, P, P, P, I, P, P, P, I, I, I, I, I, F, I, I, P],
    "plain_attn_prefill_f32": [P, LL, P, P, P, P, I, I, P, P, P, I, I, I, I, I, F, I, P],
    "plain_attn_bf16_prefill": [P, LL, P, P, P, P, I, P, P, P, I, I, I, I, I, F, I, I, P, LL, I, I, P],
    "plain_attn_bf16_decode": [P, LL, P, P, P, P, P, I, P, P, P, I, I, I, I, I, F, I, I, I, I, I, P],
    "plain_sample": [P, I, I, P, P, P, P, P, P, P, P, I, P, P, P, P, P, I, P],
    "plain_penalize": [P, I, P, P, P, P, P, P, I, P],
    "plain_logit_bias": [P, I, P, P, P, I, P],
}


def build() -> str:
    """Compile the twins if no library of the current source is there; returns its path.  The library is named
    after a hash of the source and lives beside it (``_build/``), or in a temporary folder where that cannot be
    written."""
    here = os.path.dirname(os.path.abspath(__file__))
    source = os.path.join(here, "plain_kernels.cpp")
    with open(source, "rb") as handle:
        digest = hashlib.sha256(handle.read()).hexdigest()[:12]
    folder = os.path.join(here, "_build")
    target = os.path.join(folder, f"plain_kernels-{digest}.so")
    if os.path.exists(target):
        return target
    try:
        os.makedirs(folder, exist_ok=True)
        probe = tempfile.NamedTemporaryFile(dir=folder, delete=True)
        probe.close()
    except OSError:
        folder = tempfile.mkdtemp(prefix="plain_cpp_")
        atexit.register(shutil.rmtree, folder, ignore_errors=True)
        target = os.path.join(folder, f"plain_kernels-{digest}.so")
    partial = target + f".{os.getpid()}.tmp"
    subprocess.run(["g++", "-O2", "-std=c++17", "-shared", "-fPIC", "-Wall", "-o", partial, source], check=True)
    os.replace(partial, target)
    return target


def library() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        _lib = ctypes.CDLL(build())
        for name, argtypes in SIGNATURES.items():
            fn = getattr(_lib, name)
            fn.argtypes, fn.restype = argtypes, I
        _lib.plain_bf16_to_float.argtypes = [P, P, I]
        _lib.plain_float_to_bf16.argtypes = [P, P, I]
    return _lib


def ptr(t):
    """Address of a contiguous CPU tensor, or None."""
    if t is None:
        return None
    assert t.device.type == "cpu" and t.is_contiguous()
    return t.data_ptr()


def call(name: str, *args) -> None:
    """Call a twin; tensors are passed by address, and a non-zero status is an error."""
    status = getattr(library(), name)(*[ptr(a) if isinstance(a, torch.Tensor) else a for a in args])
    if status != 0:
        raise RuntimeError(f"{name} returned {status}")
