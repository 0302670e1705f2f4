"""Plain C++ twins of the engine's kernels (``plain_kernels.cpp``), compiled with the host compiler into a
temporary folder and called through ctypes.  A twin takes the parameter list of its ``vk_*`` kernel, with host
pointers and the stream ignored.  Nothing of the engine is used here."""
from __future__ import annotations

import atexit
import ctypes
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
    "plain_gemm_bf16": [P, P, P, P, I, I, I, I, LL, LL, I, I, I, P, LL, P],
    "plain_gemm_bf16_mid": [P, P, P, P, I, I, I, I, LL, LL, I, I, I, P, LL, P],
    "plain_gemm_bf16_gated": [P, P, P, I, I, I, LL, LL, I, P],
    "plain_attn_generic": [P, LL, P, P, P, I, P, P, P, I, I, I, I, I, I, F, I, P],
    "plain_attn_bf16_prefill": [P, LL, P, P, P, P, I, P, P, P, I, I, I, I, I, F, I, P],
    "plain_attn_bf16_decode": [P, LL, P, P, P, P, P, I, P, P, P, I, I, I, I, I, F, I, I, I, P],
    "plain_sample": [P, I, I, P, P, P, P, P, P, P],
    "plain_penalize": [P, I, P, P, P, P, P, P, I, P],
    "plain_logit_bias": [P, I, P, P, P, I, P],
}


def library() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        folder = tempfile.mkdtemp(prefix="plain_cpp_")
        atexit.register(shutil.rmtree, folder, ignore_errors=True)
        target = os.path.join(folder, "plain_kernels.so")
        source = os.path.join(os.path.dirname(os.path.abspath(__file__)), "plain_kernels.cpp")
        subprocess.run(["g++", "-O2", "-std=c++17", "-shared", "-fPIC", "-Wall", "-o", target, source], check=True)
        _lib = ctypes.CDLL(target)
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
