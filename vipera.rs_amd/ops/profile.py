"""Where a step's time goes, by class of kernel, measured by the program that runs the step.

The reference prints a ``PROFILE`` line per pass with the time of each class of work (its dots by weight
type, attention, norm, rope, cache write, elementwise) and the rest
(crates/vipera-backend-cpu/src/profile.rs:226-275).  Here the classes are the step's kernels: while a
:class:`KernelTimer` is active every binding of ``ops.kernels`` that launches work is bracketed by a pair of
GPU events, and the time between each pair is added to the class that ``label`` gives the call.

The step has to run eagerly (a captured graph launches no binding).  The host must stay ahead of the GPU, or an
interval would hold the wait for the next launch: :meth:`KernelTimer.hold_back` puts a few milliseconds of
copies on the stream first, behind which the step's launches and events queue up.  Events cost the
GPU nothing between two kernels of one stream, but the step is not the captured one: a class's share is what
this gives, the step's time is the benchmark's.
"""
from __future__ import annotations

from typing import Callable, Dict, List, Optional, Tuple

import torch

from . import kernels

#: bindings that launch kernels, by name; what is not listed (shape predicates, workspaces) is left alone
LAUNCHERS = (
    "fetch_words", "embed_gather", "rmsnorm", "rope_angles", "rope_kvwrite", "swiglu", "fill_normal", "gemm_generic",
    "attn_generic", "attn_decode_f32", "attn_prefill_f32", "sample", "penalize", "logit_bias", "gemm_bf16", "gemm_bf16_qkv_rope", "gemm_bf16_follow",
    "gemm_bf16_mid_follow", "gemm_bf16_mid_qkv_rope", "gemm_bf16_gated_scaled", "attn_bf16_prefill",
    "attn_bf16_decode", "gemm_bf16_mid", "gemm_bf16_gated", "gemm_bf16_gated_tile_scaled",
)


def weight_shape(name: str, args: tuple) -> Optional[Tuple[int, int]]:
    """``(rows, columns)`` of the weight of a product binding's call, or None for a binding that is no product."""
    if name.startswith("gemm_") and len(args) >= 2 and hasattr(args[1], "shape") and args[1].dim() == 2:
        return int(args[1].shape[0]), int(args[1].shape[1])
    return None


class KernelTimer:
    """``with KernelTimer(label) as timer: <run a step eagerly>`` then ``timer.microseconds()``.

    ``label(name, args, kwargs)`` names the class of a call of binding ``name`` (default: the binding's name).
    """

    def __init__(self, label: Optional[Callable[[str, tuple, dict], str]] = None):
        self.label = label or (lambda name, args, kwargs: name)
        self.pairs: List[Tuple[str, torch.cuda.Event, torch.cuda.Event]] = []
        self._saved: Dict[str, Callable] = {}
        self._ballast: Optional[torch.Tensor] = None

    def hold_back(self, milliseconds: float = 8.0) -> None:
        """Keep the GPU busy for about ``milliseconds`` (copies of a 256 MB buffer, a fifth of a millisecond each at
        a few TB/s) so that the host gets ahead with its launches."""
        if self._ballast is None:
            self._ballast = torch.empty((2, 64 * 1024 * 1024), dtype=torch.float32, device="cuda")
        for _ in range(max(1, int(milliseconds * 5))):
            self._ballast[1].copy_(self._ballast[0])

    def __enter__(self) -> "KernelTimer":
        for name in LAUNCHERS:
            original = getattr(kernels, name)
            self._saved[name] = original
            setattr(kernels, name, self._wrap(name, original))
        return self

    def _wrap(self, name: str, original: Callable) -> Callable:
        def timed(*args, **kwargs):
            start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            start.record()
            try:
                return original(*args, **kwargs)
            finally:
                end.record()
                self.pairs.append((self.label(name, args, kwargs), start, end))
        return timed

    def __exit__(self, *exc) -> None:
        for name, original in self._saved.items():
            setattr(kernels, name, original)
        self._saved.clear()

    def microseconds(self) -> Dict[str, float]:
        """GPU time per class over everything timed so far, and ``"launches"``: how many calls that was."""
        torch.cuda.synchronize()
        out: Dict[str, float] = {}
        for label, start, end in self.pairs:
            out[label] = out.get(label, 0.0) + start.elapsed_time(end) * 1e3
        out["launches"] = float(len(self.pairs))
        return out
