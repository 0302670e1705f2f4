from . import build, kernels

__all__ = ["build", "kernels"]
