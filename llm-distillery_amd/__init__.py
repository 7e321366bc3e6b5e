"""MI355X-native distillation-loss hot path of LLM-Distillery.

Hand-written gfx950 HIP kernels behind a C ABI (libdistill_hip.so), exposed
through the reference's own Python boundary (`calculate_divergence`, `Losses`).
"""
from . import _lib  # noqa: F401
from .ops import copy16, div_topk, reduce_sum, set_option  # noqa: F401

__all__ = ["copy16", "div_topk", "reduce_sum", "set_option"]
