"""memorax_amd: MI355X-native kernels for memorax's sequence-model hot path.

Layers:
  csrc/            HIP kernels (gfx950) + the C ABI (include/memorax_amd.h)
  _lib, kernels    ctypes binding: torch device tensors -> raw pointers
  functional       differentiable ops (linear_scan, mingru_scan, linear_attention, delta_rule, ...)
  sequence_models  Memoroid-style modules: (inputs, done, initial_carry) -> (next_carry, y)
"""
from . import _lib  # noqa: F401
from .functional import (delta_rule, deltanet, gated_linear_attention, linear_attention, linear_scan,  # noqa: F401
                         mingru_scan, normalised_linear_attention)

__all__ = ["linear_scan", "mingru_scan", "linear_attention", "normalised_linear_attention", "gated_linear_attention", "delta_rule", "deltanet"]
