"""MI355X-native kernels for the DiT denoising step of DiffSynth-Engine (Flux / Wan).

Public surface:
  attention.mi355x_attention / wan_attention / attention / set_attn_implementation
  fp8_linear.enable_fp8_linear / fp8_inference
  ops.*  (tensor-level wrappers of the C-ABI kernels in libdsx.so)
  flux_dit.FluxDiTRunner / wan_dit.WanDiTRunner (fused block runners), install.accelerate_flux_dit /
  accelerate_wan_dit (a runner behind a DiT module's forward), graph.GraphedStep (a step as a HIP graph)
"""
from . import _lib  # noqa: F401
from .attention import attention, mi355x_attention, set_attn_implementation, wan_attention  # noqa: F401
from .fp8_linear import enable_fp8_linear, fp8_inference  # noqa: F401

__all__ = [
    "attention",
    "mi355x_attention",
    "wan_attention",
    "set_attn_implementation",
    "enable_fp8_linear",
    "fp8_inference",
]
