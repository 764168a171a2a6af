"""MI355X drop-in for diffsynth_engine/utils/fp8_linear.py (same two names, same signatures).

``enable_fp8_linear(module)`` casts every floating ``nn.Linear`` weight to float8_e4m3fn and sets
``module.fp8_linear_enabled`` (fp8_linear.py:7-17).  ``fp8_inference(enabled)`` is a context manager
that replaces ``torch.nn.functional.linear`` for its duration (fp8_linear.py:20-64).  Instead of
``torch._scaled_mm`` the patched linear runs the hand-written gfx950 quantise + FP8 GEMM kernels.

Two quantisation modes, chosen per weight:
  * reference-exact: the weight carries no scale; activation and weight are bare casts and both
    GEMM scales are 1.0 (what fp8_linear.py:35-48 computes);
  * scaled (default of ``enable_fp8_linear`` here): the Linear module gets a buffer ``weight_scale``
    (absmax/448, 0-dim fp32) and activations get a dynamic per-token scale.
``F.linear(input, weight, bias)`` has no slot for a scale, so the weight Parameter carries a weak
reference to its module (``_dsx_owner``) and the patched linear reads the buffer through it.  The buffer
is module state: it follows ``.to()``, is written by ``state_dict()`` as ``<name>.weight_scale`` (the key
the block runners look for) and is restored in place by ``load_state_dict``.
"""
import weakref
from contextlib import contextmanager

import torch
import torch.nn as nn
import torch.nn.functional as F

from . import ops

SCALE_BUFFER = "weight_scale"
OWNER_ATTR = "_dsx_owner"


def enable_fp8_linear(module: nn.Module, scaled: bool = True):
    _enable_fp8_linear(module, scaled)
    setattr(module, "fp8_linear_enabled", True)


def _enable_fp8_linear(module: nn.Module, scaled: bool = True):
    if isinstance(module, nn.Linear) and torch.is_floating_point(module.weight.data) \
            and module.weight.data.dtype != ops.FP8:
        # integer (e.g. GGUF) weights are left alone, as in the reference
        q, scale = ops.quantize_weight_fp8(module.weight.data, scaled=scaled)
        module.weight.data = q
        if scale is not None:
            module.register_buffer(SCALE_BUFFER, scale)
            setattr(module.weight, OWNER_ATTR, weakref.ref(module))
    for submodule in module.children():
        _enable_fp8_linear(submodule, scaled)


def weight_scale_of(weight: torch.Tensor):
    """The per-tensor scale that belongs to ``weight`` (None: a reference-style weight with unit scale)."""
    owner = getattr(weight, OWNER_ATTR, None)
    module = owner() if owner is not None else None
    if module is None:
        return None
    scale = getattr(module, SCALE_BUFFER, None)
    if scale is not None and scale.device != weight.device:
        raise RuntimeError("weight_scale of a Linear is on %s, its weight on %s" % (scale.device, weight.device))
    return scale


def fp8_linear(input: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor | None = None) -> torch.Tensor:
    """The replacement of ``F.linear`` while ``fp8_inference`` is active."""
    origin_dtype = input.dtype
    w_scale = weight_scale_of(weight)
    if weight.dtype != ops.FP8:
        # a weight that enable_fp8_linear has not converted: cast on the fly like fp8_linear.py:36
        weight, _ = ops.quantize_weight_fp8(weight, scaled=False)
    x = input if input.dtype == torch.bfloat16 else input.to(torch.bfloat16)
    origin_shape = x.shape
    x2 = x.reshape(-1, origin_shape[-1])
    a_q, a_scale = ops.quantize_fp8(x2, scaled=w_scale is not None)
    result = ops.fp8_gemm(a_q, weight, a_scale, w_scale, bias)
    if len(origin_shape) > 2:
        result = result.reshape(origin_shape[:-1] + result.shape[-1:])
    return result if origin_dtype == torch.bfloat16 else result.to(origin_dtype)


@contextmanager
def fp8_inference(enabled=True):
    if not enabled:
        yield
        return
    origin_linear = F.linear
    F.linear = fp8_linear
    try:
        yield
    finally:
        F.linear = origin_linear
