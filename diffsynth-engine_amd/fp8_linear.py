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
``F.linear(input, weight, bias)`` has no slot for a scale.  The buffer is module state: it follows ``.to()``
and ``copy.deepcopy``, is written by ``state_dict()`` as ``<name>.weight_scale`` (the key the block runners
look for) and is restored in place by ``load_state_dict``.  It reaches the patched linear two ways:
``fp8_inference`` also wraps ``nn.Linear.forward`` (the reference's LoRALinear calls it through ``super()``,
models/basic/lora.py:137-141), which announces the module's buffer for the ``F.linear`` call it makes, so
whatever else is chained onto ``F.linear`` still runs; and for code that calls ``F.linear(x, m.weight, m.bias)``
itself the weight Parameter carries a weak reference to its module (``_dsx_owner``; ``enable_fp8_linear`` on an
already converted module renews it, e.g. after a ``deepcopy``, which drops Parameter attributes).
"""
import threading
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
    elif isinstance(module, nn.Linear) and module.weight.data.dtype == ops.FP8 \
            and module._buffers.get(SCALE_BUFFER) is not None:
        setattr(module.weight, OWNER_ATTR, weakref.ref(module))  # converted earlier (and perhaps copied since)
    for submodule in module.children():
        _enable_fp8_linear(submodule, scaled)


_announced = threading.local()  # (weight, scale) of the nn.Linear.forward call in progress on this thread


def _linear_forward(self, input):
    """nn.Linear.forward while fp8_inference is active: the same F.linear call, with the module's scale announced."""
    scale = self._buffers.get(SCALE_BUFFER)
    if scale is None:
        return F.linear(input, self.weight, self.bias)
    previous = getattr(_announced, "pair", None)
    _announced.pair = (self.weight, scale)
    try:
        return F.linear(input, self.weight, self.bias)
    finally:
        _announced.pair = previous


def weight_scale_of(weight: torch.Tensor):
    """The per-tensor scale that belongs to ``weight`` (None: a reference-style weight with unit scale)."""
    pair = getattr(_announced, "pair", None)
    if pair is not None and pair[0] is weight:
        scale = pair[1]
    else:
        owner = getattr(weight, OWNER_ATTR, None)
        if owner is None:
            return None
        module = owner()
        if module is None:
            raise RuntimeError("the Linear module this scaled float8 weight was converted in is gone; its scale "
                               "went with it (keep the module, or call enable_fp8_linear on the one that holds "
                               "the weight now)")
        scale = module._buffers.get(SCALE_BUFFER)
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
    origin_linear, origin_forward = F.linear, nn.Linear.forward
    F.linear = fp8_linear
    nn.Linear.forward = _linear_forward
    try:
        yield
    finally:
        F.linear = origin_linear
        nn.Linear.forward = origin_forward
