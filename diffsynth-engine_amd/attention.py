"""MI355X attention behind the reference's attention seams.

* ``mi355x_attention(q, k, v)`` has the positional contract of the callable stored in
  ``flux_dit._attn_func`` (diffsynth_engine/models/flux/flux_dit.py:21,182,267,303): (B,H,S,D) in,
  (B,H,S,D) out, inputs may be non-contiguous views.
* ``wan_attention(q, k, v, num_heads)`` has the contract of ``wan_dit.attention``
  (diffsynth_engine/models/wan/wan_dit.py:18-22): (B,S,H*D) in and out; Lq may differ from Lk.
* ``attention(q, k, v, attn_impl="mi355x")`` takes (B,S,H,D).
* ``set_attn_implementation`` mirrors FluxDiT.set_attn_implementation (flux_dit.py:480-504) with the
  extra name ``"mi355x"``: unknown names raise ValueError, a missing library raises ImportError.
"""
from typing import Optional

import torch
import torch.nn as nn

from . import _lib, ops

SUPPORTED_IMPLEMENTATIONS = ("sdpa", "mi355x")


def _prep(t: torch.Tensor) -> torch.Tensor:
    """The kernel computes on bf16 operands (fp32 accumulation and softmax).  fp32 / fp16 tensors are rounded to
    bf16 once here, which is narrower than torch's SDPA would compute for them; the result stays within the bar the
    bf16 path is held to (2e-2 of the row maximum against fp32 SDPA of the unrounded inputs, tested)."""
    if t.dtype != torch.bfloat16:
        t = t.to(torch.bfloat16)
    if t.stride(-1) != 1 or any(s % 8 for s in t.stride()[:-1]) or t.data_ptr() % 16:
        t = t.contiguous()
    return t


def mi355x_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, attn_mask=None, dropout_p: float = 0.0,
                     is_causal: bool = False, scale: Optional[float] = None) -> torch.Tensor:
    """softmax(q k^T / sqrt(D)) v on (B,H,S,D); the SDPA arguments the DiTs never use must stay at their defaults."""
    if attn_mask is not None or dropout_p != 0.0 or is_causal:
        raise ValueError("mi355x_attention implements the unmasked, non-causal, dropout-free case only")
    dtype = q.dtype
    out = ops.attention_bhsd(_prep(q), _prep(k), _prep(v), scale=scale)
    return out if dtype == torch.bfloat16 else out.to(dtype)


def wan_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, num_heads: int) -> torch.Tensor:
    """(B,S,H*D) -> (B,S,H*D); the head split/merge of wan_dit.py:19,21 is done by strides, not copies."""
    B, Sq, HD = q.shape
    D = HD // num_heads
    dtype = q.dtype

    def split(t):
        return _prep(t).view(t.shape[0], t.shape[1], num_heads, D).transpose(1, 2)

    out = torch.empty((B, Sq, num_heads, D), dtype=torch.bfloat16, device=q.device)
    ops.attention_bhsd(split(q), split(k), split(v), out=out.transpose(1, 2))
    out = out.view(B, Sq, HD)
    return out if dtype == torch.bfloat16 else out.to(dtype)


def attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, attn_impl: Optional[str] = "mi355x",
              attn_mask: Optional[torch.Tensor] = None, scale: Optional[float] = None) -> torch.Tensor:
    """(B,S,H,D) in and out.  This package computes with its own kernels only: the reference's other backends
    (models/basic/attention.py:42-66) are the reference's to run, and asking for one here is a ValueError."""
    if attn_impl != "mi355x":
        raise ValueError(f"attn_impl must be 'mi355x' here, but got '{attn_impl}'")
    if attn_mask is not None:
        raise ValueError("attn_impl='mi355x' does not take an attention mask")
    B, Sq, H, D = q.shape
    dtype = q.dtype
    out = torch.empty((B, Sq, H, D), dtype=torch.bfloat16, device=q.device)
    ops.attention_bhsd(_prep(q).transpose(1, 2), _prep(k).transpose(1, 2), _prep(v).transpose(1, 2), scale=scale,
                       out=out.transpose(1, 2))
    return out if dtype == torch.bfloat16 else out.to(dtype)


def set_attn_implementation(attn_implementation: str, flux_dit_module=None, wan_dit_module=None):
    """Install an implementation into the reference's process-global seams.

    ``flux_dit_module`` is the imported ``diffsynth_engine.models.flux.flux_dit`` module (its global
    ``_attn_func`` is rebound), ``wan_dit_module`` the imported ``diffsynth_engine.models.wan.wan_dit``
    (its global ``attention`` is rebound).
    """
    if attn_implementation not in SUPPORTED_IMPLEMENTATIONS:
        raise ValueError(
            f"attn_implementation must be one of {SUPPORTED_IMPLEMENTATIONS}, but got '{attn_implementation}'"
        )
    if attn_implementation == "mi355x":
        _lib.load()  # ImportError if the library is not built
        flux_fn, wan_fn = mi355x_attention, wan_attention
    else:
        flux_fn = nn.functional.scaled_dot_product_attention
        wan_fn = None
    if flux_dit_module is not None:
        flux_dit_module._attn_func = flux_fn
    if wan_dit_module is not None:
        if wan_fn is None:
            raise ValueError("restoring the Wan seam needs the original function; reload the module instead")
        wan_dit_module.attention = wan_fn
    return flux_fn
