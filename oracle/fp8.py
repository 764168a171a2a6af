"""FP8 e4m3fn quantisation and the scaled linear — oracle (test infrastructure, see oracle/__init__.py).

Restates diffsynth_engine/utils/fp8_linear.py:7-64.  The cast itself is PyTorch's
``Tensor.to(torch.float8_e4m3fn)`` (fp8_linear.py:15,35-36): round-to-nearest-even onto OCP e4m3fn
(bias 7, 3 mantissa bits, max 448, subnormal step 2^-9, no inf, non-saturating: what would round
above 448 becomes NaN).
"""
import numpy as np
import torch

FP8 = torch.float8_e4m3fn
E4M3_MAX = 448.0


# ----------------------------------------------------------------------------------------------
# Bit-level restatement of the cast in numpy (independent of torch's implementation).
# ----------------------------------------------------------------------------------------------
def e4m3_to_f32(bits: np.ndarray) -> np.ndarray:
    """Decode e4m3fn bytes by the format definition: (-1)^s 2^(e-7) (1+m/8), e=0: m 2^-9, 0x7f: NaN."""
    bits = np.asarray(bits, dtype=np.uint8)
    s = (bits >> 7).astype(np.float64)
    e = ((bits >> 3) & 0xF).astype(np.int64)
    m = (bits & 0x7).astype(np.float64)
    normal = np.ldexp(1.0 + m / 8.0, e - 7)
    sub = m * 2.0 ** -9
    v = np.where(e == 0, sub, normal)
    v = np.where((bits & 0x7F) == 0x7F, np.nan, v)
    return (np.where(s == 1, -v, v)).astype(np.float32)


def _representable_magnitudes():
    codes = np.arange(0, 0x7F, dtype=np.uint8)  # 0 .. 0x7e: every finite non-negative value
    return codes, e4m3_to_f32(codes).astype(np.float64)


def e4m3_from_f32(x: np.ndarray) -> np.ndarray:
    """Round fp32 values to e4m3fn bytes by exhaustive nearest-value search with ties-to-even code.

    A value whose nearest candidate (including the would-be next value 480 = code 0x7f) is 480,
    i.e. |x| > 464 or the tie at 464 resolved to the even code... (464 ties to 448 = even mantissa),
    becomes NaN (0x7f), as do NaN and inf.
    """
    x = np.asarray(x, dtype=np.float32)
    sign = (x.view(np.uint32) >> 31).astype(np.uint8) << 7
    a = np.abs(x.astype(np.float64))
    codes, vals = _representable_magnitudes()
    vals_ext = np.concatenate([vals, [480.0]])  # 0x7f would be 480 if it were a number
    hi = np.searchsorted(vals_ext, a, side="left")  # first value >= a
    hi = np.clip(hi, 0, len(vals_ext) - 1)
    lo = np.clip(hi - 1, 0, len(vals_ext) - 1)
    d_lo = a - vals_ext[lo]
    d_hi = vals_ext[hi] - a
    pick_hi = (d_hi < d_lo) | ((d_hi == d_lo) & (hi % 2 == 0))  # tie: even code has even mantissa
    idx = np.where(pick_hi, hi, lo)
    idx = np.where(a >= 480.0, 0x7F, idx)
    idx = np.where(np.isnan(a), 0x7F, idx)
    return (idx.astype(np.uint8) | sign).astype(np.uint8)


# ----------------------------------------------------------------------------------------------
# Torch-level quantisation and linear, as the reference computes them.
# ----------------------------------------------------------------------------------------------
def cast_e4m3(x: torch.Tensor) -> torch.Tensor:
    """fp8_linear.py:35 — the bare cast."""
    return x.to(FP8)


def quantize_rowwise(x: torch.Tensor, scaled: bool = True):
    """Per-token dynamic quantisation: a = max(absmax,1e-12), s = a/448, q = cast(float(x) * (448/a)), all fp32.

    ``scaled=False`` is the reference's bare cast with unit scale.
    """
    if not scaled:
        return cast_e4m3(x), None
    xf = x.float()
    a = torch.clamp(xf.abs().amax(dim=-1), min=1e-12)
    inv = torch.full_like(a, E4M3_MAX) / a  # a true fp32 division (``448.0 / a`` would be reciprocal * 448)
    q = (xf * inv.unsqueeze(-1)).to(FP8)
    return q, a / E4M3_MAX


def quantize_weight(w: torch.Tensor, scaled: bool = True):
    """fp8_linear.py:12-17 weight cast; scaled: a = max(absmax,1e-12), s_w = a/448, q = cast(w * (448/a))."""
    if not scaled:
        return cast_e4m3(w), None
    wf = w.float()
    a = torch.clamp(wf.abs().amax(), min=1e-12)
    inv = torch.full_like(a, E4M3_MAX) / a
    return (wf * inv).to(FP8), a / E4M3_MAX


def scaled_linear(x_q, x_scale, w_q, w_scale, bias, out_dtype=torch.bfloat16):
    """fp8_linear.py:41-48: out = cast((sum_k a b) * scale_a * scale_b + bias), fp32 accumulation."""
    acc = x_q.float() @ w_q.float().t()
    if x_scale is not None:
        acc = acc * x_scale.unsqueeze(-1)
    if w_scale is not None:
        acc = acc * w_scale
    if bias is not None:
        acc = acc + bias.float()
    return acc.to(out_dtype)


def fp8_linear(x: torch.Tensor, w_q: torch.Tensor, w_scale, bias):
    """The patched F.linear (fp8_linear.py:28-60): quantise the activation, flatten leading dims, multiply."""
    shape = x.shape
    x2 = x.reshape(-1, shape[-1])
    x_q, x_s = quantize_rowwise(x2, scaled=w_scale is not None)
    out = scaled_linear(x_q, x_s, w_q, w_scale, bias, out_dtype=x.dtype)
    return out.reshape(*shape[:-1], out.shape[-1])
