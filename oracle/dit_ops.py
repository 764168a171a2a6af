"""Block-level operators of the Flux / Wan DiT — oracle (test infrastructure, see oracle/__init__.py).

Every function keeps the reference's op order and therefore its rounding points when run in bf16.
"""
import math

import torch
import torch.nn.functional as F


def sdpa(q, k, v, scale=None):
    """softmax(q k^T * scale) v with fp32 softmax — what ``_attn_func(q, k, v)`` computes
    (models/flux/flux_dit.py:21,182; models/wan/wan_dit.py:20; eager form models/basic/attention.py:114-122)."""
    d = q.shape[-1]
    scale = 1.0 / math.sqrt(d) if scale is None else scale
    s = torch.matmul(q.float(), k.float().transpose(-1, -2)) * scale
    p = torch.softmax(s, dim=-1)
    return torch.matmul(p, v.float()).to(q.dtype)


def rms_norm(x, weight, eps):
    """models/basic/transformer_helper.py:73-78: fp32 mean square, x*rsqrt -> cast -> * weight."""
    dtype = x.dtype
    var = x.to(torch.float32).square().mean(-1, keepdim=True)
    y = x * torch.rsqrt(var + eps)
    return y.to(dtype) * weight


def rope_table(ids, axes_dim, theta=10000):
    """models/basic/transformer_helper.py:46-64: per axis omega_j = theta^(-2j/dim) in float64, angle =
    pos * omega, 2x2 blocks [[cos, -sin], [sin, cos]], axes concatenated along the pair dim, fp32,
    shape (B, 1, S, sum(dim)/2, 2, 2)."""
    tables = []
    for a, dim in enumerate(axes_dim):
        pos = ids[..., a].to(torch.float64)
        omega = 1.0 / (theta ** (torch.arange(0, dim, 2, dtype=torch.float64, device=ids.device) / dim))
        ang = pos.unsqueeze(-1) * omega
        c, s = torch.cos(ang), torch.sin(ang)
        tables.append(torch.stack([c, -s, s, c], dim=-1).reshape(*ang.shape, 2, 2).float())
    return torch.cat(tables, dim=-3).unsqueeze(1)


def apply_rope(x, freqs):
    """models/flux/flux_dit.py:154-159: pairs (2i, 2i+1) -> (c x0 - s x1, s x0 + c x1), fp32 math, cast back."""
    xf = x.float().reshape(*x.shape[:-1], -1, 1, 2)
    out = freqs[..., 0] * xf[..., 0] + freqs[..., 1] * xf[..., 1]
    return out.reshape(*x.shape).type_as(x)


def layer_norm_modulate(x, scale, shift, eps=1e-6, weight=None, bias=None):
    """``norm(x) * (1 + scale) + shift`` (transformer_helper.py:17,21,35; flux_dit.py:228,233,334;
    wan_dit.py:25-26).  scale/shift broadcast over the token dim; None skips that term."""
    y = F.layer_norm(x, (x.shape[-1],), weight, bias, eps)
    if scale is not None:
        y = y * (1 + scale)
    if shift is not None:
        y = y + shift
    return y


def gated_residual(x, y, gate):
    """``x + gate * y`` (flux_dit.py:227,232,318-319; wan_dit.py:189,192)."""
    return x + (gate * y if gate is not None else y)


def gelu_tanh(x):
    """nn.GELU(approximate="tanh") (flux_dit.py:209,215,315; wan_dit.py:180)."""
    return F.gelu(x, approximate="tanh")


def timestep_embedding(t, dim=256, max_period=10000):
    """models/basic/timestep.py:6-44 with flip_sin_to_cos=True, downscale_freq_shift=0 (timestep.py:69-71):
    [cos(t w_i), sin(t w_i)], w_i = max_period^(-i/half), fp32."""
    half = dim // 2
    exponent = -math.log(max_period) * torch.arange(half, dtype=torch.float32, device=t.device) / half
    ang = t[:, None].float() * torch.exp(exponent)[None, :]
    return torch.cat([torch.cos(ang), torch.sin(ang)], dim=-1)
