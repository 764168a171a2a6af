"""Pins the oracle's block operators (CPU) against library routines, closed forms and brute force."""
import math

import pytest
import torch
import torch.nn.functional as F

from oracle import dit_ops as O


def test_sdpa_against_library_bruteforce_and_invariants():
    g = torch.Generator().manual_seed(0)
    q, k, v = (torch.randn(2, 3, 17, 16, generator=g) for _ in range(3))
    ours = O.sdpa(q, k, v)
    assert torch.allclose(ours, F.scaled_dot_product_attention(q, k, v), atol=1e-5, rtol=1e-5)
    # brute force on one (b, h, query)
    b, h, i = 1, 2, 5
    s = [sum(float(q[b, h, i, d]) * float(k[b, h, j, d]) for d in range(16)) / 4.0 for j in range(17)]
    m = max(s)
    p = [math.exp(x - m) for x in s]
    z = sum(p)
    for d in (0, 7, 15):
        ref = sum(p[j] / z * float(v[b, h, j, d]) for j in range(17))
        assert abs(float(ours[b, h, i, d]) - ref) < 1e-5
    # V constant => output constant; one key => output is that value; key permutation invariance
    assert torch.allclose(O.sdpa(q, k, torch.full_like(v, 0.3)), torch.full_like(q, 0.3), atol=1e-6)
    assert torch.allclose(O.sdpa(q, k[:, :, :1], v[:, :, :1]), v[:, :, :1].expand(-1, -1, 17, -1), atol=1e-6)
    perm = torch.randperm(17, generator=g)
    assert torch.allclose(O.sdpa(q, k[:, :, perm], v[:, :, perm]), ours, atol=1e-5)


def test_rms_norm_against_library_and_rounding_points():
    g = torch.Generator().manual_seed(1)
    x = torch.randn(2, 4, 9, 128, generator=g)
    w = 1 + 0.1 * torch.randn(128, generator=g)
    assert torch.allclose(O.rms_norm(x, w, 1e-6), F.rms_norm(x, (128,), w, 1e-6), atol=1e-5, rtol=1e-5)
    # bf16: cast after the normalisation, then a bf16 multiply (transformer_helper.py:76-77)
    xb, wb = x.bfloat16(), w.bfloat16()
    want = (xb.float() * torch.rsqrt(xb.float().square().mean(-1, keepdim=True) + 1e-6)).bfloat16() * wb
    assert torch.equal(O.rms_norm(xb, wb, 1e-6), want)


def _ids(n_txt, side):
    img = torch.zeros(side, side, 3)
    img[..., 1] += torch.arange(side)[:, None]
    img[..., 2] += torch.arange(side)[None, :]
    return torch.cat([torch.zeros(1, n_txt, 3), img.reshape(1, -1, 3)], dim=1)


def test_rope_table_closed_form_and_axis_order():
    ids = _ids(3, 4)
    t = O.rope_table(ids, (16, 56, 56), 10000)
    assert t.shape == (1, 1, 19, 64, 2, 2) and t.dtype == torch.float32
    # text rows (position 0 on every axis) carry the identity; axis 0 is 0 for every token: first 8 pairs identity
    eye = torch.eye(2).expand(64, 2, 2)
    assert torch.equal(t[0, 0, 0], eye) and torch.equal(t[0, 0, :, :8], torch.eye(2).expand(19, 8, 2, 2))
    # token (row 2, col 3): pairs 8..35 rotate by row * theta^(-2j/56), pairs 36..63 by col * theta^(-2j/56)
    tok = 3 + 2 * 4 + 3
    for j in (0, 5, 27):
        w = 10000.0 ** (-2 * j / 56)
        for base, pos in ((8, 2.0), (36, 3.0)):
            blk = t[0, 0, tok, base + j]
            c, s = math.cos(pos * w), math.sin(pos * w)
            assert torch.allclose(blk, torch.tensor([[c, -s], [s, c]], dtype=torch.float32), atol=1e-6)


def test_apply_rope_is_a_rotation_with_relative_position_property():
    g = torch.Generator().manual_seed(2)
    ids = _ids(2, 6)
    t = O.rope_table(ids, (16, 56, 56), 10000)
    x = torch.randn(1, 2, 38, 128, generator=g)
    y = O.apply_rope(x, t)
    # pos 0 => identity; per-pair norm preserved
    assert torch.equal(y[:, :, :2], x[:, :, :2])
    nx = x.reshape(1, 2, 38, 64, 2).norm(dim=-1)
    ny = y.reshape(1, 2, 38, 64, 2).norm(dim=-1)
    assert torch.allclose(nx, ny, atol=1e-5)
    # explicit pair formula (c x0 - s x1, s x0 + c x1)
    c, s = t[0, 0, :, :, 0, 0], t[0, 0, :, :, 1, 0]
    xp = x.reshape(1, 2, 38, 64, 2)
    want = torch.stack([c * xp[..., 0] - s * xp[..., 1], s * xp[..., 0] + c * xp[..., 1]], dim=-1).reshape(x.shape)
    assert torch.allclose(y, want, atol=1e-6)
    # <R(p) q, R(p') k> depends only on p - p': tokens (r,c) and (r+1,c+2) vs (r+2,c) and (r+3,c+2)
    q, k = torch.randn(128, generator=g), torch.randn(128, generator=g)
    def rot(vec, tok):
        return O.apply_rope(vec.view(1, 1, 1, 128), t[:, :, tok:tok + 1])[0, 0, 0]
    tok = lambda r, c: 2 + r * 6 + c
    d1 = torch.dot(rot(q, tok(0, 1)), rot(k, tok(1, 3)))
    d2 = torch.dot(rot(q, tok(2, 1)), rot(k, tok(3, 3)))
    assert abs(float(d1 - d2)) < 1e-4


def test_layer_norm_modulate_gelu_gated_residual():
    g = torch.Generator().manual_seed(3)
    x = torch.randn(2, 5, 64, generator=g)
    sc, sh = torch.randn(2, 1, 64, generator=g), torch.randn(2, 1, 64, generator=g)
    want = F.layer_norm(x, (64,), None, None, 1e-6) * (1 + sc) + sh
    assert torch.allclose(O.layer_norm_modulate(x, sc, sh), want, atol=1e-6)
    mu, var = x.mean(-1, keepdim=True), x.var(-1, unbiased=False, keepdim=True)
    assert torch.allclose(O.layer_norm_modulate(x, None, None), (x - mu) / torch.sqrt(var + 1e-6), atol=1e-5)
    # tanh-GELU: library routine and the explicit formula (transformer_helper.py:87-88)
    explicit = 0.5 * x * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (x + 0.044715 * torch.pow(x, 3.0))))
    assert torch.allclose(O.gelu_tanh(x), explicit, atol=1e-6)
    y, gate = torch.randn(2, 5, 64, generator=g), torch.randn(2, 1, 64, generator=g)
    assert torch.equal(O.gated_residual(x, y, gate), x + gate * y)
    assert torch.equal(O.gated_residual(x, y, None), x + y)


def test_timestep_embedding_closed_form():
    t = torch.tensor([0.0, 500.0, 1000.0])
    e = O.timestep_embedding(t, 256)
    assert e.shape == (3, 256)
    assert torch.equal(e[0, :128], torch.ones(128)) and torch.equal(e[0, 128:], torch.zeros(128))  # cos first
    for i in (0, 1, 64, 127):
        w = 10000.0 ** (-i / 128)
        assert abs(float(e[1, i]) - math.cos(500.0 * w)) < 2e-4 and abs(float(e[1, 128 + i]) - math.sin(500.0 * w)) < 2e-4
