"""Structural pins of the Wan DiT restatement in the oracle (CPU, tiny sizes)."""
import math

import torch
import torch.nn.functional as F

from oracle import dit_ops as O
from oracle import wan as ow


def _cfg(**kw):
    return dict(ow.config_14b(), dim=256, ffn_dim=512, num_heads=2, num_layers=1, **kw)


def test_rope_apply_equals_real_rotation_and_axis_split():
    hd, f, h, w = 128, 2, 3, 4
    fr = ow.freqs_cis_3d(hd, f, h, w)
    assert fr.shape == (24, 1, 64) and fr.dtype == torch.complex128
    # axis split 44/42/42 dims = 22 + 21 + 21 pairs; token (1,2,3): pair 0 by frame, pair 22 by row, pair 43 by col
    tok = 1 * 12 + 2 * 4 + 3
    for pair, pos, dim_axis, j in ((0, 1, 44, 0), (5, 1, 44, 5), (22, 2, 42, 0), (30, 2, 42, 8), (43, 3, 42, 0), (63, 3, 42, 20)):
        ang = pos * 10000.0 ** (-2 * j / dim_axis)
        assert abs(fr[tok, 0, pair].real.item() - math.cos(ang)) < 1e-12
        assert abs(fr[tok, 0, pair].imag.item() - math.sin(ang)) < 1e-12
    x = torch.randn(1, 24, 2 * hd, generator=torch.Generator().manual_seed(0))
    y = ow.rope_apply(x, fr, 2)
    xp = x.view(1, 24, 2, 64, 2)
    c, s = fr.real.float().view(1, 24, 1, 64), fr.imag.float().view(1, 24, 1, 64)
    want = torch.stack([c * xp[..., 0] - s * xp[..., 1], s * xp[..., 0] + c * xp[..., 1]], dim=-1).reshape(x.shape)
    assert torch.allclose(y, want, atol=1e-6)
    assert torch.equal(y[:, 0], x[:, 0])  # token (0,0,0) is not rotated


def test_wan_rms_norm_spans_all_heads():
    x = torch.randn(2, 5, 256, generator=torch.Generator().manual_seed(1))
    w = 1 + 0.1 * torch.randn(256, generator=torch.Generator().manual_seed(2))
    assert torch.allclose(ow.wan_rms_norm(x, w, 1e-6), F.rms_norm(x, (256,), w, 1e-6), atol=1e-5)


def test_block_identity_when_gates_and_cross_output_vanish():
    cfg = _cfg()
    sd = ow.init_params(cfg, dtype=torch.float32, bias_std=0.02)
    g = torch.Generator().manual_seed(3)
    x, ctx = torch.randn(1, 12, 256, generator=g), torch.randn(1, 5, 256, generator=g)
    fr = ow.freqs_cis_3d(128, 1, 3, 4)
    # chunk order shift_msa, scale_msa, gate_msa, shift_mlp, scale_mlp, gate_mlp: zero chunks 2 and 5
    mod = torch.randn(1, 6, 256, generator=g)
    mod[:, 2] = 0
    mod[:, 5] = 0
    sd["blocks.0.modulation"] = mod
    sd["blocks.0.cross_attn.o.weight"] = torch.zeros_like(sd["blocks.0.cross_attn.o.weight"])
    sd["blocks.0.cross_attn.o.bias"] = torch.zeros_like(sd["blocks.0.cross_attn.o.bias"])
    y = ow.dit_block(ow.Params(sd), 0, x, ctx, torch.zeros(1, 6, 256), fr, cfg)
    assert torch.equal(y, x)
    # with only gate_mlp restored the update is exactly gate * ffn(modulate(LN(x)))
    mod[:, 5] = 0.5
    sd["blocks.0.modulation"] = mod
    P = ow.Params(sd)
    y = ow.dit_block(P, 0, x, ctx, torch.zeros(1, 6, 256), fr, cfg)
    h = O.layer_norm_modulate(x, mod[:, 4:5], mod[:, 3:4], 1e-6)
    want = x + 0.5 * P.linear(O.gelu_tanh(P.linear(h, "blocks.0.ffn.0")), "blocks.0.ffn.2")
    assert torch.allclose(y, want, atol=1e-5)


def test_model_forward_shapes_and_patch_linear_equals_conv3d():
    cfg = _cfg()
    sd = ow.init_params(cfg, dtype=torch.float32, bias_std=0.02)
    g = torch.Generator().manual_seed(4)
    x = torch.randn(1, 16, 2, 6, 8, generator=g)
    out = ow.wan_dit_forward(ow.Params(sd), x, torch.randn(1, 5, 4096, generator=g), torch.tensor([500.0]), cfg)
    assert out.shape == x.shape and torch.isfinite(out).all()
    y = F.conv3d(x, sd["patch_embedding.weight"], sd["patch_embedding.bias"], stride=(1, 2, 2)).flatten(2).transpose(1, 2)
    patches = x.view(1, 16, 2, 1, 3, 2, 4, 2).permute(0, 2, 4, 6, 1, 3, 5, 7).reshape(1, 24, 64)
    lin = F.linear(patches, sd["patch_embedding.weight"].reshape(256, -1), sd["patch_embedding.bias"])
    assert torch.allclose(lin, y, atol=1e-5)
    e = ow.sinusoidal_embedding_1d(256, torch.tensor([0.0, 3.0]))
    assert torch.equal(e[0, :128], torch.ones(128)) and abs(float(e[1, 128]) - math.sin(3.0)) < 1e-6
