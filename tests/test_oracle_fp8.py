"""Pins the oracle's FP8 arithmetic (CPU): the e4m3fn cast against the format definition, known answers and
torch's own cast; the scaled linear against torch._scaled_mm and brute force."""
import numpy as np
import pytest
import torch

from oracle import fp8 as ofp8


def test_e4m3_decode_matches_format_definition_and_torch():
    codes = np.arange(256, dtype=np.uint8)
    ours = ofp8.e4m3_to_f32(codes)
    theirs = torch.from_numpy(codes).view(torch.float8_e4m3fn).float().numpy()
    assert np.array_equal(np.isnan(ours), np.isnan(theirs))
    assert np.array_equal(ours[~np.isnan(ours)], theirs[~np.isnan(theirs)])
    # spot values from the format: bias 7, max 448, min subnormal 2^-9, no inf
    assert ours[0x7E] == 448.0 and ours[0x01] == 2.0 ** -9 and ours[0x08] == 2.0 ** -6 and ours[0x38] == 1.0
    assert np.isnan(ours[0x7F]) and np.isnan(ours[0xFF]) and not np.isinf(ours[~np.isnan(ours)]).any()


def test_cast_known_answers():
    """The values probed on torch 2.10 that define the reference's quantise step (fp8_linear.py:35)."""
    x = np.array([448.0, 464.0, 465.0, 479.9, 480.0, 1e9, 2.0 ** -10, 0.001, 0.0, -0.0, 2.0 ** -9 * 1.5,
                  2.0 ** -9 * 2.5, 17.0, 18.0, 19.0, np.inf, -np.inf], dtype=np.float32)
    got = ofp8.e4m3_to_f32(ofp8.e4m3_from_f32(x))
    want = [448.0, 448.0, np.nan, np.nan, np.nan, np.nan, 0.0, 2.0 ** -9, 0.0, -0.0, 2.0 ** -8, 2.0 ** -8, 16.0,
            18.0, 20.0, np.nan, np.nan]
    for g, w in zip(got, want):
        assert (np.isnan(g) and np.isnan(w)) or g == w, (got, want)
    # ties go to the even mantissa on both sides of a binade: 17 -> 16 (m=0), 19 -> 20 (m=2)
    t = torch.from_numpy(x).to(torch.float8_e4m3fn).float().numpy()
    assert np.array_equal(np.isnan(t), np.isnan(got)) and np.array_equal(t[~np.isnan(t)], got[~np.isnan(got)])


def test_cast_bit_exact_over_all_bf16_patterns():
    bits = torch.arange(0, 65536, dtype=torch.int32).to(torch.int16)
    x = bits.view(torch.bfloat16).float()
    ours = ofp8.e4m3_from_f32(x.numpy())
    theirs = x.to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    nan_in = np.isnan(x.numpy())
    assert np.array_equal(ours[~nan_in], theirs[~nan_in])
    assert ((ours[nan_in] & 0x7F) == 0x7F).all() and ((theirs[nan_in] & 0x7F) == 0x7F).all()


def test_cast_bit_exact_over_fp32_sweep():
    g = torch.Generator().manual_seed(0)
    u = torch.randint(0, 2 ** 31 - 1, (1 << 22,), generator=g, dtype=torch.int64)
    sign = torch.randint(0, 2, (1 << 22,), generator=g, dtype=torch.int64) << 31
    x = (u | sign).to(torch.int32).view(torch.float32)
    x = x[~torch.isnan(x)]
    ours = ofp8.e4m3_from_f32(x.numpy())
    theirs = x.to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    assert np.array_equal(ours, theirs)


def test_rowwise_quant_properties():
    g = torch.Generator().manual_seed(1)
    x = (torch.randn(37, 256, generator=g) * torch.rand(37, 1, generator=g) * 50).bfloat16()
    x[5] = 0
    q, s = ofp8.quantize_rowwise(x)
    qf = q.float()
    assert not torch.isnan(qf).any()
    amax = x.float().abs().amax(-1)
    assert torch.equal(s[amax > 0], amax[amax > 0] / 448.0)
    assert torch.equal(qf.abs().amax(-1)[amax > 0], torch.full_like(amax[amax > 0], 448.0))  # absmax maps to 448
    assert (qf[5] == 0).all()
    rel = ((qf * s[:, None] - x.float()).abs() / amax.clamp_min(1e-30)[:, None]).max().item()
    assert rel <= 16.0 / 448.0 + 1e-6  # half a step of the top binade [256, 448] (step 32) relative to 448
    qb, sb = ofp8.quantize_rowwise(x, scaled=False)
    assert sb is None and torch.equal(qb.view(torch.uint8), x.to(torch.float8_e4m3fn).view(torch.uint8))


def test_scaled_linear_against_torch_scaled_mm_and_brute_force():
    """Reference call (fp8_linear.py:41-48): torch._scaled_mm(x8, w8.T, scale_a, scale_b, bias, out_dtype)."""
    g = torch.Generator().manual_seed(2)
    x = torch.randn(32, 64, generator=g).bfloat16()
    w = torch.randn(48, 64, generator=g) * 0.02
    b = torch.randn(48, generator=g).bfloat16()
    # unit scales: exactly the reference path
    xq, _ = ofp8.quantize_rowwise(x, scaled=False)
    wq, _ = ofp8.quantize_weight(w, scaled=False)
    ours = ofp8.scaled_linear(xq, None, wq, None, b)
    theirs = torch._scaled_mm(xq, wq.t(), scale_a=torch.tensor(1.0), scale_b=torch.tensor(1.0), bias=b,
                              out_dtype=torch.bfloat16)
    assert (ours.float() - theirs.float()).abs().max().item() <= 2 ** -8 * theirs.float().abs().max().item()
    # scaled: brute-force triple loop in float64 on a corner
    xq, xs = ofp8.quantize_rowwise(x)
    wq, ws = ofp8.quantize_weight(w)
    ours = ofp8.scaled_linear(xq, xs, wq, ws, b).float()
    for m in (0, 7, 31):
        for n in (0, 13, 47):
            acc = sum(float(xq[m, k].float()) * float(wq[n, k].float()) for k in range(64))
            ref = acc * float(xs[m]) * float(ws) + float(b[n])
            assert abs(float(ours[m, n]) - ref) <= 2 ** -8 * abs(ref) + 1e-6
    # fp8_linear flattens leading dims and restores them (fp8_linear.py:38-50)
    y3 = ofp8.fp8_linear(x.view(4, 8, 64), wq, ws, b)
    assert y3.shape == (4, 8, 48) and torch.equal(y3.reshape(32, 48), ofp8.fp8_linear(x, wq, ws, b))
