"""Seeded sweeps over odd shapes, strides and option combinations of the three kernel families, each case
checked against the CPU oracle.  The shapes are drawn once from a fixed seed, so a failure names its case."""
import math
import random

import pytest
import torch

from conftest import row_rel_err
from oracle import dit_ops as O
from oracle import fp8 as ofp8

pytestmark = pytest.mark.gpu


def _attention_cases(n=28):
    rnd = random.Random(1234)
    cases = []
    for i in range(n):
        B, H = rnd.choice([1, 1, 2]), rnd.randint(1, 4)
        Sq, Skv = rnd.choice([1, 7, 31, 32, 33, 63, 64, 65, 127, 255, 256, 257, rnd.randint(1, 700)]), \
            rnd.choice([1, 5, 63, 64, 65, 128, 129, 191, rnd.randint(1, 700)])
        split_q = rnd.randint(0, Sq) if rnd.random() < 0.5 else None
        split_kv = rnd.randint(0, Skv) if rnd.random() < 0.5 else None
        packed = rnd.random() < 0.5  # (B,S,H,D) storage viewed as (B,H,S,D)
        cases.append((i, B, H, Sq, Skv, split_q, split_kv, packed))
    return cases


@pytest.mark.parametrize("case", _attention_cases(), ids=lambda c: "a%d_B%d_H%d_Sq%d_Skv%d_%s_%s_%s" % c)
def test_attention_shape_sweep(dev, case):
    from diffsynth_engine_amd import ops

    i, B, H, Sq, Skv, split_q, split_kv, packed = case
    g = torch.Generator().manual_seed(100 + i)

    def mk(S):
        if packed:
            return torch.randn(B, S, H, 128, generator=g).bfloat16().transpose(1, 2)
        return torch.randn(B, H, S, 128, generator=g).bfloat16()

    q, k, v = mk(Sq), mk(Skv), mk(Skv)
    want = O.sdpa(q.float(), k.float(), v.float())
    qd, kd, vd = q.to(dev), k.to(dev), v.to(dev)
    if packed:  # .to(dev) keeps the strides of the transposed view
        assert qd.stride(1) == 128
    sq = Sq if split_q is None else split_q
    skv = Skv if split_kv is None else split_kv
    if (split_q is None and split_kv is None) or sq in (0, Sq) or skv in (0, Skv):
        got = ops.attention_bhsd(qd, kd, vd).cpu()
    else:
        # two query segments need two key segments in this entry point: split both
        o1, o2 = ops.attention_bhsd(qd[:, :, :sq], kd[:, :, :skv], vd[:, :, :skv], q2=qd[:, :, sq:],
                                    k2=kd[:, :, skv:], v2=vd[:, :, skv:])
        got = torch.cat([o1, o2], dim=2).cpu()
    err = row_rel_err(got, want)
    assert err <= 2e-2, err


def _gemm_cases(n=28):
    rnd = random.Random(4321)
    cases = []
    for i in range(n):
        M = rnd.choice([9, 16, 255, 256, 257, 511, 513, rnd.randint(9, 900)])
        N = 8 * rnd.choice([1, 2, 31, 32, 33, 64, 65, rnd.randint(1, 110)])
        K = 16 * rnd.choice([1, 2, 7, 8, 9, 16, 24, 64, rnd.randint(1, 70)])
        bias = rnd.random() < 0.7
        resid = rnd.random() < 0.5
        gate = resid and rnd.random() < 0.6
        nb = rnd.choice([1, 2, 3]) if gate else 1
        pad = rnd.choice([0, 0, 8, 24])  # output row stride beyond N
        cases.append((i, M, N, K, bias, resid, gate, nb, pad))
    return cases


@pytest.mark.parametrize("case", _gemm_cases(), ids=lambda c: "g%d_M%d_N%d_K%d_b%d_r%d_g%d_nb%d_pad%d" % c)
def test_gemm_shape_sweep(dev, case):
    from diffsynth_engine_amd import ops

    i, M, N, K, bias, resid, gate, nb, pad = case
    g = torch.Generator().manual_seed(200 + i)
    w = torch.randn(N, K, generator=g) * 0.05
    x = torch.randn(M, K, generator=g).bfloat16()
    b = torch.randn(N, generator=g).bfloat16() if bias else None
    wq, ws = ofp8.quantize_weight(w, scaled=True)
    xq, xs = ofp8.quantize_rowwise(x, scaled=True)
    proj = ofp8.scaled_linear(xq, xs, wq, ws, b)  # bf16
    want = proj
    kw = {}
    rpb = -(-M // nb)
    if resid:
        r = torch.randn(M, N, generator=g).bfloat16()
        gt = torch.randn(nb, N, generator=g).bfloat16() if gate else None
        t = proj
        if gt is not None:
            rows = torch.arange(M) // rpb
            t = (gt[rows].float() * proj.float()).bfloat16()
        want = (r.float() + t.float()).bfloat16()
        kw = dict(resid=r.to(dev), gate=None if gt is None else gt.to(dev), rows_per_batch=rpb)
    out = torch.full((M, N + pad), 7.0, dtype=torch.bfloat16, device=dev)[:, :N]
    got = ops.fp8_gemm(xq.to(dev), wq.to(dev), xs.to(dev), ws.to(dev), None if b is None else b.to(dev), out=out, **kw)
    assert got.data_ptr() == out.data_ptr()
    if pad:  # nothing written past column N
        assert bool((out.as_strided((M, pad), (N + pad, 1), N) == 7.0).all())
    d = (got.cpu().float() - want.float()).abs()
    assert d.max().item() <= 2e-2 * want.float().abs().max().item() + 2e-3, d.max().item()


def _row_cases(n=20):
    rnd = random.Random(99)
    return [(i, rnd.choice([1, 3, 4, 5, 1023, 1024, 1025, rnd.randint(1, 1500)]),
             8 * rnd.choice([1, 2, 63, 64, 65, 384, 385, 640, rnd.randint(1, 768)])) for i in range(n)]


@pytest.mark.parametrize("case", _row_cases(), ids=lambda c: "r%d_rows%d_D%d" % c)
def test_row_kernel_shape_sweep(dev, case):
    from diffsynth_engine_amd import ops

    i, rows, D = case
    g = torch.Generator().manual_seed(300 + i)
    x = (torch.randn(1, rows, D, generator=g) * 2 + 0.1).bfloat16()
    mod = (torch.randn(1, 2 * D, generator=g) * 0.5).bfloat16()
    sc, sh = mod.chunk(2, dim=1)
    # quantiser: bit-exact
    q, s = ops.quantize_fp8(x.view(rows, D).to(dev), scaled=True)
    wq, wsx = ofp8.quantize_rowwise(x.view(rows, D), scaled=True)
    assert torch.equal(s.cpu(), wsx) and torch.equal(q.cpu().view(torch.uint8), wq.view(torch.uint8))
    # AdaLN: within a bf16 ulp of the oracle for all but a sliver of elements; its e4m3 emission = quantiser of its output
    want = O.layer_norm_modulate(x, sc[:, None], sh[:, None], 1e-6)
    md = mod.to(dev)
    scd, shd = md.chunk(2, dim=1)
    y, yq, ys = ops.adaln_modulate(x.to(dev), scd, shd, want_bf16=True, want_fp8=True)
    dd = (y.cpu().float() - want.float()).abs()
    off = dd > torch.maximum(want.float().abs() * 2 ** -7, torch.tensor(2e-2 if D < 64 else 1e-6))
    assert off.float().mean().item() < 2e-3
    oq, os_ = ofp8.quantize_rowwise(y.cpu().reshape(rows, D), scaled=True)
    assert torch.equal(ys.cpu(), os_) and torch.equal(yq.cpu().view(torch.uint8).reshape(rows, D), oq.view(torch.uint8))
    # GELU
    wantg = O.gelu_tanh(x.view(rows, D))
    gy = ops.gelu_tanh(x.view(rows, D).to(dev)).cpu()
    dg = (gy.float() - wantg.float()).abs()
    assert bool((dg <= wantg.float().abs() * 2 ** -7 + 1e-6).all())
