"""GPU parity: AdaLN modulate, gated residual, tanh-GELU (+ fused e4m3 emission), Euler step — vs the bf16 oracle."""
import pytest
import torch

from oracle import dit_ops as O
from oracle import fp8 as ofp8

pytestmark = pytest.mark.gpu


def _ulp_report(got, want):
    """Fraction of elements off by more than a bf16 ulp of |want| (or 1e-6 absolute, whichever is larger),
    and max |diff| relative to max |want|."""
    d = (got.float() - want.float()).abs()
    off = d > torch.maximum(want.float().abs() * 2 ** -7, torch.tensor(1e-6))
    return off.float().mean().item(), (d.max() / want.float().abs().max()).item()


@pytest.mark.parametrize("B,S,D", [(1, 40, 3072), (2, 17, 5120), (1, 5, 64), (1, 3, 16384)])
def test_adaln_modulate(dev, B, S, D):
    from diffsynth_engine_amd import ops

    g = torch.Generator().manual_seed(D + S)
    x = (torch.randn(B, S, D, generator=g) * 2 + 0.3).bfloat16()
    mod = torch.randn(B, 6 * D, generator=g).bfloat16()
    shift, scale = mod.unsqueeze(1).chunk(6, dim=2)[:2]
    want = O.layer_norm_modulate(x, scale, shift, 1e-6)
    md = mod.to(dev)
    shd, scd = md.unsqueeze(1).chunk(6, dim=2)[:2]
    y, q, qs = ops.adaln_modulate(x.to(dev), scd, shd, want_bf16=True, want_fp8=True)
    frac, rel = _ulp_report(y.cpu(), want)
    assert frac < 1e-3 and rel <= 2 ** -6, (frac, rel)
    # the fused e4m3 emission must be the row quantiser applied to the kernel's own bf16 output
    wq, ws = ofp8.quantize_rowwise(y.cpu().reshape(-1, D), scaled=True)
    assert torch.equal(qs.cpu(), ws)
    assert torch.equal(q.cpu().view(torch.uint8).reshape(-1, D), wq.view(torch.uint8))


def test_adaln_affine_no_modulation(dev):
    """Wan norm3: LayerNorm with affine weight/bias and no scale/shift (wan_dit.py:177,190)."""
    from diffsynth_engine_amd import ops

    g = torch.Generator().manual_seed(4)
    x = torch.randn(1, 33, 5120, generator=g).bfloat16()
    w = (1 + 0.1 * torch.randn(5120, generator=g)).bfloat16()
    b = (0.1 * torch.randn(5120, generator=g)).bfloat16()
    want = O.layer_norm_modulate(x, None, None, 1e-6, w, b)
    got = ops.adaln_modulate(x.to(dev), None, None, ln_weight=w.to(dev), ln_bias=b.to(dev)).cpu()
    frac, rel = _ulp_report(got, want)
    assert frac < 1e-3 and rel <= 2 ** -6, (frac, rel)


def test_layernorm_closed_form(dev):
    """A row that is a +-1 pattern has mean 0, variance 1: LN(x) = x up to the eps term."""
    from diffsynth_engine_amd import ops

    x = torch.ones(1, 4, 3072)
    x[..., ::2] = -1
    one = torch.zeros(1, 3072).bfloat16()
    got = ops.adaln_modulate(x.bfloat16().to(dev), one.to(dev), one.to(dev)).cpu().float()
    assert torch.equal(got, x)


@pytest.mark.parametrize("B,S,D", [(1, 50, 3072), (2, 9, 5120)])
def test_gated_residual(dev, B, S, D):
    from diffsynth_engine_amd import ops

    g = torch.Generator().manual_seed(S)
    x = torch.randn(B, S, D, generator=g).bfloat16()
    y = torch.randn(B, S, D, generator=g).bfloat16()
    gate = torch.randn(B, 1, D, generator=g).bfloat16()
    want = O.gated_residual(x, y, gate)
    got = ops.gated_residual(x.to(dev), y.to(dev), gate.to(dev)).cpu()
    assert torch.equal(got, want)  # two bf16 roundings of exact fp32 ops: bit-exact
    want = O.gated_residual(x, y, None)
    assert torch.equal(ops.gated_residual(x.to(dev), y.to(dev), None).cpu(), want)


@pytest.mark.parametrize("rows,D", [(37, 12288), (5, 13824), (64, 64)])
def test_gelu_tanh(dev, rows, D):
    from diffsynth_engine_amd import ops

    g = torch.Generator().manual_seed(rows)
    x = (torch.randn(rows, D, generator=g) * 3).bfloat16()
    want = O.gelu_tanh(x)
    y, q, qs = ops.gelu_tanh(x.to(dev), want_bf16=True, want_fp8=True)
    frac, rel = _ulp_report(y.cpu(), want)
    assert frac < 1e-3 and rel <= 2 ** -7, (frac, rel)
    wq, ws = ofp8.quantize_rowwise(y.cpu(), scaled=True)
    assert torch.equal(qs.cpu(), ws) and torch.equal(q.cpu().view(torch.uint8), wq.view(torch.uint8))


def test_gelu_all_bf16_inputs(dev):
    from diffsynth_engine_amd import ops

    bits = torch.arange(0, 65536, dtype=torch.int32).to(torch.int16)
    x = bits.view(torch.bfloat16).view(8, 8192)
    want = O.gelu_tanh(x).float()
    got = ops.gelu_tanh(x.to(dev)).cpu().float()
    fin = torch.isfinite(want)
    assert torch.equal(torch.isnan(got), torch.isnan(want))
    d = (got[fin] - want[fin]).abs()
    tol = want[fin].abs() * 2 ** -7 + 1e-6
    assert bool((d <= tol).all())


def test_gelu_strided_slice_of_wider_buffer(dev):
    """The single-stream block applies GELU to columns [9216:] of the (S,21504) projection (flux_dit.py:312-315)."""
    from diffsynth_engine_amd import ops

    x = torch.randn(1, 12, 21504, generator=torch.Generator().manual_seed(0)).bfloat16()
    want = O.gelu_tanh(x[:, :, 9216:])
    got = ops.gelu_tanh(x.to(dev)[:, :, 9216:]).cpu()
    frac, rel = _ulp_report(got, want)
    assert frac < 1e-3 and rel <= 2 ** -7


def test_flow_match_euler_step(dev):
    from diffsynth_engine_amd import ops

    g = torch.Generator().manual_seed(1)
    lat, v = torch.randn(1, 16, 32, 32, generator=g), torch.randn(1, 16, 32, 32, generator=g)
    dt = torch.tensor(0.7071) - torch.tensor(0.9001)
    for dtype in (torch.float32, torch.bfloat16):
        a, b = lat.to(dtype), v.to(dtype)
        want = (a.to(torch.float32) + b * dt).to(dtype)
        got = ops.flow_match_euler_step(a.to(dev), b.to(dev), dt.item()).cpu()
        assert torch.equal(got, want)


def test_concat_gelu_builds_single_block_operand(dev):
    """[attention | gelu(mlp)] emitted as the per-token-scaled e4m3 operand of proj_out (flux_dit.py:315-317)."""
    from diffsynth_engine_amd import ops

    g = torch.Generator().manual_seed(2)
    rows, d = 21, 3072
    att = torch.randn(rows, d, generator=g).bfloat16()
    h = (torch.randn(rows, 7 * d, generator=g) * 2).bfloat16()
    want = torch.cat([att, O.gelu_tanh(h[:, 3 * d:])], dim=1)
    y, q, qs = ops.concat_gelu_tanh(att.to(dev), h.to(dev)[:, 3 * d:], want_bf16=True, want_fp8=True)
    assert torch.equal(y.cpu()[:, :d], att)
    frac, rel = _ulp_report(y.cpu(), want)
    assert frac < 1e-3 and rel <= 2 ** -7, (frac, rel)
    wq, ws = ofp8.quantize_rowwise(y.cpu(), scaled=True)
    assert torch.equal(qs.cpu(), ws) and torch.equal(q.cpu().view(torch.uint8), wq.view(torch.uint8))


def test_adaln_wave_per_row_path_many_rows(dev):
    """Rows >= 1024 take the one-wavefront-per-row kernel: same results, ragged row count."""
    from diffsynth_engine_amd import ops

    g = torch.Generator().manual_seed(8)
    for D in (3072, 5120):
        x = torch.randn(1, 1027, D, generator=g).bfloat16()
        mod = torch.randn(1, 2 * D, generator=g).bfloat16()
        sc, sh = mod.chunk(2, dim=1)
        want = O.layer_norm_modulate(x, sc[:, None], sh[:, None], 1e-6)
        md = mod.to(dev)
        scd, shd = md.chunk(2, dim=1)
        y, q, qs = ops.adaln_modulate(x.to(dev), scd, shd, want_bf16=True, want_fp8=True)
        frac, rel = _ulp_report(y.cpu(), want)
        assert frac < 1e-3 and rel <= 2 ** -6, (D, frac, rel)
        wq, ws = ofp8.quantize_rowwise(y.cpu().reshape(-1, D), scaled=True)
        assert torch.equal(qs.cpu(), ws) and torch.equal(q.cpu().view(torch.uint8).reshape(-1, D), wq.view(torch.uint8))


def test_adaln_two_wavefronts_per_row_path(dev):
    """Rows between 4096 and 5120 wide with at least 2048 of them go two to a workgroup (a pair of wavefronts
    each): an odd row count leaves the last workgroup's second row slot without a row, and 4608 columns leave
    chunk slots past the end of the row."""
    from diffsynth_engine_amd import ops

    g = torch.Generator().manual_seed(14)
    for D in (5120, 4608):
        x = torch.randn(1, 2049, D, generator=g).bfloat16()
        mod = torch.randn(1, 2 * D, generator=g).bfloat16()
        sc, sh = mod.chunk(2, dim=1)
        want = O.layer_norm_modulate(x, sc[:, None], sh[:, None], 1e-6)
        md = mod.to(dev)
        scd, shd = md.chunk(2, dim=1)
        y, q, qs = ops.adaln_modulate(x.to(dev), scd, shd, want_bf16=True, want_fp8=True)
        frac, rel = _ulp_report(y.cpu(), want)
        assert frac < 1e-3 and rel <= 2 ** -6, (D, frac, rel)
        wq, ws = ofp8.quantize_rowwise(y.cpu().reshape(-1, D), scaled=True)
        assert torch.equal(qs.cpu(), ws) and torch.equal(q.cpu().view(torch.uint8).reshape(-1, D), wq.view(torch.uint8))


def test_empty_inputs_are_accepted(dev):
    """Zero rows are a valid (empty) workload for every row kernel and for the GEMM: nothing is launched and
    an empty output comes back (the reference's torch ops accept empty batches the same way)."""
    from diffsynth_engine_amd import ops

    x = torch.zeros(0, 3072, dtype=torch.bfloat16, device=dev)
    q, s = ops.quantize_fp8(x, scaled=True)
    assert q.shape == (0, 3072) and s.shape == (0,)
    w = torch.zeros(256, 3072, dtype=torch.bfloat16, device=dev)
    wq, ws = ops.quantize_weight_fp8(w)
    assert ops.fp8_gemm(q, wq, s, ws, None).shape == (0, 256)
    assert ops.gelu_tanh(x).shape == (0, 3072)
    mod = torch.zeros(1, 3072, dtype=torch.bfloat16, device=dev)
    assert ops.adaln_modulate(x.view(1, 0, 3072), mod, mod, 1e-6).shape == (1, 0, 3072)


def test_fused_kernels_emit_the_bare_cast_without_a_scale(dev):
    """``scaled=False`` (no q_scale): the e4m3 output of AdaLN-modulate, GELU and concat-GELU is the reference's bare
    cast of their bf16 output (utils/fp8_linear.py:35), bit for bit what the stand-alone cast kernel gives, NaN
    codes beyond the format's range included."""
    from diffsynth_engine_amd import ops

    g = torch.Generator().manual_seed(21)
    for rows, D in ((300, 3072), (77, 1024), (40, 5120)):
        x = (torch.randn(1, rows, D, generator=g) * 3).bfloat16().to(dev)
        x[0, 0, :8] = torch.tensor([600.0, -600.0, 470.0, 460.0, 448.0, 1e-3, -0.0, 2e-3]).bfloat16()  # around the edges
        scale = (torch.randn(1, D, generator=g) * 2).bfloat16().to(dev)
        shift = (torch.randn(1, D, generator=g) * 50).bfloat16().to(dev)
        y = ops.adaln_modulate(x, scale, shift, 1e-6)
        q, qs = ops.adaln_modulate(x, scale, shift, 1e-6, want_bf16=False, want_fp8=True, scaled=False)
        want, _ = ops.quantize_fp8(y.view(rows, D), scaled=False)
        assert qs is None and torch.equal(q.view(rows, D).view(torch.uint8), want.view(torch.uint8))
        big = (x.view(rows, D).float() * 200).bfloat16()   # GELU keeps large positive values: some exceed 448
        yg = ops.gelu_tanh(big)
        qg, qsg = ops.gelu_tanh(big, want_bf16=False, want_fp8=True, scaled=False)
        wantg, _ = ops.quantize_fp8(yg, scaled=False)
        assert qsg is None and torch.equal(qg.view(torch.uint8), wantg.view(torch.uint8))
        assert (wantg.view(torch.uint8) & 0x7F == 0x7F).any()  # the NaN code occurs in this set-up
        pre = (torch.randn(rows, 256, generator=g) * 100).bfloat16().to(dev)
        yc = ops.concat_gelu_tanh(pre, big, want_bf16=True, want_fp8=False)
        qc, qsc = ops.concat_gelu_tanh(pre, big, want_fp8=True, scaled=False)
        wantc, _ = ops.quantize_fp8(yc, scaled=False)
        assert qsc is None and torch.equal(qc.view(torch.uint8), wantc.view(torch.uint8))
