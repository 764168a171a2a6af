"""GPU parity at the sizes the benchmark configurations name, one test group per configuration:

  configs[0]  one Flux joint block at 1024 image + 256 text tokens against the CPU oracle;
  configs[2]  joint attention at S = 4608 x 24 heads with q/k RMSNorm and the 3-axis RoPE requested from the
              attention entry point, against fp32 SDPA of the normalised / rotated operands;
  configs[3]  every one of the 19 + 38 blocks of the benchmark's step, teacher-forced (each block is fed the
              oracle's own input, so nothing is carried from block to block);
  configs[4]  one Wan2.1-14B block at 32 760 video + 512 text tokens, its three GEMM shapes and its row kernels
              at that row count.

Where the CPU would need minutes the oracle's functions are evaluated by torch on the device (same code, same
rounding points); attention errors are per query row (conftest.row_rel_err).
"""
import math

import pytest
import torch

from conftest import row_rel_err
from oracle import dit_ops as O
from oracle import flux as oflux
from oracle import fp8 as ofp8
from oracle import wan as ow

pytestmark = pytest.mark.gpu


def _cos(a, b):
    return torch.nn.functional.cosine_similarity(a.float().flatten().cpu(), b.float().flatten().cpu(), dim=0).item()


# ------------------------------------------------------------------------------------------------ configs[0]
def test_config0_joint_block_at_1024_image_and_256_text_tokens(dev):
    """BASELINE configs[0]: hidden 3072, 24 heads, 512 x 512 image -> 1024 image tokens + 256 text tokens, RoPE axes
    (16,56,56).  The HIP block against (i) the CPU oracle in the arithmetic the block runs in (scaled e4m3
    linears, bf16), held to the teacher-forced bar, and (ii) the configuration as written - the same block in fp32
    on the CPU with torch SDPA - which differs by the quantisation itself."""
    from diffsynth_engine_amd import ops
    from diffsynth_engine_amd.flux_dit import FluxDiTRunner

    sd = oflux.init_params(1, 0, dtype=torch.bfloat16, seed=0)
    g = torch.Generator().manual_seed(0)
    St, side = 256, 32
    img = torch.randn(1, side * side, 3072, generator=g).bfloat16()
    txt = torch.randn(1, St, 3072, generator=g).bfloat16()
    cond = torch.randn(1, 3072, generator=g).bfloat16()
    ids = torch.cat([torch.zeros(1, St, 3), oflux.image_ids(2 * side, 2 * side, 1, "cpu", torch.float32)], dim=1)
    freqs = O.rope_table(ids, oflux.AXES_DIM, oflux.THETA)
    want_a, want_b = oflux.joint_block(oflux.Params(sd, "fp8_scaled"), 0, img, txt, cond, freqs)
    sd32 = {k: v.float() for k, v in sd.items()}
    f32_a, f32_b = oflux.joint_block(oflux.Params(sd32, "plain"), 0, img.float(), txt.float(), cond.float(), freqs,
                                     attn=torch.nn.functional.scaled_dot_product_attention)
    R = FluxDiTRunner(sd, 1, 0, scaled=True, device=dev)
    mods = R._modulations(cond.to(dev))
    got_a, got_b = R._joint_block(0, img.to(dev), txt.to(dev), mods["blocks.0.norm1_a.linear"],
                                  mods["blocks.0.norm1_b.linear"], ops.rope_table_from_freqs(freqs).to(dev))
    assert _cos(got_a, want_a) >= 0.9995 and _cos(got_b, want_b) >= 0.9995, (_cos(got_a, want_a), _cos(got_b, want_b))
    # against fp32: what e4m3 operands cost (about 5 % of noise per Linear); the kernels may not pay more for it
    # than the oracle's fp8 mode does
    for got, want, f32 in ((got_a, want_a, f32_a), (got_b, want_b, f32_b)):
        assert _cos(got, f32) >= 0.99 and _cos(got, f32) >= _cos(want, f32) - 1e-3, (_cos(got, f32), _cos(want, f32))


# ------------------------------------------------------------------------------------------------ configs[2]
def _flux_rope_4608(dev):
    ids = torch.cat([torch.zeros(1, 512, 3), oflux.image_ids(128, 128, 1, "cpu", torch.float32)], dim=1)
    return O.rope_table(ids, oflux.AXES_DIM, oflux.THETA).to(dev)


@pytest.mark.parametrize("static_scratch", [False, True])
@pytest.mark.parametrize("wstd", [0.0, 0.1])
def test_config2_joint_attention_with_rmsnorm_and_rope_at_full_size(dev, wstd, static_scratch):
    """BASELINE configs[2] as written: B 1, H 24, D 128, S 4608 (512 text rows at position 0, then 64 x 64 image
    positions), q/k/v N(0,1), RMSNorm on q and k (weights 1, and N(1, 0.1)), RoPE (16,56,56) applied by the
    attention call, scale 1/sqrt(128).  Reference: fp32 SDPA (torch, on the device) of the operands the oracle's
    rms_norm / apply_rope produce in bf16.  Bar: 2e-2 per query row.  Both entry points (caller scratch and the
    library's static scratch)."""
    from diffsynth_engine_amd import ops

    H, S = 24, 4608
    g = torch.Generator(device=dev).manual_seed(0)
    q, k, v = [torch.randn(1, H, S, 128, generator=g, device=dev, dtype=torch.bfloat16) for _ in range(3)]
    wq = (1 + wstd * torch.randn(128, generator=g, device=dev)).bfloat16()
    wk = (1 + wstd * torch.randn(128, generator=g, device=dev)).bfloat16()
    freqs = _flux_rope_4608(dev)
    qn = O.apply_rope(O.rms_norm(q, wq, 1e-6), freqs)
    kn = O.apply_rope(O.rms_norm(k, wk, 1e-6), freqs)
    got = ops.attention_bhsd(q, k, v, rope=ops.rope_table_from_freqs(freqs), q_norm_w=wq, k_norm_w=wk,
                             static_scratch=static_scratch)
    worst = 0.0
    for h0 in range(0, H, 6):  # fp32 scores of 6 heads at a time: 0.5 GB
        want = O.sdpa(qn[:, h0:h0 + 6].float(), kn[:, h0:h0 + 6].float(), v[:, h0:h0 + 6].float())
        worst = max(worst, row_rel_err(got[:, h0:h0 + 6], want))
    assert worst <= 2e-2, worst
    # the caller's bound on the scores (what the Flux runner derives from the norm weights) must not change a bit
    bound = 1.02 * math.sqrt(128) * float(wq.float().abs().max()) * float(wk.float().abs().max())
    same = ops.attention_bhsd(q, k, v, rope=ops.rope_table_from_freqs(freqs), q_norm_w=wq, k_norm_w=wk,
                              score_bound=bound, static_scratch=static_scratch)
    assert torch.equal(got, same)


# ------------------------------------------------------------------------------------------------ configs[3]
def test_config3_every_block_of_the_full_step_teacher_forced(dev):
    """The benchmark's model (19 + 38 blocks, weights as bench.py draws them) at 4096 image + 512 text tokens.
    The oracle's FluxDiT.forward is walked block by block on the device; every block of the runner is fed the
    ORACLE's input for that block and its output is compared with the oracle's: 57 checks at the one-block bar
    (cosine >= 0.9995; a block holds 4-5 chained e4m3 quantisations), none of which inherits the chaotic
    amplification of the chained scaled-fp8 step.  A wiring or indexing mistake in any block, at any depth,
    fails its own check."""
    from bench import flux_state_dict_stream
    from diffsynth_engine_amd import ops
    from diffsynth_engine_amd.flux_dit import FluxDiTRunner

    nd, ns = 19, 38
    sd = dict(flux_state_dict_stream(nd, ns, dev, seed=0))
    R = FluxDiTRunner(sd, nd, ns, scaled=True, device=dev)
    P = oflux.Params(sd, "fp8_scaled")
    g = torch.Generator(device=dev).manual_seed(1)
    St, side = 512, 64
    img = torch.randn(1, side * side, 3072, generator=g, device=dev).bfloat16()
    txt = torch.randn(1, St, 3072, generator=g, device=dev).bfloat16()
    cond = torch.randn(1, 3072, generator=g, device=dev).bfloat16()
    freqs = _flux_rope_4608(dev)
    rope = ops.rope_table_from_freqs(freqs)
    mods = R._modulations(cond)
    worst = (1.0, "")
    for i in range(nd):
        want_a, want_b = oflux.joint_block(P, i, img, txt, cond, freqs)
        got_a, got_b = R._joint_block(i, img, txt, mods[f"blocks.{i}.norm1_a.linear"],
                                      mods[f"blocks.{i}.norm1_b.linear"], rope)
        ca, cb = _cos(got_a, want_a), _cos(got_b, want_b)
        assert ca >= 0.9995 and cb >= 0.9995, ("joint block", i, ca, cb)
        worst = min(worst, (min(ca, cb), f"blocks.{i}"))
        img, txt = want_a, want_b  # the next block's input is the oracle's output
        P._q.clear()               # (the oracle's cache of quantised weights: one block at a time)
    x = torch.cat([txt, img], dim=1)
    for i in range(ns):
        want = oflux.single_block(P, i, x, cond, freqs)
        got = R._single_block(i, x, mods[f"single_blocks.{i}.norm.linear"], rope)
        c = _cos(got, want)
        assert c >= 0.9995, ("single block", i, c)
        worst = min(worst, (c, f"single_blocks.{i}"))
        x = want
        P._q.clear()
    assert torch.isfinite(x.float()).all().item()
    print("worst teacher-forced block: %.6f (%s)" % worst)


# ------------------------------------------------------------------------------------------------ configs[4]
WAN_S, WAN_D, WAN_F = 32760, 5120, 13824  # 21 x 30 x 52 patches of the 21 x 60 x 104 latent


def _sdpa_by_heads(q, k, v, heads_per_pass=4):
    """O.sdpa a few heads at a time: the fp32 scores of all 40 heads at 32 760 tokens would be 172 GB."""
    return torch.cat([O.sdpa(q[:, h:h + heads_per_pass], k[:, h:h + heads_per_pass], v[:, h:h + heads_per_pass])
                      for h in range(0, q.shape[1], heads_per_pass)], dim=1)


def test_config4_wan_block_at_32760_video_and_512_text_tokens(dev):
    """BASELINE configs[4], one DiTBlock (wan_dit.py:185-193) at the 14B width and the full token count, fed the same
    input as the oracle's dit_block evaluated by torch on the device: self-attention over 32 760 tokens with the
    3-axis RoPE, cross-attention to 512 text tokens, FFN 13 824.  Cosine >= 0.9995 as for a Flux block."""
    from bench import wan_state_dict_stream
    from diffsynth_engine_amd.wan_dit import WanDiTRunner

    cfg = dict(ow.config_14b(), num_layers=1)
    sd = dict(wan_state_dict_stream(cfg, dev, seed=3))
    g = torch.Generator(device=dev).manual_seed(4)
    f, h, w = 21, 30, 52
    x = torch.randn(1, WAN_S, WAN_D, generator=g, device=dev).bfloat16()
    ctx = torch.randn(1, 512, WAN_D, generator=g, device=dev).bfloat16()
    t_mod = (torch.randn(1, 6, WAN_D, generator=g, device=dev) * 0.3).bfloat16()
    R = WanDiTRunner(sd, cfg, scaled=True, device=dev)
    got = R.block(0, x, ctx, t_mod, R.rope_table(f, h, w))
    assert torch.isfinite(got.float()).all().item()
    want = ow.dit_block(ow.Params(sd, "fp8_scaled"), 0, x, ctx, t_mod, ow.freqs_cis_3d(128, f, h, w).to(dev), cfg,
                        attn=_sdpa_by_heads)
    c = _cos(got, want)
    assert c >= 0.9995, c
    # the block must have changed its input by more than the tolerance, or the check above says nothing
    assert _cos(got, x) < 0.99


@pytest.mark.parametrize("K,N", [(WAN_D, WAN_D), (WAN_D, WAN_F), (WAN_F, WAN_D)])
def test_config4_gemm_shapes_at_32760_rows(dev, K, N):
    """The three Linear shapes of a Wan2.1-14B block at M = 32 760 (a ragged last tile row: 32 760 = 127 x 256 + 248;
    N = 13 824 = 54 tiles): a 256-row slice recomputed alone is bit-identical, doubling the activation scales doubles
    the output exactly, cosine >= 0.9995 and every element within bf16 rounding of the dequantised fp32 product on
    two row slices, and the gated-residual epilogue equals the oracle's bf16 op sequence on a slice."""
    from diffsynth_engine_amd import ops

    M = WAN_S
    g = torch.Generator(device=dev).manual_seed(K + N)
    x = torch.randn(M, K, generator=g, device=dev, dtype=torch.bfloat16)
    x[:, torch.randperm(K, generator=g, device=dev)[: max(1, -(-K // 1000))]] *= 20
    w = (torch.randn(N, K, generator=g, device=dev) * 0.02).to(torch.bfloat16)
    bias = torch.randn(N, generator=g, device=dev).to(torch.bfloat16)
    wq, ws = ops.quantize_weight_fp8(w)
    xq, xs = ops.quantize_fp8(x)
    full = ops.fp8_gemm(xq, wq, xs, ws, bias)
    for r0 in (1024, M - 248):  # an interior tile row and the ragged last one
        r1 = min(r0 + 256, M)
        part = ops.fp8_gemm(xq[r0:r1], wq, xs[r0:r1], ws, bias)
        assert torch.equal(full[r0:r1], part), r0
        ref = ofp8.scaled_linear(xq[r0:r1], xs[r0:r1], wq, ws, bias, out_dtype=torch.float32)
        assert _cos(full[r0:r1], ref) >= 0.9995
        assert bool(((full[r0:r1].float() - ref).abs() <= ref.abs() * 2 ** -8 + 1e-3).all())
        # quantiser codes and scales of the slice against the oracle's definition
        # (on the CPU: torch's device division by 448 is a multiplication by a reciprocal, one ulp off now and then)
        oq, osc = ofp8.quantize_rowwise(x[r0:r1].cpu())
        assert torch.equal(xq[r0:r1].cpu().view(torch.uint8), oq.view(torch.uint8)) and torch.equal(xs[r0:r1].cpu(), osc)
    plain = ops.fp8_gemm(xq, wq, xs, ws, None)
    doubled = ops.fp8_gemm(xq, wq, xs * 2, ws, None)
    assert torch.equal(doubled.float(), plain.float() * 2)
    if N == WAN_D:  # the projections whose output enters a gated residual (self_attn.o, ffn.2)
        resid = torch.randn(M, N, generator=g, device=dev, dtype=torch.bfloat16)
        gate = torch.randn(1, N, generator=g, device=dev, dtype=torch.bfloat16)
        fused = ops.fp8_gemm(xq, wq, xs, ws, bias, resid=resid, gate=gate, rows_per_batch=M)
        r0, r1 = M - 600, M
        want = O.gated_residual(resid[r0:r1], full[r0:r1], gate)
        assert torch.equal(fused[r0:r1], want)


def test_config4_row_kernels_at_32760_rows(dev):
    """AdaLN-modulate (bf16 and e4m3 emission), full-width RMSNorm + RoPE and GELU with e4m3 emission on
    32 760 x 5120 (GELU: x 13 824) buffers; the oracle is evaluated on row slices at the start, across a
    workgroup-pair boundary in the middle and at the very end."""
    from diffsynth_engine_amd import ops

    S, D = WAN_S, WAN_D
    g = torch.Generator(device=dev).manual_seed(7)
    x = (torch.randn(1, S, D, generator=g, device=dev) * 2).bfloat16()
    sc, sh = [(torch.randn(1, D, generator=g, device=dev) * 0.3).bfloat16() for _ in range(2)]
    slices = [(0, 300), (16383, 16700), (S - 257, S)]
    y = ops.adaln_modulate(x, sc, sh, 1e-6)
    yq, ys = ops.adaln_modulate(x, sc, sh, 1e-6, want_bf16=False, want_fp8=True)
    for r0, r1 in slices:
        want = O.layer_norm_modulate(x[:, r0:r1], sc[:, None], sh[:, None], 1e-6)
        d = (y[:, r0:r1].float() - want.float()).abs()
        assert d.max().item() <= 2 ** -6 * want.float().abs().max().item()
        assert (d > want.float().abs() * 2 ** -7 + 1e-6).float().mean().item() < 2e-3
        # the emitted codes are the quantisation of the kernel's own bf16 rows
        oq, osc = ofp8.quantize_rowwise(y[0, r0:r1].cpu())  # (CPU: see the GEMM test above)
        assert torch.equal(yq[0, r0:r1].cpu().view(torch.uint8), oq.view(torch.uint8)) and torch.equal(ys[r0:r1].cpu(), osc)
    w = (1 + 0.1 * torch.randn(D, generator=g, device=dev)).bfloat16()
    fr = ow.freqs_cis_3d(128, 21, 30, 52).to(dev)
    table = torch.stack((fr.real, fr.imag), dim=-1).float().reshape(1, S, 64, 2)
    got = ops.rmsnorm_rows(x, w, 1e-6, table)
    for r0, r1 in slices:
        want = ow.rope_apply(ow.wan_rms_norm(x[:, r0:r1], w, 1e-6), fr[r0:r1], 40)
        d = (got[:, r0:r1].float() - want.float()).abs()
        assert d.max().item() <= 2 ** -5 * want.float().abs().max().item()
        assert (d > want.float().abs() * 2 ** -7 + 1e-6).float().mean().item() < 2e-3
    hbuf = torch.randn(S, WAN_F, generator=g, device=dev).bfloat16()
    gq, gs = ops.gelu_tanh(hbuf, want_bf16=False, want_fp8=True)
    gy = ops.gelu_tanh(hbuf)
    for r0, r1 in slices:
        want = O.gelu_tanh(hbuf[r0:r1])
        d = (gy[r0:r1].float() - want.float()).abs()
        assert d.max().item() <= 2 ** -7 * max(want.float().abs().max().item(), 1.0)
        oq, osc = ofp8.quantize_rowwise(gy[r0:r1].cpu())
        assert torch.equal(gq[r0:r1].cpu().view(torch.uint8), oq.view(torch.uint8)) and torch.equal(gs[r0:r1].cpu(), osc)
