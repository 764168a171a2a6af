"""GPU parity: e4m3 quantisation (bit-exact) and the FP8 scaled GEMM, through the C-ABI."""
import pytest
import torch

from oracle import fp8 as ofp8

pytestmark = pytest.mark.gpu


def _all_bf16(dev):
    bits = torch.arange(0, 65536, dtype=torch.int32).to(torch.int16)
    return bits.view(torch.bfloat16).to(dev)


def test_bare_cast_bit_exact_all_bf16(dev):
    """Every bf16 bit pattern through the unscaled row quantiser == torch's cast (fp8_linear.py:35)."""
    from diffsynth_engine_amd import ops

    x = _all_bf16(dev).view(64, 1024)
    q, s = ops.quantize_fp8(x, scaled=False)
    assert s is None
    want = x.cpu().to(torch.float8_e4m3fn)
    got, want = q.cpu().view(torch.uint8), want.view(torch.uint8)
    # NaN payload sign may differ only for NaN inputs; compare NaN-ness there, bits elsewhere
    nan_in = torch.isnan(x.cpu().float())
    assert torch.equal(got[~nan_in], want[~nan_in])
    assert bool(((got[nan_in] & 0x7F) == 0x7F).all())


@pytest.mark.parametrize("M,K", [(1, 64), (7, 3072), (130, 12288), (33, 4096), (5, 16384), (3, 8)])
def test_rowwise_scaled_quant_bit_exact(dev, M, K):
    from diffsynth_engine_amd import ops

    g = torch.Generator().manual_seed(M * 1000 + K)
    x = torch.randn(M, K, generator=g)
    x[:, :: max(K // 7, 1)] *= 20.0
    if M > 2:
        x[2] = 0.0  # all-zero row: scale clamps at 1e-12/448
    x = x.bfloat16()
    q, s = ops.quantize_fp8(x.to(dev), scaled=True)
    wq, ws = ofp8.quantize_rowwise(x, scaled=True)
    assert torch.equal(s.cpu(), ws)
    assert torch.equal(q.cpu().view(torch.uint8), wq.view(torch.uint8))


def test_rowwise_quant_strided_rows(dev):
    from diffsynth_engine_amd import ops

    x = torch.randn(16, 512).bfloat16()
    xs = x.to(dev)[:, 128:384]
    q, s = ops.quantize_fp8(xs, scaled=True)
    wq, ws = ofp8.quantize_rowwise(x[:, 128:384], scaled=True)
    assert torch.equal(s.cpu(), ws) and torch.equal(q.cpu().view(torch.uint8), wq.view(torch.uint8))


def test_weight_quant_matches_oracle(dev):
    from diffsynth_engine_amd import ops

    for dtype in (torch.bfloat16, torch.float32):
        w = (torch.randn(300, 200) * 0.02).to(dtype)
        q, s = ops.quantize_weight_fp8(w.to(dev), scaled=True)
        wq, ws = ofp8.quantize_weight(w, scaled=True)
        assert torch.equal(s.cpu(), ws)
        assert torch.equal(q.cpu().view(torch.uint8), wq.view(torch.uint8))
        q, s = ops.quantize_weight_fp8(w.to(dev), scaled=False)
        assert s is None and torch.equal(q.cpu().view(torch.uint8), w.to(torch.float8_e4m3fn).view(torch.uint8))


def _gemm_case(dev, M, N, K, seed, bias=True, scaled=True):
    from diffsynth_engine_amd import ops

    g = torch.Generator().manual_seed(seed)
    w = torch.randn(N, K, generator=g) * 0.02
    x = torch.randn(M, K, generator=g)
    x[:, torch.randperm(K, generator=g)[: max(K // 1000, 1)]] *= 20.0
    x = x.bfloat16()
    b = torch.randn(N, generator=g).bfloat16() if bias else None
    wq, ws = ofp8.quantize_weight(w, scaled=scaled)
    xq, xs = ofp8.quantize_rowwise(x, scaled=scaled)
    want = ofp8.scaled_linear(xq, xs, wq, ws, b)
    got = ops.fp8_gemm(xq.to(dev), wq.to(dev), None if xs is None else xs.to(dev),
                       None if ws is None else ws.to(dev), None if b is None else b.to(dev)).cpu()
    return got.float(), want.float()


@pytest.mark.parametrize("M,N,K", [(256, 256, 128), (256, 256, 3072), (512, 768, 256), (300, 200, 64),
                                   (1000, 3072, 1024), (17, 64, 3072), (9, 264, 16), (257, 513, 144)])
def test_fp8_gemm_matches_dequantised_matmul(dev, M, N, K):
    got, want = _gemm_case(dev, M, N, K, seed=M + N + K)
    cos = torch.nn.functional.cosine_similarity(got.flatten(), want.flatten(), dim=0).item()
    assert cos >= 0.9995, cos
    # fp32 accumulation of exact e4m3 products: only summation order differs, so far tighter than the cosine bar
    err = (got - want).abs().max().item()
    assert err <= 2e-2 * want.abs().max().item() + 1e-3, err


@pytest.mark.parametrize("M", [1, 2, 8])
def test_fp8_gemv_small_m(dev, M):
    got, want = _gemm_case(dev, M, 515, 3072, seed=M)
    assert (got - want).abs().max().item() <= 2e-2 * want.abs().max().item() + 1e-3


def test_fp8_gemm_unit_scales_no_bias(dev):
    """Reference mode (fp8_linear.py:41-48): scale_a = scale_b = 1, bare casts."""
    got, want = _gemm_case(dev, 384, 512, 512, seed=5, bias=False, scaled=False)
    assert (got - want).abs().max().item() <= 2e-2 * want.abs().max().item() + 1e-3


def test_fp8_gemm_exact_on_small_integers(dev):
    """Operands that are small integers make every partial sum exact: the result must be bit-identical."""
    from diffsynth_engine_amd import ops

    g = torch.Generator().manual_seed(0)
    a = torch.randint(-3, 4, (512, 256), generator=g).float()
    w = torch.randint(-2, 3, (320, 256), generator=g).float()
    want = (a @ w.t()).bfloat16()
    got = ops.fp8_gemm(a.to(torch.float8_e4m3fn).to(dev), w.to(torch.float8_e4m3fn).to(dev)).cpu()
    assert torch.equal(got, want)


def test_gemm_rejects_bad_arguments(dev):
    from diffsynth_engine_amd import ops

    a = torch.zeros(16, 24, dtype=torch.float8_e4m3fn, device=dev)
    w = torch.zeros(16, 24, dtype=torch.float8_e4m3fn, device=dev)
    with pytest.raises(ValueError):
        ops.fp8_gemm(a, w)  # K % 16 != 0
    with pytest.raises(ValueError):
        ops.fp8_gemm(a.bfloat16(), w)


@pytest.mark.parametrize("M,N,K,B", [(512, 768, 256, 2), (300, 3072, 1024, 1), (260, 200, 128, 2), (96, 100, 64, 1)])
def test_fp8_gemm_fused_gated_residual(dev, M, N, K, B):
    """out = resid + gate * linear(x) with the gate row chosen per batch entry (flux_dit.py:227,318-319):
    the fused epilogue must reproduce the three bf16 roundings of the separate ops."""
    from diffsynth_engine_amd import ops

    g = torch.Generator().manual_seed(M + N)
    w = torch.randn(N, K, generator=g) * 0.02
    x = torch.randn(M, K, generator=g).bfloat16()
    b = torch.randn(N, generator=g).bfloat16()
    resid = torch.randn(M, N, generator=g).bfloat16()
    gate = torch.randn(B, N, generator=g).bfloat16()
    wq, ws = ofp8.quantize_weight(w)
    xq, xs = ofp8.quantize_rowwise(x)
    proj = ofp8.scaled_linear(xq, xs, wq, ws, b)
    rows = M // B
    assert rows * B == M
    want = resid + gate.repeat_interleave(rows, dim=0) * proj
    args = (xq.to(dev), wq.to(dev), xs.to(dev), ws.to(dev), b.to(dev))
    got = ops.fp8_gemm(*args, resid=resid.to(dev), gate=gate.to(dev), rows_per_batch=rows).cpu()
    plain = ops.fp8_gemm(*args).cpu()
    # identical to applying the oracle's residual arithmetic to the kernel's own projection ...
    assert torch.equal(got, resid + gate.repeat_interleave(rows, dim=0) * plain)
    # ... and within accumulation-order noise of the all-oracle result
    assert (got.float() - want.float()).abs().max().item() <= 2e-2 * want.float().abs().max().item()
    want_nogate = resid + plain
    assert torch.equal(ops.fp8_gemm(*args, resid=resid.to(dev)).cpu(), want_nogate)
    # in place on the residual buffer
    r_dev = resid.to(dev)
    ops.fp8_gemm(*args, resid=r_dev, gate=gate.to(dev), rows_per_batch=rows, out=r_dev)
    assert torch.equal(r_dev.cpu(), got)


def test_fp8_gemv_rowscale_stacks_linears(dev):
    """Three Linear layers with their own per-tensor scales evaluated as one stacked product == three products."""
    from diffsynth_engine_amd import ops

    g = torch.Generator().manual_seed(3)
    K = 3072
    x = torch.randn(2, K, generator=g).bfloat16()
    xq, xs = ofp8.quantize_rowwise(x)
    ws, ss, bs, want = [], [], [], []
    for n, std in ((515, 0.02), (64, 0.5), (1030, 0.003)):
        w = torch.randn(n, K, generator=g) * std
        b = torch.randn(n, generator=g).bfloat16()
        wq, s = ofp8.quantize_weight(w)
        ws.append(wq); ss.append(s.expand(n)); bs.append(b)
        want.append(ofp8.scaled_linear(xq, xs, wq, s, b))
    got = ops.fp8_gemv_rowscale(xq.to(dev), torch.cat(ws).to(dev), xs.to(dev), torch.cat(ss).contiguous().to(dev),
                                torch.cat(bs).to(dev)).cpu()
    want = torch.cat(want, dim=1)
    assert (got.float() - want.float()).abs().max().item() <= 1e-2 * want.float().abs().max().item()


def _rand_problem(dev, g, M, N, K, resid=False, bias=True):
    w = torch.randn(N, K, generator=g) * 0.02
    x = torch.randn(M, K, generator=g).bfloat16()
    wq, ws = ofp8.quantize_weight(w)
    xq, xs = ofp8.quantize_rowwise(x)
    kw = dict(a_q=xq.to(dev), w_q=wq.to(dev), a_scale=xs.to(dev), w_scale=ws.to(dev),
              bias=torch.randn(N, generator=g).bfloat16().to(dev) if bias else None)
    if resid:
        kw.update(resid=torch.randn(M, N, generator=g).bfloat16().to(dev),
                  gate=torch.randn(1, N, generator=g).bfloat16().to(dev), rows_per_batch=M)
    return kw


@pytest.mark.parametrize("shapes,resid", [
    ([(1024, 768, 256), (512, 768, 256)], False),        # image + text stream, same weights' shape
    ([(1024, 512, 384), (130, 1024, 128)], True),        # different N and K, ragged M, fused residual
    ([(300, 520, 256), (4, 256, 128), (700, 264, 144), (257, 256, 128)], False),   # gemv + generic-kernel members
    ([(512, 256, 128)], True),
])
def test_fp8_gemm_grouped_equals_separate_launches(dev, shapes, resid):
    """Problems submitted together give bit-identical results to one dsx_fp8_gemm(_gated_residual) call each,
    whether neighbours share a launch, fall to the small-M or generic kernel, or stand alone."""
    from diffsynth_engine_amd import ops

    g = torch.Generator().manual_seed(len(shapes) * 17 + shapes[0][0])
    probs = [_rand_problem(dev, g, M, N, K, resid=resid and M > 8) for (M, N, K) in shapes]
    want = [ops.fp8_gemm(**p).cpu() for p in probs]
    got = ops.fp8_gemm_grouped(probs)
    assert len(got) == len(want)
    for a, b in zip(got, want):
        assert torch.equal(a.cpu(), b)
    # mixed residual / no residual neighbours must not be paired, and still be right
    if len(shapes) >= 2:
        mixed = [_rand_problem(dev, g, 512, 256, 128, resid=True), _rand_problem(dev, g, 256, 512, 128, resid=False)]
        for a, p in zip(ops.fp8_gemm_grouped(mixed), mixed):
            assert torch.equal(a.cpu(), ops.fp8_gemm(**p).cpu())


def test_fp8_gemm_grouped_rejects_bad_arguments(dev):
    from diffsynth_engine_amd import ops

    g = torch.Generator().manual_seed(3)
    ok = _rand_problem(dev, g, 64, 64, 64)
    with pytest.raises(ValueError):
        ops.fp8_gemm_grouped([])
    with pytest.raises(ValueError):
        ops.fp8_gemm_grouped([ok] * 5)
    bad = dict(ok)
    bad["gate"] = torch.ones(1, 64, dtype=torch.bfloat16, device=dev)   # gate without residual
    with pytest.raises(ValueError):
        ops.fp8_gemm_grouped([ok, bad])


@pytest.mark.parametrize("M,heads,extra,batch,use_rope,use_norm", [
    (4608, 24, 3072, 1, True, True),     # a Flux joint-block qkv projection: [q | k | v]
    (1000, 2, 256 + 1024, 1, True, True),  # ragged last tile row; [q | k | v | mlp] like the single block
    (600, 3, 384, 2, True, True),        # two batch entries of 300 tokens: the table row restarts at 300
    (300, 2, 256, 1, False, True),       # RMSNorm only
    (300, 2, 256, 1, True, False),       # RoPE only
])
def test_qk_epilogue_equals_the_in_place_row_kernel(dev, M, heads, extra, batch, use_rope, use_norm):
    """The qkv GEMM whose epilogue normalises and rotates the q and k heads == the plain GEMM followed by
    dsx_rmsnorm_rope_qk in place on its output, bit for bit; v (and mlp) columns untouched."""
    from diffsynth_engine_amd import ops

    K, N = 512, 2 * heads * 128 + extra
    g = torch.Generator().manual_seed(M + heads)
    x = torch.randn(M, K, generator=g).bfloat16().to(dev)
    w = (torch.randn(N, K, generator=g) * 0.05).bfloat16().to(dev)
    bias = torch.randn(N, generator=g).bfloat16().to(dev)
    S, pos0 = M // batch, 7
    rope = None
    if use_rope:
        ang = torch.rand(batch, pos0 + S, 64, generator=g) * 6.28
        rope = torch.stack((torch.cos(ang), torch.sin(ang)), dim=-1).float().to(dev)
    wq = (1 + 0.2 * torch.randn(128, generator=g)).bfloat16().to(dev) if use_norm else None
    wk = (1 + 0.2 * torch.randn(128, generator=g)).bfloat16().to(dev) if use_norm else None
    wq8, ws = ops.quantize_weight_fp8(w)
    xq, xs = ops.quantize_fp8(x)
    plain = ops.fp8_gemm(xq, wq8, xs, ws, bias)
    want = ops.rmsnorm_rope_qk(plain.clone().view(batch, S, N), heads, heads, wq, wk, rope, pos0=pos0).view(M, N)
    got = ops.fp8_gemm(xq, wq8, xs, ws, bias, rows_per_batch=S,
                       qk=dict(heads=heads, q_norm_w=wq, k_norm_w=wk, rope=rope, pos0=pos0, eps=1e-6))
    assert torch.equal(got, want)
    assert torch.equal(got[:, 2 * heads * 128:], plain[:, 2 * heads * 128:])
    assert not torch.equal(got[:, : 2 * heads * 128], plain[:, : 2 * heads * 128])


def test_qk_epilogue_on_a_grouped_text_and_image_pair(dev):
    """Two problems in one launch, each with its own norm weights and its own first RoPE row (text rows first, then
    image rows), as the joint block submits them."""
    from diffsynth_engine_amd import ops

    heads, K, St, Si = 2, 256, 40, 300
    N = 3 * heads * 128
    g = torch.Generator().manual_seed(3)
    ang = torch.rand(1, St + Si, 64, generator=g) * 6.28
    rope = torch.stack((torch.cos(ang), torch.sin(ang)), dim=-1).float().to(dev)
    probs, wants = [], []
    for rows, pos0 in ((Si, St), (St, 0)):
        x = torch.randn(rows, K, generator=g).bfloat16().to(dev)
        w = (torch.randn(N, K, generator=g) * 0.05).bfloat16().to(dev)
        wq, wk = [(1 + 0.2 * torch.randn(128, generator=g)).bfloat16().to(dev) for _ in range(2)]
        w8, ws = ops.quantize_weight_fp8(w)
        xq, xs = ops.quantize_fp8(x)
        plain = ops.fp8_gemm(xq, w8, xs, ws, None)
        wants.append(ops.rmsnorm_rope_qk(plain.view(1, rows, N), heads, heads, wq, wk, rope, pos0=pos0).view(rows, N))
        probs.append(dict(a_q=xq, w_q=w8, a_scale=xs, w_scale=ws, rows_per_batch=rows,
                          qk=dict(heads=heads, q_norm_w=wq, k_norm_w=wk, rope=rope, pos0=pos0)))
    outs = ops.fp8_gemm_grouped(probs)
    assert torch.equal(outs[0], wants[0]) and torch.equal(outs[1], wants[1])


@pytest.mark.parametrize("kind", ["plain", "residual", "qk"])
def test_half_height_tiles_give_the_bits_of_full_tiles(dev, kind):
    """A problem with at most 128 tiles of 256 x 256 runs on tiles of 128 token rows (four waves, twice as many
    workgroups); one with more runs on 256-row tiles (eight waves).  Same wave tile and K order, so the rows of a
    small problem equal the same rows inside a large one, bit for bit, for each of the three epilogues."""
    from diffsynth_engine_amd import ops

    K, N, M_big, M_small = 1024, 3072, 3000, 1000   # 12 x 12 = 144 tiles against 4 x 12 = 48 (-> 8 x 12 of 128 rows)
    heads = 8
    g = torch.Generator().manual_seed(77)
    x = torch.randn(M_big, K, generator=g).bfloat16().to(dev)
    w = (torch.randn(N, K, generator=g) * 0.05).bfloat16().to(dev)
    bias = torch.randn(N, generator=g).bfloat16().to(dev)
    w8, ws = ops.quantize_weight_fp8(w)
    xq, xs = ops.quantize_fp8(x)
    kw_big, kw_small = {}, {}
    if kind == "residual":
        resid = torch.randn(M_big, N, generator=g).bfloat16().to(dev)
        gate = torch.randn(1, N, generator=g).bfloat16().to(dev)
        kw_big = dict(resid=resid, gate=gate, rows_per_batch=M_big)
        kw_small = dict(resid=resid[:M_small], gate=gate, rows_per_batch=M_small)
    elif kind == "qk":
        ang = torch.rand(1, M_big, 64, generator=g) * 6.28
        rope = torch.stack((torch.cos(ang), torch.sin(ang)), dim=-1).float().to(dev)
        nq, nk = [(1 + 0.2 * torch.randn(128, generator=g)).bfloat16().to(dev) for _ in range(2)]
        qk = dict(heads=heads, q_norm_w=nq, k_norm_w=nk, rope=rope, pos0=0, eps=1e-6)
        kw_big, kw_small = dict(rows_per_batch=M_big, qk=qk), dict(rows_per_batch=M_small, qk=qk)
    big = ops.fp8_gemm(xq, w8, xs, ws, bias, **kw_big)
    small = ops.fp8_gemm(xq[:M_small], w8, xs[:M_small], ws, bias, **kw_small)
    assert torch.equal(small, big[:M_small])
    # ragged heights around the 128-row tile, and a single partly filled tile
    for m in (129, 127, 9):
        kws = dict(kw_small)
        if kind == "residual":
            kws = dict(resid=kw_big["resid"][:m], gate=kw_big["gate"], rows_per_batch=m)
        elif kind == "qk":
            kws = dict(rows_per_batch=m, qk=kw_big["qk"])
        assert torch.equal(ops.fp8_gemm(xq[:m], w8, xs[:m], ws, bias, **kws), big[:m]), m


@pytest.mark.parametrize("kind", ["plain", "residual", "qk"])
@pytest.mark.parametrize("M", [4608, 700])
def test_k_extension_equals_the_concatenated_operands(dev, kind, M):
    """dsx_gemm_problem.a_ext / w_ext: K_ext more columns of the reduction axis read from operands of their own.
    The units are consumed in the order the concatenations [a | a_ext], [w | w_ext] would give, so the result is
    the concatenated product's bit for bit, with each epilogue, on 256-row and on 128-row tiles."""
    from diffsynth_engine_amd import ops

    K, E, N, heads = 1024, 128, 1536, 4
    g = torch.Generator().manual_seed(M + len(kind))
    x = torch.randn(M, K + E, generator=g).bfloat16().to(dev)
    w = (torch.randn(N, K + E, generator=g) * 0.05).bfloat16().to(dev)
    bias = torch.randn(N, generator=g).bfloat16().to(dev)
    w8, ws = ops.quantize_weight_fp8(w)
    xq, xs = ops.quantize_fp8(x)
    kw = {}
    if kind == "residual":
        kw = dict(resid=torch.randn(M, N, generator=g).bfloat16().to(dev),
                  gate=torch.randn(1, N, generator=g).bfloat16().to(dev), rows_per_batch=M)
    elif kind == "qk":
        ang = torch.rand(1, M, 64, generator=g) * 6.28
        rope = torch.stack((torch.cos(ang), torch.sin(ang)), dim=-1).float().to(dev)
        nq, nk = [(1 + 0.2 * torch.randn(128, generator=g)).bfloat16().to(dev) for _ in range(2)]
        kw = dict(rows_per_batch=M, qk=dict(heads=heads, q_norm_w=nq, k_norm_w=nk, rope=rope, pos0=0, eps=1e-6))
    whole = ops.fp8_gemm(xq, w8, xs, ws, bias, **kw)
    # the two segments as separate allocations with leading dimensions of their own
    a1, a2 = xq[:, :K].contiguous(), xq[:, K:].contiguous()
    w1, w2 = w8[:, :K].contiguous(), w8[:, K:].contiguous()
    split = ops.fp8_gemm(a1, w1, xs, ws, bias, ext=(a2, w2), **kw)
    assert torch.equal(split, whole)
    # and it is the extension that closes the gap
    assert not torch.equal(ops.fp8_gemm(a1, w1, xs, ws, bias, **kw), whole)


def test_a_pair_with_one_extended_problem_shares_a_launch(dev):
    """Two problems in one grid (the image and text linears of a joint block) of which only one continues its
    reduction axis, in either position, with different K: each gets the bits of its own single launch."""
    from diffsynth_engine_amd import ops

    g = torch.Generator().manual_seed(5)

    def problem(M, K, N, ext):
        x = torch.randn(M, K, generator=g).bfloat16().to(dev)
        w = (torch.randn(N, K, generator=g) * 0.05).bfloat16().to(dev)
        wq, ws = ops.quantize_weight_fp8(w)
        xq, xs = ops.quantize_fp8(x)
        p = dict(a_q=xq, w_q=wq, a_scale=xs, w_scale=ws, bias=torch.randn(N, generator=g).bfloat16().to(dev))
        if ext:
            p["ext"] = (torch.randn(M, 128, generator=g).mul(40).to(dev).to(ops.FP8),
                        torch.randn(N, 128, generator=g).mul(40).to(dev).to(ops.FP8))
        return p

    for first_ext in (True, False):
        big, small = problem(1024, 768, 1024, first_ext), problem(200, 1280, 512, not first_ext)
        together = ops.fp8_gemm_grouped([big, small])
        for got, p in zip(together, (big, small)):
            assert torch.equal(got, ops.fp8_gemm(p["a_q"], p["w_q"], p["a_scale"], p["w_scale"], p["bias"],
                                                 ext=p.get("ext")))


def test_k_extension_refusals(dev):
    from diffsynth_engine_amd import ops

    a, w = torch.zeros(64, 256, device=dev).to(ops.FP8), torch.zeros(64, 256, device=dev).to(ops.FP8)
    e = lambda m, k: torch.zeros(m, k, device=dev).to(ops.FP8)
    with pytest.raises(ValueError):
        ops.fp8_gemm(a, w, ext=(e(64, 64), e(64, 64)))       # K_ext % 128
    with pytest.raises(ValueError):
        ops.fp8_gemm(a, w, ext=(e(63, 128), e(64, 128)))     # rows of a_ext
    with pytest.raises(ValueError):
        ops.fp8_gemm(a[:, :128], w[:, :128], ext=(e(64, 128), e(64, 128)))  # the first segment needs two units
    with pytest.raises(ValueError):
        ops.fp8_gemm(a[:8], w, ext=(e(8, 128), e(64, 128)))  # the small-M kernel has no extension


@pytest.mark.parametrize("M,K,R", [(4608, 3072, 32), (4608, 15360, 64), (515, 1024, 128), (40, 256, 96)])
def test_lora_down_against_the_fp32_product(dev, M, K, R):
    """out[m, c R + r] = e4m3_saturating(row_scale[r] * sum_k a[m,k] d[r,k]) for every copy c, zero codes after the
    last copy.  The products
    of e4m3 codes are exact in fp32; the kernel's sum is split over wavefronts, so it may differ from torch's in the
    last bit and a value that sits on a rounding boundary may land on the neighbouring code: at most a handful of
    codes differ, each by one step."""
    from diffsynth_engine_amd import ops

    g = torch.Generator().manual_seed(M + K + R)
    a = torch.randn(M, K, generator=g).mul(60).to(dev).to(ops.FP8)
    d = torch.randn(R, K, generator=g).mul(60).to(dev).to(ops.FP8)
    rs = (torch.rand(R, generator=g) + 0.5).mul(3e-5).to(dev)
    rs[R - 1] = 1.0  # one column far beyond 448: saturates instead of turning into NaN codes
    copies = 128 // R if M > 100 else 1
    got = ops.lora_down(a, d, rs, 128, copies)
    assert got.shape == (M, 128) and got.dtype == ops.FP8
    for c in range(1, copies):  # every copy is the first one again
        assert torch.equal(got[:, c * R:(c + 1) * R].view(torch.uint8), got[:, :R].view(torch.uint8))
    # fewer valid ranks than rows of d (the rest is padding): narrower copies, more of them
    few = ops.lora_down(a, d, rs, 128, 128 // 12, ranks=12)
    for c in range(128 // 12):
        assert torch.equal(few[:, c * 12:(c + 1) * 12].view(torch.uint8), got[:, :12].view(torch.uint8))
    assert (few[:, 120:].view(torch.uint8) == 0).all()
    ref = ((a.double() @ d.double().t()) * rs.double()).float()  # (fp32 matmul of 15360 terms is itself off by ~1)
    want = ref.clamp(-448, 448).to(ops.FP8)
    gf, wf = got[:, :R].float(), want.float()
    assert torch.isfinite(gf).all()
    assert (gf[:, R - 1].abs() == 448).float().mean().item() > 0.98  # (a sum can land inside the range by chance)
    differ = gf != wf
    assert differ.float().mean().item() < 2e-3
    # a differing code is the other neighbour of the exact value on the grid: never further than one step.  (Not
    # asked of the saturating column: its scale of 1 lays bare the absolute error of a sum of 15 360 products of up to
    # 2e5 each -- the matrix pipe's fp32 accumulation is good to about 1e-5 of the partial sums' magnitude, which a
    # scale that brings typical values into e4m3's range makes invisible.)
    step = wf.abs().clamp_min(2 ** -6) * 0.125
    assert ((gf - ref.clamp(-448, 448)).abs() <= step)[:, : R - 1].all()
    assert (got[:, copies * R:].view(torch.uint8) == 0).all()


@pytest.mark.parametrize("ranks", [4, 16, 20, 48, 80, 112])
def test_lora_down_every_rank_tile_count(dev, ranks):
    """Every number of 16-rank tiles (1 to 8) has its own instantiation with its own buffer depth and wavefront count;
    ragged row counts (not a multiple of the 16-row tile) and K of one to many chunks per wavefront."""
    from diffsynth_engine_amd import ops

    R = (ranks + 31) // 32 * 32
    for M, K in ((70, 128), (33, 640), (257, 3072)):
        g = torch.Generator().manual_seed(ranks * 1000 + M + K)
        a = torch.randn(M, K, generator=g).mul(60).to(dev).to(ops.FP8)
        d = torch.zeros(R, K)
        d[:ranks] = torch.randn(ranks, K, generator=g).mul(60)
        d = d.to(dev).to(ops.FP8)
        rs = (torch.rand(R, generator=g) + 0.5).mul(100.0 / (60 * 60 * K ** 0.5)).to(dev)
        got = ops.lora_down(a, d, rs, 128, 1, ranks=ranks)
        ref = ((a.double() @ d.double().t()) * rs.double()).float()[:, :ranks]
        gf, wf = got[:, :ranks].float(), ref.clamp(-448, 448).to(ops.FP8).float()
        assert torch.isfinite(gf).all()
        assert (gf != wf).float().mean().item() < 5e-3, (M, K)
        # one grid step, or -- for values near zero, whose steps are tiny -- the matrix pipe's accumulation error:
        # about 1e-5 of the magnitude that went through the sum
        mag = ((a.float().abs() @ d.float().abs().t()) * rs)[:, :ranks]
        tol = torch.maximum(wf.abs().clamp_min(2 ** -6) * 0.125, 1e-5 * mag)
        assert ((gf - ref.clamp(-448, 448)).abs() <= tol).all(), (M, K)
        assert (got[:, ranks:].view(torch.uint8) == 0).all()
