"""The kernels see pointers and sizes, not tensors: an operand that is shorter than the sizes say would be read
past its end on the device.  The tensor-level wrappers therefore refuse, on the host and before any launch, every
operand whose shape, dtype or device does not fit the call."""
import pytest
import torch

pytestmark = pytest.mark.gpu

BF, F8 = torch.bfloat16, torch.float8_e4m3fn


def _qkv(dev, H=2, Sq=64, Skv=64):
    return [torch.randn(1, H, s, 128, device=dev).to(BF) for s in (Sq, Skv, Skv)]


def test_attention_refuses_operands_that_do_not_fit(dev):
    from diffsynth_engine_amd import ops

    q, k, v = _qkv(dev)
    ok = ops.attention_bhsd(q, k, v)
    assert ok.shape == q.shape
    bad = [dict(v=v[:, :, :32]), dict(k=k[:, :1], v=v[:, :1]), dict(k2=k), dict(k2=k, v2=v[:, :, :8]),
           dict(q2=q[:, :1]), dict(out=torch.empty(1, 2, 32, 128, device=dev, dtype=BF)),
           dict(out=torch.empty_like(q, dtype=torch.float16)), dict(q_norm_w=torch.ones(64, device=dev)),
           dict(rope=torch.zeros(1, 32, 64, 2, device=dev)), dict(rope=torch.zeros(3, 64, 64, 2, device=dev)),
           dict(rope=torch.zeros(1, 64, 64, 2)), dict(qk_norm2_max=torch.ones(2))]
    for kw in bad:
        args = dict(q=q, k=k, v=v)
        args.update(kw)
        qq, kk, vv = args.pop("q"), args.pop("k"), args.pop("v")
        with pytest.raises((ValueError, RuntimeError)):
            ops.attention_bhsd(qq, kk, vv, **args)


def test_gemm_refuses_operands_that_do_not_fit(dev):
    from diffsynth_engine_amd import ops

    a = torch.randn(40, 256, device=dev).to(BF)
    w = torch.randn(64, 256, device=dev).to(BF)
    aq, a_s = ops.quantize_fp8(a)
    wq, w_s = ops.quantize_weight_fp8(w)
    y = ops.fp8_gemm(aq, wq, a_s, w_s)
    assert y.shape == (40, 64)
    resid = torch.zeros(40, 64, device=dev, dtype=BF)
    bad = [dict(a_scale=a_s[:8]), dict(a_scale=a_s.double()), dict(w_scale=torch.ones(2, device=dev)),
           dict(bias=torch.zeros(32, device=dev, dtype=BF)), dict(bias=torch.zeros(64, dtype=BF)),
           dict(out=torch.empty(40, 32, device=dev, dtype=BF)), dict(resid=resid[:, :32]),
           dict(gate=torch.ones(1, 64, device=dev, dtype=BF)),  # a gate without a residual
           dict(resid=resid, gate=torch.ones(2, 64, device=dev, dtype=BF), rows_per_batch=10),  # 2 x 10 rows < 40
           dict(qk=dict(heads=1, q_norm_w=torch.ones(64, device=dev)))]
    for kw in bad:
        args = dict(a_scale=a_s, w_scale=w_s)
        args.update(kw)
        with pytest.raises((ValueError, RuntimeError)):  # (RuntimeError: an operand left on the host)
            ops.fp8_gemm(aq, wq, **args)
    with pytest.raises(ValueError):
        ops.fp8_gemm(aq, wq[:, :128], a_s, w_s)
    row_scale = torch.ones(64, device=dev)
    small, small_s = aq[:2], a_s[:2].contiguous()
    assert ops.fp8_gemv_rowscale(small, wq, small_s, row_scale).shape == (2, 64)
    for kw in (dict(w_row_scale=row_scale[:8]), dict(a_scale=a_s), dict(bias=torch.zeros(8, device=dev, dtype=BF)),
               dict(w_q=w)):
        args = dict(a_q=small, w_q=wq, a_scale=small_s, w_row_scale=row_scale)
        args.update(kw)
        with pytest.raises(ValueError):
            ops.fp8_gemv_rowscale(**args)


def test_row_kernels_refuse_operands_that_do_not_fit(dev):
    from diffsynth_engine_amd import ops

    x = torch.randn(1, 2, 16, 128, device=dev).to(BF)
    table = torch.zeros(1, 16, 64, 2, device=dev)
    table[..., 0] = 1
    assert torch.equal(ops.rmsnorm_rope(x, None, table), x)
    with pytest.raises(ValueError):
        ops.rmsnorm_rope(x, None, table, pos0=1)  # rows 1..16 of a 16-row table
    with pytest.raises(ValueError):
        ops.rmsnorm_rope(x, torch.ones(64, device=dev), None)
    qkv = torch.randn(1, 16, 3 * 256, device=dev).to(BF)
    ops.rmsnorm_rope_qk(qkv.clone(), 2, 2, None, None, table)
    with pytest.raises(ValueError):
        ops.rmsnorm_rope_qk(qkv.clone(), 2, 2, None, None, table[:, :8])
    with pytest.raises(ValueError):
        ops.rmsnorm_rope_qk(qkv.clone(), 2, 2, torch.ones(256, device=dev), None, table)
    rows = torch.randn(1, 16, 256, device=dev).to(BF)
    with pytest.raises(ValueError):
        ops.rmsnorm_rows(rows, torch.ones(128, device=dev))
    with pytest.raises(ValueError):
        ops.adaln_modulate(rows, None, None, ln_weight=torch.ones(128, device=dev))
    with pytest.raises(ValueError):
        ops.gated_residual(rows, rows[:, :8], None)
    with pytest.raises(ValueError):
        ops.gated_residual(rows, rows, torch.ones(3, 256, device=dev, dtype=BF))
    assert torch.equal(ops.gated_residual(rows, torch.zeros_like(rows), torch.ones(1, 256, device=dev)), rows)


def test_lora_down_refuses_operands_that_do_not_fit(dev):
    """ops.lora_down on the host, dsx_lora_down in the library: sizes the kernel's tiles and its 16-byte loads do not
    cover come back as an error before anything is launched."""
    from diffsynth_engine_amd import ops

    a = torch.randn(48, 256, device=dev).mul(50).to(F8)
    d = torch.randn(32, 256, device=dev).mul(50).to(F8)
    rs = torch.full((32,), 1e-4, device=dev)
    assert ops.lora_down(a, d, rs, 128, 4).shape == (48, 128)
    bad = [dict(d_q=d[:, :128]),                                   # K of the factors differs
           dict(a_q=a.to(BF)),                                     # not e4m3
           dict(row_scale=rs[:16]), dict(row_scale=rs.double()),   # one fp32 scale per row of d
           dict(d_q=d[:16].contiguous(), row_scale=rs[:16].contiguous()),  # rows of d: a multiple of 32
           dict(copies=5),                                         # 5 x 32 columns do not fit 128
           dict(copies=0), dict(ranks=6), dict(ranks=40),          # ranks: a multiple of 4, at most the rows of d
           dict(a_q=a[:, :192], d_q=d[:, :192].contiguous()),      # K: a multiple of 128
           dict(width=120)]                                        # output width: a multiple of 16
    for kw in bad:
        args = dict(a_q=a, d_q=d, row_scale=rs, width=128, copies=4)
        args.update(kw)
        with pytest.raises((ValueError, RuntimeError)):
            ops.lora_down(**args)
    assert ops.lora_down(a[:0], d, rs, 128, 4).shape == (0, 128)  # no rows: nothing to do
