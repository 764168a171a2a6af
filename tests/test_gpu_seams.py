"""GPU tests of the two drop-in seams as a reference user would reach them: the F.linear patch on real
nn.Modules (utils/fp8_linear.py) and the attention callables installed into module globals."""
import types

import pytest
import torch
import torch.nn as nn
import torch.nn.functional as F

from conftest import row_rel_err
from oracle import dit_ops as O
from oracle import fp8 as ofp8

pytestmark = pytest.mark.gpu


class _Mlp(nn.Module):
    def __init__(self):
        super().__init__()
        self.net = nn.Sequential(nn.Linear(256, 512), nn.GELU(approximate="tanh"), nn.Linear(512, 128, bias=False))

    def forward(self, x):
        return self.net(x)


@pytest.mark.parametrize("scaled", [True, False])
def test_enable_fp8_linear_and_fp8_inference_on_a_module(dev, scaled):
    """enable_fp8_linear casts every floating nn.Linear weight in place and sets the flag FluxDiT.forward reads
    (fp8_linear.py:7-17, flux_dit.py:404); under fp8_inference every nn.Linear.forward reaches the patched
    F.linear (2-D and >2-D inputs, with and without bias)."""
    from diffsynth_engine_amd import enable_fp8_linear, fp8_inference

    torch.manual_seed(0)
    m = _Mlp().to(torch.bfloat16)
    ref_w = [m.net[0].weight.detach().clone(), m.net[2].weight.detach().clone()]
    ref_b = m.net[0].bias.detach().clone()
    m = m.to(dev)
    enable_fp8_linear(m, scaled=scaled)
    assert m.fp8_linear_enabled is True
    assert m.net[0].weight.dtype == torch.float8_e4m3fn and m.net[0].bias.dtype == torch.bfloat16
    assert ("net.0.weight_scale" in m.state_dict()) == scaled  # the per-tensor scale is module state
    x = torch.randn(3, 20, 256, generator=torch.Generator().manual_seed(1)).bfloat16()
    orig = F.linear
    with fp8_inference(getattr(m, "fp8_linear_enabled", False)):
        y3 = m(x.to(dev))
        y2 = m(x[0].to(dev))
    assert F.linear is orig
    # oracle: the same two linears through the reference arithmetic
    wq0, ws0 = ofp8.quantize_weight(ref_w[0], scaled)
    wq1, ws1 = ofp8.quantize_weight(ref_w[1], scaled)
    h = O.gelu_tanh(ofp8.fp8_linear(x, wq0, ws0, ref_b))
    want = ofp8.fp8_linear(h, wq1, ws1, None)
    assert y3.shape == (3, 20, 128) and y2.shape == (20, 128) and y3.dtype == torch.bfloat16
    cos = F.cosine_similarity(y3.cpu().float().flatten(), want.float().flatten(), dim=0).item()
    assert cos >= 0.9995, cos
    assert torch.equal(y2.cpu(), y3[0].cpu())
    # weights quantised by the kernel are bit-identical to the oracle's
    assert torch.equal(m.net[0].weight.data.cpu().view(torch.uint8), wq0.view(torch.uint8))


def test_flux_seam_called_the_way_flux_joint_attention_calls_it(dev):
    """_attn_func(q, k, v) positional, (B,H,S,D) non-contiguous views in, `.transpose(1,2).reshape` and `.to(dtype)`
    applied to the result (flux_dit.py:182-184)."""
    from diffsynth_engine_amd import set_attn_implementation

    fake_flux_dit = types.SimpleNamespace(_attn_func=F.scaled_dot_product_attention)
    set_attn_implementation("mi355x", flux_dit_module=fake_flux_dit)
    B, S, H = 2, 200, 4
    qkv = torch.randn(B, S, 3 * H * 128, generator=torch.Generator().manual_seed(2)).bfloat16()
    qd, kd, vd = qkv.to(dev).view(B, S, 3 * H, 128).transpose(1, 2).chunk(3, dim=1)
    hs = fake_flux_dit._attn_func(qd, kd, vd)
    hs = hs.transpose(1, 2).reshape(B, -1, H * 128).to(qd.dtype)
    q, k, v = qkv.view(B, S, 3 * H, 128).transpose(1, 2).chunk(3, dim=1)
    want = O.sdpa(q.float(), k.float(), v.float()).transpose(1, 2).reshape(B, S, H * 128)
    assert row_rel_err(hs.cpu().view(B, S, H, 128), want.view(B, S, H, 128)) <= 2e-2
    set_attn_implementation("sdpa", flux_dit_module=fake_flux_dit)
    assert fake_flux_dit._attn_func is F.scaled_dot_product_attention


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16])
def test_wider_inputs_are_rounded_to_bf16_once_and_stay_inside_the_bar(dev, dtype):
    """The reference runs CLIP/T5 in other dtypes through the same callables; outputs come back in the input dtype.
    The kernel's arithmetic is bf16 operands with fp32 accumulation whatever arrives: fp32 and fp16 q, k, v are
    rounded to bf16 once on the way in, which is narrower than what torch's SDPA would compute for them.  The cost
    of that rounding is held to the same bar as a bf16 call, against fp32 SDPA of the UNROUNDED inputs, at a
    sequence length where it has accumulated (scores of size ~sqrt(128) * 2^-9 relative error each)."""
    from diffsynth_engine_amd import mi355x_attention

    g = torch.Generator().manual_seed(3)
    q, k, v = [torch.randn(1, 2, 1152, 128, generator=g).to(dtype) for _ in range(3)]
    assert not torch.equal(q.float(), q.bfloat16().float())  # the inputs do carry bits bf16 drops
    out = mi355x_attention(q.to(dev), k.to(dev), v.to(dev))
    assert out.dtype == dtype
    want = O.sdpa(q.float(), k.float(), v.float())
    err = row_rel_err(out.cpu(), want)
    assert err <= 2e-2, err
    # and the rounding is the whole difference: the same call on pre-rounded inputs gives the same bits
    same = mi355x_attention(q.bfloat16().to(dev), k.bfloat16().to(dev), v.bfloat16().to(dev))
    assert torch.equal(same.to(dtype).cpu(), out.cpu())


def test_weight_scale_travels_with_the_module_state(dev):
    """enable_fp8_linear -> state_dict() -> block-runner storage, and -> load_state_dict into another converted
    module: the per-tensor scale is a buffer of the Linear (`<name>.weight_scale`), so neither path can take an
    already scaled e4m3 weight at unit scale (wrong by 448 / absmax per layer, with no error)."""
    from diffsynth_engine_amd import enable_fp8_linear, fp8_inference, ops
    from diffsynth_engine_amd.flux_dit import ingest_state_dict

    torch.manual_seed(3)
    m = _Mlp().to(torch.bfloat16).to(dev)
    enable_fp8_linear(m)
    sd = m.state_dict()
    assert sd["net.0.weight"].dtype == torch.float8_e4m3fn and sd["net.0.weight_scale"].dim() == 0
    x = torch.randn(40, 256, generator=torch.Generator().manual_seed(4)).bfloat16().to(dev)
    with fp8_inference():
        want = m.net[0](x)
    lin, _ = ingest_state_dict({k: sd[k] for k in sorted(sd)}, dev, scaled=True)  # bias, weight, weight_scale order
    a_q, a_s = ops.quantize_fp8(x)
    assert torch.equal(lin["net.0"](a_q, a_s), want)
    # a second module converted from other weights takes this one's state in place, scale included
    torch.manual_seed(5)
    m2 = _Mlp().to(torch.bfloat16).to(dev)
    with torch.no_grad():
        m2.net[0].weight.mul_(3)
    enable_fp8_linear(m2)
    assert not torch.equal(m2.net[0].weight_scale, m.net[0].weight_scale)
    m2.load_state_dict(sd)
    with fp8_inference():
        assert torch.equal(m2.net[0](x), want)
    # without its scale the weight is refused rather than mis-scaled
    del sd["net.0.weight_scale"]
    with pytest.raises(ValueError, match="net.0"):
        ingest_state_dict(sd, dev, scaled=True)


def test_weight_scale_survives_deepcopy_and_a_dead_owner_is_an_error(dev):
    """copy.deepcopy drops Python attributes of a Parameter, the buffer it keeps: under fp8_inference the copy
    computes what the original does (through nn.Linear.forward, which announces the module's scale).  A direct
    F.linear call with a scaled weight whose module is gone raises instead of running at unit scale, and
    enable_fp8_linear on the copy renews the link for such callers."""
    import copy
    import gc

    from diffsynth_engine_amd import enable_fp8_linear, fp8_inference

    torch.manual_seed(11)
    m = _Mlp().to(torch.bfloat16).to(dev)
    enable_fp8_linear(m)
    x = torch.randn(24, 256, generator=torch.Generator().manual_seed(12)).bfloat16().to(dev)
    forward_before, linear_before = nn.Linear.forward, F.linear
    with fp8_inference():
        assert F.linear is not linear_before
        want = m(x)
        direct = F.linear(x, m.net[0].weight, m.net[0].bias)
        assert torch.equal(direct, m.net[0](x))
    c = copy.deepcopy(m)
    assert not hasattr(c.net[0].weight, "_dsx_owner") and c.net[0].weight_scale.item() == m.net[0].weight_scale.item()
    with fp8_inference():
        assert torch.equal(c(x), want)
    assert nn.Linear.forward is forward_before and F.linear is linear_before
    enable_fp8_linear(c)  # already converted: only the link is renewed
    with fp8_inference():
        assert torch.equal(F.linear(x, c.net[0].weight, c.net[0].bias), direct)
    w, b = m.net[0].weight, m.net[0].bias
    del m
    gc.collect()
    with fp8_inference():
        with pytest.raises(RuntimeError, match="scale"):
            F.linear(x, w, b)
