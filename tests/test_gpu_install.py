"""accelerate_flux_dit / accelerate_wan_dit / restore_forward: a module with the reference's parameter names gets
the fused runner behind its ``forward`` (the block bodies flux_dit.py:219-236,308-321 and wan_dit.py:185-193 are
what the runner replaces), from nothing but ``module.state_dict()``."""
import pytest
import torch
import torch.nn as nn

from oracle import flux as oflux
from oracle import wan as ow

pytestmark = pytest.mark.gpu


class Shell(nn.Module):
    """A module tree that holds a flat state dict under its dotted names (what FluxDiT / WanDiT look like to
    ``state_dict()``); its own forward is a marker."""

    def forward(self, *args, **kwargs):
        return "module's own forward"


def shell_from(sd, device):
    root = Shell()
    for name, t in sd.items():
        *path, leaf = name.split(".")
        m = root
        for p in path:
            if p not in m._modules:
                m.add_module(p, nn.Module())
            m = m._modules[p]
        m.register_parameter(leaf, nn.Parameter(t.to(device), requires_grad=False))
    return root


def _flux_inputs(dev):
    g = torch.Generator().manual_seed(4)
    return dict(hidden_states=torch.randn(1, 16, 16, 24, generator=g).bfloat16().to(dev),
                timestep=torch.tensor([500.0], device=dev), prompt_emb=torch.randn(1, 24, 4096, generator=g).bfloat16().to(dev),
                pooled_prompt_emb=torch.randn(1, 768, generator=g).bfloat16().to(dev),
                guidance=torch.tensor([3.5], device=dev), text_ids=torch.zeros(1, 24, 3, device=dev))


def test_flux_module_runs_the_runner_and_can_be_restored(dev):
    from diffsynth_engine_amd.flux_dit import FluxDiTRunner
    from diffsynth_engine_amd.install import accelerate_flux_dit, restore_forward

    sd = oflux.init_params(2, 3, dtype=torch.bfloat16, seed=3, bias_std=0.02)
    dit = shell_from(sd, dev)
    inp = _flux_inputs(dev)
    assert dit(**inp) == "module's own forward"
    runner = accelerate_flux_dit(dit)
    assert (runner.num_double, runner.num_single, runner.scaled) == (2, 3, True)  # counted, not assumed
    got = dit(**inp)  # through nn.Module.__call__
    want = FluxDiTRunner(sd, 2, 3, scaled=True, device=dev)(**inp)
    assert torch.equal(got, want)
    # and the runner computes the model: against the oracle on the same weights
    ref = oflux.flux_dit_forward(oflux.Params(sd, "fp8_scaled"), **{k: v.cpu() for k, v in inp.items()},
                                 num_double=2, num_single=3)
    cos = torch.nn.functional.cosine_similarity(got.float().flatten().cpu(), ref.float().flatten(), dim=0).item()
    assert cos >= 0.995, cos
    restore_forward(dit)
    assert dit(**inp) == "module's own forward" and "_dsx_runner" not in dit.__dict__
    restore_forward(dit)  # a second call is a no-op


def test_flux_module_converted_by_either_enable_fp8_linear(dev):
    """Weights already in e4m3: with ``weight_scale`` buffers (this package's enable_fp8_linear) the runner takes
    the scales; bare e4m3 weights (the reference's enable_fp8_linear, fp8_linear.py:7-17) run at unit scale."""
    from diffsynth_engine_amd import ops
    from diffsynth_engine_amd.flux_dit import FluxDiTRunner
    from diffsynth_engine_amd.install import accelerate_flux_dit

    sd = oflux.init_params(1, 1, dtype=torch.bfloat16, seed=5, bias_std=0.02)
    inp = _flux_inputs(dev)
    scaled_sd, bare_sd = {}, {}
    for k, v in sd.items():
        if k.endswith(".weight") and v.dim() == 2:
            q, s = ops.quantize_weight_fp8(v.to(dev), scaled=True)
            scaled_sd[k], scaled_sd[k[:-len(".weight")] + ".weight_scale"] = q, s
            bare_sd[k] = v.to(dev).to(torch.float8_e4m3fn)
        else:
            scaled_sd[k] = bare_sd[k] = v
    r_scaled = accelerate_flux_dit(shell_from(scaled_sd, dev))
    assert r_scaled.scaled and torch.equal(r_scaled(**inp), FluxDiTRunner(sd, 1, 1, scaled=True, device=dev)(**inp))
    r_bare = accelerate_flux_dit(shell_from(bare_sd, dev))
    assert not r_bare.scaled and torch.equal(r_bare(**inp), FluxDiTRunner(sd, 1, 1, scaled=False, device=dev)(**inp))


def test_wan_module_runs_the_runner_with_dims_read_off_the_checkpoint(dev):
    from diffsynth_engine_amd.install import accelerate_wan_dit, restore_forward
    from diffsynth_engine_amd.wan_dit import WanDiTRunner

    cfg = dict(ow.config_14b(), dim=512, ffn_dim=1024, num_heads=4, num_layers=2)
    sd = ow.init_params(cfg, dtype=torch.bfloat16, seed=1, bias_std=0.02)
    dit = shell_from(sd, dev)
    g = torch.Generator().manual_seed(3)
    x = torch.randn(1, 16, 2, 12, 16, generator=g).bfloat16().to(dev)
    ctx = torch.randn(1, 32, 4096, generator=g).bfloat16().to(dev)
    t = torch.tensor([500.0]).bfloat16().to(dev)
    runner = accelerate_wan_dit(dit)
    for key in ("dim", "num_heads", "num_layers", "out_dim", "freq_dim", "eps"):
        assert runner.cfg[key] == cfg[key], key
    assert tuple(runner.cfg["patch_size"]) == tuple(cfg["patch_size"])
    got = dit(x, ctx, t)
    assert torch.equal(got, WanDiTRunner(sd, cfg, scaled=True, device=dev)(x, ctx, t))
    assert torch.equal(got, dit(x=x, context=ctx, timestep=t))  # the pipeline's keyword form, wan_video.py:294-368
    restore_forward(dit)
    assert dit(x, ctx, t) == "module's own forward"
