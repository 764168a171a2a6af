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


class _LoRA:
    """The attributes of the reference's LoRA objects that LoRALinear.forward uses (models/basic/lora.py:9-32)."""

    def __init__(self, scale, rank, alpha, up, down, as_linear):
        self.scale, self.rank, self.alpha = scale, rank, alpha
        if as_linear:  # LoRALinear.add_lora wraps the factors in bias-free Linears (lora.py:92-99)
            self.up, self.down = nn.Linear(up.shape[1], up.shape[0], bias=False), nn.Linear(down.shape[1], down.shape[0], bias=False)
            self.up.weight.data, self.down.weight.data = up, down
        else:
            self.up, self.down = up, down


def _give_lora(dit, name, lora):
    sub = dit.get_submodule(name)
    if "_lora_dict" not in sub.__dict__:
        object.__setattr__(sub, "_lora_dict", {})
    sub._lora_dict["lora%d" % len(sub._lora_dict)] = lora


def test_unfused_loras_of_the_module_reach_the_runner(dev):
    """LoRALinear.forward (lora.py:137-141): w_x + sum of scale * alpha / rank * up(down(x)) over ``_lora_dict``;
    a weight a LoRA was fused into brings an ``_original_weight`` copy in the state dict, which must not be run."""
    from diffsynth_engine_amd.flux_dit import FluxDiTRunner
    from diffsynth_engine_amd.install import accelerate_flux_dit

    sd = oflux.init_params(1, 1, dtype=torch.bfloat16, seed=7, bias_std=0.02)
    dit = shell_from(sd, dev)
    g = torch.Generator().manual_seed(8)
    direct = FluxDiTRunner(sd, 1, 1, scaled=True, device=dev)
    for i, (name, r) in enumerate({"blocks.0.attn.a_to_qkv": 16, "blocks.0.ff_b.2": 8, "single_blocks.0.proj_out": 4}.items()):
        n, k = sd[name + ".weight"].shape
        down = (torch.randn(r, k, generator=g) * 0.05).bfloat16().to(dev)
        up = (torch.randn(n, r, generator=g) * 0.05).bfloat16().to(dev)
        _give_lora(dit, name, _LoRA(0.8, r, 2 * r, up, down, as_linear=bool(i % 2)))
        direct.add_lora(name, down, up, 0.8 * (2 * r) / r)
    dit.get_submodule("blocks.0.attn.a_to_out").register_buffer(
        "_original_weight", torch.zeros_like(sd["blocks.0.attn.a_to_out.weight"]).to(dev))
    inp = _flux_inputs(dev)
    got = accelerate_flux_dit(dit)(**inp)
    assert torch.equal(got, direct(**inp))
    assert not torch.equal(got, FluxDiTRunner(sd, 1, 1, scaled=True, device=dev)(**inp))  # the LoRAs are in there
    # factors that do not fit their Linear are refused, not run
    n, k = sd["blocks.0.norm1_a.linear.weight"].shape
    _give_lora(dit, "blocks.0.norm1_a.linear", _LoRA(1.0, 4, 4, torch.zeros(n, 4, device=dev), torch.zeros(4, k + 16, device=dev), False))
    with pytest.raises(ValueError):
        accelerate_flux_dit(dit)


def test_wan_runner_with_unfused_loras_matches_the_oracle(dev):
    """One Wan block with low-rank pairs on a projection that feeds RMSNorm (q), on one behind a gated residual (o),
    on a cross-attention k and on the first FFN layer, against the oracle with the same pairs."""
    from diffsynth_engine_amd.install import accelerate_wan_dit

    cfg = dict(ow.config_14b(), dim=512, ffn_dim=1024, num_heads=4, num_layers=1)
    sd = ow.init_params(cfg, dtype=torch.bfloat16, seed=11, bias_std=0.02)
    dit = shell_from(sd, dev)
    P = ow.Params(sd, "fp8_scaled")
    g = torch.Generator().manual_seed(12)
    for name, r in {"blocks.0.self_attn.q": 16, "blocks.0.self_attn.o": 8, "blocks.0.cross_attn.k": 4, "blocks.0.ffn.0": 32}.items():
        n, k = sd[name + ".weight"].shape
        down = (torch.randn(r, k, generator=g) * 0.05).bfloat16()
        up = (torch.randn(n, r, generator=g) * 0.05).bfloat16()
        P.lora[name] = [(down, up, 0.5)]
        _give_lora(dit, name, _LoRA(0.5, r, r, up.to(dev), down.to(dev), as_linear=True))
    f, h, w = 2, 6, 8
    S = f * h * w
    x = torch.randn(1, S, 512, generator=g).bfloat16()
    ctx = torch.randn(1, 40, 512, generator=g).bfloat16()
    t_mod = (torch.randn(1, 6, 512, generator=g) * 0.3).bfloat16()
    freqs = ow.freqs_cis_3d(128, f, h, w)
    want = ow.dit_block(P, 0, x, ctx, t_mod, freqs, cfg)
    plain = ow.dit_block(ow.Params(sd, "fp8_scaled"), 0, x, ctx, t_mod, freqs, cfg)
    cos = lambda a, b: torch.nn.functional.cosine_similarity(a.float().flatten().cpu(), b.float().flatten().cpu(), dim=0).item()
    assert cos(plain, want) < 0.9999  # the low-rank terms matter in this set-up
    R = accelerate_wan_dit(dit)
    got = R.block(0, x.to(dev), ctx.to(dev), t_mod.to(dev), R.rope_table(f, h, w))
    assert cos(got, want) >= 0.9995, cos(got, want)
