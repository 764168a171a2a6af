"""A whole denoising step recorded as a HIP graph: every replay has to give what the eager step gives.

The replays are separated by eager work and synchronisations of the program's own, and each is checked, because
a graph that is only right on its first replay (a recorded memset node, a stale pointer) passes a single check."""
import pytest
import torch

from oracle import flux as oflux

pytestmark = pytest.mark.gpu


def _inputs(side, n_txt, seed, dev):
    g = torch.Generator().manual_seed(seed)
    return dict(hidden_states=torch.randn(1, 16, side, side, generator=g).bfloat16().to(dev),
                timestep=torch.tensor([float(100 + 37 * seed % 900)], device=dev),
                prompt_emb=torch.randn(1, n_txt, 4096, generator=g).bfloat16().to(dev),
                pooled_prompt_emb=torch.randn(1, 768, generator=g).bfloat16().to(dev),
                guidance=torch.tensor([3.5], device=dev), text_ids=torch.zeros(1, n_txt, 3, device=dev))


def test_flux_step_graph_replays_equal_eager(dev):
    from diffsynth_engine_amd.flux_dit import FluxDiTRunner
    from diffsynth_engine_amd.graph import GraphedStep

    sd = {k: v.to(dev) for k, v in oflux.init_params(2, 2, dtype=torch.bfloat16, seed=11, bias_std=0.02).items()}
    runner = FluxDiTRunner(sd, 2, 2, scaled=True, device=dev)
    step = GraphedStep(runner, **_inputs(32, 64, 0, dev))
    for r in range(1, 5):
        inp = _inputs(32, 64, r, dev)
        eager = runner(**inp).clone()
        torch.cuda.synchronize()
        filler = torch.randn(512, 512, device=dev) @ torch.randn(512, 512, device=dev)  # unrelated eager work
        got = step(**inp).clone()
        torch.cuda.synchronize()
        assert torch.isfinite(filler).all().item()
        assert torch.equal(got, eager), r
    with pytest.raises(ValueError):
        step(hidden_states=torch.zeros(1, 16, 16, 16, device=dev, dtype=torch.bfloat16))


def test_wan_step_graph_replays_equal_eager(dev):
    from oracle import wan as ow

    from diffsynth_engine_amd.graph import GraphedStep
    from diffsynth_engine_amd.wan_dit import WanDiTRunner

    cfg = dict(ow.config_14b(), dim=512, ffn_dim=1024, num_heads=4, num_layers=2)
    sd = ow.init_params(cfg, dtype=torch.bfloat16, seed=1, bias_std=0.02)
    runner = WanDiTRunner(sd, cfg, scaled=True, device=dev)

    def inputs(seed):
        g = torch.Generator().manual_seed(seed)
        return dict(x=torch.randn(1, 16, 2, 12, 16, generator=g).bfloat16().to(dev),
                    context=torch.randn(1, 32, 4096, generator=g).bfloat16().to(dev),
                    timestep=torch.tensor([float(200 + 100 * seed)], device=dev).bfloat16())

    step = GraphedStep(runner, **inputs(0))
    for r in range(1, 4):
        inp = inputs(r)
        eager = runner(**inp).clone()
        torch.cuda.synchronize()
        got = step(**inp).clone()
        torch.cuda.synchronize()
        assert torch.equal(got, eager), r
