"""Pins the scheduler / sampler restatements (oracle AND host mirror) against the reference's golden files."""
import os

import pytest
import torch
from safetensors.torch import load_file

from oracle import sampler as osamp

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def _allclose(a, b):
    return torch.allclose(a, b, atol=1e-3, rtol=1e-3)  # the reference's assertTensorEqual (tests/common/test_case.py:42-58)


def _flux_schedule(mod):
    # the call made by tests/test_algorithm/test_scheduler.py:45-59 and test_sampler.py:21-42
    mu = mod.calculate_shift(1024 // 16 * 1024 // 16)
    if mod is osamp:
        return mod.recified_flow_schedule(20, mu=mu, sigma_min=1.0 / 20, sigma_max=1.0, use_dynamic_shifting=True)
    return mod.RecifitedFlowScheduler(use_dynamic_shifting=True).schedule(20, mu=mu, sigma_min=1.0 / 20, sigma_max=1.0)


def test_recified_flow_schedule_matches_reference_golden():
    from diffsynth_engine_amd import sampler as host

    gold = load_file(os.path.join(GOLD, "recifited_flow_20steps_flux.safetensors"))
    for mod in (osamp, host):
        sigmas, timesteps = _flux_schedule(mod)
        assert sigmas.shape == gold["sigmas"].shape and timesteps.shape == gold["timesteps"].shape
        assert _allclose(sigmas, gold["sigmas"]) and _allclose(timesteps, gold["timesteps"])
    assert abs(osamp.calculate_shift(256) - 0.5) < 1e-12 and abs(osamp.calculate_shift(4096) - 1.15) < 1e-12


def test_flow_match_euler_step_matches_reference_golden():
    gold = load_file(os.path.join(GOLD, "flow_match_euler_i10_rows256.safetensors"))
    sigmas, _ = _flux_schedule(osamp)
    got = osamp.flow_match_euler_step(gold["origin_sample"], gold["model_output"], sigmas, 10)
    assert _allclose(got, gold["prev_sample"])
    # static shift form (Wan uses shift 5.0): s*t / (1 + (s-1)*t), endpoints fixed
    sig, ts = osamp.recified_flow_schedule(10, shift=5.0, sigma_min=0.0, sigma_max=1.0)
    assert abs(float(sig[0]) - 1.0) < 1e-6 and float(sig[-1]) == 0.0 and abs(float(ts[0]) - 1000.0) < 1e-3
    mid = 0.5
    assert abs(5 * mid / (1 + 4 * mid) - 5.0 / 6.0) < 1e-12


@pytest.mark.gpu
def test_device_sampler_step_matches_reference_golden(dev):
    from diffsynth_engine_amd import sampler as host

    gold = load_file(os.path.join(GOLD, "flow_match_euler_i10_rows256.safetensors"))
    sigmas, timesteps = _flux_schedule(host)
    s = host.FlowMatchEulerSampler()
    s.initialize(None, timesteps, sigmas, None)
    got = s.step(gold["origin_sample"].to(dev), gold["model_output"].to(dev), 10).cpu()
    assert torch.equal(got, osamp.flow_match_euler_step(gold["origin_sample"], gold["model_output"], sigmas, 10))
    assert _allclose(got, gold["prev_sample"])
