"""Scheduler and sampler either side of the DiT call, with the reference's class and method names.

``RecifitedFlowScheduler.schedule`` (algorithm/noise_scheduler/flow_match/recifited_flow.py:33-47) is a
handful of host-side scalar operations and stays in torch; ``FlowMatchEulerSampler.step``
(algorithm/sampler/flow_match/flow_match_euler.py:11-19) runs as one libdsx kernel on the device so that the
denoising loop never leaves the GPU between DiT calls.
"""
import math

import torch

from . import ops


def calculate_shift(image_seq_len, base_seq_len: int = 256, max_seq_len: int = 4096, base_shift: float = 0.5,
                    max_shift: float = 1.15):
    """pipelines/flux_image.py:166-176."""
    m = (max_shift - base_shift) / (max_seq_len - base_seq_len)
    b = base_shift - m * base_seq_len
    return image_seq_len * m + b


class RecifitedFlowScheduler:
    def __init__(self, shift=1.0, sigma_min=0.001, sigma_max=1.0, num_train_timesteps=1000,
                 use_dynamic_shifting=False):
        self.shift = shift
        self.sigma_min = sigma_min
        self.sigma_max = sigma_max
        self.num_train_timesteps = num_train_timesteps
        self.use_dynamic_shifting = use_dynamic_shifting

    def schedule(self, num_inference_steps: int, mu: float | None = None, sigma_min: float | None = None,
                 sigma_max: float | None = None):
        sigma_min = self.sigma_min if sigma_min is None else sigma_min
        sigma_max = self.sigma_max if sigma_max is None else sigma_max
        sigmas = torch.linspace(sigma_max, sigma_min, num_inference_steps)
        if self.use_dynamic_shifting:
            if mu is None:
                raise ValueError("dynamic shifting needs mu")
            sigmas = math.exp(mu) / (math.exp(mu) + (1 / sigmas - 1))
        else:
            sigmas = self.shift * sigmas / (1 + (self.shift - 1) * sigmas)
        timesteps = sigmas * self.num_train_timesteps
        return torch.cat([sigmas, sigmas.new_zeros([1])]), timesteps


class FlowMatchEulerSampler:
    def initialize(self, init_latents, timesteps, sigmas, mask=None):
        self.init_latents = init_latents
        self.timesteps = timesteps
        self.sigmas = sigmas
        self.mask = mask
        # the step needs sigma[i+1] - sigma[i] as a host scalar; fetch the table once, not once per step
        self._sigmas_host = [float(s) for s in torch.as_tensor(sigmas, dtype=torch.float32).cpu()]

    def step(self, latents, model_outputs, i):
        if self.mask is not None:
            model_outputs = model_outputs * self.mask + self.init_latents * (1 - self.mask)
        s = torch.tensor(self._sigmas_host[i : i + 2], dtype=torch.float32)
        dt = float(s[1] - s[0])  # fp32 difference, as torch computes sigmas[i+1] - sigmas[i]
        if latents.dtype != model_outputs.dtype:
            latents = latents.to(model_outputs.dtype)
        return ops.flow_match_euler_step(latents, model_outputs, dt)

    def add_noise(self, latents, noise, sigma):
        return (1 - sigma) * latents + noise * sigma
