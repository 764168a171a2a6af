"""Flow-match scheduler and Euler sampler either side of the DiT call — oracle (test infrastructure,
see oracle/__init__.py).  Pinned against the reference's own golden files (tests/golden/)."""
import math

import torch


def calculate_shift(image_seq_len, base_seq_len=256, max_seq_len=4096, base_shift=0.5, max_shift=1.15):
    """pipelines/flux_image.py:166-176: linear interpolation of the dynamic-shift mu in the token count."""
    m = (max_shift - base_shift) / (max_seq_len - base_seq_len)
    return image_seq_len * m + (base_shift - m * base_seq_len)


def recified_flow_schedule(num_inference_steps, mu=None, sigma_min=0.001, sigma_max=1.0, shift=1.0,
                           num_train_timesteps=1000, use_dynamic_shifting=False):
    """algorithm/noise_scheduler/flow_match/recifited_flow.py:33-47: linspace sigmas, then either the dynamic
    time shift e^mu / (e^mu + (1/t - 1)) (Flux) or the static shift s t / (1 + (s-1) t); timesteps = sigma * 1000;
    a trailing zero sigma."""
    sigmas = torch.linspace(sigma_max, sigma_min, num_inference_steps)
    if use_dynamic_shifting:
        sigmas = math.exp(mu) / (math.exp(mu) + (1 / sigmas - 1) ** 1.0)
    else:
        sigmas = shift * sigmas / (1 + (shift - 1) * sigmas)
    timesteps = sigmas * num_train_timesteps
    return torch.cat([sigmas, sigmas.new_zeros([1])]), timesteps


def flow_match_euler_step(latents, model_outputs, sigmas, i):
    """algorithm/sampler/flow_match/flow_match_euler.py:11-19 (no inpainting mask):
    latents.float() + model_outputs * (sigma[i+1] - sigma[i]), cast to the model output dtype."""
    dt = sigmas[i + 1] - sigmas[i]
    out = latents.to(dtype=torch.float32) + model_outputs * dt
    return out.to(dtype=model_outputs.dtype)
