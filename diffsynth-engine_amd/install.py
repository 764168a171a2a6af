"""Put a fused block runner behind a DiT module's ``forward``.

The two seams (attention.py, fp8_linear.py) replace what the reference's modules call; the block runners replace
the module bodies themselves (FluxJointTransformerBlock.forward, FluxSingleTransformerBlock.forward,
diffsynth_engine/models/flux/flux_dit.py:219-236,308-321; DiTBlock.forward, models/wan/wan_dit.py:185-193).  A
pipeline keeps calling ``self.dit(...)`` (pipelines/flux_image.py:513-526, pipelines/wan_video.py:294-368):

    from diffsynth_engine_amd.install import accelerate_flux_dit
    accelerate_flux_dit(pipe.dit)          # pipe.dit(...) now runs FluxDiTRunner.forward

The runner is built from ``module.state_dict()`` (the reference's parameter names) on the module's device and keeps
its own e4m3 copy of every Linear weight; the module's parameters stay as they are, so ``restore_forward`` gives the
original behaviour back.  Unfused LoRAs the module's LoRALinear layers carry at that moment are attached to the
runner's linears.  Later changes to the module
(``load_state_dict``, LoRAs added, removed, fused or rescaled) do not reach the runner: call ``accelerate_*`` again.
"""
from typing import Optional

import torch
import torch.nn as nn

from . import ops
from .flux_dit import SCALE_SUFFIX, FluxDiTRunner
from .wan_dit import WanDiTRunner

_ORIGINAL = "_dsx_original_forward"
RUNNER = "_dsx_runner"


def _device_of(module: nn.Module) -> torch.device:
    for p in module.parameters():
        return p.device
    raise ValueError("the module has no parameters")


def _scaled_mode(state_dict, scaled: Optional[bool]) -> bool:
    """Scaled e4m3 (per-token x per-tensor) unless the module already holds bare e4m3 weights without scales, the
    state the reference's ``enable_fp8_linear`` leaves (utils/fp8_linear.py:15): those run with unit scales."""
    if scaled is not None:
        return scaled
    for key, t in state_dict.items():
        if key.endswith(".weight") and t.dim() == 2 and t.dtype == ops.FP8 \
                and key[: -len(".weight")] + SCALE_SUFFIX not in state_dict:
            return False
    return True


def _state_dict(module: nn.Module):
    """``module.state_dict()`` without the copies LoRALinear keeps of weights it has fused a LoRA into
    (``_original_weight``, models/basic/lora.py:66,119-120): the fused ``weight`` is the one to run."""
    return {k: v for k, v in module.state_dict().items() if not k.endswith("._original_weight")}


def _attach_loras(module: nn.Module, runner) -> int:
    """Unfused LoRAs of the module's LoRALinear layers (``_lora_dict``, models/basic/lora.py:63,80-100: name ->
    LoRA with ``scale``, ``alpha``, ``rank`` and ``up`` / ``down`` as bias-free Linears or plain tensors) go to the
    runner's linears of the same names; LoRALinear.forward adds ``scale * alpha / rank * up(down(x))`` (:29-32,137-141)."""
    n = 0
    for name, sub in module.named_modules():
        for lora in getattr(sub, "_lora_dict", {}).values():
            up = lora.up.weight if isinstance(lora.up, nn.Module) else lora.up
            down = lora.down.weight if isinstance(lora.down, nn.Module) else lora.down
            runner.add_lora(name, down.detach(), up.detach(), float(lora.scale) * float(lora.alpha) / float(lora.rank))
            n += 1
    return n


def _rebind(module: nn.Module, runner):
    if _ORIGINAL not in module.__dict__:
        # the bound method the instance had: a class attribute normally, an instance attribute if someone
        # rebound it before
        object.__setattr__(module, _ORIGINAL, module.__dict__.get("forward"))
    object.__setattr__(module, RUNNER, runner)
    object.__setattr__(module, "forward", runner.forward)  # nn.Module.__call__ looks `forward` up on the instance first
    return runner


def accelerate_flux_dit(dit: nn.Module, scaled: Optional[bool] = None, **runner_options) -> FluxDiTRunner:
    """``dit``: a module with FluxDiT's parameter names (flux_dit.py:338-364).  Returns the runner that now
    answers ``dit(hidden_states, timestep, prompt_emb, pooled_prompt_emb, guidance, text_ids, image_ids=None)``."""
    sd = _state_dict(dit)
    runner = FluxDiTRunner(sd, scaled=_scaled_mode(sd, scaled), device=_device_of(dit), **runner_options)
    _attach_loras(dit, runner)
    return _rebind(dit, runner)


def accelerate_wan_dit(dit: nn.Module, cfg: Optional[dict] = None, scaled: Optional[bool] = None) -> WanDiTRunner:
    """``dit``: a module with WanDiT's parameter names (wan_dit.py:247-299).  ``cfg``: the constructor arguments
    of conf/models/wan/dit/*.json; left out, they are read off the parameter shapes.  Returns the runner that now
    answers ``dit(x, context, timestep, clip_feature=None, y=None)``."""
    sd = _state_dict(dit)
    runner = WanDiTRunner(sd, cfg, scaled=_scaled_mode(sd, scaled), device=_device_of(dit))
    _attach_loras(dit, runner)
    return _rebind(dit, runner)


def restore_forward(module: nn.Module) -> None:
    """Undo ``accelerate_*``: the module computes with its own code again and the runner is dropped."""
    if _ORIGINAL not in module.__dict__:
        return
    original = module.__dict__[_ORIGINAL]
    for name in (_ORIGINAL, RUNNER, "forward"):
        module.__dict__.pop(name, None)
    if original is not None:
        object.__setattr__(module, "forward", original)
