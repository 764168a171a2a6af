"""Writes input/output vectors of the reference's WanDiT (text-to-video) at reduced size.

WanDiT's wiring (diffsynth_engine/models/wan/wan_dit.py: modulation chunk order, the 3-axis complex
RoPE split, full-width q/k RMSNorm, cross-attention without gate, head modulation, patch / unpatch
orders) is fixed by no closed form, and the reference holds no WanDiT test or fixture.  This script
builds the reference's own class in the build container with a reduced config (dim 40, 2 heads of 20,
2 layers, ffn 48, text dim 12, freq dim 16, patch (1,2,2)), fp32 on the CPU, runs one DiTBlock and the
whole forward on seeded inputs, and saves inputs, parameters and outputs:

    python tests/golden/make_wan_fixtures.py [/root/reference]

The root package's __init__ is bypassed (it imports the pipelines, whose dependencies are absent): an
empty module object with the real __path__ stands for ``diffsynth_engine``; every module wan_dit.py
imports is then the reference's own file.  The result, wan_dit.safetensors (under 1 MB), is data.
"""
import os
import sys
import types

import torch
from safetensors.torch import save_file

sys.dont_write_bytecode = True  # the reference tree is read-only: leave no __pycache__ in it
ref = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
here = os.path.dirname(os.path.abspath(__file__))

root = types.ModuleType("diffsynth_engine")
root.__path__ = [os.path.join(ref, "diffsynth_engine")]
sys.modules["diffsynth_engine"] = root

from diffsynth_engine.models.wan import wan_dit as wd  # noqa: E402

torch.manual_seed(777)
cfg = dict(dim=40, in_dim=4, ffn_dim=48, out_dim=4, text_dim=12, freq_dim=16, eps=1e-6, patch_size=(1, 2, 2),
           num_heads=2, num_layers=2)
out = {}

with torch.no_grad():
    model = wd.WanDiT(has_image_input=False, device="cpu", dtype=torch.float32, **cfg)
    model.eval()
    for name, p in model.named_parameters():
        if p.ndim >= 2 and "modulation" not in name:
            p.copy_(torch.randn_like(p) * 0.3)
        elif "norm" in name and name.endswith("weight"):
            p.copy_(1.0 + 0.3 * torch.randn_like(p))
        else:
            p.copy_(torch.randn_like(p) * 0.5)
    for k, v in model.state_dict().items():
        out["param." + k] = v.detach().clone()

    x = torch.randn(1, 4, 3, 4, 6)            # (b, c, frames, height, width) -> f,h,w = 3,2,3 = 18 tokens
    context = torch.randn(1, 5, 12)
    timestep = torch.tensor([412.0])
    out.update({"model.x": x, "model.context": context, "model.timestep": timestep,
                "model.out": model(x, context, timestep).contiguous()})

    # one block on its own, with the per-token RoPE table WanDiT.forward builds for a (3,2,3) grid
    f, h, w = 3, 2, 3
    freqs = torch.cat([model.freqs[0][:f].view(f, 1, 1, -1).expand(f, h, w, -1),
                       model.freqs[1][:h].view(1, h, 1, -1).expand(f, h, w, -1),
                       model.freqs[2][:w].view(1, 1, w, -1).expand(f, h, w, -1)], dim=-1).reshape(f * h * w, 1, -1)
    xb = torch.randn(1, f * h * w, cfg["dim"])
    cb = torch.randn(1, 5, cfg["dim"])
    t_mod = torch.randn(1, 6, cfg["dim"])
    out.update({"block.x": xb, "block.context": cb, "block.t_mod": t_mod,
                "block.freqs_real": torch.view_as_real(freqs).contiguous(),
                "block.out": model.blocks[1](xb, cb, t_mod, freqs).contiguous()})

save_file(out, os.path.join(here, "wan_dit.safetensors"))
print(len(out), "tensors;", sum(v.numel() * v.element_size() for v in out.values()) // 1024, "KiB")
