"""Writes input/output vectors of the reference's WanDiT in its image-to-video form at reduced size.

has_image_input=True (conf/models/wan/dit/14b-i2v.json) changes three places of
diffsynth_engine/models/wan/wan_dit.py that no closed form fixes and no reference test covers: the latents are
concatenated with the encoded image along channels before the patch embedding (:331), the CLIP feature goes
through the ``img_emb`` MLP (LayerNorm, Linear, erf-GELU, Linear, LayerNorm; :195-211) and is put IN FRONT of the
text context (:333), and every cross-attention splits that context at row 257 and adds a second attention over
the image rows with its own k/v projections and k norm (:136-152).  This script builds the reference's own class
in the build container with a reduced config, fp32 on the CPU, and saves inputs, parameters and outputs of the
whole forward and of one block:

    python tests/golden/make_wan_i2v_fixtures.py [/root/reference]

The package root is bypassed as in make_wan_fixtures.py.  WanDiT.__init__ hard-codes the CLIP width 1280 for
``img_emb``; the model object gets an ``MLP`` of the reference's class at width 24 instead (a 1280 x 1280 weight
would make the fixture 6 MB), everything else is what the constructor built.  The result,
wan_i2v.safetensors, is data.
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

torch.manual_seed(4242)
CLIP_DIM, N_IMG, N_TXT = 24, 257, 5  # the split at row 257 is hard-coded in CrossAttention.forward
cfg = dict(dim=40, in_dim=8, ffn_dim=48, out_dim=4, text_dim=12, freq_dim=16, eps=1e-6, patch_size=(1, 2, 2),
           num_heads=2, num_layers=2)
out = {}

with torch.no_grad():
    model = wd.WanDiT(has_image_input=True, device="cpu", dtype=torch.float32, **cfg)
    model.img_emb = wd.MLP(CLIP_DIM, cfg["dim"], device="cpu", dtype=torch.float32)
    model.eval()
    for name, p in model.named_parameters():
        if p.ndim >= 2 and "modulation" not in name:
            p.copy_(torch.randn_like(p) * 0.3)
        elif ("norm" in name or name in ("img_emb.proj.0.weight", "img_emb.proj.4.weight")) and name.endswith("weight"):
            p.copy_(1.0 + 0.3 * torch.randn_like(p))
        else:
            p.copy_(torch.randn_like(p) * 0.5)
    for k, v in model.state_dict().items():
        out["param." + k] = v.detach().clone()

    x = torch.randn(1, 4, 3, 4, 6)  # (b, c, frames, height, width) -> f,h,w = 3,2,3 = 18 tokens
    y = torch.randn(1, 4, 3, 4, 6)  # the encoded image (and mask) channels, concatenated after x
    context = torch.randn(1, N_TXT, 12)
    clip = torch.randn(1, N_IMG, CLIP_DIM)
    timestep = torch.tensor([305.0])
    out.update({"model.x": x, "model.y": y, "model.context": context, "model.clip_feature": clip,
                "model.timestep": timestep,
                "model.out": model(x, context, timestep, clip_feature=clip, y=y).contiguous(),
                "img_emb.out": model.img_emb(clip).contiguous()})

    f, h, w = 3, 2, 3
    freqs = torch.cat([model.freqs[0][:f].view(f, 1, 1, -1).expand(f, h, w, -1),
                       model.freqs[1][:h].view(1, h, 1, -1).expand(f, h, w, -1),
                       model.freqs[2][:w].view(1, 1, w, -1).expand(f, h, w, -1)], dim=-1).reshape(f * h * w, 1, -1)
    xb = torch.randn(1, f * h * w, cfg["dim"])
    cb = torch.randn(1, N_IMG + N_TXT, cfg["dim"])  # [image rows | text rows], already embedded
    t_mod = torch.randn(1, 6, cfg["dim"])
    out.update({"block.x": xb, "block.context": cb, "block.t_mod": t_mod,
                "block.freqs_real": torch.view_as_real(freqs).contiguous(),
                "block.out": model.blocks[1](xb, cb, t_mod, freqs).contiguous()})

save_file(out, os.path.join(here, "wan_i2v.safetensors"))
print(len(out), "tensors;", sum(v.numel() * v.element_size() for v in out.values()) // 1024, "KiB")
