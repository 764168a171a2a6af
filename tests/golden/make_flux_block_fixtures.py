"""Writes input/output vectors of the reference's Flux DiT blocks and model forward at reduced size.

The wiring of FluxJointTransformerBlock, FluxSingleTransformerBlock, AdaLayerNormContinuous and
FluxDiT.forward (diffsynth_engine/models/flux/flux_dit.py) is fixed by no closed form or library
routine, and the reference's only fixture on this path needs the Flux.1-dev checkpoint.  This script
runs those classes in the build container, fp32 on the CPU, on tiny seeded inputs, and saves inputs,
parameters and outputs:

    python tests/golden/make_flux_block_fixtures.py [/root/reference]

How the file is loaded (and what is NOT the reference's here):
  * the root package's __init__ is bypassed (it pulls in the pipelines, whose dependencies modelscope,
    flufl.lock and imageio are absent): an empty module object with the real __path__ stands for
    ``diffsynth_engine`` so that the sub-modules flux_dit.py imports are the reference's own files;
  * ``diffsynth_engine.utils.gguf`` imports the third-party ``gguf`` package (absent); the only name
    flux_dit.py takes from it is the context manager ``gguf_inference``, which for ordinary (non-GGUF)
    weights calls the original F.linear unchanged; a null context stands for it;
  * the blocks take their width and head count as constructor arguments (dim 32, 2 heads of 16);
    FluxDiT.__init__ hard-codes Flux.1-dev's sizes (12 G parameters), so the model object is created
    without calling it and given sub-modules of the same classes at reduced width (2 joint + 2 single
    blocks); FluxDiT.forward, patchify, unpatchify and prepare_image_ids run unmodified.

The result, flux_blocks.safetensors (under 1 MB), is data.
"""
import contextlib
import os
import sys
import types

import torch
import torch.nn as nn
from safetensors.torch import save_file

sys.dont_write_bytecode = True  # the reference tree is read-only: leave no __pycache__ in it
ref = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
here = os.path.dirname(os.path.abspath(__file__))

root = types.ModuleType("diffsynth_engine")
root.__path__ = [os.path.join(ref, "diffsynth_engine")]
sys.modules["diffsynth_engine"] = root
gguf_stub = types.ModuleType("diffsynth_engine.utils.gguf")
gguf_stub.gguf_inference = contextlib.nullcontext
sys.modules["diffsynth_engine.utils.gguf"] = gguf_stub

from diffsynth_engine.models.flux import flux_dit as fd  # noqa: E402
from diffsynth_engine.models.basic.transformer_helper import RoPEEmbedding  # noqa: E402
from diffsynth_engine.models.basic.timestep import TimestepEmbeddings  # noqa: E402

torch.manual_seed(4321)
DIM, HEADS, AXES = 32, 2, [4, 6, 6]
N_TXT, LAT_H, LAT_W = 3, 4, 6            # 2x3 = 6 image tokens
f32 = dict(device="cpu", dtype=torch.float32)
out = {}


def randomise(module):
    # nn.Linear's default init leaves biases tiny and RMSNorm weights at 1: make every parameter matter
    for name, p in module.named_parameters():
        p.copy_(torch.randn_like(p) * (0.3 if name.endswith("weight") and p.ndim == 2 else 0.5)
                + (1.0 if p.ndim == 1 and "norm_" in name else 0.0))


def put(prefix, module, **tensors):
    for k, v in module.state_dict().items():
        out[f"{prefix}.param.{k}"] = v.detach().clone()
    for k, v in tensors.items():
        out[f"{prefix}.{k}"] = v.detach().clone().contiguous()


with torch.no_grad():
    n_img = (LAT_H // 2) * (LAT_W // 2)
    ids_txt = torch.zeros(1, N_TXT, 3)
    ids_img = torch.zeros(LAT_H // 2, LAT_W // 2, 3)
    ids_img[..., 1] += torch.arange(LAT_H // 2)[:, None]
    ids_img[..., 2] += torch.arange(LAT_W // 2)[None, :]
    ids = torch.cat([ids_txt, ids_img.reshape(1, -1, 3)], dim=1)
    rope = RoPEEmbedding(DIM, 10000, AXES)(ids)
    img = torch.randn(1, n_img, DIM)
    txt = torch.randn(1, N_TXT, DIM)
    temb = torch.randn(1, DIM)

    blk = fd.FluxJointTransformerBlock(DIM, HEADS, **f32)
    randomise(blk)
    o_img, o_txt = blk(img, txt, temb, rope)
    put("joint", blk, img=img, txt=txt, temb=temb, ids=ids, out_img=o_img, out_txt=o_txt)

    blk = fd.FluxSingleTransformerBlock(DIM, HEADS, **f32)
    randomise(blk)
    x = torch.cat([txt, img], dim=1)
    o_x, _ = blk(x, txt, temb, rope)
    put("single", blk, x=x, temb=temb, ids=ids, out=o_x)

    m = fd.AdaLayerNormContinuous(DIM, **f32)
    randomise(m)
    put("adacont", m, x=img, cond=temb, out=m(img, temb))

    model = fd.FluxDiT.__new__(fd.FluxDiT)
    nn.Module.__init__(model)
    model.pos_embedder = RoPEEmbedding(DIM, 10000, AXES)
    model.time_embedder = TimestepEmbeddings(256, DIM, **f32)
    model.guidance_embedder = TimestepEmbeddings(256, DIM, **f32)
    model.pooled_text_embedder = nn.Sequential(nn.Linear(12, DIM), nn.SiLU(), nn.Linear(DIM, DIM))
    model.context_embedder = nn.Linear(20, DIM)
    model.x_embedder = nn.Linear(64, DIM)
    model.blocks = nn.ModuleList([fd.FluxJointTransformerBlock(DIM, HEADS, **f32) for _ in range(2)])
    model.single_blocks = nn.ModuleList([fd.FluxSingleTransformerBlock(DIM, HEADS, **f32) for _ in range(2)])
    model.final_norm_out = fd.AdaLayerNormContinuous(DIM, **f32)
    model.final_proj_out = nn.Linear(DIM, 64)
    model.eval()
    randomise(model)
    latents = torch.randn(1, 16, LAT_H, LAT_W)
    inputs = dict(hidden_states=latents, timestep=torch.tensor([637.0]), prompt_emb=torch.randn(1, N_TXT, 20),
                  pooled_prompt_emb=torch.randn(1, 12), guidance=torch.tensor([3.5]), text_ids=ids_txt)
    y = model(**inputs)
    put("model", model, out=y, **inputs)

save_file(out, os.path.join(here, "flux_blocks.safetensors"))
print(len(out), "tensors;", sum(v.numel() for v in out.values()) * 4 // 1024, "KiB")
