"""Writes input/output vectors of the reference's Flux DiT forward UNDER ITS FP8 PATCH at head dim 128.

flux_blocks.safetensors (make_flux_block_fixtures.py) is fp32 at head dim 16: the oracle can read it, the HIP
kernels (head dim 128, e4m3 linears) cannot.  This script runs the reference's own classes in bf16 on the CPU
with ``enable_fp8_linear`` + ``fp8_inference`` active (diffsynth_engine/utils/fp8_linear.py:7-64: bare e4m3
casts, unit scales, torch._scaled_mm), at a size the kernels accept directly: hidden 256 = 2 heads x 128, RoPE
axes (16,56,56), 1 joint + 1 single block, 24 text + 24 image tokens:

    python tests/golden/make_flux_fp8_fixture.py [/root/reference]

Loading follows make_flux_block_fixtures.py: the root package's __init__ is bypassed (its pipelines need
modelscope / flufl.lock / imageio, absent here), a null context stands for ``gguf_inference`` (module needs the
absent ``gguf`` package; for ordinary weights it calls F.linear unchanged), and FluxDiT.__init__ (which
hard-codes Flux.1-dev's 12 G parameters) is not called: the model object gets sub-modules of the reference's
classes at reduced width and FluxDiT.forward runs unmodified.

Weights are drawn N(0, 1/fan_in) so that activations stay far below 448 (the reference's cast does not
saturate).  Linear weights are saved as the e4m3 bytes enable_fp8_linear left in the module (uint8), everything
else as bf16.  The result, flux_fp8_d128.safetensors (~3.6 MB), is data.
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
from diffsynth_engine.utils.fp8_linear import enable_fp8_linear  # noqa: E402

torch.manual_seed(1234)
DIM, HEADS, AXES = 256, 2, [16, 56, 56]
N_TXT, LAT_H, LAT_W = 24, 8, 12  # 4 x 6 = 24 image tokens
TXT_DIM, POOLED_DIM = 64, 32
bf = dict(device="cpu", dtype=torch.bfloat16)
out = {}

with torch.no_grad():
    model = fd.FluxDiT.__new__(fd.FluxDiT)
    nn.Module.__init__(model)
    model.pos_embedder = RoPEEmbedding(DIM, 10000, AXES)
    model.time_embedder = TimestepEmbeddings(256, DIM, **bf)
    model.guidance_embedder = TimestepEmbeddings(256, DIM, **bf)
    model.pooled_text_embedder = nn.Sequential(nn.Linear(POOLED_DIM, DIM, **bf), nn.SiLU(), nn.Linear(DIM, DIM, **bf))
    model.context_embedder = nn.Linear(TXT_DIM, DIM, **bf)
    model.x_embedder = nn.Linear(64, DIM, **bf)
    model.blocks = nn.ModuleList([fd.FluxJointTransformerBlock(DIM, HEADS, **bf)])
    model.single_blocks = nn.ModuleList([fd.FluxSingleTransformerBlock(DIM, HEADS, **bf)])
    model.final_norm_out = fd.AdaLayerNormContinuous(DIM, **bf)
    model.final_proj_out = nn.Linear(DIM, 64, **bf)
    model.eval()
    for name, p in model.named_parameters():
        if p.ndim == 2:  # Linear weight: keep every layer's output O(1); AdaLN projections half of that
            std = (0.5 if ".norm" in name or "norm_out" in name else 1.0) / p.shape[1] ** 0.5
            p.copy_((torch.randn(p.shape) * std).to(p.dtype))
        elif name.endswith(".bias"):
            p.copy_((torch.randn(p.shape) * 0.1).to(p.dtype))
        else:  # RMSNorm weights
            p.copy_((1.0 + 0.2 * torch.randn(p.shape)).to(p.dtype))
    enable_fp8_linear(model)  # the reference's: weights -> float8_e4m3fn in place, fp8_linear_enabled = True
    assert model.fp8_linear_enabled and model.x_embedder.weight.dtype == torch.float8_e4m3fn
    inputs = dict(hidden_states=torch.randn(1, 16, LAT_H, LAT_W).bfloat16(), timestep=torch.tensor([637.0]),
                  prompt_emb=torch.randn(1, N_TXT, TXT_DIM).bfloat16(),
                  pooled_prompt_emb=torch.randn(1, POOLED_DIM).bfloat16(), guidance=torch.tensor([3.5]),
                  text_ids=torch.zeros(1, N_TXT, 3))
    y = model(**inputs)  # FluxDiT.forward enters fp8_inference itself (flux_dit.py:404-405)
    assert y.dtype == torch.bfloat16 and torch.isfinite(y.float()).all()
    for k, v in model.state_dict().items():
        out["param." + k] = v.view(torch.uint8).clone() if v.dtype == torch.float8_e4m3fn else v.clone()
    for k, v in inputs.items():
        out["in." + k] = v.clone().contiguous()
    out["out"] = y.clone().contiguous()

save_file(out, os.path.join(here, "flux_fp8_d128.safetensors"))
print(len(out), "tensors;", sum(v.numel() * v.element_size() for v in out.values()) // 1024, "KiB; |out| max",
      float(y.float().abs().max()), "std", float(y.float().std()))
