"""Writes input/output vectors of the reference's conditioning and RoPE helper modules.

These are the functions of the path whose WIRING (chunk orders, axis concatenation order, sin/cos
order) no library routine or closed form fixes.  They live in two reference files that import only
torch, so they are loaded here by file path (the package itself is never imported), run in fp32 on
the CPU with tiny seeded inputs, and their inputs, parameters and outputs are saved:

    python tests/golden/make_leaf_module_fixtures.py [/root/reference]

  diffsynth_engine/models/basic/transformer_helper.py   AdaLayerNorm (6-way and single=True),
                                                        AdaLayerNormSingle, RoPEEmbedding, RMSNorm
  diffsynth_engine/models/basic/timestep.py             TimestepEmbeddings
  diffsynth_engine/utils/fp8_linear.py                  enable_fp8_linear + fp8_inference on one nn.Linear
                                                        (bf16, CPU torch._scaled_mm), 3-D and 2-D inputs

Runs in the build container only; the result, leaf_modules.safetensors (a few tens of KB), is data.
"""
import importlib.util
import os
import sys

import torch
from safetensors.torch import save_file

sys.dont_write_bytecode = True  # the reference tree is read-only: leave no __pycache__ in it
ref = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
here = os.path.dirname(os.path.abspath(__file__))


def load(rel, name):
    spec = importlib.util.spec_from_file_location(name, os.path.join(ref, rel))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


th = load("diffsynth_engine/models/basic/transformer_helper.py", "_ref_transformer_helper")
ts = load("diffsynth_engine/models/basic/timestep.py", "_ref_timestep")
fl = load("diffsynth_engine/utils/fp8_linear.py", "_ref_fp8_linear")

torch.manual_seed(1234)
out = {}
dim, B, S = 32, 2, 5
f32 = dict(device="cpu", dtype=torch.float32)


def put(prefix, module, **tensors):
    for k, v in module.state_dict().items():
        out[f"{prefix}.param.{k}"] = v.detach().clone()
    for k, v in tensors.items():
        out[f"{prefix}.{k}"] = v.detach().clone().contiguous()


with torch.no_grad():
    x = torch.randn(B, S, dim)
    emb = torch.randn(B, dim)

    m = th.AdaLayerNorm(dim, single=False, **f32)
    y, gate_msa, shift_mlp, scale_mlp, gate_mlp = m(x, emb)
    put("ada6", m, x=x, emb=emb, out=y, gate_msa=gate_msa, shift_mlp=shift_mlp, scale_mlp=scale_mlp,
        gate_mlp=gate_mlp)

    m = th.AdaLayerNorm(dim, single=True, **f32)
    put("ada2", m, x=x, emb=emb, out=m(x, emb))

    m = th.AdaLayerNormSingle(dim, **f32)
    y, gate = m(x, emb)
    put("ada3", m, x=x, emb=emb, out=y, gate=gate)

    axes = [4, 6, 6]
    ids = torch.stack([torch.zeros(B, S), torch.arange(S).float().repeat(B, 1) * 3 + 1,
                       torch.arange(S).float().flip(0).repeat(B, 1) + 2], dim=-1)
    m = th.RoPEEmbedding(sum(axes), 10000, axes)
    put("rope", m, ids=ids, axes=torch.tensor(axes), out=m(ids))

    m = th.RMSNorm(16, eps=1e-6, **f32)
    m.weight.copy_(torch.randn(16))
    xr = torch.randn(B, 3, S, 16)
    put("rmsnorm", m, x=xr, out=m(xr))

    m = ts.TimestepEmbeddings(dim_in=16, dim_out=dim, **f32)
    t = torch.tensor([0.0, 3.5, 999.0])
    put("timestep", m, t=t, proj=m.time_proj(t), out=m(t, torch.float32))

    lin = torch.nn.Linear(32, 48, dtype=torch.bfloat16)
    lin.weight.copy_(torch.randn(48, 32) * 0.5)
    lin.bias.copy_(torch.randn(48))
    w_bf16 = lin.weight.detach().clone()
    fl.enable_fp8_linear(lin)
    assert lin.weight.dtype == torch.float8_e4m3fn and lin.fp8_linear_enabled
    x3 = (torch.randn(2, 5, 32) * 3).to(torch.bfloat16)
    x3[0, 0, 0] = 460.0     # rounds to 448, the largest finite e4m3 value
    x2 = (torch.randn(7, 32) * 0.01).to(torch.bfloat16)   # subnormal range of e4m3
    with fl.fp8_inference(True):
        y3 = torch.nn.functional.linear(x3, lin.weight, lin.bias)
        y2 = torch.nn.functional.linear(x2, lin.weight, lin.bias)
    assert torch.nn.functional.linear is not None
    out.update({"fp8.weight_bf16": w_bf16, "fp8.weight_e4m3_bits": lin.weight.detach().view(torch.uint8).clone(),
                "fp8.bias": lin.bias.detach().clone(), "fp8.x3": x3, "fp8.y3": y3.contiguous(), "fp8.x2": x2,
                "fp8.y2": y2.contiguous()})

save_file(out, os.path.join(here, "leaf_modules.safetensors"))
print({k: tuple(v.shape) for k, v in out.items()})
