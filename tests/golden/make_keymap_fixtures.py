"""Writes input/output vectors of the reference's Flux checkpoint key conversion.

FluxDiTStateDictConverter.convert (diffsynth_engine/models/flux/flux_dit.py:24-123) renames and re-packs
third-party checkpoints; which names map where is data no formula fixes.  This script feeds the
reference's own converter synthetic state dicts in the original ("civitai") and the diffusers layouts --
every key its tables know, for two joint and two single blocks, tiny tensors (each filled with its own
value so that concatenation order and the swapped halves of the final modulation show), plus keys it must
drop -- and saves what went in and what came out:

    python tests/golden/make_keymap_fixtures.py [/root/reference]

The reference module is loaded as in make_flux_block_fixtures.py (root package __init__ bypassed, a null
context for gguf_inference).  The result, flux_keymaps.safetensors, is data.
"""
import contextlib
import json
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
gguf_stub = types.ModuleType("diffsynth_engine.utils.gguf")
gguf_stub.gguf_inference = contextlib.nullcontext
sys.modules["diffsynth_engine.utils.gguf"] = gguf_stub

from diffsynth_engine.models.flux import flux_dit as fd  # noqa: E402

tables = json.load(open(os.path.join(ref, "diffsynth_engine", "conf", "models", "flux", "flux_dit.json")))
counter = [0]


def tensor(name):
    counter[0] += 1
    rows = 6144 if "adaLN_modulation" in name else 4   # the converter swaps this one at row 3072
    shape = (rows,) if name.endswith(("bias", "scale")) else (rows, 2)
    return torch.full(shape, float(counter[0])) + torch.arange(rows).reshape(-1, *([1] * (len(shape) - 1))) / 8192.0


civitai = {}
for k in tables["civitai"]["rename_dict"]:
    civitai["model.diffusion_model." + k] = tensor(k)
for k in tables["civitai"]["suffix_rename_dict"]:
    for n in (0, 1):
        block = "double_blocks" if k.startswith(("img_", "txt_")) else "single_blocks"
        civitai[f"model.diffusion_model.{block}.{n}.{k}"] = tensor(k)
civitai["model.diffusion_model.not_a_flux_key.weight"] = tensor("x.weight")

diffusers = {}
for k in tables["diffusers"]["global_rename_dict"]:
    for leaf in ("weight", "bias"):
        diffusers[f"{k}.{leaf}"] = tensor(leaf)
for k in tables["diffusers"]["rename_dict"]:
    for n in (0, 1):
        for leaf in ("weight", "bias"):
            diffusers[f"transformer_blocks.{n}.{k}.{leaf}"] = tensor(leaf)
for k in tables["diffusers"]["rename_dict_single"]:
    for n in (0, 1):
        for leaf in ("weight", "bias"):
            diffusers[f"single_transformer_blocks.{n}.{k}.{leaf}"] = tensor(leaf)
diffusers["transformer_blocks.0.unknown_module.weight"] = tensor("x.weight")

conv = fd.FluxDiTStateDictConverter()
out = {}
for tag, sd in (("civitai", civitai), ("diffusers", diffusers)):
    res = conv.convert(dict(sd))
    for k, v in sd.items():
        out[f"in.{tag}::{k}"] = v.clone()
    for k, v in res.items():
        out[f"out.{tag}::{k}"] = v.clone()
    print(tag, len(sd), "->", len(res))
save_file(out, os.path.join(here, "flux_keymaps.safetensors"))
print(sum(v.numel() * 4 for v in out.values()) // 1024, "KiB")
