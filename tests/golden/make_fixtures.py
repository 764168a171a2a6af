"""Copies the reference-held golden DATA this path's neighbours are pinned against into tests/golden/.

Run once in the build container (the reference tree is not available on the GPU box):
    python tests/golden/make_fixtures.py [/root/reference]
Only data files are read (safetensors, which execute nothing); no reference code is imported.
  recifited_flow_20steps_flux.safetensors   sigmas[21], timesteps[20]      (copied whole, 300 B)
  flow_match_euler_i10.safetensors          origin_sample / model_output / prev_sample, F32 [1,4096,64];
                                            rows 0..255 of each are kept (192 KiB instead of 3 MiB)
"""
import os
import shutil
import sys

from safetensors.torch import load_file, save_file

ref = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
src = os.path.join(ref, "tests", "data", "expect", "algorithm")
dst = os.path.dirname(os.path.abspath(__file__))
shutil.copyfile(os.path.join(src, "recifited_flow_20steps_flux.safetensors"),
                os.path.join(dst, "recifited_flow_20steps_flux.safetensors"))
os.chmod(os.path.join(dst, "recifited_flow_20steps_flux.safetensors"), 0o644)
t = load_file(os.path.join(src, "flow_match_euler_i10.safetensors"))
save_file({k: v[:, :256].contiguous() for k, v in t.items()},
          os.path.join(dst, "flow_match_euler_i10_rows256.safetensors"))
print({k: tuple(v.shape) for k, v in t.items()})
