"""Builds libdsx.so (the C-ABI library of gfx950 kernels) in-tree with hipcc.

Run as ``python -m diffsynth_engine_amd.build`` or call :func:`build_library`.
hipcc cross-compiles for gfx950 without a GPU present.
"""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB_PATH = os.path.join(HERE, "libdsx.so")
SOURCES = ["capi.hip", "quant.hip", "fp8_gemm.hip", "attn_fwd.hip", "attn_plain.hip", "attn_plain16.hip", "epilogue.hip", "lora.hip"]

# -packed-fp32-ops: keep the compiler from forming v_pk_*_f32 out of scalar float code.
HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]


def _run(cmd):
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    # the host pass does not know the amdgcn feature flag and says so once per file; drop that line
    out = "\n".join(l for l in proc.stdout.splitlines() if "is not a recognized feature" not in l)
    if proc.returncode != 0:
        raise RuntimeError("command failed: %s\n%s" % (" ".join(cmd), out))
    return out


def build_library(verbose=True):
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    objdir = os.path.join(HERE, "build")
    os.makedirs(objdir, exist_ok=True)
    objs = [os.path.join(objdir, s.replace(".hip", ".o")) for s in SOURCES]

    def compile_one(pair):
        src, obj = pair
        return _run([hipcc] + HIPCC_FLAGS + ["-c", os.path.join(CSRC, src), "-o", obj])

    with ThreadPoolExecutor(max_workers=min(len(SOURCES), 8)) as ex:
        outs = list(ex.map(compile_one, zip(SOURCES, objs)))
    outs.append(_run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB_PATH] + objs))
    if verbose:
        for o in outs:
            if o.strip():
                print(o)
        print("built", LIB_PATH)
    return LIB_PATH


if __name__ == "__main__":
    build_library()
    sys.exit(0)
