"""CPU-side checks of the drop-in boundary: the library loads, exports every declared symbol,
and the host-side mirrors keep the reference's error conventions.  No kernel is launched."""
import ctypes
import os
import re

import pytest
import torch
import torch.nn.functional as F

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_symbols():
    text = open(os.path.join(ROOT, "include", "dsx.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(dsx_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    from diffsynth_engine_amd import _lib

    lib = _lib.load()
    names = _declared_symbols()
    assert len(names) >= 12
    for n in names:
        assert hasattr(lib, n), n
    assert sorted(_lib.SIGNATURES) == names  # the ctypes table and the header agree


def test_abi_version_and_strerror():
    from diffsynth_engine_amd import _lib

    lib = _lib.load()
    assert lib.dsx_abi_version() == 7
    assert _lib.strerror(0) == "ok"
    for code in (-1, -2, -3, -4, -5, -6):
        assert _lib.strerror(code) and "unknown" not in _lib.strerror(code)
    assert "unknown" in _lib.strerror(-99)


def test_attn_params_struct_layout_matches_header():
    from diffsynth_engine_amd import _lib

    # q,k,v,o,sq,skv = 6*16; 12 stride pairs * 16; 3 int32 + float; rope, rope_sb, rope_rows;
    # 2*16 norm pointers; two floats; workspace pointer + byte count
    assert ctypes.sizeof(_lib.AttnParams) == 6 * 16 + 12 * 16 + 16 + 8 + 8 + 8 + 32 + 8 + 16 + 8


def test_null_and_shape_errors_without_touching_the_gpu():
    from diffsynth_engine_amd import _lib

    lib = _lib.load()
    assert lib.dsx_fp8_gemm(None, 16, None, 16, None, None, None, None, 16, 16, 16, 16, None) == _lib.DSX_ENULL
    buf = ctypes.create_string_buffer(4096)
    p = ctypes.addressof(buf)
    p16 = (p + 15) & ~15
    assert lib.dsx_fp8_gemm(p16, 24, p16, 24, None, None, None, p16, 16, 16, 16, 24, None) == _lib.DSX_EBADSHAPE
    assert lib.dsx_fp8_gemm(p16 + 1, 16, p16, 16, None, None, None, p16, 16, 16, 16, 16, None) == _lib.DSX_EALIGN
    assert lib.dsx_quant_fp8_rowwise(p16, 12, p16, 12, None, 4, 12, None) == _lib.DSX_EBADSHAPE
    assert lib.dsx_attn_fwd(None, None) == _lib.DSX_ENULL
    P = _lib.AttnParams()
    P.head_dim, P.batch, P.heads = 64, 1, 1
    assert lib.dsx_attn_fwd(P, None) == _lib.DSX_EBADSHAPE
    assert lib.dsx_gelu_tanh(p16, 8, None, 8, None, 8, None, 1, 8, None) == _lib.DSX_ENULL
    assert lib.dsx_adaln_modulate(p16, 12, None, None, 0, 1, None, None, 1e-6, p16, 12, None, 0, None, 1, 12,
                                  None) == _lib.DSX_EBADSHAPE
    with pytest.raises(ValueError):
        _lib.check(_lib.DSX_EALIGN, "x")
    with pytest.raises(RuntimeError):
        _lib.check(_lib.DSX_EARCH, "x")


def test_missing_library_is_an_import_error(monkeypatch):
    from diffsynth_engine_amd import _lib

    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", "/nonexistent/libdsx.so")
    with pytest.raises(ImportError):
        _lib.load()


def test_attention_name_validation_mirrors_reference():
    """Unknown implementation names raise ValueError (flux_dit.py:483-486)."""
    import types

    from diffsynth_engine_amd import mi355x_attention, set_attn_implementation

    with pytest.raises(ValueError):
        set_attn_implementation("sage_attn_typo")
    fake = types.SimpleNamespace(_attn_func=F.scaled_dot_product_attention)
    set_attn_implementation("mi355x", flux_dit_module=fake)
    assert fake._attn_func is mi355x_attention
    set_attn_implementation("sdpa", flux_dit_module=fake)
    assert fake._attn_func is F.scaled_dot_product_attention


def test_cpu_tensors_are_refused_not_silently_computed():
    from diffsynth_engine_amd import mi355x_attention, ops

    q = torch.zeros(1, 1, 8, 128, dtype=torch.bfloat16)
    with pytest.raises(RuntimeError):
        mi355x_attention(q, q, q)
    with pytest.raises(RuntimeError):
        ops.quantize_fp8(torch.zeros(2, 16, dtype=torch.bfloat16))


def test_fp8_inference_patches_and_restores_f_linear():
    """Same observable behaviour as fp8_linear.py:20-64; additionally restores on exceptions."""
    from diffsynth_engine_amd import fp8_inference
    from diffsynth_engine_amd import fp8_linear as mod

    orig = F.linear
    with fp8_inference(False):
        assert F.linear is orig
    with fp8_inference():
        assert F.linear is mod.fp8_linear
    assert F.linear is orig
    with pytest.raises(KeyError):
        with fp8_inference(True):
            raise KeyError("boom")
    assert F.linear is orig


def test_graft_entry_build_checks_pass_on_the_built_library(monkeypatch):
    """build() compiles and then checks the import and the ABI version; here the compile step is skipped and
    the checks run against the library already in the tree."""
    import __graft_entry__ as entry
    from diffsynth_engine_amd import build as build_mod

    monkeypatch.setattr(build_mod, "build_library", lambda verbose=True: build_mod.LIB_PATH)
    entry.build()


def test_attention_workspace_size_query():
    """dsx_attn_workspace_bytes needs no GPU: with RoPE / q-k RMSNorm requested it asks for the bf16 copy of k
    (q is treated inside the attention kernel), otherwise (no GPU to split work over) for nothing."""
    from diffsynth_engine_amd import _lib

    lib = _lib.load()
    P = _lib.AttnParams()
    P.sq[0], P.sq[1], P.skv[0], P.skv[1] = 512, 4096, 512, 4096
    P.batch, P.heads, P.head_dim = 2, 24, 128
    if not torch.cuda.is_available():
        assert lib.dsx_attn_workspace_bytes(P) == 0
    buf = ctypes.create_string_buffer(64)
    P.k_norm_w[0] = ctypes.addressof(buf)
    need = lib.dsx_attn_workspace_bytes(P)
    assert need >= 2 * 2 * 24 * 4608 * 128
    if not torch.cuda.is_available():
        assert need == 2 * 2 * 24 * 4608 * 128
    P.head_dim = 64
    assert lib.dsx_attn_workspace_bytes(P) == 0
    assert lib.dsx_attn_workspace_bytes(None) == 0


def test_graphed_step_refuses_host_inputs():
    """A host tensor cannot be an input of a recorded step (its copy to the device cannot be recorded): refused
    before anything touches the GPU."""
    import torch

    from diffsynth_engine_amd.graph import GraphedStep

    with pytest.raises(RuntimeError):
        GraphedStep(lambda **kw: None, x=torch.zeros(4))


def _host_attn_params(buf, sq=64, skv=64):
    """dsx_attn_params over a host buffer: good enough for everything dsx_attn_fwd checks before it launches."""
    from diffsynth_engine_amd import _lib

    p16 = (ctypes.addressof(buf) + 15) & ~15
    P = _lib.AttnParams()
    for name in ("q", "k", "v", "o"):
        getattr(P, name)[0] = p16
        getattr(P, name + "_sb")[0], getattr(P, name + "_sh")[0], getattr(P, name + "_ss")[0] = 0, 128, 128
    P.sq[0], P.skv[0], P.batch, P.heads, P.head_dim = sq, skv, 1, 1, 128
    P.softmax_scale = 0.0884
    return P, p16


def test_attention_refuses_what_its_kernels_would_mis_address():
    """Checked on the host before any launch: overlapping key/value rows, a RoPE table with fewer rows than the
    joint sequence, RoPE with Sq != Skv, and k-side pre-processing without the scratch it needs."""
    from diffsynth_engine_amd import _lib

    lib = _lib.load()
    buf = ctypes.create_string_buffer(1 << 16)
    P, p16 = _host_attn_params(buf)
    P.k_ss[0] = 64
    assert lib.dsx_attn_fwd(P, None) == _lib.DSX_EBADSHAPE
    P, p16 = _host_attn_params(buf)
    P.v_ss[0] = 120
    assert lib.dsx_attn_fwd(P, None) == _lib.DSX_EBADSHAPE
    P, p16 = _host_attn_params(buf)
    P.rope, P.rope_rows = p16, 63  # one row short
    assert lib.dsx_attn_fwd(P, None) == _lib.DSX_EBADSHAPE
    P.rope_rows = 64
    assert lib.dsx_attn_fwd(P, None) == _lib.DSX_EWORKSPACE  # k has to be rotated into scratch that was not given
    P.workspace, P.workspace_bytes = p16, 2 * 64 * 128 - 16
    assert lib.dsx_attn_fwd(P, None) == _lib.DSX_EWORKSPACE  # too small
    P, p16 = _host_attn_params(buf, sq=64, skv=32)
    P.rope, P.rope_rows = p16, 64
    assert lib.dsx_attn_fwd(P, None) == _lib.DSX_EBADSHAPE  # fused RoPE is for self / joint attention
    P, p16 = _host_attn_params(buf)
    P.k_norm_w[0] = p16
    assert lib.dsx_attn_fwd(P, None) == _lib.DSX_EWORKSPACE
    with pytest.raises(ValueError):
        _lib.check(_lib.DSX_EWORKSPACE, "x")


def test_device_side_score_bound_and_head_norm_guards():
    """qk_norm2_max describes q and k as given, so it is refused together with any fused pre-processing (before the
    scratch question is even asked) and when misaligned; head_norm2_max needs rows made of whole 128-wide heads; the
    probe knows eight kinds."""
    from diffsynth_engine_amd import _lib

    lib = _lib.load()
    buf = ctypes.create_string_buffer(1 << 16)
    P, p16 = _host_attn_params(buf)
    P.qk_norm2_max = p16 + 2
    assert lib.dsx_attn_fwd(P, None) == _lib.DSX_EALIGN
    P.qk_norm2_max = p16
    P.q_norm_w[0] = p16
    assert lib.dsx_attn_fwd(P, None) == _lib.DSX_EBADSHAPE
    P, p16 = _host_attn_params(buf)
    P.qk_norm2_max, P.rope, P.rope_rows = p16, p16, 64
    assert lib.dsx_attn_fwd(P, None) == _lib.DSX_EBADSHAPE
    assert lib.dsx_attn_fwd_static(P, None) == _lib.DSX_EBADSHAPE
    # dsx_rmsnorm_rows(x, ldx, w, eps, rope, rope_sb, rows_per_batch, out, ldo, rows, D, head_norm2_max, stream)
    assert lib.dsx_rmsnorm_rows(p16, 192, p16, 1e-6, None, 0, 4, p16, 192, 4, 192, p16, None) == _lib.DSX_EBADSHAPE
    assert lib.dsx_rmsnorm_rows(p16, 256, p16, 1e-6, None, 0, 4, p16, 256, 4, 256, p16 + 2, None) == _lib.DSX_EALIGN
    assert lib.dsx_rmsnorm_rows(p16, 256, p16, 1e-6, None, 0, 4, p16, 256, 0, 256, p16, None) == _lib.DSX_OK  # no rows
    for kind in (-1, 8):
        assert lib.dsx_mfma_ceiling_probe(kind, p16, 1, 1, p16, None, None) == _lib.DSX_EBADSHAPE
    assert lib.dsx_mfma_ceiling_probe(7, None, 1, 1, p16, None, None) == _lib.DSX_ENULL
    assert lib.dsx_gelu_erf(p16, 12, p16, 12, None, 0, None, 4, 12, None) == _lib.DSX_EBADSHAPE  # D % 8


def test_gemm_refuses_leading_dimensions_beyond_its_32_bit_tile_offsets():
    from diffsynth_engine_amd import _lib

    lib = _lib.load()
    buf = ctypes.create_string_buffer(4096)
    p16 = (ctypes.addressof(buf) + 15) & ~15
    big = 1 << 24
    assert lib.dsx_fp8_gemm(p16, big, p16, 128, None, None, None, p16, 256, 16, 256, 128, None) == _lib.DSX_EBADSHAPE
    assert lib.dsx_fp8_gemm(p16, 128, p16, big, None, None, None, p16, 256, 16, 256, 128, None) == _lib.DSX_EBADSHAPE
    n = 1 << 30  # 2^24 x 2^24 tiles of 64 x 64
    assert lib.dsx_fp8_gemm(p16, 128, p16, 128, None, None, None, p16, n, n, n, 128, None) == _lib.DSX_EBADSHAPE


def test_gemm_problem_struct_layout_and_qk_epilogue_checks():
    """dsx_gemm_problem: 17 eight-byte fields, then the q/k epilogue's two weight pointers, table pointer, three
    int64, a float and an int32.  The q/k epilogue is refused (before any launch) with a residual, with fewer columns
    than 2 * heads * 128, with a RoPE table that ends before the last token's row, and outside the tile kernel's shapes."""
    from diffsynth_engine_amd import _lib

    assert ctypes.sizeof(_lib.GemmProblem) == 17 * 8 + 2 * 8 + 8 + 3 * 8 + 4 + 4 + 5 * 8
    lib = _lib.load()
    buf = ctypes.create_string_buffer(1 << 12)
    p16 = (ctypes.addressof(buf) + 15) & ~15

    def problem(**kw):
        base = dict(a=p16, lda=128, w=p16, ldw=128, out=p16, ldo=512, M=64, N=512, K=128, rows_per_batch=64,
                    qk_heads=2, rope=p16, rope_rows=64, norm_eps=1e-6)
        base.update(kw)
        return (_lib.GemmProblem * 1)(_lib.GemmProblem(**base))

    assert lib.dsx_fp8_gemm_grouped(problem(resid=p16, ldr=512), 1, None) == _lib.DSX_EBADSHAPE
    assert lib.dsx_fp8_gemm_grouped(problem(qk_heads=3), 1, None) == _lib.DSX_EBADSHAPE       # 768 columns needed
    assert lib.dsx_fp8_gemm_grouped(problem(rope_rows=63), 1, None) == _lib.DSX_EBADSHAPE
    assert lib.dsx_fp8_gemm_grouped(problem(rope_pos0=1), 1, None) == _lib.DSX_EBADSHAPE       # rows 1..64 of 64
    assert lib.dsx_fp8_gemm_grouped(problem(K=144, lda=144, ldw=144), 1, None) == _lib.DSX_EBADSHAPE  # K % 128
    assert lib.dsx_fp8_gemm_grouped(problem(M=8), 1, None) == _lib.DSX_EBADSHAPE               # the GEMV path has none
    assert lib.dsx_fp8_gemm_grouped(problem(rope=p16 + 4), 1, None) == _lib.DSX_EALIGN


def test_header_compiles_as_c99_and_agrees_with_the_ctypes_mirrors(tmp_path):
    """include/dsx.h is a C header (the boundary is a C ABI): it has to compile with a C compiler, and the struct
    sizes a C caller sees must be the ones the ctypes mirrors use."""
    import shutil
    import subprocess

    from diffsynth_engine_amd import _lib

    cc = shutil.which("gcc") or shutil.which("cc")
    if cc is None:
        pytest.skip("no C compiler")
    src = tmp_path / "h.c"
    src.write_text('#include <stdio.h>\n#include "dsx.h"\nint main(void) { printf("%zu %zu %d %lld\\n", '
                   'sizeof(dsx_attn_params), sizeof(dsx_gemm_problem), DSX_ABI_VERSION, '
                   '(long long)DSX_ATTN_STATIC_SCRATCH_BYTES); return 0; }\n')
    exe = tmp_path / "h"
    subprocess.run([cc, "-std=c99", "-Wall", "-Wextra", "-pedantic", "-Werror", "-I", os.path.join(ROOT, "include"),
                    str(src), "-o", str(exe)], check=True)
    attn, gemm, abi, scratch = map(int, subprocess.run([str(exe)], check=True, capture_output=True, text=True).stdout.split())
    assert attn == ctypes.sizeof(_lib.AttnParams) and gemm == ctypes.sizeof(_lib.GemmProblem)
    assert abi == _lib.ABI_VERSION == _lib.load().dsx_abi_version()
    assert scratch == _lib.load().dsx_attn_static_scratch_bytes()
