"""ctypes binding of libdsx.so (declarations follow include/dsx.h one to one).

There is no fallback: if the library has not been built, or a call is made without a gfx950
device, the error is raised to the caller.
"""
import ctypes
import os

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libdsx.so")

c_void_p = ctypes.c_void_p
c_int64 = ctypes.c_int64
c_int = ctypes.c_int
c_float = ctypes.c_float

DSX_OK = 0
DSX_EBADSHAPE = -1
DSX_EALIGN = -2
DSX_EARCH = -3
DSX_ELAUNCH = -4
DSX_ENULL = -5
DSX_EWORKSPACE = -6
ABI_VERSION = 7


class AttnParams(ctypes.Structure):
    """Mirror of ``dsx_attn_params``."""

    _fields_ = [
        ("q", c_void_p * 2),
        ("k", c_void_p * 2),
        ("v", c_void_p * 2),
        ("o", c_void_p * 2),
        ("sq", c_int64 * 2),
        ("skv", c_int64 * 2),
        ("q_sb", c_int64 * 2), ("q_sh", c_int64 * 2), ("q_ss", c_int64 * 2),
        ("k_sb", c_int64 * 2), ("k_sh", c_int64 * 2), ("k_ss", c_int64 * 2),
        ("v_sb", c_int64 * 2), ("v_sh", c_int64 * 2), ("v_ss", c_int64 * 2),
        ("o_sb", c_int64 * 2), ("o_sh", c_int64 * 2), ("o_ss", c_int64 * 2),
        ("batch", ctypes.c_int32), ("heads", ctypes.c_int32), ("head_dim", ctypes.c_int32),
        ("softmax_scale", c_float),
        ("rope", c_void_p),
        ("rope_sb", c_int64),
        ("rope_rows", c_int64),
        ("q_norm_w", c_void_p * 2),
        ("k_norm_w", c_void_p * 2),
        ("norm_eps", c_float),
        ("score_bound", ctypes.c_float),
        ("workspace", c_void_p),
        ("workspace_bytes", c_int64),
        ("qk_norm2_max", c_void_p),
    ]


class GemmProblem(ctypes.Structure):
    """Mirror of ``dsx_gemm_problem``."""

    _fields_ = [
        ("a", c_void_p), ("lda", c_int64),
        ("w", c_void_p), ("ldw", c_int64),
        ("a_scale", c_void_p),
        ("w_scale", c_void_p),
        ("bias", c_void_p),
        ("resid", c_void_p), ("ldr", c_int64),
        ("gate", c_void_p), ("gate_sb", c_int64),
        ("rows_per_batch", c_int64),
        ("out", c_void_p), ("ldo", c_int64),
        ("M", c_int64), ("N", c_int64), ("K", c_int64),
        ("q_norm_w", c_void_p), ("k_norm_w", c_void_p),
        ("rope", c_void_p), ("rope_sb", c_int64), ("rope_pos0", c_int64), ("rope_rows", c_int64),
        ("norm_eps", c_float),
        ("qk_heads", ctypes.c_int32),
        ("a_ext", c_void_p), ("lda_ext", c_int64),
        ("w_ext", c_void_p), ("ldw_ext", c_int64),
        ("K_ext", c_int64),
    ]


GEMM_GROUP_MAX = 4

# name -> (restype, argtypes); every symbol include/dsx.h declares
SIGNATURES = {
    "dsx_abi_version": (c_int, []),
    "dsx_strerror": (ctypes.c_char_p, [c_int]),
    "dsx_check_device": (c_int, []),
    "dsx_quant_fp8_rowwise": (c_int, [c_void_p, c_int64, c_void_p, c_int64, c_void_p, c_int64, c_int64, c_void_p]),
    "dsx_absmax": (c_int, [c_void_p, c_int64, c_int, c_void_p, c_void_p]),
    "dsx_cast_fp8_scaled": (c_int, [c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int64, c_void_p]),
    "dsx_fp8_gemm": (c_int, [c_void_p, c_int64, c_void_p, c_int64, c_void_p, c_void_p, c_void_p, c_void_p,
                             c_int64, c_int64, c_int64, c_int64, c_void_p]),
    "dsx_fp8_gemm_gated_residual": (c_int, [c_void_p, c_int64, c_void_p, c_int64, c_void_p, c_void_p, c_void_p,
                                            c_void_p, c_int64, c_void_p, c_int64, c_int64, c_void_p, c_int64,
                                            c_int64, c_int64, c_int64, c_void_p]),
    "dsx_fp8_gemm_grouped": (c_int, [ctypes.POINTER(GemmProblem), c_int, c_void_p]),
    "dsx_lora_down": (c_int, [c_void_p, c_int64, c_void_p, c_int64, c_void_p, c_void_p, c_int64, c_int64, c_int64,
                              c_int64, c_int64, c_int64, c_int64, c_void_p]),
    "dsx_fp8_gemv_rowscale": (c_int, [c_void_p, c_int64, c_void_p, c_int64, c_void_p, c_void_p, c_void_p, c_void_p,
                                      c_int64, c_int64, c_int64, c_int64, c_void_p]),
    "dsx_concat_gelu_tanh": (c_int, [c_void_p, c_int64, c_int64, c_void_p, c_int64, c_void_p, c_int64, c_void_p,
                                     c_int64, c_void_p, c_int64, c_int64, c_void_p]),
    "dsx_attn_fwd": (c_int, [ctypes.POINTER(AttnParams), c_void_p]),
    "dsx_attn_workspace_bytes": (c_int64, [ctypes.POINTER(AttnParams)]),
    "dsx_attn_fwd_static": (c_int, [ctypes.POINTER(AttnParams), c_void_p]),
    "dsx_attn_static_scratch_bytes": (c_int64, []),
    "dsx_rmsnorm_rope": (c_int, [c_void_p, c_int64, c_int64, c_int64, c_void_p, c_float, c_void_p, c_int64,
                                 c_int64, c_void_p, c_int64, c_int64, c_int64, ctypes.c_int32, ctypes.c_int32,
                                 c_int64, c_void_p]),
    "dsx_rmsnorm_rope_qk": (c_int, [c_void_p, c_int64, c_int64, ctypes.c_int32, ctypes.c_int32, c_void_p, c_void_p,
                                    c_float, c_void_p, c_int64, c_int64, ctypes.c_int32, c_int64, c_void_p]),
    "dsx_rmsnorm_rows": (c_int, [c_void_p, c_int64, c_void_p, c_float, c_void_p, c_int64, c_int64, c_void_p, c_int64,
                                 c_int64, c_int64, c_void_p, c_void_p]),
    "dsx_adaln_modulate": (c_int, [c_void_p, c_int64, c_void_p, c_void_p, c_int64, c_int64, c_void_p, c_void_p,
                                   c_float, c_void_p, c_int64, c_void_p, c_int64, c_void_p, c_int64, c_int64,
                                   c_void_p]),
    "dsx_gated_residual": (c_int, [c_void_p, c_int64, c_void_p, c_int64, c_void_p, c_int64, c_int64, c_void_p,
                                   c_int64, c_int64, c_int64, c_void_p]),
    "dsx_gelu_tanh": (c_int, [c_void_p, c_int64, c_void_p, c_int64, c_void_p, c_int64, c_void_p, c_int64, c_int64,
                              c_void_p]),
    "dsx_gelu_erf": (c_int, [c_void_p, c_int64, c_void_p, c_int64, c_void_p, c_int64, c_void_p, c_int64, c_int64,
                             c_void_p]),
    "dsx_flow_match_euler_step": (c_int, [c_void_p, c_void_p, c_float, c_void_p, c_int64, c_int, c_void_p]),
    "dsx_mfma_ceiling_probe": (c_int, [c_int, c_void_p, c_int64, ctypes.c_int32, c_void_p, ctypes.POINTER(c_int64),
                                       c_void_p]),
}

_lib = None


def load():
    """Load libdsx.so once and attach argument types.  Raises ImportError if it is not built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            "libdsx.so is not built (%s missing); run `python -m diffsynth_engine_amd.build`" % LIB_PATH
        )
    try:
        lib = ctypes.CDLL(LIB_PATH)
    except OSError as e:  # missing HIP runtime etc.
        raise ImportError("cannot load %s: %s" % (LIB_PATH, e)) from e
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    if lib.dsx_abi_version() != ABI_VERSION:
        raise ImportError("libdsx.so ABI version %d, expected %d" % (lib.dsx_abi_version(), ABI_VERSION))
    _lib = lib
    return lib


def strerror(code):
    return load().dsx_strerror(code).decode()


def check(code, what):
    """Turn a DSX_* return code into the exception the reference's conventions call for."""
    if code == DSX_OK:
        return
    msg = "%s: %s (dsx error %d)" % (what, strerror(code), code)
    if code in (DSX_EARCH, DSX_ELAUNCH):
        raise RuntimeError(msg)
    raise ValueError(msg)
