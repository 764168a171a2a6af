"""Tensor-level wrappers of the C-ABI kernels.

PyTorch is used for device memory and the current stream only; every function below launches
hand-written gfx950 kernels from libdsx.so on ``torch.cuda.current_stream()`` and raises if the
library is missing or the tensors are not on a GPU.
"""
import math
from typing import Optional, Tuple

import torch

from . import _lib

FP8 = torch.float8_e4m3fn
_BF16 = torch.bfloat16


def _stream():
    return torch.cuda.current_stream().cuda_stream


def _ptr(t: Optional[torch.Tensor]):
    return None if t is None else t.data_ptr()


def _require_cuda(*tensors):
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise RuntimeError("diffsynth_engine_amd kernels need tensors on an MI355X device, got %s" % t.device)


def _rows_2d(x: torch.Tensor) -> Tuple[torch.Tensor, int]:
    """View x as (rows, D) with unit stride in the last dim; returns the view and its row stride."""
    if x.stride(-1) != 1:
        x = x.contiguous()
    D = x.shape[-1]
    if x.dim() == 2:
        return x, x.stride(0)
    x2 = x.reshape(-1, D) if x.is_contiguous() else None
    if x2 is None:
        # a column slice of a contiguous (…, Dfull) buffer keeps a uniform row stride
        ld = x.stride(-2)
        ok = all(x.stride(i) == x.stride(i + 1) * x.shape[i + 1] for i in range(x.dim() - 2))
        if not ok:
            x = x.contiguous()
            return x.reshape(-1, D), D
        x2 = x.as_strided((x.numel() // D, D), (ld, 1), x.storage_offset())
        return x2, ld
    return x2, D


def quantize_fp8(x: torch.Tensor, scaled: bool = True):
    """bf16 (…,K) -> (e4m3 (…,K), per-row fp32 scales or None).

    ``scaled=False`` is the reference's bare ``input.to(torch.float8_e4m3fn)``
    (diffsynth_engine/utils/fp8_linear.py:35); ``scaled=True`` divides each row by absmax/448 first.
    """
    _require_cuda(x)
    if x.dtype != _BF16:
        raise ValueError("quantize_fp8 expects bf16, got %s" % x.dtype)
    x2, ldx = _rows_2d(x)
    M, K = x2.shape
    q = torch.empty((M, K), dtype=FP8, device=x.device)
    scale = torch.empty((M,), dtype=torch.float32, device=x.device) if scaled else None
    rc = _lib.load().dsx_quant_fp8_rowwise(_ptr(x2), ldx, _ptr(q), K, _ptr(scale), M, K, _stream())
    _lib.check(rc, "dsx_quant_fp8_rowwise")
    return q.view(*x.shape[:-1], K), scale


def quantize_weight_fp8(w: torch.Tensor, scaled: bool = True):
    """Weight cast of enable_fp8_linear (fp8_linear.py:15): returns (e4m3 weight, 0-dim fp32 scale or None)."""
    _require_cuda(w)
    if w.dtype not in (_BF16, torch.float32):
        w = w.to(_BF16)
    w = w.contiguous()
    lib = _lib.load()
    is_fp32 = int(w.dtype == torch.float32)
    scale = amax = None
    if scaled:
        amax = torch.zeros((), dtype=torch.float32, device=w.device)
        scale = torch.empty((), dtype=torch.float32, device=w.device)
        _lib.check(lib.dsx_absmax(_ptr(w), w.numel(), is_fp32, _ptr(amax), _stream()), "dsx_absmax")
    q = torch.empty(w.shape, dtype=FP8, device=w.device)
    _lib.check(lib.dsx_cast_fp8_scaled(_ptr(w), is_fp32, _ptr(amax), _ptr(scale), _ptr(q), w.numel(), _stream()),
               "dsx_cast_fp8_scaled")
    return q, scale


def _gemm_problem(a_q, w_q, a_scale=None, w_scale=None, bias=None, out=None, resid=None, gate=None,
                  rows_per_batch=None, qk=None, ext=None):
    """Validate one GEMM and describe it as a ``dsx_gemm_problem``; returns (problem, out, keep-alive refs).

    ``qk``: optional dict(heads=H, q_norm_w=, k_norm_w=, rope=(B|1, S, 64, 2) fp32 table or None, pos0=, eps=) for a
    packed qkv projection: per-head RMSNorm + RoPE of the q and k heads in the GEMM's epilogue (rows_per_batch =
    tokens per batch entry; token t of an entry takes table row pos0 + t)."""
    _require_cuda(a_q, w_q)
    if a_q.dtype != FP8 or w_q.dtype != FP8:
        raise ValueError("fp8_gemm expects float8_e4m3fn operands")
    if a_q.dim() != 2 or w_q.dim() != 2 or a_q.shape[1] != w_q.shape[1]:
        raise ValueError("fp8_gemm shape mismatch: a %s, w %s" % (tuple(a_q.shape), tuple(w_q.shape)))
    if a_q.stride(1) != 1:
        a_q = a_q.contiguous()
    if w_q.stride(1) != 1:
        w_q = w_q.contiguous()
    M, K = a_q.shape
    N = w_q.shape[0]
    if out is None:
        out = torch.empty((M, N), dtype=_BF16, device=a_q.device)
    elif out.dtype != _BF16 or out.shape != (M, N) or out.stride(1) != 1:
        raise ValueError("fp8_gemm: bad `out`")
    if bias is not None:
        if bias.numel() != N:
            raise ValueError("fp8_gemm: bias has %d entries for N = %d" % (bias.numel(), N))
        if bias.dtype != _BF16:
            bias = bias.to(_BF16)
        bias = bias.contiguous()
    if a_scale is not None:
        if a_scale.dtype != torch.float32 or a_scale.numel() != M:
            raise ValueError("fp8_gemm: a_scale must hold one fp32 value per row of a")
        a_scale = a_scale.contiguous()
    if w_scale is not None and (w_scale.dtype != torch.float32 or w_scale.numel() != 1):
        raise ValueError("fp8_gemm: w_scale must be one fp32 value")
    _require_cuda(a_scale, w_scale, bias, out, resid, gate)
    gate_sb = 0
    if resid is not None:
        if resid.dtype != _BF16 or resid.shape != (M, N) or resid.stride(1) != 1:
            raise ValueError("fp8_gemm: `resid` must be bf16 (M,N) with unit column stride")
        if gate is not None:
            gate = gate.reshape(-1, N)
            if gate.dtype != _BF16 or gate.stride(1) != 1:
                gate = gate.to(_BF16).contiguous()
            rpb = rows_per_batch or max(M, 1)
            if gate.shape[0] > 1 and gate.shape[0] * rpb < M:
                raise ValueError("fp8_gemm: %d gate rows of %d tokens do not cover M = %d" % (gate.shape[0], rpb, M))
            gate_sb = gate.stride(0) if gate.shape[0] > 1 else 0
    elif gate is not None:
        raise ValueError("fp8_gemm: `gate` needs `resid`")
    prob = _lib.GemmProblem(
        a=_ptr(a_q), lda=a_q.stride(0), w=_ptr(w_q), ldw=w_q.stride(0), a_scale=_ptr(a_scale), w_scale=_ptr(w_scale),
        bias=_ptr(bias), resid=_ptr(resid), ldr=resid.stride(0) if resid is not None else 0, gate=_ptr(gate),
        gate_sb=gate_sb, rows_per_batch=(rows_per_batch or max(M, 1)), out=_ptr(out), ldo=out.stride(0), M=M, N=N, K=K)
    keep = [a_q, w_q, a_scale, w_scale, bias, resid, gate]
    if qk is not None:
        if resid is not None:
            raise ValueError("fp8_gemm: the q/k epilogue and the residual epilogue exclude each other")
        wq, wk, rope = qk.get("q_norm_w"), qk.get("k_norm_w"), qk.get("rope")
        wq = None if wq is None else wq.to(_BF16).contiguous()
        wk = None if wk is None else wk.to(_BF16).contiguous()
        if any(w is not None and w.numel() != 128 for w in (wq, wk)):
            raise ValueError("fp8_gemm: q/k RMSNorm weights have 128 entries")
        prob.q_norm_w, prob.k_norm_w = _ptr(wq), _ptr(wk)
        prob.qk_heads, prob.norm_eps = int(qk["heads"]), float(qk.get("eps", 1e-6))
        if rope is not None:
            if rope.dtype != torch.float32 or rope.dim() != 4 or rope.shape[2:] != (64, 2):
                raise ValueError("rope table must be fp32 (B|1, S, 64, 2)")
            # the kernel takes table row (m / rows_per_batch) of the batch axis on trust: it must be there
            batches = -(-M // prob.rows_per_batch)
            if rope.shape[0] not in (1, batches):
                raise ValueError("fp8_gemm: a rope table of batch %d beside %d batch entries of %d rows"
                                 % (rope.shape[0], batches, prob.rows_per_batch))
            rope = rope.contiguous()
            prob.rope, prob.rope_rows = _ptr(rope), rope.shape[1]
            prob.rope_sb = rope.stride(0) if rope.shape[0] > 1 else 0
            prob.rope_pos0 = int(qk.get("pos0", 0))
        keep += [wq, wk, rope]
    if ext is not None:
        # (a_ext (M, K_ext), w_ext (N, K_ext)): more columns of the reduction axis, e.g. an unfused low-rank update
        a_e, w_e = ext
        _require_cuda(a_e, w_e)
        if a_e.dtype != FP8 or w_e.dtype != FP8 or a_e.dim() != 2 or w_e.dim() != 2 or a_e.shape[0] != M \
                or w_e.shape[0] != N or a_e.shape[1] != w_e.shape[1] or a_e.stride(1) != 1 or w_e.stride(1) != 1:
            raise ValueError("fp8_gemm: `ext` must be e4m3 (M, K_ext) and (N, K_ext) with unit column stride")
        prob.a_ext, prob.lda_ext, prob.w_ext, prob.ldw_ext = _ptr(a_e), a_e.stride(0), _ptr(w_e), w_e.stride(0)
        prob.K_ext = a_e.shape[1]
        keep += [a_e, w_e]
    return prob, out, tuple(keep)


def fp8_gemm(a_q: torch.Tensor, w_q: torch.Tensor, a_scale: Optional[torch.Tensor] = None,
             w_scale: Optional[torch.Tensor] = None, bias: Optional[torch.Tensor] = None,
             out: Optional[torch.Tensor] = None, resid: Optional[torch.Tensor] = None,
             gate: Optional[torch.Tensor] = None, rows_per_batch: Optional[int] = None, qk=None,
             ext=None) -> torch.Tensor:
    """out[m,n] = bf16((sum_k a[m,k] w[n,k]) * a_scale[m] * w_scale + bias[n]); a (M,K), w (N,K) e4m3.

    With ``resid`` (M,N) the gated residual is fused: out = resid + gate * that, gate (B,N) or None,
    rows_per_batch = rows of a per batch entry (default: all M rows share gate row 0).
    With ``qk`` (see _gemm_problem) the q and k heads of a packed qkv projection leave normalised and rotated.
    With ``ext`` = (a_ext (M,E), w_ext (N,E)) the sum runs over E more columns, as if a and w were [a | a_ext] and
    [w | w_ext]."""
    if qk is not None or ext is not None:  # options the problem description carries and the flat entry points do not
        return fp8_gemm_grouped([dict(a_q=a_q, w_q=w_q, a_scale=a_scale, w_scale=w_scale, bias=bias, out=out,
                                      resid=resid, gate=gate, rows_per_batch=rows_per_batch, qk=qk, ext=ext)])[0]
    pr, out, _keep = _gemm_problem(a_q, w_q, a_scale, w_scale, bias, out, resid, gate, rows_per_batch)
    lib = _lib.load()
    if resid is None:
        rc = lib.dsx_fp8_gemm(pr.a, pr.lda, pr.w, pr.ldw, pr.a_scale, pr.w_scale, pr.bias, pr.out, pr.ldo,
                              pr.M, pr.N, pr.K, _stream())
        _lib.check(rc, "dsx_fp8_gemm")
        return out
    rc = lib.dsx_fp8_gemm_gated_residual(pr.a, pr.lda, pr.w, pr.ldw, pr.a_scale, pr.w_scale, pr.bias, pr.resid, pr.ldr,
                                         pr.gate, pr.gate_sb, pr.rows_per_batch, pr.out, pr.ldo, pr.M, pr.N, pr.K,
                                         _stream())
    _lib.check(rc, "dsx_fp8_gemm_gated_residual")
    return out


def fp8_gemm_grouped(problems):
    """Several independent GEMMs in one submission; ``problems`` is a list of dicts with the keyword
    arguments of :func:`fp8_gemm`.  Neighbouring problems share a launch when the kernel allows it
    (see ``dsx_fp8_gemm_grouped``).  Returns the list of outputs."""
    if not 0 < len(problems) <= _lib.GEMM_GROUP_MAX:
        raise ValueError("fp8_gemm_grouped takes 1..%d problems" % _lib.GEMM_GROUP_MAX)
    built = [_gemm_problem(**kw) for kw in problems]
    arr = (_lib.GemmProblem * len(built))(*[b[0] for b in built])
    rc = _lib.load().dsx_fp8_gemm_grouped(arr, len(built), _stream())
    _lib.check(rc, "dsx_fp8_gemm_grouped")
    return [b[1] for b in built]


def lora_down(a_q: torch.Tensor, d_q: torch.Tensor, row_scale: torch.Tensor, width: int = 128, copies: int = 1,
              ranks: Optional[int] = None) -> torch.Tensor:
    """(M, width) e4m3: columns c ranks + r (r < ranks, c < copies) hold
    e4m3_saturating(row_scale[r] * sum_k a_q[m,k] d_q[r,k]), the rest zero codes; the operand `ext` of :func:`fp8_gemm`
    for an unfused low-rank update.  d_q: the stacked down factors, zero rows from `ranks` (default: all) up to
    R = d_q.shape[0], a multiple of 32 and at most 128."""
    _require_cuda(a_q, d_q, row_scale)
    if a_q.dtype != FP8 or d_q.dtype != FP8 or a_q.dim() != 2 or d_q.dim() != 2 or a_q.shape[1] != d_q.shape[1] \
            or a_q.stride(1) != 1 or not d_q.is_contiguous():
        raise ValueError("lora_down expects e4m3 a (M,K) and contiguous d (R,K)")
    M, K = a_q.shape
    R = d_q.shape[0]
    if row_scale.dtype != torch.float32 or row_scale.numel() != R or not row_scale.is_contiguous():
        raise ValueError("lora_down: row_scale must hold one contiguous fp32 value per row of d")
    out = torch.empty((M, width), dtype=FP8, device=a_q.device)
    rc = _lib.load().dsx_lora_down(_ptr(a_q), a_q.stride(0), _ptr(d_q), K, _ptr(row_scale), _ptr(out), width, M, K, R,
                                   R if ranks is None else ranks, copies, width, _stream())
    _lib.check(rc, "dsx_lora_down")
    return out


def fp8_gemv_rowscale(a_q: torch.Tensor, w_q: torch.Tensor, a_scale: Optional[torch.Tensor],
                      w_row_scale: torch.Tensor, bias: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Small-M (<= 8) product against a stack of Linear weights with one fp32 weight scale per output row."""
    _require_cuda(a_q, w_q, a_scale, w_row_scale, bias)
    if a_q.dtype != FP8 or w_q.dtype != FP8 or a_q.dim() != 2 or w_q.dim() != 2 or a_q.shape[1] != w_q.shape[1]:
        raise ValueError("fp8_gemv_rowscale expects e4m3 a (M,K) and w (N,K)")
    if a_q.stride(1) != 1:
        a_q = a_q.contiguous()
    if w_q.stride(1) != 1:
        w_q = w_q.contiguous()
    M, K = a_q.shape
    N = w_q.shape[0]
    if w_row_scale.dtype != torch.float32 or w_row_scale.numel() != N or not w_row_scale.is_contiguous():
        raise ValueError("fp8_gemv_rowscale: w_row_scale must hold one contiguous fp32 value per row of w")
    if a_scale is not None and (a_scale.dtype != torch.float32 or a_scale.numel() != M or not a_scale.is_contiguous()):
        raise ValueError("fp8_gemv_rowscale: a_scale must hold one contiguous fp32 value per row of a")
    if bias is not None:
        if bias.numel() != N:
            raise ValueError("fp8_gemv_rowscale: bias has %d entries for N = %d" % (bias.numel(), N))
        bias = bias.to(_BF16).contiguous()
    out = torch.empty((M, N), dtype=_BF16, device=a_q.device)
    rc = _lib.load().dsx_fp8_gemv_rowscale(_ptr(a_q), a_q.stride(0), _ptr(w_q), w_q.stride(0), _ptr(a_scale),
                                           _ptr(w_row_scale), _ptr(bias), _ptr(out), N, M, N, K, _stream())
    _lib.check(rc, "dsx_fp8_gemv_rowscale")
    return out


def _bhsd_strides(t: torch.Tensor):
    if t.stride(3) != 1:
        raise ValueError("attention operands need unit stride in the head dim")
    return t.stride(0), t.stride(1), t.stride(2)


def rope_table_from_freqs(freqs: torch.Tensor) -> torch.Tensor:
    """Reference RoPE table (B,1,S,64,2,2) [[c,-s],[s,c]] (transformer_helper.py:54-64) -> (B,S,64,2) (c,s) fp32."""
    if freqs.dim() != 6 or freqs.shape[-2:] != (2, 2):
        raise ValueError("expected a (B,1,S,P,2,2) rotary table")
    return torch.stack((freqs[:, 0, :, :, 0, 0], freqs[:, 0, :, :, 1, 0]), dim=-1).float().contiguous()


def attention_bhsd(q, k, v, *, q2=None, k2=None, v2=None, scale: Optional[float] = None,
                   rope: Optional[torch.Tensor] = None, q_norm_w=None, k_norm_w=None, q2_norm_w=None,
                   k2_norm_w=None, eps: float = 1e-6, out: Optional[torch.Tensor] = None,
                   out2: Optional[torch.Tensor] = None, score_bound: float = 0.0, split_keys: bool = True,
                   static_scratch: bool = False, qk_norm2_max: Optional[torch.Tensor] = None):
    """softmax(q k^T * scale) v over the concatenation [segment 1, segment 2] of rows.

    q, k, v: (B,H,S,128) bf16 views with unit stride in the last dim (any other strides).
    q2/k2/v2: optional second segment (same strides as the first), appended after the first.
    rope: optional (B or 1, Sq, 64, 2) fp32 (cos, sin) table applied in-kernel to q and k;
    *_norm_w: optional (128,) bf16 RMSNorm weights applied before RoPE.
    A scratch buffer of dsx_attn_workspace_bytes is allocated here when the call needs one: k is normalised /
    rotated once into it by a row kernel (q is treated as the attention kernel loads it), and the key range of a
    sparsely filled last round of workgroups is split over the idle compute units (split_keys=False: no scratch
    is offered for that, one workgroup walks the whole key axis of its unit).
    static_scratch: go through dsx_attn_fwd_static, the entry point that allocates nothing: the library's own
    static device array serves as scratch (calls on one GPU must then not overlap) and a call that needs more
    than it holds raises.
    score_bound: optional promise |scale * q.k| <= score_bound for every pair (after RMSNorm/RoPE); when it is
    small enough the kernel skips the running softmax maximum (same result).  0 = no promise.
    qk_norm2_max: optional fp32 device tensor of two values, upper bounds of |q row|^2 and |k row|^2 over every
    head row the call reads (rmsnorm_rows(..., head_norm2_max=) leaves them); the kernels read it on the device
    and skip the running maximum when the bound it implies is small enough.  Not with rope / *_norm_w.
    Returns out (B,H,Sq1,128)-shaped view semantics: writes `out` (B,Sq1,H,128 layout allowed via strides).
    """
    _require_cuda(q, k, v)
    for t in (q, k, v, q2, k2, v2):
        if t is not None and t.dtype != _BF16:
            raise ValueError("attention expects bf16 tensors, got %s" % t.dtype)
    B, H, S1, D = q.shape
    if D != 128:
        raise ValueError("head_dim must be 128, got %d" % D)
    if k.shape != v.shape or k.shape[:2] != (B, H) or k.shape[3] != D:
        raise ValueError("attention: q %s, k %s, v %s do not fit" % (tuple(q.shape), tuple(k.shape), tuple(v.shape)))
    if (k2 is None) != (v2 is None) or (k2 is not None and (k2.shape != v2.shape or k2.shape[:2] != (B, H)
                                                            or k2.shape[3] != D)):
        raise ValueError("attention: the second key/value segment does not fit the first")
    if q2 is not None and (q2.shape[:2] != (B, H) or q2.shape[3] != D):
        raise ValueError("attention: the second query segment does not fit the first")
    for t, s_ in ((out, S1), (out2, None if q2 is None else q2.shape[2])):
        if t is not None and (t.dtype != _BF16 or tuple(t.shape) != (B, H, s_, D)):
            raise ValueError("attention: `out` must be bf16 (B,H,Sq,128)")
    _require_cuda(q2, k2, v2, out, out2, rope, qk_norm2_max)
    P = _lib.AttnParams()
    S2 = 0 if q2 is None else q2.shape[2]
    Skv1 = k.shape[2]
    Skv2 = 0 if k2 is None else k2.shape[2]
    if out is None:
        out = torch.empty((B, S1, H, D), dtype=_BF16, device=q.device).transpose(1, 2)
    if q2 is not None and out2 is None:
        out2 = torch.empty((B, S2, H, D), dtype=_BF16, device=q.device).transpose(1, 2)

    P.q[0], P.q[1] = _ptr(q), _ptr(q2)
    P.k[0], P.k[1] = _ptr(k), _ptr(k2)
    P.v[0], P.v[1] = _ptr(v), _ptr(v2)
    P.o[0], P.o[1] = _ptr(out), _ptr(out2)
    P.sq[0], P.sq[1] = S1, S2
    P.skv[0], P.skv[1] = Skv1, Skv2
    for name, t1, t2 in (("q", q, q2), ("k", k, k2), ("v", v, v2), ("o", out, out2)):
        for g, t in enumerate((t1, t2)):
            if t is not None:
                sb, sh, ss = _bhsd_strides(t)
                getattr(P, name + "_sb")[g], getattr(P, name + "_sh")[g], getattr(P, name + "_ss")[g] = sb, sh, ss
    P.batch, P.heads, P.head_dim = B, H, D
    P.softmax_scale = float(scale) if scale is not None else 1.0 / math.sqrt(D)
    keep = []
    if rope is not None:
        if rope.dtype != torch.float32 or rope.dim() != 4 or rope.shape[1:] != (S1 + S2, 64, 2) \
                or rope.shape[0] not in (1, B):
            raise ValueError("rope table must be fp32 (B|1, Sq, 64, 2)")
        rope = rope.contiguous()
        keep.append(rope)
        P.rope = _ptr(rope)
        P.rope_sb = rope.stride(0) if rope.shape[0] > 1 else 0
        P.rope_rows = rope.shape[1]
    for i, (qw, kw) in enumerate(((q_norm_w, k_norm_w), (q2_norm_w, k2_norm_w))):
        for name, w in (("q_norm_w", qw), ("k_norm_w", kw)):
            if w is not None:
                if w.numel() != D:
                    raise ValueError("attention: RMSNorm weights have %d entries" % D)
                w = w.to(_BF16).contiguous()
                keep.append(w)
                getattr(P, name)[i] = _ptr(w)
    P.norm_eps = eps
    P.score_bound = float(score_bound)
    if qk_norm2_max is not None:
        if qk_norm2_max.dtype != torch.float32 or qk_norm2_max.numel() != 2 or not qk_norm2_max.is_contiguous() \
                or qk_norm2_max.device != q.device:
            raise ValueError("qk_norm2_max must be two contiguous fp32 values on the device of q")
        keep.append(qk_norm2_max)
        P.qk_norm2_max = _ptr(qk_norm2_max)
    lib = _lib.load()
    # scratch for the one-off k pre-pass and for splitting the key range of a partly filled last round
    if static_scratch:
        _lib.check(lib.dsx_attn_fwd_static(P, _stream()), "dsx_attn_fwd_static")
        return (out, out2) if q2 is not None else out
    k_side = rope is not None or any(w is not None for w in (k_norm_w, k2_norm_w))
    need = lib.dsx_attn_workspace_bytes(P) if (split_keys or k_side) else 0
    if need > 0:
        ws = torch.empty(need, dtype=torch.uint8, device=q.device)
        keep.append(ws)
        P.workspace, P.workspace_bytes = _ptr(ws), need
    rc = lib.dsx_attn_fwd(P, _stream())
    _lib.check(rc, "dsx_attn_fwd")
    return (out, out2) if q2 is not None else out


def _rope_table(rope: torch.Tensor, batch: int, rows: int) -> torch.Tensor:
    """A (B|1, >= rows, 64, 2) fp32 (cos, sin) table on the device, contiguous; the kernels read `rows` rows of it per
    batch entry and cannot see where it ends."""
    _require_cuda(rope)
    if rope.dtype != torch.float32 or rope.dim() != 4 or rope.shape[2:] != (64, 2) or rope.shape[0] not in (1, batch) \
            or rope.shape[1] < rows:
        raise ValueError("rope table must be fp32 (B|1, >= %d, 64, 2), got %s" % (rows, tuple(rope.shape)))
    return rope.contiguous()


def rmsnorm_rope(x: torch.Tensor, norm_w: Optional[torch.Tensor], rope: Optional[torch.Tensor], pos0: int = 0,
                 eps: float = 1e-6, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """RMSNorm (per head, 128) then RoPE of a (B,H,S,128) bf16 view; returns a dense (B,H,S,128) tensor."""
    _require_cuda(x)
    B, H, S, D = x.shape
    if D != 128 or x.dtype != _BF16:
        raise ValueError("rmsnorm_rope expects bf16 (B,H,S,128)")
    if out is None:
        out = torch.empty((B, H, S, D), dtype=_BF16, device=x.device)
    elif out.dtype != _BF16 or out.shape != x.shape:
        raise ValueError("rmsnorm_rope: `out` must match x")
    if norm_w is not None:
        if norm_w.numel() != D:
            raise ValueError("rmsnorm_rope: the RMSNorm weight has %d entries" % D)
        norm_w = norm_w.to(_BF16).contiguous()
    rope_sb = 0
    if rope is not None:
        rope = _rope_table(rope, B, pos0 + S)
        rope_sb = rope.stride(0) if rope.shape[0] > 1 else 0
    xs, os_ = _bhsd_strides(x), _bhsd_strides(out)
    rc = _lib.load().dsx_rmsnorm_rope(_ptr(x), xs[0], xs[1], xs[2], _ptr(norm_w), eps, _ptr(rope), rope_sb, pos0,
                                      _ptr(out), os_[0], os_[1], os_[2], B, H, S, _stream())
    _lib.check(rc, "dsx_rmsnorm_rope")
    return out


def rmsnorm_rope_qk(qkv: torch.Tensor, heads_q: int, heads_k: int, q_norm_w: Optional[torch.Tensor],
                    k_norm_w: Optional[torch.Tensor], rope: Optional[torch.Tensor], pos0: int = 0,
                    eps: float = 1e-6) -> torch.Tensor:
    """In-place RMSNorm + RoPE of the q and k heads of a packed projection ``qkv`` (B, S, >= (hq+hk)*128):
    heads [0,hq) with q_norm_w, [hq,hq+hk) with k_norm_w; the remaining columns (v, ...) are untouched."""
    _require_cuda(qkv)
    if qkv.dim() != 3 or qkv.dtype != _BF16 or qkv.stride(2) != 1 or qkv.shape[2] < (heads_q + heads_k) * 128:
        raise ValueError("rmsnorm_rope_qk expects bf16 (B, S, >= (heads_q+heads_k)*128) with unit column stride")
    B, S, _ = qkv.shape
    if any(w is not None and w.numel() != 128 for w in (q_norm_w, k_norm_w)):
        raise ValueError("rmsnorm_rope_qk: RMSNorm weights have 128 entries")
    if q_norm_w is not None:
        q_norm_w = q_norm_w.to(_BF16).contiguous()
    if k_norm_w is not None:
        k_norm_w = k_norm_w.to(_BF16).contiguous()
    rope_sb = 0
    if rope is not None:
        rope = _rope_table(rope, B, pos0 + S)
        rope_sb = rope.stride(0) if rope.shape[0] > 1 else 0
    rc = _lib.load().dsx_rmsnorm_rope_qk(_ptr(qkv), qkv.stride(0), qkv.stride(1), heads_q, heads_k, _ptr(q_norm_w),
                                         _ptr(k_norm_w), eps, _ptr(rope), rope_sb, pos0, B, S, _stream())
    _lib.check(rc, "dsx_rmsnorm_rope_qk")
    return qkv


def rmsnorm_rows(x: torch.Tensor, weight: torch.Tensor, eps: float = 1e-6, rope: Optional[torch.Tensor] = None,
                 out: Optional[torch.Tensor] = None, head_norm2_max: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Wan-style RMSNorm over the full last dim of (B,S,D) (or (rows,D)) bf16, optionally followed by RoPE on
    every 128-wide head with the fp32 (B|1, S, 64, 2) (cos, sin) table.
    head_norm2_max: optional one-element fp32 device tensor, raised to the largest squared 2-norm of a 128-wide
    head of an output row (never lowered: zero it before the first contributing call)."""
    _require_cuda(x)
    if x.dtype != _BF16:
        raise ValueError("rmsnorm_rows expects bf16")
    shp = x.shape
    D = shp[-1]
    x2, ldx = _rows_2d(x)
    rows = x2.shape[0]
    rows_per_batch = shp[-2] if x.dim() >= 2 else rows
    rope_sb = 0
    if rope is not None:
        rope = rope.contiguous()
        if rope.dtype != torch.float32 or rope.shape[-3:] != (rows_per_batch, 64, 2):
            raise ValueError("rope table must be fp32 (B|1, S, 64, 2)")
        rope_sb = rope.stride(0) if rope.dim() == 4 and rope.shape[0] > 1 else 0
    if out is None:
        out = torch.empty((rows, D), dtype=_BF16, device=x.device)
        o2, ldo = out, D
    else:
        o2, ldo = _rows_2d(out)
    if weight.numel() != D:
        raise ValueError("rmsnorm_rows: the weight has %d entries for D = %d" % (weight.numel(), D))
    w = weight.to(_BF16).contiguous()
    _require_cuda(w, rope, out)
    if head_norm2_max is not None and (head_norm2_max.dtype != torch.float32 or head_norm2_max.numel() != 1
                                       or head_norm2_max.device != x.device):
        raise ValueError("head_norm2_max must be one fp32 value on the device of x")
    rc = _lib.load().dsx_rmsnorm_rows(_ptr(x2), ldx, _ptr(w), eps, _ptr(rope), rope_sb, rows_per_batch, _ptr(o2), ldo,
                                      rows, D, _ptr(head_norm2_max), _stream())
    _lib.check(rc, "dsx_rmsnorm_rows")
    return out.view(shp)


def adaln_modulate(x: torch.Tensor, scale: Optional[torch.Tensor], shift: Optional[torch.Tensor],
                   eps: float = 1e-6, ln_weight=None, ln_bias=None, want_bf16: bool = True,
                   want_fp8: bool = False, scaled: bool = True):
    """LayerNorm(x) * (1 + scale) + shift per token; x (B,S,D) bf16, scale/shift (B,D) or (B,1,D) bf16.

    Returns y (bf16) and/or (q e4m3, q_scale fp32 per token) depending on want_*; ``scaled=False``: q is the
    reference's bare cast of y (unit scale, utils/fp8_linear.py:35) and q_scale is None.
    """
    _require_cuda(x)
    if x.dtype != _BF16:
        raise ValueError("adaln_modulate expects bf16")
    shp = x.shape
    D = shp[-1]
    B = shp[0] if x.dim() == 3 else 1
    x2, ldx = _rows_2d(x)
    rows = x2.shape[0]
    mod_sb = 0

    def prep(t):
        nonlocal mod_sb
        if t is None:
            return None
        t = t.reshape(-1, D)  # a view for (B,D), (B,1,D) and chunk() slices of a (B,k*D) projection
        if t.dtype != _BF16:
            t = t.to(_BF16)
        if t.stride(1) != 1:
            t = t.contiguous()
        if t.shape[0] not in (1, B):
            raise ValueError("modulation must have one row per batch entry")
        sb = t.stride(0) if t.shape[0] > 1 else 0
        if mod_sb and sb and mod_sb != sb:
            raise ValueError("scale and shift must share a batch stride")
        mod_sb = sb or mod_sb
        return t

    scale_t, shift_t = prep(scale), prep(shift)
    if any(t is not None and t.numel() != D for t in (ln_weight, ln_bias)):
        raise ValueError("adaln_modulate: the LayerNorm affine has D = %d entries" % D)
    ln_weight = None if ln_weight is None else ln_weight.to(_BF16).contiguous()
    ln_bias = None if ln_bias is None else ln_bias.to(_BF16).contiguous()
    _require_cuda(scale_t, shift_t, ln_weight, ln_bias)
    y = torch.empty((rows, D), dtype=_BF16, device=x.device) if want_bf16 else None
    q = torch.empty((rows, D), dtype=FP8, device=x.device) if want_fp8 else None
    qs = torch.empty((rows,), dtype=torch.float32, device=x.device) if want_fp8 and scaled else None
    rc = _lib.load().dsx_adaln_modulate(_ptr(x2), ldx, _ptr(scale_t), _ptr(shift_t), mod_sb, max(rows // B, 1),
                                        _ptr(ln_weight), _ptr(ln_bias), eps, _ptr(y), D, _ptr(q), D, _ptr(qs), rows,
                                        D, _stream())
    _lib.check(rc, "dsx_adaln_modulate")
    res = []
    if want_bf16:
        res.append(y.view(shp))
    if want_fp8:
        res += [q.view(shp), qs]
    return res[0] if len(res) == 1 else tuple(res)


def gated_residual(x: torch.Tensor, y: torch.Tensor, gate: Optional[torch.Tensor],
                   out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """x + gate * y (gate (B,D) / (B,1,D) or None); bf16, rounding bf16(x + bf16(gate*y))."""
    _require_cuda(x, y, gate, out)
    if x.dtype != _BF16 or y.dtype != _BF16 or x.shape != y.shape:
        raise ValueError("gated_residual expects two bf16 tensors of one shape")
    shp = x.shape
    D = shp[-1]
    B = shp[0] if x.dim() == 3 else 1
    x2, ldx = _rows_2d(x)
    y2, ldy = _rows_2d(y)
    rows = x2.shape[0]
    gate_sb = 0
    if gate is not None:
        gate = gate.reshape(-1, D)
        if gate.shape[0] not in (1, B):
            raise ValueError("gated_residual: the gate must have one row per batch entry")
        if gate.dtype != _BF16:
            gate = gate.to(_BF16)
        if gate.stride(1) != 1:
            gate = gate.contiguous()
        gate_sb = gate.stride(0) if gate.shape[0] > 1 else 0
    if out is None:
        out = torch.empty((rows, D), dtype=_BF16, device=x.device)
        o2, ldo = out, D
    else:
        o2, ldo = _rows_2d(out)
    rc = _lib.load().dsx_gated_residual(_ptr(x2), ldx, _ptr(y2), ldy, _ptr(gate), gate_sb, max(rows // B, 1),
                                        _ptr(o2), ldo, rows, D, _stream())
    _lib.check(rc, "dsx_gated_residual")
    return out.view(shp)


def gelu_tanh(x: torch.Tensor, want_bf16: bool = True, want_fp8: bool = False, out: Optional[torch.Tensor] = None,
              erf: bool = False, scaled: bool = True):
    """tanh-GELU (``erf``: the exact erf form of nn.GELU()) over the last dim of a bf16 tensor (a column slice of
    a wider buffer is fine).  ``scaled=False``: the e4m3 output is the bare cast (unit scale, q_scale None)."""
    _require_cuda(x, out)
    if x.dtype != _BF16:
        raise ValueError("gelu_tanh expects bf16")
    shp = x.shape
    D = shp[-1]
    x2, ldx = _rows_2d(x)
    rows = x2.shape[0]
    y, ldy = None, D
    if want_bf16:
        if out is not None:
            y, ldy = _rows_2d(out)
        else:
            y = torch.empty((rows, D), dtype=_BF16, device=x.device)
    q = torch.empty((rows, D), dtype=FP8, device=x.device) if want_fp8 else None
    qs = torch.empty((rows,), dtype=torch.float32, device=x.device) if want_fp8 and scaled else None
    fn = _lib.load().dsx_gelu_erf if erf else _lib.load().dsx_gelu_tanh
    _lib.check(fn(_ptr(x2), ldx, _ptr(y), ldy, _ptr(q), D, _ptr(qs), rows, D, _stream()),
               "dsx_gelu_erf" if erf else "dsx_gelu_tanh")
    res = []
    if want_bf16:
        res.append(out if out is not None else y.view(shp))
    if want_fp8:
        res += [q.view(shp), qs]
    return res[0] if len(res) == 1 else tuple(res)


def concat_gelu_tanh(prefix: torch.Tensor, x: torch.Tensor, want_bf16: bool = False, want_fp8: bool = True,
                     scaled: bool = True):
    """[prefix | gelu_tanh(x)] along the last dim for 2-D (rows, D) views; bf16 and/or per-token e4m3 output
    (``scaled=False``: the bare cast, q_scale None)."""
    _require_cuda(prefix, x)
    if prefix.dtype != _BF16 or x.dtype != _BF16 or prefix.dim() != 2 or x.dim() != 2:
        raise ValueError("concat_gelu_tanh expects 2-D bf16 tensors")
    p2, ldp = _rows_2d(prefix)
    x2, ldx = _rows_2d(x)
    rows, Dp = p2.shape
    D = x2.shape[1]
    Dt = Dp + D
    y = torch.empty((rows, Dt), dtype=_BF16, device=x.device) if want_bf16 else None
    q = torch.empty((rows, Dt), dtype=FP8, device=x.device) if want_fp8 else None
    qs = torch.empty((rows,), dtype=torch.float32, device=x.device) if want_fp8 and scaled else None
    rc = _lib.load().dsx_concat_gelu_tanh(_ptr(p2), ldp, Dp, _ptr(x2), ldx, _ptr(y), Dt, _ptr(q), Dt, _ptr(qs), rows,
                                          D, _stream())
    _lib.check(rc, "dsx_concat_gelu_tanh")
    res = ([y] if want_bf16 else []) + ([q, qs] if want_fp8 else [])
    return res[0] if len(res) == 1 else tuple(res)


def flow_match_euler_step(latents: torch.Tensor, model_outputs: torch.Tensor, dt: float) -> torch.Tensor:
    """latents + model_outputs * dt in fp32, cast back (flow_match_euler.py:11-19)."""
    _require_cuda(latents, model_outputs)
    if latents.dtype != model_outputs.dtype or latents.dtype not in (_BF16, torch.float32):
        raise ValueError("flow_match_euler_step expects matching bf16 or fp32 tensors")
    a, b = latents.contiguous(), model_outputs.contiguous()
    out = torch.empty_like(a)
    rc = _lib.load().dsx_flow_match_euler_step(_ptr(a), _ptr(b), float(dt), _ptr(out), a.numel(),
                                               int(a.dtype == torch.float32), _stream())
    _lib.check(rc, "dsx_flow_match_euler_step")
    return out
