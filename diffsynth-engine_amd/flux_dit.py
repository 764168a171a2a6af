"""Fused MI355X runner of the Flux DiT denoising step.

Same inputs/outputs and state-dict names as ``FluxDiT.forward``
(diffsynth_engine/models/flux/flux_dit.py:392-461), but the block bodies
(FluxJointTransformerBlock.forward :219-236, FluxSingleTransformerBlock.forward :308-321,
FluxJointAttention.forward :161-194) are issued as a fixed sequence of libdsx kernels:

  AdaLN-modulate (+ e4m3 emission) -> FP8 GEMM -> RMSNorm+RoPE in place -> flash attention reading
  q/k/v straight out of the packed qkv projection by stride (text-first joint sequence from two base
  pointers, no chunk/concat copies) -> quantise -> FP8 GEMM with the gated residual in its epilogue
  -> AdaLN-modulate -> FP8 GEMM -> GELU (+ e4m3 emission) -> FP8 GEMM with gated residual.

Every AdaLN projection consumes the same silu(conditioning) (transformer_helper.py:14,33;
flux_dit.py:332), so all of them are stacked into one weight matrix at construction and evaluated
by a single HBM-bound pass per step.

All Linear layers run as per-token x per-tensor scaled e4m3 GEMMs (``scaled=True``) or with the
reference's bare casts and unit scales (``scaled=False``, utils/fp8_linear.py:28-60).
"""
import math
from typing import Dict, Optional

import torch

from . import ops

HEAD_DIM = 128  # the attention kernel's head width; hidden size and head count come from the checkpoint
AXES_DIM = (16, 56, 56)
THETA = 10000
EPS = 1e-6
SCALE_SUFFIX = ".weight_scale"  # per-tensor scale of an already quantised weight, as enable_fp8_linear's buffer names it


def _lora_factors(down: torch.Tensor, up: torch.Tensor, coef: float, n: int, k: int, dev):
    """(down e4m3 (r', K), its scale, up e4m3 (N, r'), its scale x coef) with the rank zero-padded to a multiple of
    128: the up product then has a whole 128-byte K unit and runs on the tile kernel with the residual epilogue
    (13.8 us for 4608 x 3072 at rank 16) instead of the ragged-K kernel (45.8 us)."""
    if tuple(down.shape[1:]) != (k,) or up.shape[0] != n or up.shape[1] != down.shape[0]:
        raise ValueError("LoRA factors (%s, %s) do not fit a Linear %d -> %d" % (tuple(down.shape), tuple(up.shape), k, n))
    r = down.shape[0]
    rp = (r + 127) // 128 * 128  # a whole 128-byte K unit: both products then run on the tile kernel
    d = torch.zeros((rp, k), dtype=torch.bfloat16, device=dev)
    d[:r] = down.to(dev, torch.bfloat16)
    u = torch.zeros((n, rp), dtype=torch.bfloat16, device=dev)
    u[:, :r] = up.to(dev, torch.bfloat16)
    dq, ds = ops.quantize_weight_fp8(d, scaled=True)
    uq, us = ops.quantize_weight_fp8(u, scaled=True)
    return dq, ds, uq, (us * coef).float()


class _Linear:
    """An e4m3 weight (N,K) with its per-tensor scale and bf16 bias, plus optional unfused LoRA pairs.

    Unfused low-rank updates (LoRALinear.forward, models/basic/lora.py:29-32,137-141: y += c * up(down(x))) ride the
    main product as 128 more columns of its reduction axis whenever the layer runs on the tile kernel in scaled mode:
    ``t = down(x)`` comes from one small HBM-bound kernel (ops.lora_down) as e4m3 on the row's own scale grid, and
    ``c * up / s_w`` is stored next to the weight as the matching 128 columns (each rank repeated as often as 128
    columns allow, every copy carrying its share of t), so that
    ``s_x[m] s_w (sum_k xq wq + sum_r t u) = x W^T + c up(down(x))`` comes out of ONE accumulation with every
    epilogue (bias, gated residual, q/k RMSNorm + RoPE) unchanged.  Elsewhere (unit-scale mode, whose arithmetic is
    the reference's bare casts with the coefficient applied in bf16; products with at most 8 rows; ranks beyond 128;
    updates so strong that t would leave e4m3's range)
    the update is two more products added through residual epilogues."""

    __slots__ = ("w", "s", "b", "n", "k", "loras", "scaled", "prequantised", "_raw", "_ext")

    def __init__(self, weight: torch.Tensor, bias: Optional[torch.Tensor], scaled: bool):
        self.prequantised = weight.dtype == ops.FP8
        if self.prequantised:
            self.w, self.s = weight, None  # the scale arrives under its own key (ingest_state_dict)
        else:
            self.w, self.s = ops.quantize_weight_fp8(weight, scaled=scaled)
        self.b = None if bias is None else bias.to(torch.bfloat16).contiguous()
        self.n, self.k = self.w.shape
        self.loras = []  # (down_q (r,K), down_scale, up_q (N,r), up_scale * coefficient): the two-product form
        self._raw = []   # (down, up, coefficient) as given: the extension form is built from these on first use
        self._ext = None
        self.scaled = scaled

    def add_lora(self, down: torch.Tensor, up: torch.Tensor, coef: float):
        """Unfused low-rank update y += coef * up(down(x)) (models/basic/lora.py:29-32,137-141); both factors are
        stored as e4m3 like every other Linear under fp8 inference."""
        self.loras.append(_lora_factors(down, up, coef, self.n, self.k, self.w.device))
        self._raw.append((down, up, float(coef)))
        self._ext = None

    def _extension(self):
        """(stacked down factors e4m3 (R,K), per-row scale fp32 (R), extension weight e4m3 (N,128), copies, columns per copy) or None when
        the updates of this layer do not fit the extension form."""
        if self._ext is None:
            dev, f32 = self.w.device, torch.float32
            total = sum(d.shape[0] for d, _, _ in self._raw)
            if self.s is None or total > 128 or self.k % 128 or self.k < 256 or self.n % 8:
                self._ext = False
            else:
                # Every rank is laid down `copies` times, each copy carrying 1 / copies of t: the few terms of a
                # low-rank product would otherwise have to be as large, each, as the sum of K terms they sit beside,
                # and e4m3 ends at 448.  The 128 columns are there anyway.
                ranks = (total + 3) // 4 * 4   # columns of one copy (written four at a time)
                R = (total + 31) // 32 * 32    # rows of the stacked down factors (whole MFMA tiles)
                copies = min(128 // ranks, 32)
                d_all = torch.zeros((R, self.k), dtype=ops.FP8, device=dev)
                rs = torch.zeros((R,), dtype=f32, device=dev)
                u_all = torch.zeros((self.n, 128), dtype=ops.FP8, device=dev)
                r0, fits = 0, True
                for down, up, coef in self._raw:
                    r = down.shape[0]
                    dq, ds = ops.quantize_weight_fp8(down.to(dev, torch.bfloat16).contiguous(), scaled=True)
                    # what the main product's scales leave to be multiplied in: c * up / s_w, on its own e4m3 grid
                    uq, us = ops.quantize_weight_fp8((up.to(dev, f32) * coef / self.s).contiguous(), scaled=True)
                    d_all[r0:r0 + r] = dq
                    rs[r0:r0 + r] = ds * us / copies
                    for c in range(copies):
                        u_all[:, c * ranks + r0:c * ranks + r0 + r] = uq
                    r0 += r
                    # t of a row of N(0,1)-like codes (rms 448 / 4) against the longest down row, four deviations
                    # out, has to stay inside e4m3; an update too strong for that takes the two-product form
                    t_far = 4.0 * 112.0 * dq.float().norm(dim=1).max() * ds * us / copies
                    fits = fits and bool(t_far <= 448.0)
                self._ext = (d_all, rs, u_all, copies, ranks) if fits else False
        return self._ext or None

    def _rides_main_product(self, a_q) -> bool:
        return bool(self.loras) and a_q.shape[0] > 8 and self._extension() is not None

    def problem(self, a_q, a_s, out=None, resid=None, gate=None, rows_per_batch=None, qk=None):
        """Keyword arguments of ``ops.fp8_gemm`` for this layer applied to ``a_q`` (low-rank updates included when
        they ride the main product: their down projection is launched here)."""
        ext = None
        if self._rides_main_product(a_q):
            d_all, rs, u_all, copies, ranks = self._extension()
            ext = (ops.lora_down(a_q, d_all, rs, 128, copies, ranks), u_all)
        return dict(a_q=a_q, w_q=self.w, a_scale=a_s if self.s is not None else None, w_scale=self.s, bias=self.b,
                    out=out, resid=resid, gate=gate, rows_per_batch=rows_per_batch, qk=qk, ext=ext)

    def __call__(self, a_q, a_s, out=None, resid=None, gate=None, rows_per_batch=None, qk=None):
        if not self.loras or self._rides_main_product(a_q):
            return ops.fp8_gemm(**self.problem(a_q, a_s, out, resid, gate, rows_per_batch, qk))
        if qk is not None:  # the low-rank terms are added after the main product: q/k can only be prepared after them
            raise ValueError("a LoRA on a qkv projection needs qk_prep='attention'")
        main = dict(a_q=a_q, w_q=self.w, a_scale=a_s if self.s is not None else None, w_scale=self.s, bias=self.b)
        if resid is None:  # y = main + sum(lora): the low-rank products are added by residual epilogues
            # the main product and the first down projection read the same operand and have the same (plain)
            # epilogue: one launch, in which the few tiles of the projection run beside the main product's
            dq, ds, _, _ = self.loras[0]
            y, h0 = ops.fp8_gemm_grouped([dict(main, out=out), dict(a_q=a_q, w_q=dq, a_scale=a_s, w_scale=ds, bias=None)])
            hs_list = [h0] + [ops.fp8_gemm(a_q, dq, a_s, ds, None) for dq, ds, _, _ in self.loras[1:]]
            for h, (_, _, uq, us) in zip(hs_list, self.loras):
                hq, hs = ops.quantize_fp8(h, scaled=True)
                ops.fp8_gemm(hq, uq, hs, us, None, resid=y, out=y)
            return y
        lows = []
        for dq, ds, uq, us in self.loras:
            hq, hs = ops.quantize_fp8(ops.fp8_gemm(a_q, dq, a_s, ds, None), scaled=True)
            lows.append((hq, hs, uq, us))
        # resid + gate*(main + lora) = (resid + gate*lora) + gate*main: every term rides a GEMM epilogue
        acc = resid
        for hq, hs, uq, us in lows:
            acc = ops.fp8_gemm(hq, uq, hs, us, None, resid=acc, gate=gate, rows_per_batch=rows_per_batch)
        return ops.fp8_gemm(**dict(main, out=out, resid=acc, gate=gate, rows_per_batch=rows_per_batch))


def _gemm_pair(la: "_Linear", pa: dict, lb: "_Linear", pb: dict):
    """Two independent linears (image and text stream): one grouped submission, unless one of them carries low-rank
    updates in the two-product form."""
    if any(L.loras and not L._rides_main_product(p["a_q"]) for L, p in ((la, pa), (lb, pb))):
        return la(**pa), lb(**pb)
    return ops.fp8_gemm_grouped([la.problem(**pa), lb.problem(**pb)])


def ingest_state_dict(state_dict, device, scaled: bool, as_linear=None):
    """Turns a checkpoint into runner storage, whatever order its keys come in (a safetensors file lists
    ``x.bias`` before ``x.weight``; the reference loads through ``load_state_dict``, which does not care).

    ``state_dict`` is a mapping or any iterable of (name, tensor) pairs; the latter lets a caller stream a
    12B-parameter model through without ever holding it unquantised: every 2-D ``.weight`` is quantised as it
    arrives, biases and ``.weight_scale`` entries wait until all weights are in.  ``as_linear(key, tensor)``
    may return a 2-D view for keys that are Linear layers in disguise (a Conv3d whose kernel equals its
    stride).  Returns (linears by name, every other tensor by full key, bf16 on the device).  A float8 weight
    must bring its scale (``<name>.weight_scale``, which enable_fp8_linear's modules emit) when ``scaled`` is set:
    taking it at unit scale would be wrong by 448/absmax per layer without any error."""
    device = torch.device(device)
    lin: Dict[str, _Linear] = {}
    other: Dict[str, torch.Tensor] = {}
    biases: Dict[str, torch.Tensor] = {}
    scales: Dict[str, torch.Tensor] = {}
    items = state_dict.items() if hasattr(state_dict, "items") else state_dict
    for key, t in items:
        if key.endswith(SCALE_SUFFIX):
            scales[key[: -len(SCALE_SUFFIX)]] = t.to(device, torch.float32).reshape(())
            continue
        w2 = as_linear(key, t) if as_linear is not None else None
        if w2 is None and key.endswith(".weight") and t.dim() == 2:
            w2 = t
        if w2 is not None:
            lin[key[: -len(".weight")]] = _Linear(w2.to(device), None, scaled)
        elif key.endswith(".bias"):
            biases[key[: -len(".bias")]] = t.to(device, torch.bfloat16).contiguous()
        else:
            other[key] = (t.to(device, torch.bfloat16) if torch.is_floating_point(t) else t.to(device)).contiguous()
    for name, sc in scales.items():
        if name not in lin:
            raise KeyError("%s%s has no matching weight" % (name, SCALE_SUFFIX))
        if not lin[name].prequantised:
            raise ValueError("%s%s given for a weight that is not float8_e4m3fn" % (name, SCALE_SUFFIX))
        lin[name].s = sc
    for name, b in biases.items():
        if name in lin:
            lin[name].b = b
        else:
            other[name + ".bias"] = b  # the affine bias of a norm layer
    if scaled:
        missing = [n for n, L in lin.items() if L.prequantised and L.s is None]
        if missing:
            raise ValueError("float8 weights without a scale in scaled mode (pass `<name>%s` or use scaled=False "
                             "for reference-style unit scales): %s" % (SCALE_SUFFIX, ", ".join(missing[:4])))
    return lin, other


def count_blocks(names, prefix: str) -> int:
    """1 + the largest index i among names of the form ``<prefix><i>.…`` (0 if there is none)."""
    n = 0
    for name in names:
        if name.startswith(prefix):
            head = name[len(prefix):].split(".", 1)[0]
            if head.isdigit():
                n = max(n, int(head) + 1)
    return n


class FluxDiTRunner:
    """Holds quantised weights of a Flux-architecture DiT and runs one denoising step.  The hidden size comes
    from the checkpoint (``x_embedder.weight``); heads are 128 wide (``heads`` = hidden / 128 unless given)."""

    def __init__(self, state_dict, num_double: Optional[int] = None, num_single: Optional[int] = None,
                 scaled: bool = True, device="cuda:0", heads: Optional[int] = None, axes_dim=AXES_DIM,
                 qk_prep: str = "gemm"):
        self.device = torch.device(device)
        self.scaled = scaled
        # Where the per-head RMSNorm and the RoPE rotation of q and k happen (flux_dit.py:165-171,179-180,297-301):
        # "gemm": in the epilogue of the qkv projection, on the tile the GEMM is about to store (no pass of its
        # own; the attention call is then plain); "attention": requested from the attention entry point (k in one
        # row pass into scratch, q as the attention kernel loads it).  Same arithmetic, same bits.
        if qk_prep not in ("gemm", "attention"):
            raise ValueError("qk_prep must be 'gemm' or 'attention', got %r" % (qk_prep,))
        self.qk_prep = qk_prep
        self.lin, other = ingest_state_dict(state_dict, self.device, scaled)
        # block counts: given, or as many as the checkpoint holds (FluxDiT builds 19 + 38, flux_dit.py:352-356)
        if num_double is None:
            num_double = count_blocks(self.lin, "blocks.")
        if num_single is None:
            num_single = count_blocks(self.lin, "single_blocks.")
        self.num_double, self.num_single = num_double, num_single
        self.norm_w: Dict[str, torch.Tensor] = {}
        for key, t in other.items():
            if key.endswith(".weight") and t.dim() == 1:
                self.norm_w[key[: -len(".weight")]] = t
            else:
                raise KeyError("unexpected entry %s %s in a Flux DiT state dict" % (key, tuple(t.shape)))
        self.hidden = self.lin["x_embedder"].n
        self.heads = heads if heads is not None else self.hidden // HEAD_DIM
        self.axes_dim = tuple(axes_dim)
        if self.heads * HEAD_DIM != self.hidden or sum(self.axes_dim) != HEAD_DIM:
            raise ValueError("FluxDiTRunner needs hidden = heads * 128 and RoPE axes that sum to 128, got hidden %d, "
                             "heads %d, axes %s" % (self.hidden, self.heads, self.axes_dim))
        self.has_guidance = "guidance_embedder.timestep_embedder.0" in self.lin
        # After RMSNorm over the head dim every q and k row has norm <= sqrt(128) * max|weight| and RoPE keeps
        # norms, so |q.k| / sqrt(128) <= sqrt(128) * max|w_q| * max|w_k|: the attention kernel is told so and
        # drops its running maximum where that keeps exp2 in range (2 % slack for the bf16 roundings).
        self.score_bound: Dict[str, float] = {}
        wmax = {k: float(v.float().abs().max()) for k, v in self.norm_w.items()}
        for i in range(num_double):
            pre = f"blocks.{i}.attn."
            if all(pre + n in wmax for n in ("norm_q_a", "norm_q_b", "norm_k_a", "norm_k_b")):
                self.score_bound[f"blocks.{i}."] = 1.02 * math.sqrt(HEAD_DIM) * max(
                    wmax[pre + "norm_q_a"], wmax[pre + "norm_q_b"]) * max(wmax[pre + "norm_k_a"], wmax[pre + "norm_k_b"])
        for i in range(num_single):
            pre = f"single_blocks.{i}."
            if pre + "norm_q_a" in wmax and pre + "norm_k_a" in wmax:
                self.score_bound[pre] = 1.02 * math.sqrt(HEAD_DIM) * wmax[pre + "norm_q_a"] * wmax[pre + "norm_k_a"]
        self._stack_modulation()

    def _stack_modulation(self):
        """One (N_total, hidden) e4m3 matrix holding every AdaLN projection, with a weight scale per row."""
        names = []
        for i in range(self.num_double):
            names += [f"blocks.{i}.norm1_a.linear", f"blocks.{i}.norm1_b.linear"]
        names += [f"single_blocks.{i}.norm.linear" for i in range(self.num_single)]
        names.append("final_norm_out.linear")
        self.mod_loras: Dict[str, list] = {}
        self.mod_slices, off = {}, 0
        ws, ss, bs = [], [], []
        one = torch.ones((), dtype=torch.float32, device=self.device)
        for n in names:
            L = self.lin.pop(n)
            self.mod_slices[n] = (off, off + L.n)
            off += L.n
            ws.append(L.w)
            ss.append((L.s if L.s is not None else one).expand(L.n))
            bs.append(L.b if L.b is not None else torch.zeros(L.n, dtype=torch.bfloat16, device=self.device))
        self.mod_w = torch.cat(ws, dim=0)
        self.mod_row_scale = torch.cat(ss).contiguous()
        self.mod_bias = torch.cat(bs).contiguous()

    def add_lora(self, name: str, down: torch.Tensor, up: torch.Tensor, coef: float = 1.0):
        """Attach an unfused LoRA (``coef`` = scale * alpha / rank) to the Linear called ``name``, the stacked
        AdaLN projections included."""
        if name in self.mod_slices:  # a slice of the stacked matrix: its low-rank terms are added per step
            lo, hi = self.mod_slices[name]
            self.mod_loras.setdefault(name, []).append(
                _lora_factors(down, up, coef, hi - lo, self.mod_w.shape[1], self.device))
            return
        self.lin[name].add_lora(down, up, coef)

    def _qk_in_gemm(self, rows, *layers) -> bool:
        """q/k are prepared in the GEMM epilogue unless a projection carries low-rank updates in the two-product
        form (added after the main product, so the projection is complete only after them) or a problem is
        outside what the tile kernel that carries the epilogue takes (more than 8 rows, K a multiple of 128)."""
        return (self.qk_prep == "gemm" and not any(L.loras and L._extension() is None for L in layers)
                and min(rows) > 8 and all(L.k % 128 == 0 and L.n % 8 == 0 for L in layers))

    # ------------------------------------------------------------------ small helpers
    def _linear_bf16(self, x: torch.Tensor, name: str) -> torch.Tensor:
        """quantise + GEMM for a bf16 activation (embedders and M=1 conditioning projections)."""
        shp = x.shape
        a_q, a_s = ops.quantize_fp8(x.reshape(-1, shp[-1]), scaled=self.scaled)
        y = self.lin[name](a_q, a_s)
        return y.view(*shp[:-1], y.shape[-1])

    def _timestep_mlp(self, name: str, t: torch.Tensor) -> torch.Tensor:
        """TimestepEmbeddings (models/basic/timestep.py:66-81): cos/sin features -> Linear -> SiLU -> Linear."""
        half = 128
        freq = torch.exp(-math.log(10000) * torch.arange(half, dtype=torch.float32, device=t.device) / half)
        ang = t[:, None].float() * freq[None, :]
        emb = torch.cat([torch.cos(ang), torch.sin(ang)], dim=-1).to(torch.bfloat16)
        h = self._linear_bf16(emb, name + ".timestep_embedder.0")
        return self._linear_bf16(torch.nn.functional.silu(h), name + ".timestep_embedder.2")

    def _rope(self, text_ids: torch.Tensor, image_ids: torch.Tensor) -> torch.Tensor:
        """(B,S,64,2) fp32 (cos, sin) table of RoPEEmbedding (transformer_helper.py:39-64), float64 angles."""
        ids = torch.cat((text_ids, image_ids), dim=1).to(torch.float64)
        cols = []
        for a, dim in enumerate(self.axes_dim):
            omega = 1.0 / (THETA ** (torch.arange(0, dim, 2, dtype=torch.float64, device=ids.device) / dim))
            ang = ids[..., a].unsqueeze(-1) * omega
            cols.append(torch.stack((torch.cos(ang), torch.sin(ang)), dim=-1))
        return torch.cat(cols, dim=-2).float().contiguous()

    def _modulations(self, cond: torch.Tensor) -> Dict[str, torch.Tensor]:
        """linear(silu(cond)) of every AdaLN layer: one pass over the stacked weights."""
        a_q, a_s = ops.quantize_fp8(torch.nn.functional.silu(cond), scaled=self.scaled)
        out = ops.fp8_gemv_rowscale(a_q, self.mod_w, a_s, self.mod_row_scale, self.mod_bias)
        for name, loras in self.mod_loras.items():  # LoRALinear.forward: w_x += lora(x), lora.py:137-141
            lo, hi = self.mod_slices[name]
            piece = out[:, lo:hi]
            for dq, ds, uq, us in loras:
                hq, hs = ops.quantize_fp8(ops.fp8_gemm(a_q, dq, a_s, ds, None), scaled=True)
                ops.fp8_gemm(hq, uq, hs, us, None, resid=piece, out=piece)
        return {n: out[:, lo:hi] for n, (lo, hi) in self.mod_slices.items()}

    def _modulate_q(self, x, scale, shift):
        """LayerNorm-modulate straight to the GEMM operand format."""
        return ops.adaln_modulate(x, scale, shift, EPS, want_bf16=False, want_fp8=True, scaled=self.scaled)

    def _gelu_q(self, h):
        return ops.gelu_tanh(h, want_bf16=False, want_fp8=True, scaled=self.scaled)

    # ------------------------------------------------------------------ blocks
    def _joint_block(self, i: int, img, txt, mod_a, mod_b, rope):
        """img (B,Si,d), txt (B,St,d); mod_*: (B, 6d) = shift_msa, scale_msa, gate_msa, shift_mlp, scale_mlp,
        gate_mlp (transformer_helper.py:20)."""
        pre = f"blocks.{i}."
        B, Si, d = img.shape
        HEADS = self.heads
        St = txt.shape[1]
        ma, mb = mod_a.chunk(6, dim=1), mod_b.chunk(6, dim=1)
        L = self.lin
        nw = self.norm_w
        qa, sa = self._modulate_q(img, ma[1], ma[0])
        qb, sb = self._modulate_q(txt, mb[1], mb[0])
        in_gemm = self._qk_in_gemm((B * Si, B * St), L[pre + "attn.a_to_qkv"], L[pre + "attn.b_to_qkv"])
        qk_a = qk_b = None
        if in_gemm:  # text rows take RoPE rows [0, St), image rows [St, St + Si) of every batch entry
            qk_a = dict(heads=HEADS, q_norm_w=nw[pre + "attn.norm_q_a"], k_norm_w=nw[pre + "attn.norm_k_a"], rope=rope,
                        pos0=St, eps=EPS)
            qk_b = dict(heads=HEADS, q_norm_w=nw[pre + "attn.norm_q_b"], k_norm_w=nw[pre + "attn.norm_k_b"], rope=rope,
                        pos0=0, eps=EPS)
        qkv_a, qkv_b = _gemm_pair(L[pre + "attn.a_to_qkv"], dict(a_q=qa.view(-1, d), a_s=sa, rows_per_batch=Si, qk=qk_a),
                                  L[pre + "attn.b_to_qkv"], dict(a_q=qb.view(-1, d), a_s=sb, rows_per_batch=St, qk=qk_b))
        qkv_a = qkv_a.view(B, Si, 3 * HEADS, HEAD_DIM).transpose(1, 2)
        qkv_b = qkv_b.view(B, St, 3 * HEADS, HEAD_DIM).transpose(1, 2)
        # With one batch entry the text and image rows of an intermediate share one [text; image] buffer, so
        # that the row kernels between the GEMM pairs (quantise, GELU) run once over both streams; with more
        # entries the rows of one stream would not be evenly strided for the GEMM.
        joint = B == 1
        if joint:
            o = torch.empty((1, St + Si, HEADS, HEAD_DIM), dtype=torch.bfloat16, device=img.device)
            o_b, o_a = o[:, :St], o[:, St:]
        else:
            o_b = torch.empty((B, St, HEADS, HEAD_DIM), dtype=torch.bfloat16, device=img.device)
            o_a = torch.empty((B, Si, HEADS, HEAD_DIM), dtype=torch.bfloat16, device=img.device)
        qb_, kb_, vb_ = qkv_b[:, :HEADS], qkv_b[:, HEADS:2 * HEADS], qkv_b[:, 2 * HEADS:]
        qa_, ka_, va_ = qkv_a[:, :HEADS], qkv_a[:, HEADS:2 * HEADS], qkv_a[:, 2 * HEADS:]
        # joint attention over [text; image] rows; q and k either arrive prepared from the GEMM epilogue or go in
        # with the per-stream RMSNorm weights and the RoPE table
        if in_gemm:
            ops.attention_bhsd(qb_, kb_, vb_, q2=qa_, k2=ka_, v2=va_, out=o_b.transpose(1, 2), out2=o_a.transpose(1, 2),
                               score_bound=self.score_bound.get(pre, 0.0))
        else:
            ops.attention_bhsd(qb_, kb_, vb_, q2=qa_, k2=ka_, v2=va_, rope=rope,
                               q_norm_w=nw[pre + "attn.norm_q_b"], k_norm_w=nw[pre + "attn.norm_k_b"],
                               q2_norm_w=nw[pre + "attn.norm_q_a"], k2_norm_w=nw[pre + "attn.norm_k_a"], eps=EPS,
                               out=o_b.transpose(1, 2), out2=o_a.transpose(1, 2),
                               score_bound=self.score_bound.get(pre, 0.0))
        # The two streams run the same sequence on different weights (flux_dit.py:226-234): out-projection +
        # gated residual, LN-modulate, MLP + gated residual.  Each pair of linears goes out as one grouped
        # submission so that the 512-token text problem runs beside the image problem instead of after it.
        xa, xb = img.reshape(B * Si, d), txt.reshape(B * St, d)
        if joint:
            qo, so = ops.quantize_fp8(o.view(St + Si, d), scaled=self.scaled)
            qb, qa = qo[:St], qo[St:]
            sb, sa = (so[:St], so[St:]) if so is not None else (None, None)
        else:
            qa, sa = ops.quantize_fp8(o_a.view(B * Si, d), scaled=self.scaled)
            qb, sb = ops.quantize_fp8(o_b.view(B * St, d), scaled=self.scaled)
        xa, xb = _gemm_pair(L[pre + "attn.a_to_out"], dict(a_q=qa, a_s=sa, resid=xa, gate=ma[2], rows_per_batch=Si),
                            L[pre + "attn.b_to_out"], dict(a_q=qb, a_s=sb, resid=xb, gate=mb[2], rows_per_batch=St))
        qa, sa = self._modulate_q(xa.view(B, Si, d), ma[4], ma[3])
        qb, sb = self._modulate_q(xb.view(B, St, d), mb[4], mb[3])
        if joint:
            h = torch.empty((St + Si, L[pre + "ff_a.0"].n), dtype=torch.bfloat16, device=img.device)
            _gemm_pair(L[pre + "ff_a.0"], dict(a_q=qa.view(-1, d), a_s=sa, out=h[St:]),
                       L[pre + "ff_b.0"], dict(a_q=qb.view(-1, d), a_s=sb, out=h[:St]))
            qh, sh_ = self._gelu_q(h)
            qb, qa = qh[:St], qh[St:]
            sb, sa = (sh_[:St], sh_[St:]) if sh_ is not None else (None, None)
        else:
            ha, hb = _gemm_pair(L[pre + "ff_a.0"], dict(a_q=qa.view(-1, d), a_s=sa),
                                L[pre + "ff_b.0"], dict(a_q=qb.view(-1, d), a_s=sb))
            qa, sa = self._gelu_q(ha)
            qb, sb = self._gelu_q(hb)
        xa, xb = _gemm_pair(L[pre + "ff_a.2"], dict(a_q=qa, a_s=sa, resid=xa, gate=ma[5], rows_per_batch=Si),
                            L[pre + "ff_b.2"], dict(a_q=qb, a_s=sb, resid=xb, gate=mb[5], rows_per_batch=St))
        return xa.view(B, Si, d), xb.view(B, St, d)

    def _single_block(self, i: int, x, mod, rope):
        """x (B,S,d); mod (B,3d) = shift, scale, gate (transformer_helper.py:34)."""
        pre = f"single_blocks.{i}."
        B, S, d = x.shape
        HEADS = self.heads
        L = self.lin
        shift, scale, gate = mod.chunk(3, dim=1)
        q, sc = self._modulate_q(x, scale, shift)
        nw = self.norm_w
        in_gemm = self._qk_in_gemm((B * S,), L[pre + "to_qkv_mlp"])
        qk = dict(heads=HEADS, q_norm_w=nw[pre + "norm_q_a"], k_norm_w=nw[pre + "norm_k_a"], rope=rope, pos0=0,
                  eps=EPS) if in_gemm else None
        h = L[pre + "to_qkv_mlp"](q.view(-1, d), sc, rows_per_batch=S, qk=qk)  # (B*S, 7d): [q | k | v | mlp]
        att = torch.empty((B, S, HEADS, HEAD_DIM), dtype=torch.bfloat16, device=x.device)
        qkv = h.view(B, S, 7 * d)[:, :, : 3 * d].unflatten(2, (3 * HEADS, HEAD_DIM)).transpose(1, 2)
        q_, k_, v_ = qkv[:, :HEADS], qkv[:, HEADS:2 * HEADS], qkv[:, 2 * HEADS:]
        if in_gemm:
            ops.attention_bhsd(q_, k_, v_, out=att.transpose(1, 2), score_bound=self.score_bound.get(pre, 0.0))
        else:
            ops.attention_bhsd(q_, k_, v_, rope=rope, q_norm_w=nw[pre + "norm_q_a"], k_norm_w=nw[pre + "norm_k_a"],
                               eps=EPS, out=att.transpose(1, 2), score_bound=self.score_bound.get(pre, 0.0))
        # cat([attention, gelu(mlp)]) (flux_dit.py:315-317) is never materialised in bf16: one kernel reads both
        # parts and emits the e4m3 operand of proj_out with its per-token scale
        q, sc = ops.concat_gelu_tanh(att.view(B * S, d), h[:, 3 * d:], want_fp8=True, scaled=self.scaled)
        out = L[pre + "proj_out"](q, sc, resid=x.reshape(B * S, d), gate=gate, rows_per_batch=S)
        return out.view(B, S, d)

    # ------------------------------------------------------------------ step
    @torch.no_grad()
    def forward(self, hidden_states, timestep, prompt_emb, pooled_prompt_emb, guidance, text_ids, image_ids=None,
                use_gradient_checkpointing=False, **kwargs):
        """FluxDiT.forward's signature (flux_dit.py:392-402); the trailing arguments concern training and are ignored.
        text_ids / image_ids / guidance may have batch 1 beside a larger batch of latents (the pipeline's batched
        classifier-free guidance, pipelines/flux_image.py:389-399): they broadcast."""
        dev = self.device
        bf = torch.bfloat16
        B, C, Hh, Ww = hidden_states.shape
        # The RoPE table of the last call is kept while the id tensors are the same objects, unmodified (a denoising
        # loop passes the same ids forty times; building the table is ~30 small launches).  Not under stream capture:
        # a recorded step must rebuild the table from whatever its input buffers hold at replay.
        src = (text_ids, image_ids, text_ids._version, -1 if image_ids is None else image_ids._version, B, Hh, Ww)
        old, rope = getattr(self, "_rope_src", None), None
        capturing = torch.cuda.is_current_stream_capturing()
        if not capturing and old is not None and old[0] is text_ids and old[1] is image_ids and old[2:] == src[2:]:
            rope = self._rope_table
        else:
            if image_ids is None:
                image_ids = torch.zeros(Hh // 2, Ww // 2, 3, device=dev)
                image_ids[..., 1] += torch.arange(Hh // 2, device=dev)[:, None]
                image_ids[..., 2] += torch.arange(Ww // 2, device=dev)[None, :]
                image_ids = image_ids.reshape(1, -1, 3).repeat(text_ids.shape[0], 1, 1)
            for name, ids in (("text_ids", text_ids), ("image_ids", image_ids)):
                if ids.shape[0] not in (1, B):
                    raise ValueError("%s has batch %d beside latents of batch %d" % (name, ids.shape[0], B))
            if text_ids.shape[0] != image_ids.shape[0]:  # one of them broadcasts: the RoPE table is built per entry
                text_ids, image_ids = (t.expand(B, *t.shape[1:]) for t in (text_ids, image_ids))
            rope = self._rope(text_ids.to(dev), image_ids.to(dev))
            if not capturing:
                self._rope_src, self._rope_table = src, rope
        cond = self._timestep_mlp("time_embedder", timestep)
        if self.has_guidance and guidance is not None:
            cond = cond + self._timestep_mlp("guidance_embedder", guidance * 1000)
        pooled = self._linear_bf16(pooled_prompt_emb.to(bf), "pooled_text_embedder.0")
        cond = cond + self._linear_bf16(torch.nn.functional.silu(pooled), "pooled_text_embedder.2")
        txt = self._linear_bf16(prompt_emb.to(bf), "context_embedder")
        x = hidden_states.to(bf).view(B, C, Hh // 2, 2, Ww // 2, 2).permute(0, 2, 4, 1, 3, 5)
        img = self._linear_bf16(x.reshape(B, (Hh // 2) * (Ww // 2), C * 4), "x_embedder")

        mods = self._modulations(cond)
        for i in range(self.num_double):
            img, txt = self._joint_block(i, img, txt, mods[f"blocks.{i}.norm1_a.linear"],
                                         mods[f"blocks.{i}.norm1_b.linear"], rope)
        St = txt.shape[1]
        x = torch.cat([txt, img], dim=1)
        for i in range(self.num_single):
            x = self._single_block(i, x, mods[f"single_blocks.{i}.norm.linear"], rope)
        x = x[:, St:]
        scale, shift = mods["final_norm_out.linear"].chunk(2, dim=1)  # AdaLayerNormContinuous: scale first (:333)
        q, s = self._modulate_q(x, scale, shift)
        out = self.lin["final_proj_out"](q.view(-1, self.hidden), s).view(B, Hh // 2, Ww // 2, C, 2, 2)
        return out.permute(0, 3, 1, 4, 2, 5).reshape(B, C, Hh, Ww)

    __call__ = forward
