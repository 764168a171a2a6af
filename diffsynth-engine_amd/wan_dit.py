"""Fused MI355X runner of the Wan2.1 DiT denoising step (text-to-video, and image-to-video when the checkpoint
holds the ``has_image_input`` entries).

Same inputs/outputs and state-dict names as ``WanDiT.forward``
(diffsynth_engine/models/wan/wan_dit.py:319-351).  ``DiTBlock.forward`` (:185-193) is issued as:

  AdaLN-modulate (+ e4m3) -> q/k/v FP8 GEMMs -> RMSNorm over the model dim + RoPE on q, k (one row kernel
  each) -> flash attention over the (B,S,H*D) projections by stride -> quantise -> o GEMM with the gated
  residual in its epilogue -> LayerNorm(affine) (+ e4m3) -> cross-attention against the text keys/values
  (Lq != Lk) -> o GEMM with plain residual -> AdaLN-modulate -> FFN GEMM -> GELU (+ e4m3) -> FFN GEMM with
  gated residual.

Image-to-video (conf/models/wan/dit/14b-i2v.json; wan_dit.py:136-152,195-211,329-333): the encoded image rides
along as extra latent channels, the CLIP feature goes through the ``img_emb`` MLP and its 257 rows are put in
front of the text context, and every cross-attention adds a second attention of the same queries over those rows
(own k/v projections and k norm) before the o projection.

The reference wires FP8 for Flux only (models/flux/flux_dit.py:404; pipelines/base.py:164-165 raises for the
rest); here every Linear of the Wan DiT runs through the same scaled e4m3 GEMM as Flux.
"""
import math
from typing import Dict, Optional

import torch

from . import ops
from .flux_dit import _Linear, _gemm_pair, count_blocks, ingest_state_dict


IMAGE_ROWS = 257  # CLIP tokens in front of the text context (the split is hard-coded, wan_dit.py:138-139)


def wan_config_from_shapes(shapes: Dict[str, tuple], eps: float = 1e-6) -> dict:
    """The constructor arguments of WanDiT (wan_dit.py:247-262; conf/models/wan/dit/*.json) that the runner needs,
    read off a checkpoint's tensor shapes: ``shapes`` maps state-dict names to shapes.  Heads are 128 wide (the
    attention kernel's head width: 40 heads at dim 5120, 12 at 1536, as in the reference's configurations); eps
    is not in a checkpoint (1e-6 in every configuration the reference ships)."""
    conv = tuple(shapes["patch_embedding.weight"])  # (dim, in_dim, pf, ph, pw)
    if len(conv) != 5:
        raise ValueError("patch_embedding.weight must be the 5-D Conv3d weight, got shape %s" % (conv,))
    dim, patch = conv[0], tuple(conv[2:])
    if dim % 128:
        raise ValueError("WanDiTRunner needs dim = heads * 128, got dim %d" % dim)
    layers = count_blocks((k for k in shapes if k.endswith(".weight")), "blocks.")
    out_features = shapes["head.head.weight"][0]
    return {"dim": dim, "in_dim": conv[1], "ffn_dim": shapes["blocks.0.ffn.0.weight"][0],
            "out_dim": out_features // math.prod(patch), "text_dim": shapes["text_embedding.0.weight"][1],
            "freq_dim": shapes["time_embedding.0.weight"][1], "eps": eps, "patch_size": patch,
            "num_heads": dim // 128, "num_layers": layers,
            "has_image_input": "img_emb.proj.1.weight" in shapes}


class WanDiTRunner:
    def __init__(self, state_dict, cfg: Optional[dict] = None, scaled: bool = True, device="cuda:0"):
        self.device = torch.device(device)
        self.scaled = scaled
        # self-attention reads the largest head norms of q and k on the device and drops the running softmax
        # maximum when they allow it (False: always the running maximum)
        self.device_score_bound = True
        shapes: Dict[str, tuple] = {}

        def conv_as_linear(key, t):  # Conv3d with kernel == stride is a Linear over each patch
            shapes[key] = tuple(t.shape)
            return t.reshape(t.shape[0], -1) if key == "patch_embedding.weight" else None

        # key order does not matter: biases are attached once every weight is known; what is not a Linear
        # (modulation vectors, norm weights and the affine bias of norm3) lands in `vec` under its full key
        self.lin, self.vec = ingest_state_dict(state_dict, self.device, scaled, as_linear=conv_as_linear)
        # dims: given (the reference's conf/models/wan/dit/*.json), or read off the checkpoint's shapes
        self.cfg = dict(wan_config_from_shapes(shapes) if cfg is None else cfg)
        self.has_image_input = "img_emb.proj.1" in self.lin

    def add_lora(self, name: str, down: torch.Tensor, up: torch.Tensor, coef: float = 1.0):
        """Attach an unfused LoRA (``coef`` = scale * alpha / rank, models/basic/lora.py:29-32,137-141) to the
        Linear called ``name``."""
        self.lin[name].add_lora(down, up, coef)

    # ------------------------------------------------------------------ helpers
    def _linear_bf16(self, x, name):
        shp = x.shape
        a_q, a_s = ops.quantize_fp8(x.reshape(-1, shp[-1]), scaled=self.scaled)
        y = self.lin[name](a_q, a_s)
        return y.view(*shp[:-1], y.shape[-1])

    def _q(self, y):
        return ops.quantize_fp8(y, scaled=self.scaled)

    def _modulate_q(self, x, scale, shift, w=None, b=None):
        return ops.adaln_modulate(x, scale, shift, self.cfg["eps"], ln_weight=w, ln_bias=b, want_bf16=False,
                                  want_fp8=True, scaled=self.scaled)

    def rope_table(self, f, h, w, theta=10000.0):
        """(1, f*h*w, 64, 2) fp32 (cos, sin): head dim split (d - 2*(d//3), d//3, d//3) over (frame, row, col)
        with float64 angles pos * theta^(-2j/dim_axis) (wan_dit.py:38-51,335-346)."""
        hd = self.cfg["dim"] // self.cfg["num_heads"]
        dev = self.device

        def axis(dim, end):
            fr = 1.0 / (theta ** (torch.arange(0, dim, 2, device=dev)[: dim // 2].double() / dim))
            return torch.outer(torch.arange(end, device=dev).double(), fr)

        af, ah, aw = axis(hd - 2 * (hd // 3), f), axis(hd // 3, h), axis(hd // 3, w)
        ang = torch.cat([af.view(f, 1, 1, -1).expand(f, h, w, -1), ah.view(1, h, 1, -1).expand(f, h, w, -1),
                         aw.view(1, 1, w, -1).expand(f, h, w, -1)], dim=-1).reshape(1, f * h * w, -1)
        return torch.stack((torch.cos(ang), torch.sin(ang)), dim=-1).float().contiguous()

    def _attention(self, q, k, v, qk_norm2_max=None):
        """(B,S,H*D) projections -> (B,S,H*D) attention output, head split/merge by strides (wan_dit.py:18-22).
        qk_norm2_max: the largest squared head norms of q and k, on the device (see ops.attention_bhsd)."""
        H = self.cfg["num_heads"]
        B, Sq, HD = q.shape
        D = HD // H
        sp = lambda t: t.view(t.shape[0], t.shape[1], H, D).transpose(1, 2)
        out = torch.empty((B, Sq, H, D), dtype=torch.bfloat16, device=q.device)
        ops.attention_bhsd(sp(q), sp(k), sp(v), out=out.transpose(1, 2), qk_norm2_max=qk_norm2_max)
        return out.view(B * Sq, HD)

    # ------------------------------------------------------------------ block
    def quantise_context(self, context):
        """The cross-attention operand of every block: the embedded context as e4m3 rows with their scales, text
        rows and (image-to-video) the 257 CLIP rows in front of them separately (CrossAttention.forward,
        wan_dit.py:136-152).  The same for every block of a step, so the step does it once."""
        B, _, d = context.shape
        img = None
        if self.has_image_input:
            img, context = context[:, :IMAGE_ROWS], context[:, IMAGE_ROWS:]
        parts = []
        for t in (context, img):
            parts.append(None if t is None else self._q(t.reshape(B * t.shape[1], d)) + (t.shape[1],))
        return parts

    def block(self, i, x, context, t_mod, rope, context_q=None):
        """DiTBlock.forward; x (B,S,d), context (B,Sc,d) already embedded, t_mod (B,6,d); ``context_q``: what
        quantise_context(context) returned, when the caller has it already."""
        p = f"blocks.{i}."
        L, V, eps = self.lin, self.vec, self.cfg["eps"]
        B, S, d = x.shape
        mod = (V[p + "modulation"] + t_mod).reshape(B, 6 * d)  # shift_msa, scale_msa, gate_msa, shift_mlp, ...
        m = mod.chunk(6, dim=1)
        x2 = x.reshape(B * S, d)
        # self-attention
        hq, hs = self._modulate_q(x, m[1], m[0])
        hq = hq.view(B * S, d)
        # The RMSNorm runs over all heads at once, so no static bound on a head's scores exists; the norm kernels
        # leave the largest squared head norm of q and of k on the device and the attention kernels read it there
        # (|q.k| <= |q||k|): with ordinary activations the running softmax maximum is not needed.
        nm = torch.zeros(2, dtype=torch.float32, device=x.device) if self.device_score_bound else None
        q = ops.rmsnorm_rows(L[p + "self_attn.q"](hq, hs).view(B, S, d), V[p + "self_attn.norm_q.weight"], eps, rope,
                             head_norm2_max=None if nm is None else nm[0:1])
        k = ops.rmsnorm_rows(L[p + "self_attn.k"](hq, hs).view(B, S, d), V[p + "self_attn.norm_k.weight"], eps, rope,
                             head_norm2_max=None if nm is None else nm[1:2])
        v = L[p + "self_attn.v"](hq, hs).view(B, S, d)
        aq, asc = self._q(self._attention(q, k, v, nm))
        x2 = L[p + "self_attn.o"](aq, asc, resid=x2, gate=m[2], rows_per_batch=S)
        # cross-attention (no gate on the residual)
        hq, hs = self._modulate_q(x2.view(B, S, d), None, None, V[p + "norm3.weight"], V[p + "norm3.bias"])
        q = ops.rmsnorm_rows(L[p + "cross_attn.q"](hq.view(B * S, d), hs).view(B, S, d),
                             V[p + "cross_attn.norm_q.weight"], eps)
        # k and v projections of the context share their operand: one launch, side by side
        (cq, cs, Sc), img = context_q if context_q is not None else self.quantise_context(context)
        k, v = _gemm_pair(L[p + "cross_attn.k"], dict(a_q=cq, a_s=cs), L[p + "cross_attn.v"], dict(a_q=cq, a_s=cs))
        k = ops.rmsnorm_rows(k.view(B, Sc, d), V[p + "cross_attn.norm_k.weight"], eps)
        a = self._attention(q, k, v.view(B, Sc, d))
        if img is not None:  # the same queries over the image rows; the two outputs are added in bf16
            iq, isc, Si = img
            k, v = _gemm_pair(L[p + "cross_attn.k_img"], dict(a_q=iq, a_s=isc),
                              L[p + "cross_attn.v_img"], dict(a_q=iq, a_s=isc))
            k = ops.rmsnorm_rows(k.view(B, Si, d), V[p + "cross_attn.norm_k_img.weight"], eps)
            a = ops.gated_residual(a, self._attention(q, k, v.view(B, Si, d)), None)
        aq, asc = self._q(a)
        x2 = L[p + "cross_attn.o"](aq, asc, resid=x2, gate=None, rows_per_batch=S)
        # feed-forward
        hq, hs = self._modulate_q(x2.view(B, S, d), m[4], m[3])
        h = L[p + "ffn.0"](hq.view(B * S, d), hs)
        gq, gs = ops.gelu_tanh(h, want_bf16=False, want_fp8=True, scaled=self.scaled)
        x2 = L[p + "ffn.2"](gq, gs, resid=x2, gate=m[5], rows_per_batch=S)
        return x2.view(B, S, d)

    # ------------------------------------------------------------------ step
    def _img_emb(self, clip_feature):
        """MLP.forward (wan_dit.py:195-211): LayerNorm (affine, eps 1e-5) -> Linear -> erf-GELU -> Linear -> LayerNorm."""
        V = self.vec
        h = ops.adaln_modulate(clip_feature.to(torch.bfloat16), None, None, 1e-5, ln_weight=V["img_emb.proj.0.weight"],
                               ln_bias=V["img_emb.proj.0.bias"])
        h = self._linear_bf16(ops.gelu_tanh(self._linear_bf16(h, "img_emb.proj.1"), erf=True), "img_emb.proj.3")
        return ops.adaln_modulate(h, None, None, 1e-5, ln_weight=V["img_emb.proj.4.weight"],
                                  ln_bias=V["img_emb.proj.4.bias"])

    @torch.no_grad()
    def forward(self, x, context, timestep, clip_feature=None, y=None):
        """``clip_feature`` (B,257,clip_dim) and ``y`` (B,c_y,f,h,w): the image-to-video inputs (both or neither)."""
        cfg = self.cfg
        d = cfg["dim"]
        pf, ph, pw = cfg["patch_size"]
        bf = torch.bfloat16
        half = cfg["freq_dim"] // 2
        ang = torch.outer(timestep.to(torch.float64),
                          torch.pow(10000, -torch.arange(half, dtype=torch.float64, device=self.device).div(half)))
        emb = torch.cat([torch.cos(ang), torch.sin(ang)], dim=1).to(bf)
        t = self._linear_bf16(torch.nn.functional.silu(self._linear_bf16(emb, "time_embedding.0")), "time_embedding.2")
        t_mod = self._linear_bf16(torch.nn.functional.silu(t), "time_projection.1").unflatten(1, (6, d))
        ctx = ops.gelu_tanh(self._linear_bf16(context.to(bf), "text_embedding.0"))
        ctx = self._linear_bf16(ctx, "text_embedding.2")
        if self.has_image_input != (clip_feature is not None and y is not None):
            raise ValueError("clip_feature and y go with an image-to-video checkpoint, and only with one")
        if self.has_image_input:
            if clip_feature.shape[1] != IMAGE_ROWS:
                raise ValueError("clip_feature must have %d rows, got %d" % (IMAGE_ROWS, clip_feature.shape[1]))
            x = torch.cat([x, y.to(x.dtype)], dim=1)                         # (b, c_x + c_y, f, h, w)  (:331)
            ctx = torch.cat([self._img_emb(clip_feature), ctx], dim=1)  # image rows first           (:333)
        B, C, Fr, Hh, Ww = x.shape
        f, h, w = Fr // pf, Hh // ph, Ww // pw
        patches = x.to(bf).view(B, C, f, pf, h, ph, w, pw).permute(0, 2, 4, 6, 1, 3, 5, 7)
        hs = self._linear_bf16(patches.reshape(B, f * h * w, C * pf * ph * pw), "patch_embedding")
        rope = self.rope_table(f, h, w)
        ctx_q = self.quantise_context(ctx)
        for i in range(cfg["num_layers"]):
            hs = self.block(i, hs, ctx, t_mod, rope, ctx_q)
        # Head.forward (wan_dit.py:234-237).  The reference adds the (B, d) embedding to the (1, 2, d) table as it
        # stands, so a batch of two (its batched classifier-free guidance, pipelines/wan_video.py:233-248, where both
        # entries carry the same timestep) gets ONE (shift, scale) pair, shift from entry 0 and scale from entry 1;
        # the same expression is evaluated here and shared by the batch (larger batches do not broadcast there either).
        shift, scale = (self.vec["head.modulation"] + t).chunk(2, dim=1)
        hq, hsc = self._modulate_q(hs, scale.reshape(1, d).expand(B, d), shift.reshape(1, d).expand(B, d))
        out = self.lin["head.head"](hq.view(-1, d), hsc)
        c = cfg["out_dim"]
        return out.view(B, f, h, w, pf, ph, pw, c).permute(0, 7, 1, 4, 2, 5, 3, 6).reshape(B, c, f * pf, h * ph, w * pw)

    __call__ = forward
