"""Wan2.1 DiT block and model forward — oracle (test infrastructure, see oracle/__init__.py).

Restates diffsynth_engine/models/wan/wan_dit.py:18-351 (text-to-video, and image-to-video where the parameter
dict holds the has_image_input=True entries) as functions over a flat parameter dict whose keys are the
reference's state-dict names.  The reference has no WanDiT test; wiring is pinned by vectors its own WanDiT
class wrote at reduced size in both forms (tests/test_oracle_leaf_goldens.py) and by structural invariants
(tests/test_oracle_wan.py).  ``linear_mode`` as in oracle/flux.py.
"""
import math

import torch
import torch.nn.functional as F

from . import dit_ops as O
from .flux import Params  # same parameter container / fp8 linear modes


def config_14b():
    """conf/models/wan/dit/14b-t2v.json"""
    return dict(dim=5120, in_dim=16, ffn_dim=13824, out_dim=16, text_dim=4096, freq_dim=256, eps=1e-6,
                patch_size=(1, 2, 2), num_heads=40, num_layers=40)


IMAGE_ROWS = 257  # CLIP tokens in front of the text context (the split is hard-coded, wan_dit.py:138-139)


def init_params(cfg, dtype=torch.bfloat16, device="cpu", seed=0, std=0.02, bias_std=0.0, clip_dim=None):
    """Random WanDiT parameters (shapes from WanDiT.__init__, wan_dit.py:248-299); with ``clip_dim`` the
    image-to-video form (cross_attn.k_img / v_img / norm_k_img per block and the img_emb MLP, 1280 wide in the
    reference)."""
    g = torch.Generator(device="cpu").manual_seed(seed)
    d, f = cfg["dim"], cfg["ffn_dim"]
    t = {}

    def lin(name, n_in, n_out):
        t[name + ".weight"] = (torch.randn(n_out, n_in, generator=g) * std).to(dtype).to(device)
        b = torch.randn(n_out, generator=g) * bias_std if bias_std else torch.zeros(n_out)
        t[name + ".bias"] = b.to(dtype).to(device)

    pf, ph, pw = cfg["patch_size"]
    t["patch_embedding.weight"] = (torch.randn(d, cfg["in_dim"], pf, ph, pw, generator=g) * std).to(dtype).to(device)
    t["patch_embedding.bias"] = torch.zeros(d, dtype=dtype, device=device)
    lin("text_embedding.0", cfg["text_dim"], d)
    lin("text_embedding.2", d, d)
    lin("time_embedding.0", cfg["freq_dim"], d)
    lin("time_embedding.2", d, d)
    lin("time_projection.1", d, 6 * d)
    for i in range(cfg["num_layers"]):
        p = f"blocks.{i}."
        for a in ("self_attn", "cross_attn"):
            for n in ("q", "k", "v", "o"):
                lin(p + f"{a}.{n}", d, d)
            t[p + f"{a}.norm_q.weight"] = (1 + 0.1 * torch.randn(d, generator=g)).to(dtype).to(device)
            t[p + f"{a}.norm_k.weight"] = (1 + 0.1 * torch.randn(d, generator=g)).to(dtype).to(device)
        t[p + "norm3.weight"] = (1 + 0.1 * torch.randn(d, generator=g)).to(dtype).to(device)
        t[p + "norm3.bias"] = (0.1 * torch.randn(d, generator=g)).to(dtype).to(device)
        if clip_dim:
            lin(p + "cross_attn.k_img", d, d)
            lin(p + "cross_attn.v_img", d, d)
            t[p + "cross_attn.norm_k_img.weight"] = (1 + 0.1 * torch.randn(d, generator=g)).to(dtype).to(device)
        lin(p + "ffn.0", d, f)
        lin(p + "ffn.2", f, d)
        t[p + "modulation"] = (torch.randn(1, 6, d, generator=g) / d ** 0.5).to(dtype).to(device)
    lin("head.head", d, cfg["out_dim"] * pf * ph * pw)
    t["head.modulation"] = (torch.randn(1, 2, d, generator=g) / d ** 0.5).to(dtype).to(device)
    if clip_dim:
        for i, n in ((0, clip_dim), (4, d)):
            t[f"img_emb.proj.{i}.weight"] = (1 + 0.1 * torch.randn(n, generator=g)).to(dtype).to(device)
            t[f"img_emb.proj.{i}.bias"] = (0.1 * torch.randn(n, generator=g)).to(dtype).to(device)
        lin("img_emb.proj.1", clip_dim, clip_dim)
        lin("img_emb.proj.3", clip_dim, d)
    return t


def freqs_cis_3d(head_dim, f, h, w, theta=10000.0):
    """precompute_freqs_cis_3d + the per-token table of WanDiT.forward (wan_dit.py:38-51,335-346): the head
    dim splits into (head_dim - 2*(head_dim//3), head_dim//3, head_dim//3) for (frame, row, col); each axis gets
    complex128 phases e^{i pos theta^(-2j/dim_axis)}; the three are concatenated per token -> (f*h*w, 1, head_dim/2)."""
    def axis(dim, end):
        fr = 1.0 / (theta ** (torch.arange(0, dim, 2)[: dim // 2].double() / dim))
        ang = torch.outer(torch.arange(end), fr)
        return torch.polar(torch.ones_like(ang), ang)

    df = head_dim - 2 * (head_dim // 3)
    ff, fh, fw = axis(df, f), axis(head_dim // 3, h), axis(head_dim // 3, w)
    return torch.cat([ff.view(f, 1, 1, -1).expand(f, h, w, -1), fh.view(1, h, 1, -1).expand(f, h, w, -1),
                      fw.view(1, 1, w, -1).expand(f, h, w, -1)], dim=-1).reshape(f * h * w, 1, -1)


def rope_apply(x, freqs, num_heads):
    """wan_dit.py:54-58: float64 complex multiply on adjacent pairs of each head, cast back."""
    b, s, hd = x.shape
    xc = torch.view_as_complex(x.to(torch.float64).reshape(b, s, num_heads, -1, 2))
    return torch.view_as_real(xc * freqs).flatten(2).to(x.dtype)


def wan_rms_norm(x, weight, eps):
    """wan_dit.py:61-78 over the full model dim: norm(x.float()).to(dtype) * weight."""
    xf = x.float()
    return (xf * torch.rsqrt(xf.pow(2).mean(dim=-1, keepdim=True) + eps)).to(x.dtype) * weight


def attention(q, k, v, num_heads, attn=O.sdpa):
    """wan_dit.py:18-22: (B,S,H*D) -> (B,H,S,D) -> SDPA -> back."""
    b, sq, hd = q.shape
    d = hd // num_heads
    sp = lambda t: t.view(t.shape[0], t.shape[1], num_heads, d).transpose(1, 2)
    o = attn(sp(q), sp(k), sp(v))
    return o.transpose(1, 2).reshape(b, sq, hd)


def dit_block(P, i, x, context, t_mod, freqs, cfg, attn=O.sdpa):
    """DiTBlock.forward (wan_dit.py:185-193); chunk order shift_msa, scale_msa, gate_msa, shift_mlp, scale_mlp,
    gate_mlp; norm1/norm2 without affine, norm3 with; the cross-attention residual has no gate."""
    p = f"blocks.{i}."
    eps, H = cfg["eps"], cfg["num_heads"]
    shift_msa, scale_msa, gate_msa, shift_mlp, scale_mlp, gate_mlp = (P[p + "modulation"] + t_mod).chunk(6, dim=1)
    h = O.layer_norm_modulate(x, scale_msa, shift_msa, eps)
    q = wan_rms_norm(P.linear(h, p + "self_attn.q"), P[p + "self_attn.norm_q.weight"], eps)
    k = wan_rms_norm(P.linear(h, p + "self_attn.k"), P[p + "self_attn.norm_k.weight"], eps)
    v = P.linear(h, p + "self_attn.v")
    a = attention(rope_apply(q, freqs, H), rope_apply(k, freqs, H), v, H, attn)
    x = x + gate_msa * P.linear(a, p + "self_attn.o")
    h = O.layer_norm_modulate(x, None, None, eps, P[p + "norm3.weight"], P[p + "norm3.bias"])
    q = wan_rms_norm(P.linear(h, p + "cross_attn.q"), P[p + "cross_attn.norm_q.weight"], eps)
    # CrossAttention.forward (wan_dit.py:136-152): with image input the first 257 context rows are the embedded
    # CLIP tokens; they get their own k/v projections and k norm, and the two attention outputs are added
    img, ctx = (context[:, :IMAGE_ROWS], context[:, IMAGE_ROWS:]) if p + "cross_attn.k_img.weight" in P.t else (None, context)
    k = wan_rms_norm(P.linear(ctx, p + "cross_attn.k"), P[p + "cross_attn.norm_k.weight"], eps)
    v = P.linear(ctx, p + "cross_attn.v")
    a = attention(q, k, v, H, attn)
    if img is not None:
        k_img = wan_rms_norm(P.linear(img, p + "cross_attn.k_img"), P[p + "cross_attn.norm_k_img.weight"], eps)
        a = a + attention(q, k_img, P.linear(img, p + "cross_attn.v_img"), H, attn)
    x = x + P.linear(a, p + "cross_attn.o")
    h = O.layer_norm_modulate(x, scale_mlp, shift_mlp, eps)
    return x + gate_mlp * P.linear(O.gelu_tanh(P.linear(h, p + "ffn.0")), p + "ffn.2")


def sinusoidal_embedding_1d(dim, position):
    """wan_dit.py:29-35: float64 [cos | sin] of position * 10000^(-j/(dim/2)), cast to the position dtype."""
    half = dim // 2
    ang = torch.outer(position.type(torch.float64),
                      torch.pow(10000, -torch.arange(half, dtype=torch.float64, device=position.device).div(half)))
    return torch.cat([torch.cos(ang), torch.sin(ang)], dim=1).to(position.dtype)


def img_emb(P, clip_feature):
    """MLP.forward (wan_dit.py:195-211): LayerNorm (affine, eps 1e-5) -> Linear -> erf-GELU -> Linear -> LayerNorm."""
    n = clip_feature.shape[-1]
    h = F.layer_norm(clip_feature, (n,), P["img_emb.proj.0.weight"], P["img_emb.proj.0.bias"], 1e-5)
    h = P.linear(F.gelu(P.linear(h, "img_emb.proj.1")), "img_emb.proj.3")
    return F.layer_norm(h, (h.shape[-1],), P["img_emb.proj.4.weight"], P["img_emb.proj.4.bias"], 1e-5)


def wan_dit_forward(P, x, context, timestep, cfg, attn=O.sdpa, clip_feature=None, y=None):
    """WanDiT.forward (wan_dit.py:319-351); ``clip_feature`` (B,257,clip_dim) and ``y`` (B,c_y,f,h,w) for the
    image-to-video form."""
    d = cfg["dim"]
    pf, ph, pw = cfg["patch_size"]
    t = P.linear(F.silu(P.linear(sinusoidal_embedding_1d(cfg["freq_dim"], timestep), "time_embedding.0")),
                 "time_embedding.2")
    t_mod = P.linear(F.silu(t), "time_projection.1").unflatten(1, (6, d))
    context = P.linear(F.gelu(P.linear(context, "text_embedding.0"), approximate="tanh"), "text_embedding.2")
    if clip_feature is not None:
        x = torch.cat([x, y], dim=1)                                   # (b, c_x + c_y, f, h, w)  (:331)
        context = torch.cat([img_emb(P, clip_feature), context], dim=1)  # image rows first           (:333)
    # Conv3d with kernel == stride is a Linear over each (c, pf, ph, pw) patch
    B, C, Fr, Hh, Ww = x.shape
    f, h, w = Fr // pf, Hh // ph, Ww // pw
    patches = x.view(B, C, f, pf, h, ph, w, pw).permute(0, 2, 4, 6, 1, 3, 5, 7).reshape(B, f * h * w, C * pf * ph * pw)
    P.t["patch_embedding_as_linear.weight"] = P["patch_embedding.weight"].reshape(d, -1)
    P.t["patch_embedding_as_linear.bias"] = P["patch_embedding.bias"]
    x = P.linear(patches, "patch_embedding_as_linear")
    freqs = freqs_cis_3d(d // cfg["num_heads"], f, h, w).to(x.device)
    for i in range(cfg["num_layers"]):
        x = dit_block(P, i, x, context, t_mod, freqs, cfg, attn)
    shift, scale = (P["head.modulation"] + t).chunk(2, dim=1)  # Head.forward (wan_dit.py:234-237)
    x = P.linear(O.layer_norm_modulate(x, scale, shift, cfg["eps"]), "head.head")
    # unpatchify 'b (f h w) (x y z c) -> b c (f x) (h y) (w z)' (wan_dit.py:307-317)
    c = cfg["out_dim"]
    return x.view(B, f, h, w, pf, ph, pw, c).permute(0, 7, 1, 4, 2, 5, 3, 6).reshape(B, c, f * pf, h * ph, w * pw)
