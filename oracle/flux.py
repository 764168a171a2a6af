"""Flux DiT blocks and the full denoising-step forward — oracle (test infrastructure, see oracle/__init__.py).

Restates diffsynth_engine/models/flux/flux_dit.py:126-335,392-461 as functions over a flat dict of
parameters whose keys are the reference's state-dict names (``blocks.3.attn.a_to_qkv.weight`` ...).
Wiring is pinned by vectors the reference's own classes wrote at reduced width
(tests/test_oracle_leaf_goldens.py) and by structural invariants (tests/test_oracle_flux.py).

``linear_mode``:
  "plain"       F.linear in the tensors' dtype (the reference without enable_fp8_linear)
  "fp8_ref"     reference fp8 path: bare e4m3 casts, unit scales (utils/fp8_linear.py:28-60)
  "fp8_scaled"  per-tensor weight scale + per-token activation scale
"""
import torch
import torch.nn.functional as F

from . import dit_ops as O
from . import fp8

HIDDEN = 3072
HEADS = 24
HEAD_DIM = 128
AXES_DIM = (16, 56, 56)
THETA = 10000
EPS = 1e-6


class Params:
    """Flat parameter dict plus, in the fp8 modes, a cache of quantised weights."""

    def __init__(self, tensors, linear_mode="plain", heads=HEADS, head_dim=HEAD_DIM, axes_dim=AXES_DIM):
        assert linear_mode in ("plain", "fp8_ref", "fp8_scaled")
        self.t = tensors
        self.linear_mode = linear_mode
        self._q = {}
        self.lora = {}  # layer name -> list of (down (r,K), up (N,r), coefficient)
        # geometry: Flux.1-dev's unless a test builds a reduced model (flux_dit.py:343,352-356)
        self.heads, self.head_dim, self.axes_dim = heads, head_dim, tuple(axes_dim)

    def __getitem__(self, k):
        return self.t[k]

    def linear(self, x, name):
        """nn.Linear, or LoRALinear.forward when low-rank pairs are attached (models/basic/lora.py:29-32,137-141:
        w_x = linear(x); w_x += scale * alpha / rank * up(down(x)), every F.linear through the fp8 patch)."""
        y = self._linear(x, self.t[name + ".weight"], self.t.get(name + ".bias"), name)
        for j, (down, up, coef) in enumerate(self.lora.get(name, ())):
            h = self._linear(x, down, None, f"{name}#lora{j}.down")
            y = y + coef * self._linear(h, up, None, f"{name}#lora{j}.up")
        return y

    def _linear(self, x, w, b, key):
        if self.linear_mode == "plain":
            return F.linear(x, w, b)
        if key not in self._q:
            self._q[key] = fp8.quantize_weight(w, scaled=self.linear_mode == "fp8_scaled")
        w_q, w_s = self._q[key]
        return fp8.fp8_linear(x, w_q, w_s, b)


def init_params(num_double=19, num_single=38, dtype=torch.bfloat16, device="cpu", seed=0, std=0.02,
                guidance=True, bias_std=0.0):
    """Random Flux.1-dev-architecture parameters: Linear weights N(0, std), biases N(0, bias_std) (0 = zeros),
    RMSNorm weights 1.  Shapes follow FluxDiT.__init__ (flux_dit.py:341-364)."""
    g = torch.Generator(device="cpu").manual_seed(seed)
    t = {}

    def lin(name, n_in, n_out):
        t[name + ".weight"] = (torch.randn(n_out, n_in, generator=g) * std).to(dtype).to(device)
        if bias_std:
            t[name + ".bias"] = (torch.randn(n_out, generator=g) * bias_std).to(dtype).to(device)
        else:
            t[name + ".bias"] = torch.zeros(n_out, dtype=dtype, device=device)

    d = HIDDEN
    lin("time_embedder.timestep_embedder.0", 256, d)
    lin("time_embedder.timestep_embedder.2", d, d)
    if guidance:
        lin("guidance_embedder.timestep_embedder.0", 256, d)
        lin("guidance_embedder.timestep_embedder.2", d, d)
    lin("pooled_text_embedder.0", 768, d)
    lin("pooled_text_embedder.2", d, d)
    lin("context_embedder", 4096, d)
    lin("x_embedder", 64, d)
    for i in range(num_double):
        p = f"blocks.{i}."
        lin(p + "norm1_a.linear", d, 6 * d)
        lin(p + "norm1_b.linear", d, 6 * d)
        lin(p + "attn.a_to_qkv", d, 3 * d)
        lin(p + "attn.b_to_qkv", d, 3 * d)
        for n in ("norm_q_a", "norm_k_a", "norm_q_b", "norm_k_b"):
            t[p + f"attn.{n}.weight"] = torch.ones(HEAD_DIM, dtype=dtype, device=device)
        lin(p + "attn.a_to_out", d, d)
        lin(p + "attn.b_to_out", d, d)
        lin(p + "ff_a.0", d, 4 * d)
        lin(p + "ff_a.2", 4 * d, d)
        lin(p + "ff_b.0", d, 4 * d)
        lin(p + "ff_b.2", 4 * d, d)
    for i in range(num_single):
        p = f"single_blocks.{i}."
        lin(p + "norm.linear", d, 3 * d)
        lin(p + "to_qkv_mlp", d, 7 * d)
        t[p + "norm_q_a.weight"] = torch.ones(HEAD_DIM, dtype=dtype, device=device)
        t[p + "norm_k_a.weight"] = torch.ones(HEAD_DIM, dtype=dtype, device=device)
        lin(p + "proj_out", 5 * d, d)
    lin("final_norm_out.linear", d, 2 * d)
    lin("final_proj_out", d, 64)
    return t


def _heads(x, heads=HEADS, head_dim=HEAD_DIM):
    """(B,S,3*H*D) -> q,k,v each (B,H,S,D): view as (B,S,3H,D), transpose, chunk(3) (flux_dit.py:165-167)."""
    B, S, _ = x.shape
    x = x.view(B, S, 3 * heads, head_dim).transpose(1, 2)
    return x.chunk(3, dim=1)


def _merge(x):
    B, H, S, D = x.shape
    return x.transpose(1, 2).reshape(B, S, H * D)


def joint_attention(P, pre, a, b, freqs, attn=O.sdpa):
    """FluxJointAttention.forward (flux_dit.py:161-194); a = image stream, b = text stream, text first."""
    q_a, k_a, v_a = _heads(P.linear(a, pre + "a_to_qkv"), P.heads, P.head_dim)
    q_a = O.rms_norm(q_a, P[pre + "norm_q_a.weight"], EPS)
    k_a = O.rms_norm(k_a, P[pre + "norm_k_a.weight"], EPS)
    q_b, k_b, v_b = _heads(P.linear(b, pre + "b_to_qkv"), P.heads, P.head_dim)
    q_b = O.rms_norm(q_b, P[pre + "norm_q_b.weight"], EPS)
    k_b = O.rms_norm(k_b, P[pre + "norm_k_b.weight"], EPS)
    q = torch.cat([q_b, q_a], dim=2)
    k = torch.cat([k_b, k_a], dim=2)
    v = torch.cat([v_b, v_a], dim=2)
    q, k = O.apply_rope(q, freqs), O.apply_rope(k, freqs)
    h = _merge(attn(q, k, v)).to(q.dtype)
    n_txt = b.shape[1]
    h_b, h_a = h[:, :n_txt], h[:, n_txt:]
    return P.linear(h_a, pre + "a_to_out"), P.linear(h_b, pre + "b_to_out")


def ada_layer_norm6(P, name, x, emb):
    """AdaLayerNorm.forward, 6-way (transformer_helper.py:13-22): chunk order
    shift_msa, scale_msa, gate_msa, shift_mlp, scale_mlp, gate_mlp."""
    e = P.linear(F.silu(emb), name + ".linear").unsqueeze(1)
    shift_msa, scale_msa, gate_msa, shift_mlp, scale_mlp, gate_mlp = e.chunk(6, dim=2)
    return O.layer_norm_modulate(x, scale_msa, shift_msa, EPS), gate_msa, shift_mlp, scale_mlp, gate_mlp


def ada_layer_norm3(P, name, x, emb):
    """AdaLayerNormSingle.forward (transformer_helper.py:32-36): chunk order shift, scale, gate."""
    e = P.linear(F.silu(emb), name + ".linear")
    shift, scale, gate = e.chunk(3, dim=1)
    return O.layer_norm_modulate(x, scale[:, None], shift[:, None], EPS), gate


def ada_layer_norm_continuous(P, name, x, cond):
    """AdaLayerNormContinuous.forward (flux_dit.py:331-335): chunk order scale, shift."""
    e = P.linear(F.silu(cond), name + ".linear")
    scale, shift = torch.chunk(e, 2, dim=1)
    return O.layer_norm_modulate(x, scale[:, None], shift[:, None], EPS)


def joint_block(P, i, a, b, temb, freqs, attn=O.sdpa):
    """FluxJointTransformerBlock.forward (flux_dit.py:219-236)."""
    pre = f"blocks.{i}."
    na, gate_msa_a, shift_mlp_a, scale_mlp_a, gate_mlp_a = ada_layer_norm6(P, pre + "norm1_a", a, temb)
    nb, gate_msa_b, shift_mlp_b, scale_mlp_b, gate_mlp_b = ada_layer_norm6(P, pre + "norm1_b", b, temb)
    attn_a, attn_b = joint_attention(P, pre + "attn.", na, nb, freqs, attn)

    a = O.gated_residual(a, attn_a, gate_msa_a)
    na = O.layer_norm_modulate(a, scale_mlp_a, shift_mlp_a, EPS)
    ff = P.linear(O.gelu_tanh(P.linear(na, pre + "ff_a.0")), pre + "ff_a.2")
    a = O.gated_residual(a, ff, gate_mlp_a)

    b = O.gated_residual(b, attn_b, gate_msa_b)
    nb = O.layer_norm_modulate(b, scale_mlp_b, shift_mlp_b, EPS)
    ff = P.linear(O.gelu_tanh(P.linear(nb, pre + "ff_b.0")), pre + "ff_b.2")
    b = O.gated_residual(b, ff, gate_mlp_b)
    return a, b


def single_block(P, i, x, temb, freqs, attn=O.sdpa):
    """FluxSingleTransformerBlock.forward + process_attention (flux_dit.py:294-321);
    AdaLayerNormSingle chunk order shift, scale, gate (transformer_helper.py:32-36)."""
    pre = f"single_blocks.{i}."
    n, gate = ada_layer_norm3(P, pre + "norm", x, temb)
    h = P.linear(n, pre + "to_qkv_mlp")
    d = P.heads * P.head_dim
    qkv, mlp = h[:, :, : 3 * d], h[:, :, 3 * d:]
    q, k, v = _heads(qkv, P.heads, P.head_dim)
    q = O.rms_norm(q, P[pre + "norm_q_a.weight"], EPS)
    k = O.rms_norm(k, P[pre + "norm_k_a.weight"], EPS)
    q, k = O.apply_rope(q, freqs), O.apply_rope(k, freqs)
    att = _merge(attn(q, k, v)).to(q.dtype)
    mlp = O.gelu_tanh(mlp)
    out = gate.unsqueeze(1) * P.linear(torch.cat([att, mlp], dim=2), pre + "proj_out")
    return x + out


def timestep_mlp(P, name, t, dtype):
    """TimestepEmbeddings.forward (models/basic/timestep.py:78-81)."""
    e = O.timestep_embedding(t, 256).to(dtype)
    e = P.linear(e, name + ".timestep_embedder.0")
    return P.linear(F.silu(e), name + ".timestep_embedder.2")


def image_ids(height, width, batch, device, dtype):
    """FluxDiT.prepare_image_ids (flux_dit.py:376-390): (0, row, col) per 2x2 latent patch."""
    ids = torch.zeros(height // 2, width // 2, 3)
    ids[..., 1] += torch.arange(height // 2)[:, None]
    ids[..., 2] += torch.arange(width // 2)[None, :]
    return ids.reshape(1, -1, 3).repeat(batch, 1, 1).to(device=device, dtype=dtype)


def patchify(x):
    """'B C (H P) (W Q) -> B (H W) (C P Q)', P=Q=2 (flux_dit.py:366-368)."""
    B, C, H, W = x.shape
    x = x.view(B, C, H // 2, 2, W // 2, 2).permute(0, 2, 4, 1, 3, 5)
    return x.reshape(B, (H // 2) * (W // 2), C * 4)


def unpatchify(x, height, width):
    """'B (H W) (C P Q) -> B C (H P) (W Q)' (flux_dit.py:370-374)."""
    B, _, CPQ = x.shape
    C = CPQ // 4
    x = x.view(B, height // 2, width // 2, C, 2, 2).permute(0, 3, 1, 4, 2, 5)
    return x.reshape(B, C, height, width)


def flux_dit_forward(P, hidden_states, timestep, prompt_emb, pooled_prompt_emb, guidance, text_ids,
                     num_double=19, num_single=38, attn=O.sdpa):
    """FluxDiT.forward (flux_dit.py:392-461).  ``timestep`` is on the 0..1000 scale; guidance is
    multiplied by 1000 inside (flux_dit.py:413)."""
    dtype = hidden_states.dtype
    img_ids = image_ids(hidden_states.shape[-2], hidden_states.shape[-1], hidden_states.shape[0],
                        hidden_states.device, dtype)
    cond = timestep_mlp(P, "time_embedder", timestep, dtype)
    if guidance is not None and "guidance_embedder.timestep_embedder.0.weight" in P.t:
        cond = cond + timestep_mlp(P, "guidance_embedder", guidance * 1000, dtype)
    cond = cond + P.linear(F.silu(P.linear(pooled_prompt_emb, "pooled_text_embedder.0")), "pooled_text_embedder.2")
    txt = P.linear(prompt_emb, "context_embedder")
    freqs = O.rope_table(torch.cat((text_ids, img_ids), dim=1), P.axes_dim, THETA)
    height, width = hidden_states.shape[-2:]
    img = P.linear(patchify(hidden_states), "x_embedder")
    for i in range(num_double):
        img, txt = joint_block(P, i, img, txt, cond, freqs, attn)
    x = torch.cat([txt, img], dim=1)
    for i in range(num_single):
        x = single_block(P, i, x, cond, freqs, attn)
    x = x[:, txt.shape[1]:]
    x = ada_layer_norm_continuous(P, "final_norm_out", x, cond)
    x = P.linear(x, "final_proj_out")
    return unpatchify(x, height, width)
