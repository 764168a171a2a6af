"""The oracle's conditioning / RoPE / RMSNorm / timestep functions against vectors written by the
reference's own modules (tests/golden/make_leaf_module_fixtures.py made them in the build container
from diffsynth_engine/models/basic/transformer_helper.py and timestep.py; fp32, CPU).

These pin what no closed form fixes: the chunk orders of AdaLayerNorm (6-way) and AdaLayerNormSingle,
the axis -> pair concatenation order and 2x2 block layout of RoPEEmbedding, the cos-first order of the
timestep embedding, and RMSNorm's cast-then-scale order.
"""
import os

import pytest
import torch
from safetensors.torch import load_file

from oracle import dit_ops as O
from oracle import flux as OF

G = load_file(os.path.join(os.path.dirname(__file__), "golden", "leaf_modules.safetensors"))


def _params(prefix, name):
    return OF.Params({f"{name}.{k[len(prefix) + 7:]}": v for k, v in G.items() if k.startswith(prefix + ".param.")})


def _close(a, b, tol=2e-6):
    assert a.shape == b.shape, (a.shape, b.shape)
    assert (a - b).abs().max().item() <= tol * max(1.0, b.abs().max().item())


def test_ada_layer_norm_six_way_chunk_order():
    P = _params("ada6", "n")
    out = OF.ada_layer_norm6(P, "n", G["ada6.x"], G["ada6.emb"])
    for got, key in zip(out, ("out", "gate_msa", "shift_mlp", "scale_mlp", "gate_mlp")):
        _close(got, G["ada6." + key])


def test_ada_layer_norm_six_way_detects_a_swapped_chunk():
    # the fixture separates the candidates: shift and scale swapped must NOT match
    P = _params("ada6", "n")
    e = P.linear(torch.nn.functional.silu(G["ada6.emb"]), "n.linear").unsqueeze(1)
    scale_wrong, shift_wrong = e.chunk(6, dim=2)[:2]
    wrong = O.layer_norm_modulate(G["ada6.x"], scale_wrong, shift_wrong, 1e-6)
    assert (wrong - G["ada6.out"]).abs().max().item() > 1e-2


def test_ada_layer_norm_single_chunk_order():
    P = _params("ada3", "n")
    out, gate = OF.ada_layer_norm3(P, "n", G["ada3.x"], G["ada3.emb"])
    _close(out, G["ada3.out"])
    _close(gate, G["ada3.gate"])


def test_rope_embedding_table():
    axes = [int(a) for a in G["rope.axes"]]
    got = O.rope_table(G["rope.ids"], axes, 10000)
    assert got.dtype == torch.float32
    assert torch.equal(got, G["rope.out"]), (got - G["rope.out"]).abs().max()


def test_rms_norm():
    got = O.rms_norm(G["rmsnorm.x"], G["rmsnorm.param.weight"], 1e-6)
    _close(got, G["rmsnorm.out"], 1e-6)


def test_timestep_embedding_and_mlp():
    proj = O.timestep_embedding(G["timestep.t"], 16)
    _close(proj, G["timestep.proj"], 1e-6)
    P = _params("timestep", "te")
    # the oracle's MLP wrapper embeds with 256 channels (the model's value); restate its two linears here
    e = P.linear(proj, "te.timestep_embedder.0")
    out = P.linear(torch.nn.functional.silu(e), "te.timestep_embedder.2")
    _close(out, G["timestep.out"], 1e-5)


# ---- block and model wiring: vectors written by the reference's own flux_dit.py classes at reduced
# ---- width (tests/golden/make_flux_block_fixtures.py): dim 32, 2 heads of 16, RoPE axes (4, 6, 6)
B = load_file(os.path.join(os.path.dirname(__file__), "golden", "flux_blocks.safetensors"))
GEOM = dict(heads=2, head_dim=16, axes_dim=(4, 6, 6))


def _bparams(prefix, name=""):
    return OF.Params({name + k[len(prefix) + 7:]: v for k, v in B.items() if k.startswith(prefix + ".param.")}, **GEOM)


def test_joint_block_against_reference_vectors():
    P = _bparams("joint", "blocks.0.")
    freqs = O.rope_table(B["joint.ids"], GEOM["axes_dim"], 10000)
    img, txt = OF.joint_block(P, 0, B["joint.img"], B["joint.txt"], B["joint.temb"], freqs)
    _close(img, B["joint.out_img"], 2e-5)
    _close(txt, B["joint.out_txt"], 2e-5)


def test_joint_block_fixture_separates_text_first_from_image_first():
    # image-first concatenation (the plausible mistake) must not reproduce the vectors
    P = _bparams("joint", "blocks.0.")
    ids = B["joint.ids"]
    n_txt = B["joint.txt"].shape[1]
    swapped = torch.cat([ids[:, n_txt:], ids[:, :n_txt]], dim=1)
    freqs = O.rope_table(swapped, GEOM["axes_dim"], 10000)
    txt, img = OF.joint_block(P, 0, B["joint.txt"], B["joint.img"], B["joint.temb"], freqs)  # roles swapped
    assert (img - B["joint.out_img"]).abs().max().item() > 1e-2


def test_single_block_against_reference_vectors():
    P = _bparams("single", "single_blocks.0.")
    freqs = O.rope_table(B["single.ids"], GEOM["axes_dim"], 10000)
    _close(OF.single_block(P, 0, B["single.x"], B["single.temb"], freqs), B["single.out"], 2e-5)


def test_ada_layer_norm_continuous_chunk_order():
    P = _bparams("adacont", "n.")
    _close(OF.ada_layer_norm_continuous(P, "n", B["adacont.x"], B["adacont.cond"]), B["adacont.out"], 1e-5)


def test_model_forward_against_reference_vectors():
    P = _bparams("model")
    got = OF.flux_dit_forward(P, B["model.hidden_states"], B["model.timestep"], B["model.prompt_emb"],
                              B["model.pooled_prompt_emb"], B["model.guidance"], B["model.text_ids"],
                              num_double=2, num_single=2)
    _close(got, B["model.out"], 5e-5)


# ---- WanDiT: vectors written by the reference's own class at reduced size (tests/golden/make_wan_fixtures.py)
W = load_file(os.path.join(os.path.dirname(__file__), "golden", "wan_dit.safetensors"))
WCFG = dict(dim=40, in_dim=4, ffn_dim=48, out_dim=4, text_dim=12, freq_dim=16, eps=1e-6, patch_size=(1, 2, 2),
            num_heads=2, num_layers=2)


def _wparams():
    from oracle import wan as OW
    return OW, OW.Params({k[6:]: v.clone() for k, v in W.items() if k.startswith("param.")})


def test_wan_rope_table_against_reference_vectors():
    OW, _ = _wparams()
    got = torch.view_as_real(OW.freqs_cis_3d(WCFG["dim"] // WCFG["num_heads"], 3, 2, 3))
    assert got.dtype == torch.float64
    _close(got, W["block.freqs_real"], 1e-12)


def test_wan_block_against_reference_vectors():
    OW, P = _wparams()
    freqs = torch.view_as_complex(W["block.freqs_real"])
    got = OW.dit_block(P, 1, W["block.x"], W["block.context"], W["block.t_mod"], freqs, WCFG)
    _close(got, W["block.out"], 2e-5)


def test_wan_model_forward_against_reference_vectors():
    OW, P = _wparams()
    got = OW.wan_dit_forward(P, W["model.x"], W["model.context"], W["model.timestep"], WCFG)
    _close(got, W["model.out"], 5e-5)


# ---- WanDiT, image-to-video form (has_image_input=True; tests/golden/make_wan_i2v_fixtures.py)
WI = load_file(os.path.join(os.path.dirname(__file__), "golden", "wan_i2v.safetensors"))
WICFG = dict(WCFG, in_dim=8)


def _wiparams(drop=()):
    from oracle import wan as OW
    return OW, OW.Params({k[6:]: v.clone() for k, v in WI.items() if k.startswith("param.") and
                          not any(d in k for d in drop)})


def test_wan_i2v_img_emb_against_reference_vectors():
    OW, P = _wiparams()
    _close(OW.img_emb(P, WI["model.clip_feature"]), WI["img_emb.out"], 2e-5)
    # tanh-GELU in place of the erf form is a different function at this bar
    import torch.nn.functional as F
    h = F.layer_norm(WI["model.clip_feature"], (24,), P["img_emb.proj.0.weight"], P["img_emb.proj.0.bias"], 1e-5)
    h = P.linear(F.gelu(P.linear(h, "img_emb.proj.1"), approximate="tanh"), "img_emb.proj.3")
    wrong = F.layer_norm(h, (40,), P["img_emb.proj.4.weight"], P["img_emb.proj.4.bias"], 1e-5)
    assert (wrong - WI["img_emb.out"]).abs().max() > 1e-3


def test_wan_i2v_block_against_reference_vectors():
    OW, P = _wiparams()
    freqs = torch.view_as_complex(WI["block.freqs_real"])
    got = OW.dit_block(P, 1, WI["block.x"], WI["block.context"], WI["block.t_mod"], freqs, WICFG)
    _close(got, WI["block.out"], 2e-5)
    # negative controls: without the image branch (all 262 rows as text), and with the image rows taken from the
    # END of the context instead of its first 257 rows, the block is a different function
    _, Pt = _wiparams(drop=("k_img", "v_img"))
    assert (OW.dit_block(Pt, 1, WI["block.x"], WI["block.context"], WI["block.t_mod"], freqs, WICFG)
            - WI["block.out"]).abs().max() > 1e-2
    swapped = torch.cat([WI["block.context"][:, 257:], WI["block.context"][:, :257]], dim=1)
    assert (OW.dit_block(P, 1, WI["block.x"], swapped, WI["block.t_mod"], freqs, WICFG)
            - WI["block.out"]).abs().max() > 1e-2


def test_wan_i2v_model_forward_against_reference_vectors():
    OW, P = _wiparams()
    got = OW.wan_dit_forward(P, WI["model.x"], WI["model.context"], WI["model.timestep"], WICFG,
                             clip_feature=WI["model.clip_feature"], y=WI["model.y"])
    _close(got, WI["model.out"], 5e-5)
    # channel order of the concat: [x | y], not [y | x]
    wrong = OW.wan_dit_forward(P, WI["model.y"], WI["model.context"], WI["model.timestep"], WICFG,
                               clip_feature=WI["model.clip_feature"], y=WI["model.x"])
    assert (wrong - WI["model.out"]).abs().max() > 1e-2


# ---- the reference's fp8 patch of F.linear (diffsynth_engine/utils/fp8_linear.py) on one nn.Linear
def test_reference_fp8_linear_vectors():
    from oracle import fp8
    w_q, w_s = fp8.quantize_weight(G["fp8.weight_bf16"], scaled=False)
    assert w_s is None
    assert torch.equal(w_q.view(torch.uint8), G["fp8.weight_e4m3_bits"])
    # numpy bit-level cast agrees with what enable_fp8_linear stored
    bits = fp8.e4m3_from_f32(G["fp8.weight_bf16"].float().numpy())
    assert (bits == G["fp8.weight_e4m3_bits"].numpy()).all()
    for x, y in ((G["fp8.x3"], G["fp8.y3"]), (G["fp8.x2"], G["fp8.y2"])):
        got = fp8.fp8_linear(x, w_q, None, G["fp8.bias"])
        assert got.shape == y.shape and got.dtype == y.dtype
        # same products, fp32 accumulation in a different order: at most one bf16 ulp apart
        d = (got.float() - y.float()).abs()
        assert (d <= y.float().abs() * 2 ** -7 + 1e-6).all(), d.max()
        assert (d > 0).float().mean().item() < 0.05


# ---- the reference's FluxDiT.forward UNDER ITS FP8 PATCH, bf16, head dim 128 (tests/golden/make_flux_fp8_fixture.py:
# ---- hidden 256 = 2 heads x 128, RoPE axes (16,56,56), 1 joint + 1 single block, enable_fp8_linear + fp8_inference)
def load_fp8_d128_fixture():
    """(state dict with float8_e4m3fn Linear weights, inputs, output) of flux_fp8_d128.safetensors."""
    raw = load_file(os.path.join(os.path.dirname(__file__), "golden", "flux_fp8_d128.safetensors"))
    sd = {k[len("param."):]: (v.view(torch.float8_e4m3fn) if v.dtype == torch.uint8 else v)
          for k, v in raw.items() if k.startswith("param.")}
    inputs = {k[len("in."):]: v for k, v in raw.items() if k.startswith("in.")}
    return sd, inputs, raw["out"]


def test_fp8_reference_mode_against_the_references_own_fp8_forward():
    """The oracle's "fp8_ref" mode (bare e4m3 casts, unit scales, fp32 accumulation, bf16 rounding points of the
    torch op sequence) against what the reference computed with torch._scaled_mm on the CPU.  With the attention
    backend the reference used there (torch's bf16 SDPA) the oracle reproduces the reference's output BIT FOR
    BIT: every chunk order, rounding point, bias and cast of the fp8 path is pinned.  With the oracle's own fp32
    softmax attention the difference is that backend's bf16 arithmetic alone."""
    sd, inputs, want = load_fp8_d128_fixture()
    P = OF.Params(sd, "fp8_ref", heads=2, head_dim=128, axes_dim=(16, 56, 56))
    same = OF.flux_dit_forward(P, **inputs, num_double=1, num_single=1,
                               attn=torch.nn.functional.scaled_dot_product_attention)
    assert same.dtype == torch.bfloat16 and torch.equal(same, want)
    got = OF.flux_dit_forward(P, **inputs, num_double=1, num_single=1)
    cos = torch.nn.functional.cosine_similarity(got.float().flatten(), want.float().flatten(), dim=0).item()
    assert cos >= 0.9998, cos
    # the scaled mode is a different function of the same weights: the fixture tells the two apart
    Ps = OF.Params({k: (v.float() if v.dtype == torch.float8_e4m3fn else v) for k, v in sd.items()}, "fp8_scaled",
                   heads=2, head_dim=128, axes_dim=(16, 56, 56))
    other = OF.flux_dit_forward(Ps, **inputs, num_double=1, num_single=1)
    assert not torch.equal(other, want)
