"""The HIP runner against vectors the REFERENCE ITSELF computed (not the oracle's restatement), and the
checkpoint chain foreign layout -> convert_flux_state_dict -> runner.

tests/golden/flux_fp8_d128.safetensors holds FluxDiT.forward of the reference under its own fp8 patch
(diffsynth_engine/utils/fp8_linear.py:7-64; bf16, unit scales) at a size the kernels take directly: hidden 256 =
2 heads x 128, RoPE axes (16,56,56), 1 joint + 1 single block, 24 text + 24 image tokens, non-zero biases and
non-trivial RMSNorm weights (tests/golden/make_flux_fp8_fixture.py)."""
import random

import pytest
import torch

from oracle import flux as oflux
from test_oracle_leaf_goldens import load_fp8_d128_fixture

pytestmark = pytest.mark.gpu


def _cos(a, b):
    return torch.nn.functional.cosine_similarity(a.float().flatten().cpu(), b.float().flatten().cpu(), dim=0).item()


def test_runner_in_reference_mode_matches_the_references_own_fp8_forward(dev):
    """scaled=False is the reference's arithmetic: bare e4m3 casts of activations and weights, unit scales
    (fp8_linear.py:35-48).  The fixture's Linear weights are the e4m3 bytes the reference's enable_fp8_linear left
    in its modules, so both sides multiply the same codes.  The oracle with the reference's attention backend
    reproduces this output bit for bit (tests/test_oracle_leaf_goldens.py); with its own fp32-softmax attention it
    reaches cosine 0.99990.  The kernels are held to 0.9995, the one-block bar of every teacher-forced test."""
    from diffsynth_engine_amd.flux_dit import FluxDiTRunner

    sd, inputs, want = load_fp8_d128_fixture()
    R = FluxDiTRunner({k: v.to(dev) for k, v in sd.items()}, 1, 1, scaled=False, device=dev)
    assert (R.hidden, R.heads) == (256, 2)
    got = R(**{k: v.to(dev) for k, v in inputs.items()}).cpu()
    assert got.shape == want.shape and got.dtype == torch.bfloat16
    c = _cos(got, want)
    assert c >= 0.9995, c
    assert (got.float() - want.float()).abs().max().item() <= 2 ** -3 * want.float().abs().max().item()


# ---- engine names -> the two foreign checkpoint layouts (the inverse of what FluxDiTStateDictConverter.convert,
# ---- flux_dit.py:24-123, does; checkpoint.py's forward direction is pinned by the reference converter's own
# ---- vectors in tests/test_checkpoint_keymaps.py)
_BFL_TOP = {"time_embedder.timestep_embedder.0": "time_in.in_layer", "time_embedder.timestep_embedder.2": "time_in.out_layer",
            "guidance_embedder.timestep_embedder.0": "guidance_in.in_layer",
            "guidance_embedder.timestep_embedder.2": "guidance_in.out_layer",
            "pooled_text_embedder.0": "vector_in.in_layer", "pooled_text_embedder.2": "vector_in.out_layer",
            "context_embedder": "txt_in", "x_embedder": "img_in", "final_proj_out": "final_layer.linear",
            "final_norm_out.linear": "final_layer.adaLN_modulation.1"}


def _to_black_forest(sd):
    out = {}
    for name, t in sd.items():
        mod, _, leaf = name.rpartition(".")
        if mod in _BFL_TOP:
            if mod == "final_norm_out.linear":  # engine (scale, shift) -> original (shift, scale)
                half = t.shape[0] // 2
                t = torch.cat([t[half:], t[:half]], dim=0)
            out[f"model.diffusion_model.{_BFL_TOP[mod]}.{leaf}"] = t
            continue
        parts = name.split(".")
        i, rest = parts[1], ".".join(parts[2:])
        if parts[0] == "blocks":
            for s, stream in (("a", "img"), ("b", "txt")):
                table = {f"attn.{s}_to_qkv": f"{stream}_attn.qkv", f"attn.{s}_to_out": f"{stream}_attn.proj",
                         f"ff_{s}.0": f"{stream}_mlp.0", f"ff_{s}.2": f"{stream}_mlp.2", f"norm1_{s}.linear": f"{stream}_mod.lin"}
                if mod.split(".", 2)[2] in table:
                    out[f"model.diffusion_model.double_blocks.{i}.{table[mod.split('.', 2)[2]]}.{leaf}"] = t
                elif rest == f"attn.norm_q_{s}.weight":
                    out[f"model.diffusion_model.double_blocks.{i}.{stream}_attn.norm.query_norm.scale"] = t
                elif rest == f"attn.norm_k_{s}.weight":
                    out[f"model.diffusion_model.double_blocks.{i}.{stream}_attn.norm.key_norm.scale"] = t
        else:
            table = {"to_qkv_mlp": "linear1", "proj_out": "linear2", "norm.linear": "modulation.lin"}
            key = mod.split(".", 2)[2]
            if key in table:
                out[f"model.diffusion_model.single_blocks.{i}.{table[key]}.{leaf}"] = t
            elif rest == "norm_q_a.weight":
                out[f"model.diffusion_model.single_blocks.{i}.norm.query_norm.scale"] = t
            elif rest == "norm_k_a.weight":
                out[f"model.diffusion_model.single_blocks.{i}.norm.key_norm.scale"] = t
    assert len(out) == len(sd)
    return out


def _to_diffusers(sd, hidden):
    top = {"context_embedder": "context_embedder", "x_embedder": "x_embedder",
           "time_embedder.timestep_embedder.0": "time_text_embed.timestep_embedder.linear_1",
           "time_embedder.timestep_embedder.2": "time_text_embed.timestep_embedder.linear_2",
           "guidance_embedder.timestep_embedder.0": "time_text_embed.guidance_embedder.linear_1",
           "guidance_embedder.timestep_embedder.2": "time_text_embed.guidance_embedder.linear_2",
           "pooled_text_embedder.0": "time_text_embed.text_embedder.linear_1",
           "pooled_text_embedder.2": "time_text_embed.text_embedder.linear_2",
           "final_norm_out.linear": "norm_out.linear", "final_proj_out": "proj_out"}
    double = {"norm1_a.linear": "norm1.linear", "norm1_b.linear": "norm1_context.linear", "attn.a_to_out": "attn.to_out.0",
              "attn.b_to_out": "attn.to_add_out", "ff_a.0": "ff.net.0.proj", "ff_a.2": "ff.net.2",
              "ff_b.0": "ff_context.net.0.proj", "ff_b.2": "ff_context.net.2", "attn.norm_q_a": "attn.norm_q",
              "attn.norm_k_a": "attn.norm_k", "attn.norm_q_b": "attn.norm_added_q", "attn.norm_k_b": "attn.norm_added_k"}
    single = {"norm.linear": "norm.linear", "proj_out": "proj_out", "norm_q_a": "attn.norm_q", "norm_k_a": "attn.norm_k"}
    out = {}
    for name, t in sd.items():
        mod, _, leaf = name.rpartition(".")
        if mod in top:
            out[f"{top[mod]}.{leaf}"] = t
            continue
        parts = mod.split(".")
        i, key = parts[1], ".".join(parts[2:])
        if parts[0] == "blocks":
            pre = f"transformer_blocks.{i}."
            if key == "attn.a_to_qkv":
                for n, piece in zip(("attn.to_q", "attn.to_k", "attn.to_v"), t.split(hidden, dim=0)):
                    out[f"{pre}{n}.{leaf}"] = piece.contiguous()
            elif key == "attn.b_to_qkv":
                for n, piece in zip(("attn.add_q_proj", "attn.add_k_proj", "attn.add_v_proj"), t.split(hidden, dim=0)):
                    out[f"{pre}{n}.{leaf}"] = piece.contiguous()
            else:
                out[f"{pre}{double[key]}.{leaf}"] = t
        else:
            pre = f"single_transformer_blocks.{i}."
            if key == "to_qkv_mlp":
                q, k, v, mlp = t.split([hidden, hidden, hidden, t.shape[0] - 3 * hidden], dim=0)
                for n, piece in (("attn.to_q", q), ("attn.to_k", k), ("attn.to_v", v), ("proj_mlp", mlp)):
                    out[f"{pre}{n}.{leaf}"] = piece.contiguous()
            else:
                out[f"{pre}{single[key]}.{leaf}"] = t
    return out


@pytest.mark.parametrize("layout", ["black_forest", "diffusers"])
def test_foreign_checkpoint_through_the_converter_into_the_runner(dev, layout):
    """FluxDiTStateDictConverter.convert -> from_state_dict -> fp8 (flux_dit.py:24-123,463-478; fp8_linear.py:7-17)
    as one chain: a bf16 state dict in a third-party layout, keys in shuffled and in sorted order (a safetensors
    file lists `x.bias` before `x.weight`), non-zero biases, goes through convert_flux_state_dict into the runner,
    which quantises it (scaled mode).  The step output is bit-identical to the runner built from the engine-layout
    dict, and matches the oracle given the same engine-layout weights."""
    from diffsynth_engine_amd.checkpoint import convert_flux_state_dict
    from diffsynth_engine_amd.flux_dit import FluxDiTRunner

    sd8, inputs, _ = load_fp8_d128_fixture()
    engine = {k: (v.float().bfloat16() if v.dtype == torch.float8_e4m3fn else v) for k, v in sd8.items()}
    assert any(k.endswith(".bias") and float(v.float().abs().max()) > 0 for k, v in engine.items())
    foreign = _to_black_forest(engine) if layout == "black_forest" else _to_diffusers(engine, 256)
    assert not set(foreign) & set(engine) or layout == "diffusers"  # (diffusers shares two top-level names)
    inp = {k: v.to(dev) for k, v in inputs.items()}
    base = FluxDiTRunner(engine, 1, 1, scaled=True, device=dev)(**inp)
    keys = sorted(foreign)
    assert any(a.endswith(".bias") and a[:-5] + ".weight" in keys[i:] for i, a in enumerate(keys))  # a bias comes first
    for order in (keys, random.Random(5).sample(keys, len(keys))):
        converted = convert_flux_state_dict({k: foreign[k] for k in order})
        assert sorted(converted) == sorted(engine)
        got = FluxDiTRunner(converted, 1, 1, scaled=True, device=dev)(**inp)
        assert torch.equal(got, base)
    want = oflux.flux_dit_forward(oflux.Params(engine, "fp8_scaled", heads=2, head_dim=128, axes_dim=(16, 56, 56)),
                                  **inputs, num_double=1, num_single=1)
    assert _cos(base, want) >= 0.999, _cos(base, want)
    # dropping the biases must be visible at this bar, or the comparison above would not notice a lost bias
    nobias = {k: (torch.zeros_like(v) if k.endswith(".bias") else v) for k, v in engine.items()}
    assert _cos(FluxDiTRunner(nobias, 1, 1, scaled=True, device=dev)(**inp), want) < 0.99
