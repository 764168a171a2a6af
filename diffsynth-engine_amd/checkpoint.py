"""Checkpoint key maps for the Flux DiT: third-party layouts -> the state-dict names the runner takes.

Mirrors ``FluxDiTStateDictConverter.convert`` (diffsynth_engine/models/flux/flux_dit.py:24-123, tables in
conf/models/flux/flux_dit.json): the layout is detected from marker keys, tensors are renamed, separate
q/k/v (and, for single blocks, the MLP input) projections are concatenated into the packed projections the
engine uses, and the two halves of the original final-layer modulation are swapped (shift,scale ->
scale,shift).  Tensors are passed through untouched otherwise; quantisation happens when the runner (or
``enable_fp8_linear``) takes them.
"""
from typing import Dict

import torch

_BLACK_FOREST_TOP = {          # original ("civitai") layout, top-level modules
    "time_in.in_layer": "time_embedder.timestep_embedder.0",
    "time_in.out_layer": "time_embedder.timestep_embedder.2",
    "guidance_in.in_layer": "guidance_embedder.timestep_embedder.0",
    "guidance_in.out_layer": "guidance_embedder.timestep_embedder.2",
    "vector_in.in_layer": "pooled_text_embedder.0",
    "vector_in.out_layer": "pooled_text_embedder.2",
    "txt_in": "context_embedder",
    "img_in": "x_embedder",
    "final_layer.linear": "final_proj_out",
    "final_layer.adaLN_modulation.1": "final_norm_out.linear",
}


def _bfl_double(rest: str):
    """'img_attn.qkv.weight' -> 'attn.a_to_qkv.weight' ... (image stream = a, text stream = b)."""
    stream, _, tail = rest.partition("_")
    if stream not in ("img", "txt"):
        return None
    s = "a" if stream == "img" else "b"
    table = {
        "attn.qkv": f"attn.{s}_to_qkv", "attn.proj": f"attn.{s}_to_out", "mlp.0": f"ff_{s}.0", "mlp.2": f"ff_{s}.2",
        "mod.lin": f"norm1_{s}.linear",
    }
    if tail == "attn.norm.query_norm.scale":
        return f"attn.norm_q_{s}.weight"
    if tail == "attn.norm.key_norm.scale":
        return f"attn.norm_k_{s}.weight"
    mod, _, leaf = tail.rpartition(".")
    return f"{table[mod]}.{leaf}" if mod in table and leaf in ("weight", "bias") else None


def _bfl_single(rest: str):
    table = {"linear1": "to_qkv_mlp", "linear2": "proj_out", "modulation.lin": "norm.linear"}
    if rest == "norm.query_norm.scale":
        return "norm_q_a.weight"
    if rest == "norm.key_norm.scale":
        return "norm_k_a.weight"
    mod, _, leaf = rest.rpartition(".")
    return f"{table[mod]}.{leaf}" if mod in table and leaf in ("weight", "bias") else None


def _from_black_forest(sd: Dict[str, torch.Tensor]) -> Dict[str, torch.Tensor]:
    out = {}
    for name, t in sd.items():
        if name.startswith("model.diffusion_model."):
            name = name[len("model.diffusion_model."):]
        mod, _, leaf = name.rpartition(".")
        if mod in _BLACK_FOREST_TOP and leaf in ("weight", "bias"):
            if mod == "final_layer.adaLN_modulation.1":
                half = t.shape[0] // 2  # stored (shift, scale); AdaLayerNormContinuous chunks (scale, shift)
                t = torch.cat([t[half:], t[:half]], dim=0)
            out[f"{_BLACK_FOREST_TOP[mod]}.{leaf}"] = t
            continue
        parts = name.split(".")
        if parts[0] == "double_blocks" and len(parts) > 2:
            new = _bfl_double(".".join(parts[2:]))
            if new:
                out[f"blocks.{parts[1]}.{new}"] = t
        elif parts[0] == "single_blocks" and len(parts) > 2:
            new = _bfl_single(".".join(parts[2:]))
            if new:
                out[f"single_blocks.{parts[1]}.{new}"] = t
    return out


_DIFFUSERS_TOP = {
    "context_embedder": "context_embedder",
    "x_embedder": "x_embedder",
    "time_text_embed.timestep_embedder.linear_1": "time_embedder.timestep_embedder.0",
    "time_text_embed.timestep_embedder.linear_2": "time_embedder.timestep_embedder.2",
    "time_text_embed.guidance_embedder.linear_1": "guidance_embedder.timestep_embedder.0",
    "time_text_embed.guidance_embedder.linear_2": "guidance_embedder.timestep_embedder.2",
    "time_text_embed.text_embedder.linear_1": "pooled_text_embedder.0",
    "time_text_embed.text_embedder.linear_2": "pooled_text_embedder.2",
    "norm_out.linear": "final_norm_out.linear",
    "proj_out": "final_proj_out",
}
_DIFFUSERS_DOUBLE = {
    "norm1.linear": "norm1_a.linear", "norm1_context.linear": "norm1_b.linear",
    "attn.to_q": "attn.a_to_q", "attn.to_k": "attn.a_to_k", "attn.to_v": "attn.a_to_v",
    "attn.to_out.0": "attn.a_to_out",
    "attn.add_q_proj": "attn.b_to_q", "attn.add_k_proj": "attn.b_to_k", "attn.add_v_proj": "attn.b_to_v",
    "attn.to_add_out": "attn.b_to_out",
    "ff.net.0.proj": "ff_a.0", "ff.net.2": "ff_a.2", "ff_context.net.0.proj": "ff_b.0", "ff_context.net.2": "ff_b.2",
    "attn.norm_q": "attn.norm_q_a", "attn.norm_k": "attn.norm_k_a",
    "attn.norm_added_q": "attn.norm_q_b", "attn.norm_added_k": "attn.norm_k_b",
    "proj_out": "proj_out",
}
_DIFFUSERS_SINGLE = {
    "attn.to_q": "a_to_q", "attn.to_k": "a_to_k", "attn.to_v": "a_to_v", "attn.norm_q": "norm_q_a",
    "attn.norm_k": "norm_k_a", "norm.linear": "norm.linear", "proj_mlp": "mlp_in", "proj_out": "proj_out",
}


def _from_diffusers(sd: Dict[str, torch.Tensor]) -> Dict[str, torch.Tensor]:
    out = {}
    for name, t in sd.items():
        mod, _, leaf = name.rpartition(".")
        if leaf not in ("weight", "bias"):
            continue
        if mod in _DIFFUSERS_TOP:
            out[f"{_DIFFUSERS_TOP[mod]}.{leaf}"] = t
            continue
        parts = mod.split(".")
        if parts[0] == "transformer_blocks" and ".".join(parts[2:]) in _DIFFUSERS_DOUBLE:
            out[f"blocks.{parts[1]}.{_DIFFUSERS_DOUBLE['.'.join(parts[2:])]}.{leaf}"] = t
        elif parts[0] == "single_transformer_blocks" and ".".join(parts[2:]) in _DIFFUSERS_SINGLE:
            out[f"single_blocks.{parts[1]}.{_DIFFUSERS_SINGLE['.'.join(parts[2:])]}.{leaf}"] = t
    # packed projections: rows [q | k | v] (joint blocks, both streams) and [q | k | v | mlp] (single blocks)
    for name in [n for n in out if ".mlp_in." in n]:
        q, k, v = (name.replace(".mlp_in.", f".a_to_{c}.") for c in "qkv")
        out[name.replace(".mlp_in.", ".to_qkv_mlp.")] = torch.cat([out.pop(q), out.pop(k), out.pop(v), out.pop(name)], dim=0)
    for s in ("a", "b"):
        for name in [n for n in out if f".{s}_to_q." in n]:
            k, v = name.replace(f".{s}_to_q.", f".{s}_to_k."), name.replace(f".{s}_to_q.", f".{s}_to_v.")
            out[name.replace(f".{s}_to_q.", f".{s}_to_qkv.")] = torch.cat([out.pop(name), out.pop(k), out.pop(v)], dim=0)
    return out


def convert_flux_state_dict(state_dict: Dict[str, torch.Tensor]) -> Dict[str, torch.Tensor]:
    """Return a state dict with the engine's FluxDiT parameter names, whatever layout came in."""
    if "txt_in.weight" in state_dict or "model.diffusion_model.txt_in.weight" in state_dict:
        return _from_black_forest(state_dict)
    if "time_text_embed.timestep_embedder.linear_1.weight" in state_dict:
        return _from_diffusers(state_dict)
    return state_dict
