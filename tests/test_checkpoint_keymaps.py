"""Checkpoint key conversion against vectors written by the reference's own FluxDiTStateDictConverter
(tests/golden/make_keymap_fixtures.py): same output names, same tensors (concatenation order of the packed
projections, swapped halves of the final modulation), unknown keys dropped, native layout passed through."""
import os

import torch
from safetensors.torch import load_file

from diffsynth_engine_amd.checkpoint import convert_flux_state_dict

G = load_file(os.path.join(os.path.dirname(__file__), "golden", "flux_keymaps.safetensors"))


def _case(tag):
    src = {k.split("::", 1)[1]: v for k, v in G.items() if k.startswith(f"in.{tag}::")}
    want = {k.split("::", 1)[1]: v for k, v in G.items() if k.startswith(f"out.{tag}::")}
    return src, want


def _check(tag):
    src, want = _case(tag)
    got = convert_flux_state_dict(src)
    assert sorted(got) == sorted(want)
    for k in want:
        assert got[k].shape == want[k].shape and torch.equal(got[k], want[k]), k


def test_original_layout():
    _check("civitai")


def test_original_layout_without_the_model_prefix():
    src, want = _case("civitai")
    src = {k.replace("model.diffusion_model.", ""): v for k, v in src.items()}
    got = convert_flux_state_dict(src)
    assert sorted(got) == sorted(want) and all(torch.equal(got[k], want[k]) for k in want)


def test_diffusers_layout():
    _check("diffusers")


def test_native_layout_is_returned_as_is():
    _, want = _case("civitai")
    assert convert_flux_state_dict(want) is want
