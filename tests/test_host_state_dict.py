"""Host logic of the block runners' checkpoint ingestion, on the CPU (already quantised weights: no kernel runs).

The reference loads through ``load_state_dict`` (diffsynth_engine/models/flux/flux_dit.py:463-478), which does not
depend on key order; a safetensors file lists ``x.bias`` before ``x.weight``."""
import pytest
import torch

FP8 = torch.float8_e4m3fn


def _tiny():
    g = torch.Generator().manual_seed(0)
    sd = {}
    for name, (n, k) in {"blocks.0.attn.a_to_qkv": (48, 16), "final_proj_out": (8, 16)}.items():
        sd[name + ".weight"] = (torch.randn(n, k, generator=g)).to(FP8)
        sd[name + ".weight_scale"] = torch.rand((), generator=g) + 0.5
        sd[name + ".bias"] = torch.randn(n, generator=g)
    sd["blocks.0.attn.norm_q_a.weight"] = torch.ones(128)
    sd["blocks.0.norm3.weight"] = torch.ones(16)
    sd["blocks.0.norm3.bias"] = torch.randn(16, generator=g)
    sd["blocks.0.modulation"] = torch.randn(1, 6, 16, generator=g)
    return sd


@pytest.mark.parametrize("order", ["sorted", "reversed", "insertion"])
def test_ingestion_does_not_depend_on_key_order(order):
    from diffsynth_engine_amd.flux_dit import ingest_state_dict

    sd = _tiny()
    keys = {"sorted": sorted(sd), "reversed": sorted(sd, reverse=True), "insertion": list(sd)}[order]
    assert order != "sorted" or keys.index("final_proj_out.bias") < keys.index("final_proj_out.weight")
    lin, other = ingest_state_dict(((k, sd[k]) for k in keys), "cpu", scaled=True)
    assert sorted(lin) == ["blocks.0.attn.a_to_qkv", "final_proj_out"]
    for name, L in lin.items():
        assert torch.equal(L.b.float(), sd[name + ".bias"].bfloat16().float())
        assert torch.equal(L.s, sd[name + ".weight_scale"].float()) and L.s.dim() == 0
        assert torch.equal(L.w.view(torch.uint8), sd[name + ".weight"].view(torch.uint8))
    # what is not a Linear keeps its full key, the affine bias of a norm layer included
    assert sorted(other) == ["blocks.0.attn.norm_q_a.weight", "blocks.0.modulation", "blocks.0.norm3.bias",
                             "blocks.0.norm3.weight"]


def test_quantised_weight_without_its_scale_is_refused_in_scaled_mode():
    from diffsynth_engine_amd.flux_dit import ingest_state_dict

    sd = _tiny()
    del sd["final_proj_out.weight_scale"]
    with pytest.raises(ValueError, match="final_proj_out"):
        ingest_state_dict(sd, "cpu", scaled=True)
    lin, _ = ingest_state_dict(sd, "cpu", scaled=False)  # the reference's unit-scale weights carry none
    assert lin["final_proj_out"].s is None and lin["blocks.0.attn.a_to_qkv"].s is not None


def test_scale_without_a_weight_is_an_error():
    from diffsynth_engine_amd.flux_dit import ingest_state_dict

    sd = _tiny()
    sd["nowhere.weight_scale"] = torch.ones(())
    with pytest.raises(KeyError):
        ingest_state_dict(sd, "cpu", scaled=True)


def test_flux_runner_refuses_entries_it_has_no_use_for():
    from diffsynth_engine_amd.flux_dit import FluxDiTRunner

    sd = _tiny()
    with pytest.raises(KeyError, match="modulation|norm3"):
        FluxDiTRunner(sd, 0, 0, scaled=True, device="cpu")


def test_wan_dims_and_flux_block_counts_are_read_off_a_checkpoint():
    """WanDiT's constructor arguments (wan_dit.py:247-262, conf/models/wan/dit/*.json) from tensor shapes alone
    (reduced widths; text-to-video twice and the image-to-video form); Flux block counts from the key names."""
    from diffsynth_engine_amd.flux_dit import count_blocks
    from diffsynth_engine_amd.wan_dit import wan_config_from_shapes
    from oracle import wan as ow

    base = ow.config_14b()
    for cfg, clip in ((dict(base, dim=256, ffn_dim=640, num_heads=2, num_layers=3), None),
                      (dict(base, dim=384, ffn_dim=512, num_heads=3, num_layers=2, out_dim=8, freq_dim=64, text_dim=96), None),
                      (dict(base, dim=128, ffn_dim=256, num_heads=1, num_layers=2, in_dim=36, patch_size=(1, 2, 2)), 80)):
        small = cfg
        sd = ow.init_params(small, dtype=torch.bfloat16, seed=0, **({"clip_dim": clip} if clip else {}))
        got = wan_config_from_shapes({k: tuple(v.shape) for k, v in sd.items()})
        for key in ("dim", "in_dim", "ffn_dim", "out_dim", "text_dim", "freq_dim", "eps", "num_heads", "num_layers"):
            assert got[key] == small[key], (key, got[key], small[key])
        assert tuple(got["patch_size"]) == tuple(small["patch_size"]) and got["has_image_input"] == bool(clip)
    names = ["blocks.0.attn.a_to_qkv", "blocks.18.ff_a.0", "single_blocks.37.proj_out", "single_blocks.4.norm.linear", "x_embedder"]
    assert (count_blocks(names, "blocks."), count_blocks(names, "single_blocks.")) == (19, 38)
    assert count_blocks(["x_embedder"], "blocks.") == 0
    with pytest.raises(ValueError):
        wan_config_from_shapes({"patch_embedding.weight": (100, 16, 1, 2, 2)})
