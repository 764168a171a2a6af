"""CPU restatement of the reference's DiT denoising-step arithmetic — TEST INFRASTRUCTURE ONLY.

Nothing under ``diffsynth_engine_amd`` imports this package.  Its only users are ``tests/``,
``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py``, where it is the checker
(or the timed CPU baseline), never the product path.

Each function cites the reference file:line it restates (paths relative to the root of
modelscope/DiffSynth-Engine v0.1.1).  The arithmetic of the path lives in PyTorch
(``torch >= 2.4.1`` per the reference's pyproject.toml:17): ``F.scaled_dot_product_attention``,
``torch._scaled_mm``, ``Tensor.to(torch.float8_e4m3fn)``, ``nn.LayerNorm``, ``nn.GELU``.

How each function is pinned (tests/test_oracle_*.py):
  fp8.e4m3_from_f32_bits / e4m3_to_f32   numpy bit-level restatement; pinned exhaustively against
                                          torch's own cast over all 65 536 bf16 patterns, a 2^22 fp32
                                          sweep, and known answers (448, 464->448, 465->NaN, 2^-10->0, ...)
  fp8.quantize_rowwise / scaled_linear    pinned against torch._scaled_mm on CPU and brute force
  dit_ops.sdpa                            pinned against F.scaled_dot_product_attention, brute-force
                                          loops on tiny shapes, and softmax invariants
  dit_ops.rope_table / apply_rope         pinned by closed forms: 2-D rotation, norm preservation,
                                          pos=0 identity, R(a)R(b)=R(a+b), relative-position property
  dit_ops.rms_norm / layer_norm_modulate  pinned against F.rms_norm / F.layer_norm
  dit_ops.gelu_tanh                       pinned against F.gelu(approximate="tanh") and the NewGELU formula
  dit_ops.timestep_embedding              pinned by the closed form sin/cos(t * 10000^(-i/half))
  sampler.*                               pinned against the reference's own golden files
                                          tests/data/expect/algorithm/{flow_match_euler_i10,
                                          recifited_flow_20steps_flux}.safetensors (copied as fixtures)
  flux.ada_layer_norm6 / ada_layer_norm3 / rope_table / rms_norm / timestep_embedding, fp8.fp8_linear
                                          pinned against vectors written by the reference's own leaf modules
                                          (models/basic/transformer_helper.py, models/basic/timestep.py,
                                          utils/fp8_linear.py; tests/golden/make_leaf_module_fixtures.py)
  flux.joint_block / single_block / ada_layer_norm_continuous / flux_dit_forward
                                          pinned against vectors written by the reference's own
                                          FluxJointTransformerBlock, FluxSingleTransformerBlock,
                                          AdaLayerNormContinuous and FluxDiT.forward at reduced width
                                          (tests/golden/make_flux_block_fixtures.py), plus structural invariants
  wan.freqs_cis_3d / dit_block / wan_dit_forward
                                          pinned against vectors written by the reference's own WanDiT at
                                          reduced size (tests/golden/make_wan_fixtures.py)
The reference's only fixture on this path (tests/data/expect/flux/flux_dit.safetensors) needs the
12B-parameter Flux.1-dev checkpoint and is not usable offline; full-size real-weight parity is unpinned.
"""
