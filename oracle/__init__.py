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
  flux.* / wan.* block and model wiring   PARITY UNPINNED by any reference-held vector: the only
                                          reference fixture on this path (tests/data/expect/flux/flux_dit.safetensors)
                                          needs the 12B-parameter Flux.1-dev checkpoint.  Pinned only by
                                          structural invariants (zero gates => identity, text rows see no
                                          rotation, chunk orders checked against hand-built cases).
"""
