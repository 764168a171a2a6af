#!/usr/bin/env python3
"""Benchmark of the DiT denoising-step hot path on one MI355X.

Headline workload: one full Flux.1-dev-architecture DiT denoising step (19 double-stream + 38
single-stream blocks, hidden 3072, 24 heads x 128, 1024x1024 image = 4096 image tokens + 512 text
tokens, batch 1), random-init weights N(0, 0.02) quantised to e4m3 with per-tensor scales, activations
quantised per token, synthetic N(0,1) inputs.  A "step" is one FluxDiTRunner.forward.

Prints ONE JSON line.  `roofline` describes the dominant kernel (the FP8 GEMM, ~80 % of the step's
flops): algorithmic flops 2*M*N*K of every large GEMM launched in the timed region divided by the sum of
their durations, measured with events on the launch stream.  `cpu_baseline` times the CPU oracle
(pure-torch restatement of the reference path) on the host cores for a bounded sample.
Secondary figures (attention kernel TFLOP/s at S=4608, per-shape GEMM TFLOP/s, HBM GB/s of the
bandwidth-bound kernels) ride along under "detail".  `--workload wan14b` times one Wan2.1-14B step instead
(40 layers, 32 760 video tokens) and prints its own line.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_FP8 = 5.0e15   # MI355X dense fp8 MFMA, flop/s
PEAK_BF16 = 2.5e15  # MI355X dense bf16 MFMA, flop/s
PEAK_HBM = 8.0e12   # bytes/s

HIDDEN, HEADS, HEAD_DIM = 3072, 24, 128
N_IMG, N_TXT = 4096, 512


def flux_state_dict_stream(num_double, num_single, device, seed=0, std=0.02):
    """Yield (name, tensor) pairs of a random Flux.1-dev-architecture DiT, generated on the device one tensor
    at a time (weights N(0,std) bf16, biases 0, RMSNorm weights 1) so that the runner can quantise as it goes.
    std=None draws every Linear N(0, 1/fan_in) instead (AdaLN projections at half that deviation): every layer's
    output then stays O(1), far below e4m3's 448, which the reference's unscaled casts need."""
    import torch

    g = torch.Generator(device=device).manual_seed(seed)
    d = HIDDEN

    def lin(name, n_in, n_out):
        s = std if std is not None else (0.5 if "norm" in name else 1.0) / n_in ** 0.5
        yield name + ".weight", (torch.randn(n_out, n_in, generator=g, device=device) * s).to(torch.bfloat16)
        yield name + ".bias", torch.zeros(n_out, dtype=torch.bfloat16, device=device)

    def ones(name):
        yield name + ".weight", torch.ones(HEAD_DIM, dtype=torch.bfloat16, device=device)

    yield from lin("time_embedder.timestep_embedder.0", 256, d)
    yield from lin("time_embedder.timestep_embedder.2", d, d)
    yield from lin("guidance_embedder.timestep_embedder.0", 256, d)
    yield from lin("guidance_embedder.timestep_embedder.2", d, d)
    yield from lin("pooled_text_embedder.0", 768, d)
    yield from lin("pooled_text_embedder.2", d, d)
    yield from lin("context_embedder", 4096, d)
    yield from lin("x_embedder", 64, d)
    for i in range(num_double):
        p = f"blocks.{i}."
        yield from lin(p + "norm1_a.linear", d, 6 * d)
        yield from lin(p + "norm1_b.linear", d, 6 * d)
        yield from lin(p + "attn.a_to_qkv", d, 3 * d)
        yield from lin(p + "attn.b_to_qkv", d, 3 * d)
        for n in ("norm_q_a", "norm_k_a", "norm_q_b", "norm_k_b"):
            yield from ones(p + "attn." + n)
        yield from lin(p + "attn.a_to_out", d, d)
        yield from lin(p + "attn.b_to_out", d, d)
        yield from lin(p + "ff_a.0", d, 4 * d)
        yield from lin(p + "ff_a.2", 4 * d, d)
        yield from lin(p + "ff_b.0", d, 4 * d)
        yield from lin(p + "ff_b.2", 4 * d, d)
    for i in range(num_single):
        p = f"single_blocks.{i}."
        yield from lin(p + "norm.linear", d, 3 * d)
        yield from lin(p + "to_qkv_mlp", d, 7 * d)
        yield from ones(p + "norm_q_a")
        yield from ones(p + "norm_k_a")
        yield from lin(p + "proj_out", 5 * d, d)
    yield from lin("final_norm_out.linear", d, 2 * d)
    yield from lin("final_proj_out", d, 64)


def wan_state_dict_stream(cfg, device, seed=0, std=0.02):
    """(name, tensor) pairs of a random Wan2.1-architecture DiT (text-to-video variant), generated on the
    device one tensor at a time: Linear weights N(0,std) bf16, biases 0, norm weights 1, modulation tables
    N(0,1)/sqrt(dim)."""
    import torch

    g = torch.Generator(device=device).manual_seed(seed)
    d, f = cfg["dim"], cfg["ffn_dim"]
    bf = torch.bfloat16

    def lin(name, n_in, n_out):
        yield name + ".weight", (torch.randn(n_out, n_in, generator=g, device=device) * std).to(bf)
        yield name + ".bias", torch.zeros(n_out, dtype=bf, device=device)

    pf, ph, pw = cfg["patch_size"]
    yield "patch_embedding.weight", (torch.randn(d, cfg["in_dim"], pf, ph, pw, generator=g, device=device) * std).to(bf)
    yield "patch_embedding.bias", torch.zeros(d, dtype=bf, device=device)
    yield from lin("text_embedding.0", cfg["text_dim"], d)
    yield from lin("text_embedding.2", d, d)
    yield from lin("time_embedding.0", cfg["freq_dim"], d)
    yield from lin("time_embedding.2", d, d)
    yield from lin("time_projection.1", d, 6 * d)
    for i in range(cfg["num_layers"]):
        p = f"blocks.{i}."
        for a in ("self_attn", "cross_attn"):
            for n in ("q", "k", "v", "o"):
                yield from lin(p + f"{a}.{n}", d, d)
            yield p + f"{a}.norm_q.weight", torch.ones(d, dtype=bf, device=device)
            yield p + f"{a}.norm_k.weight", torch.ones(d, dtype=bf, device=device)
        yield p + "norm3.weight", torch.ones(d, dtype=bf, device=device)
        yield p + "norm3.bias", torch.zeros(d, dtype=bf, device=device)
        yield from lin(p + "ffn.0", d, f)
        yield from lin(p + "ffn.2", f, d)
        yield p + "modulation", (torch.randn(1, 6, d, generator=g, device=device) / d ** 0.5).to(bf)
    yield from lin("head.head", d, cfg["out_dim"] * pf * ph * pw)
    yield "head.modulation", (torch.randn(1, 2, d, generator=g, device=device) / d ** 0.5).to(bf)


def run_wan(torch, dev, layers, steps, warmup, with_cpu_baseline):
    """BASELINE configs[4]: one Wan2.1-14B DiT denoising step, 21 x 60 x 104 latent = 32 760 tokens, 512 text
    tokens, `layers` of the 40 layers; every Linear through the scaled e4m3 GEMM.  Returns the result line."""
    from diffsynth_engine_amd.wan_dit import WanDiTRunner

    class _A:
        pass

    args = _A()
    args.steps, args.warmup, args.no_cpu_baseline = steps, warmup, not with_cpu_baseline
    cfg = dict(dim=5120, in_dim=16, ffn_dim=13824, out_dim=16, text_dim=4096, freq_dim=256, eps=1e-6,
               patch_size=(1, 2, 2), num_heads=40, num_layers=layers)
    runner = WanDiTRunner(wan_state_dict_stream(cfg, dev), cfg, scaled=True, device=dev)
    g = torch.Generator(device=dev).manual_seed(0)
    x = torch.randn(1, 16, 21, 60, 104, generator=g, device=dev).to(torch.bfloat16)
    ctx = torch.randn(1, 512, 4096, generator=g, device=dev).to(torch.bfloat16)
    t = torch.tensor([500.0], device=dev)
    from diffsynth_engine_amd import ops

    at, gt = AttnTimer(torch, ops), GemmTimer(torch, ops)
    with at, gt:  # bracketed like the timed steps: says how many events a step takes, and creates the first of them
        for _ in range(args.warmup):
            out = runner(x, ctx, t)
    if args.warmup:
        at.prepare(len(at.records) // args.warmup * args.steps)
        gt.prepare(len(gt.records) // args.warmup * args.steps)
    torch.cuda.synchronize()
    with at, gt:
        t0 = time.perf_counter()
        for _ in range(args.steps):
            out = runner(x, ctx, t)
        torch.cuda.synchronize()
        ms = (time.perf_counter() - t0) * 1e3 / args.steps
        n_attn, attn_flops, attn_secs = at.summary()
        n_gemm, gemm_flops, gemm_secs = gt.summary()
    assert torch.isfinite(out.float()).all().item(), "non-finite output"
    # the same step with the device-side score bound off (every self-attention keeps its running maximum)
    runner.device_score_bound = False
    runner(x, ctx, t)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(2):
        runner(x, ctx, t)
    torch.cuda.synchronize()
    ms_scan = (time.perf_counter() - t0) * 1e3 / 2
    runner.device_score_bound = True
    # sampled-row parity of the timed configuration: the last layer's self-attention shape through the same entry
    # point (the largest head norms of q and k on the device, as the step's norm kernels leave them) against
    # torch's fp32 SDPA on a few query rows of three heads
    gq = torch.Generator(device=dev).manual_seed(1)
    q, k, v = [torch.randn(1, 32760, 5120, generator=gq, device=dev, dtype=torch.bfloat16) for _ in range(3)]
    n2 = lambda tt: tt.view(32760 * 40, 128).float().square().sum(-1).max()
    o = runner._attention(q, k, v, torch.stack([n2(q), n2(k)])).view(1, 32760, 40, 128)
    rows = torch.tensor([0, 255, 16383, 32759], device=dev)
    for h in (0, 21, 39):
        hs = lambda tt: tt.view(1, 32760, 40, 128)[:, :, h].float()
        ref = torch.nn.functional.scaled_dot_product_attention(hs(q)[:, rows].unsqueeze(1), hs(k).unsqueeze(1),
                                                               hs(v).unsqueeze(1))[:, 0]
        err = ((o[:, rows, h].float() - ref).abs().amax(-1) / ref.abs().amax(-1)).max().item()
        assert err <= 2e-2, "attention row check failed: %g" % err
    del q, k, v, o
    S, d, f, L = 21 * 30 * 52, cfg["dim"], cfg["ffn_dim"], cfg["num_layers"]
    gemm = L * (2.0 * S * d * d * 4 + 2.0 * S * d * f * 2 + 2.0 * S * d * d * 2 + 2.0 * 512 * d * d * 2)
    attn = L * (4.0 * S * S * d + 4.0 * S * 512 * d)
    t_ideal = gemm / PEAK_FP8 + attn / PEAK_BF16
    return {
        "metric": "wan2.1_14b_480p_fp8_dit_step_ms", "value": round(ms, 1), "unit": "ms", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms, 1), "higher_is_better": False,
        "scaling": "weak", "vs_baseline": None, "dtype": "fp8_e4m3 GEMM (fp32 accumulate) + bf16 attention",
        "data": "synthetic",
        "config": {"workload": "BASELINE configs[4]: Wan2.1-14B-architecture DiT, one denoising step, %d layers, "
                               "32760 video tokens (21x60x104 latent) + 512 text tokens, batch 1, random init" % L},
        # dominant kernel: attn_plain16_kernel (53 % of the step's flops); self- and cross-attention launches together
        "roofline": {"bound": "mfma", "achieved": round(attn_flops / attn_secs / 1e12, 1), "peak": PEAK_BF16 / 1e12,
                     "unit": "TFLOP/s", "frac": round(attn_flops / attn_secs / PEAK_BF16, 4),
                     "traffic": WAN_ATTN_TRAFFIC_BYTES, "kernel": "attn_plain16_kernel", "launches": n_attn,
                     "avg_launch_us": round(attn_secs / max(n_attn, 1) * 1e6, 1)},
        "detail": {"fp8_gemm_in_step": {"launches": n_gemm, "tflops": round(gemm_flops / gemm_secs / 1e12, 1),
                                        "frac_fp8_peak": round(gemm_flops / gemm_secs / PEAK_FP8, 4),
                                        "ms_per_step": round(gemm_secs * 1e3 / args.steps, 1)},
                   "attention_in_step": {"ms_per_step": round(attn_secs * 1e3 / args.steps, 1)},
                   "ms_per_step_without_device_score_bound": round(ms_scan, 1)},
        "step_roofline": {"algorithmic_tflop": round((gemm + attn) / 1e12, 1), "ideal_ms": round(t_ideal * 1e3, 1),
                          "frac": round(t_ideal * 1e3 / ms, 4)},
        "cpu_baseline": None if args.no_cpu_baseline else wan_cpu_baseline(cfg, S)}


def step_flops(num_double, num_single, n_img=N_IMG, n_txt=N_TXT):
    """Algorithmic flops of one step: 2MNK of every Linear with M > 1 plus 4*S^2*D*H per attention."""
    d, S = HIDDEN, n_img + n_txt
    per_tok_double = 2 * d * (3 * d + d + 4 * d + 4 * d)
    gemm = num_double * S * per_tok_double + num_single * S * 2 * d * (7 * d + 5 * d)
    gemm += n_txt * 2 * 4096 * d + n_img * 2 * 64 * d + n_img * 2 * d * 64
    attn = (num_double + num_single) * 4 * S * S * HEAD_DIM * HEADS
    return gemm, attn


_HIP = None


def _hip_runtime():
    """The HIP runtime this process already has loaded (torch's), through ctypes: for timing events with flags that
    torch.cuda.Event does not expose."""
    global _HIP
    if _HIP is None:
        import ctypes

        path = next(tok for tok in open("/proc/self/maps").read().split() if "libamdhip64" in tok)
        hip = ctypes.CDLL(path)
        hip.hipEventCreateWithFlags.argtypes = [ctypes.POINTER(ctypes.c_void_p), ctypes.c_uint]
        hip.hipEventRecord.argtypes = [ctypes.c_void_p, ctypes.c_void_p]
        hip.hipEventElapsedTime.argtypes = [ctypes.POINTER(ctypes.c_float), ctypes.c_void_p, ctypes.c_void_p]
        _HIP = hip
    return _HIP


class _HipEvent:
    """A HIP timing event without the system-scope fence of a default event (hipEventDisableSystemFence): the
    brackets around the 155 GEMM launches of a step then cost 0.45 ms per step instead of 1.0 ms, and a bracket
    holds 2 us less that is not the kernel."""

    def __init__(self, torch):
        import ctypes

        self._ct, self._torch, self.h = ctypes, torch, ctypes.c_void_p()
        rc = _hip_runtime().hipEventCreateWithFlags(ctypes.byref(self.h), 0x20000000)  # hipEventDisableSystemFence
        if rc:
            raise RuntimeError("hipEventCreateWithFlags failed: %d" % rc)

    def record(self):  # on torch's current stream, the stream handed to the C-ABI
        rc = _hip_runtime().hipEventRecord(self.h, self._ct.c_void_p(self._torch.cuda.current_stream().cuda_stream))
        if rc:
            raise RuntimeError("hipEventRecord failed: %d" % rc)

    def elapsed_time(self, later):  # ms
        ms = self._ct.c_float()
        rc = _hip_runtime().hipEventElapsedTime(self._ct.byref(ms), self.h, later.h)
        if rc:
            raise RuntimeError("hipEventElapsedTime failed: %d" % rc)
        return ms.value


class _EventBrackets:
    """Event pairs around calls on the launch stream (torch's current stream, which is the stream handed to the
    C-ABI), with the flops of each call.

    Events come from a pool that `prepare` fills BEFORE a timed region: the first record of a new timing event
    makes the HIP runtime allocate its signal, hundreds at a time cost the host tens of milliseconds (30 ms in one
    piece in the first GPU process of a freshly started machine), and a timed region of five steps that creates its
    3100 events as it goes is host-bound through its first step and reads 3-6 ms per step more than the steps take."""

    def __init__(self, torch, ops):
        self.torch, self.ops = torch, ops
        self.records, self.pool = [], []

    kind = "hip events without system-scope fence"

    def _new_pair(self):
        if _EventBrackets.kind.startswith("hip"):
            try:
                return _HipEvent(self.torch), _HipEvent(self.torch)
            except (StopIteration, OSError, AttributeError, RuntimeError):  # runtime not found through /proc: torch's
                _EventBrackets.kind = "torch.cuda.Event"
        return self.torch.cuda.Event(enable_timing=True), self.torch.cuda.Event(enable_timing=True)

    def _pair(self):
        return self.pool.pop() if self.pool else self._new_pair()

    def prepare(self, pairs):
        """Leaves `pairs` event pairs in the pool, each recorded once (that is what creates them), keeps the pairs
        of earlier records for re-use and forgets those records."""
        self.pool += [(e0, e1) for e0, e1, _ in self.records]
        del self.records[:]
        while len(self.pool) < pairs:
            e0, e1 = self._new_pair()
            e0.record()
            e1.record()
            self.pool.append((e0, e1))
        self.torch.cuda.synchronize()

    def bracket(self, fn, flops):
        e0, e1 = self._pair()
        e0.record()
        out = fn()
        e1.record()
        self.records.append((e0, e1, flops))
        return out

    def summary(self):
        self.torch.cuda.synchronize()
        secs = sum(e0.elapsed_time(e1) for e0, e1, _ in self.records) * 1e-3
        return len(self.records), sum(f for _, _, f in self.records), secs


class GemmTimer(_EventBrackets):
    """Brackets every fp8_gemm launch (single, or two problems sharing one grid) and accumulates algorithmic flops
    for launches with M > 8."""

    def __init__(self, torch, ops):
        super().__init__(torch, ops)
        self._orig = ops.fp8_gemm
        self._orig_grouped = ops.fp8_gemm_grouped

    def __enter__(self):
        orig, orig_grouped = self._orig, self._orig_grouped

        def timed(a_q, w_q, *args, **kw):
            M, K = a_q.shape
            if M <= 8 or kw.get("qk") is not None:  # (a q/k-epilogue call goes through the grouped entry, timed there)
                return orig(a_q, w_q, *args, **kw)
            return self.bracket(lambda: orig(a_q, w_q, *args, **kw), 2.0 * M * K * w_q.shape[0])

        def timed_grouped(problems):
            return self.bracket(lambda: orig_grouped(problems),
                                sum(2.0 * p["a_q"].shape[0] * p["a_q"].shape[1] * p["w_q"].shape[0] for p in problems))

        self.ops.fp8_gemm = timed
        self.ops.fp8_gemm_grouped = timed_grouped
        return self

    def __exit__(self, *exc):
        self.ops.fp8_gemm = self._orig
        self.ops.fp8_gemm_grouped = self._orig_grouped


class AttnTimer(_EventBrackets):
    """Brackets every ops.attention_bhsd call of a step and accumulates the algorithmic flops
    4 * Sq * Skv * D * H * B of each (a call with fused q/k pre-processing includes its k row pass)."""

    def __init__(self, torch, ops):
        super().__init__(torch, ops)
        self._orig = ops.attention_bhsd

    def __enter__(self):
        orig = self._orig

        def timed(q, k, v, *args, q2=None, k2=None, **kw):
            B, H, Sq, D = q.shape
            Sq += 0 if q2 is None else q2.shape[2]
            Skv = k.shape[2] + (0 if k2 is None else k2.shape[2])
            return self.bracket(lambda: orig(q, k, v, *args, q2=q2, k2=k2, **kw), 4.0 * B * H * Sq * Skv * D)

        self.ops.attention_bhsd = timed
        return self

    def __exit__(self, *exc):
        self.ops.attention_bhsd = self._orig


def time_kernel(torch, fn, args_list=None, reps=10):
    """Seconds per call of ``fn`` with the host taken out of the measurement: the calls are recorded into one HIP
    graph and the graph is replayed, so a 6 us kernel is not reported at the 12 us it takes Python to launch it.
    ``args_list``: one argument tuple per call of the recorded sequence; bandwidth-bound kernels get a rotation of
    buffers larger than the 256 MB Infinity Cache so that every call reads HBM.  Without it ``fn()`` is recorded
    ten times on the same operands (matrix kernels: the caches are left as they are).  At least 100 calls are
    timed (``reps`` replays); the figure is their mean."""
    calls = [()] * 10 if args_list is None else list(args_list)
    for a in calls[:3]:
        fn(*a)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        for a in calls:
            fn(*a)
    graph.replay()  # warm-up: with the three eager calls above, at least 20 calls before the timed ones
    graph.replay()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    e0.record()
    for _ in range(reps):
        graph.replay()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) * 1e-3 / (reps * len(calls))


def _rotation(torch, make, nbytes):
    """Enough distinct buffers to exceed the Infinity Cache (256 MB) plus the L2s."""
    return [(make(),) for _ in range(max(3, -(-(320 << 20) // nbytes)))]


def mfma_ceiling(torch, dev):
    """What the matrix pipes sustain on this box with nothing else going on: MFMAs on register operands, two
    wavefronts per SIMD on every compute unit, all-zero and random operand bits (random bits draw more power and the
    clock management lowers the clock).  The roofline fractions of this file use the published dense peaks; these
    figures say how much of the gap to them is the machine's and how much the kernels'."""
    import ctypes

    from diffsynth_engine_amd import _lib

    lib = _lib.load()
    cus = torch.cuda.get_device_properties(dev).multi_processor_count
    sink = torch.zeros(1, device=dev)
    out = {}
    g = torch.Generator(device=dev).manual_seed(0)
    for kind, name, iters in ((0, "bf16_32x32x16", 40000), (1, "fp8_32x32x64", 20000), (2, "bf16_16x16x32", 40000),
                              (3, "fp8_16x16x128", 20000), (4, "bf16_32x32x16_both_operands_change", 40000),
                              (5, "fp8_32x32x64_both_operands_change", 20000),
                              (6, "bf16_16x16x32_both_operands_change", 40000),
                              (7, "fp8_16x16x128_both_operands_change", 20000)):
        for fill in ("zero", "random"):
            if fill == "zero":
                bits = torch.zeros(16 * 256, dtype=torch.int32, device=dev)
            elif kind & 1 == 0:  # random finite bf16 pairs / e4m3 quadruples (no NaN patterns)
                bits = torch.randn(16 * 256 * 2, generator=g, device=dev).bfloat16().view(torch.int32)
            else:
                bits = torch.randn(16 * 256 * 4, generator=g, device=dev).to(torch.float8_e4m3fn).view(torch.int32)
            flops = ctypes.c_int64(0)
            stream = torch.cuda.current_stream().cuda_stream
            launch = lambda: _lib.check(lib.dsx_mfma_ceiling_probe(kind, bits.data_ptr(), iters, 2 * cus, sink.data_ptr(),
                                                                   ctypes.byref(flops), stream), "dsx_mfma_ceiling_probe")
            launch()
            torch.cuda.synchronize()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for _ in range(3):
                launch()
            e1.record()
            torch.cuda.synchronize()
            t = e0.elapsed_time(e1) * 1e-3 / 3
            out[f"{name}_{fill}"] = {"ms": round(t * 1e3, 2), "tflops": round(flops.value / t / 1e12, 1)}
    return out


def micro_benchmarks(torch, ops, dev):
    """Per-kernel figures at the sizes of the Flux-1024 step: configs[1] GEMM shapes, configs[2] attention,
    and the bandwidth-bound kernels."""
    detail = {}
    g = torch.Generator(device=dev).manual_seed(0)
    M = N_IMG + N_TXT
    gem = {}
    for K, N in ((3072, 9216), (3072, 3072), (3072, 12288), (12288, 3072), (3072, 21504), (15360, 3072)):
        x = torch.randn(M, K, generator=g, device=dev, dtype=torch.bfloat16)
        x[:, torch.randperm(K, generator=g, device=dev)[: max(1, -(-K // 1000))]] *= 20
        w = (torch.randn(N, K, generator=g, device=dev) * 0.02).to(torch.bfloat16)
        bias = torch.randn(N, generator=g, device=dev).to(torch.bfloat16)
        wq, ws = ops.quantize_weight_fp8(w)
        xq, xs = ops.quantize_fp8(x)
        out = torch.empty(M, N, dtype=torch.bfloat16, device=dev)
        t = time_kernel(torch, lambda: ops.fp8_gemm(xq, wq, xs, ws, bias, out=out))
        xs_rot = _rotation(torch, lambda: x.clone(), M * K * 2)
        tq = time_kernel(torch, lambda xx: ops.quantize_fp8(xx), xs_rot)
        del xs_rot
        fl = 2.0 * M * N * K
        gem[f"{K}x{N}"] = {"us": round(t * 1e6, 1), "tflops": round(fl / t / 1e12, 1),
                           "frac_fp8_peak": round(fl / t / PEAK_FP8, 4),
                           "quant_us": round(tq * 1e6, 1), "quant_gbps": round((M * K * 3 + 4 * M) / tq / 1e9, 1)}
        del x, w, wq, xq, out
    detail["fp8_gemm_M4608"] = gem

    S = M
    q = torch.randn(1, HEADS, S, HEAD_DIM, generator=g, device=dev, dtype=torch.bfloat16)
    k = torch.randn(1, HEADS, S, HEAD_DIM, generator=g, device=dev, dtype=torch.bfloat16)
    v = torch.randn(1, HEADS, S, HEAD_DIM, generator=g, device=dev, dtype=torch.bfloat16)
    out = torch.empty(1, S, HEADS, HEAD_DIM, dtype=torch.bfloat16, device=dev).transpose(1, 2)
    fl = 4.0 * S * S * HEAD_DIM * HEADS
    t = time_kernel(torch, lambda: ops.attention_bhsd(q, k, v, out=out))
    att = {"plain": {"us": round(t * 1e6, 1), "tflops": round(fl / t / 1e12, 1), "frac_bf16_peak": round(fl / t / PEAK_BF16, 4),
                     "kernel_launches": 1}}
    # fused RMSNorm + 3-axis RoPE (16,56,56), ids: 512 text rows at 0, then (0,r,c) over 64x64
    ids = torch.zeros(1, S, 3, dtype=torch.float64, device=dev)
    rc = torch.arange(64, device=dev, dtype=torch.float64)
    ids[0, N_TXT:, 1] = rc.repeat_interleave(64)
    ids[0, N_TXT:, 2] = rc.repeat(64)
    cols = []
    for a, dim in enumerate((16, 56, 56)):
        omega = 1.0 / (10000 ** (torch.arange(0, dim, 2, dtype=torch.float64, device=dev) / dim))
        ang = ids[..., a].unsqueeze(-1) * omega
        cols.append(torch.stack((torch.cos(ang), torch.sin(ang)), dim=-1))
    rope = torch.cat(cols, dim=-2).float().contiguous()
    w1 = torch.ones(HEAD_DIM, dtype=torch.bfloat16, device=dev)
    # q/k RMSNorm + 3-axis RoPE requested from the attention entry point (one C call): q is treated as the
    # attention kernel loads it, k once into caller scratch by a row kernel ahead of it.
    # "..._score_bound": the caller also states the bound on |scale * q.k| that unit RMSNorm weights imply
    # (sqrt(128), with 2 % for the bf16 roundings), which lets the kernel drop its running maximum
    for key, bound in (("rmsnorm_rope_then_attention_one_call", 0.0),
                       ("rmsnorm_rope_then_attention_one_call_score_bound", 1.02 * HEAD_DIM ** 0.5)):
        t = time_kernel(torch, lambda: ops.attention_bhsd(q, k, v, out=out, rope=rope, q_norm_w=w1, k_norm_w=w1,
                                                          score_bound=bound))
        att[key] = {"us": round(t * 1e6, 1), "tflops": round(fl / t / 1e12, 1),
                    "frac_bf16_peak": round(fl / t / PEAK_BF16, 4),
                    "kernel_launches": 2}  # one C call, two launches: the k row pass, then attention (q as it loads)
    detail["attention_S4608_H24_D128"] = att

    mod = torch.randn(1, 3 * HIDDEN, generator=g, device=dev, dtype=torch.bfloat16)
    sh, sc, gt = mod.chunk(3, dim=1)
    xs_rot = _rotation(torch, lambda: torch.randn(1, S, HIDDEN, generator=g, device=dev, dtype=torch.bfloat16),
                       S * HIDDEN * 2)
    y = torch.randn(1, S, HIDDEN, generator=g, device=dev, dtype=torch.bfloat16)
    t1 = time_kernel(torch, lambda x: ops.adaln_modulate(x, sc, sh, want_bf16=True), xs_rot)
    t1q = time_kernel(torch, lambda x: ops.adaln_modulate(x, sc, sh, want_bf16=False, want_fp8=True), xs_rot)
    t2 = time_kernel(torch, lambda x: ops.gated_residual(x, y, gt), xs_rot)
    del xs_rot
    hs_rot = _rotation(torch, lambda: torch.randn(S, 4 * HIDDEN, generator=g, device=dev, dtype=torch.bfloat16),
                       S * 4 * HIDDEN * 2)
    t3 = time_kernel(torch, lambda h: ops.gelu_tanh(h), hs_rot)
    t3q = time_kernel(torch, lambda h: ops.gelu_tanh(h, want_bf16=False, want_fp8=True), hs_rot)
    del hs_rot
    n = S * HIDDEN
    def hbm(t, nbytes):  # algorithmic bytes over time, and as a fraction of the 8 TB/s peak
        return {"us": round(t * 1e6, 1), "gbps": round(nbytes / t / 1e9, 1), "frac_hbm": round(nbytes / t / PEAK_HBM, 4)}

    detail["epilogues"] = {
        "adaln_modulate_bf16": hbm(t1, 4 * n), "adaln_modulate_fp8": hbm(t1q, 3 * n), "gated_residual": hbm(t2, 6 * n),
        "gelu_tanh_bf16": hbm(t3, 16 * n), "gelu_tanh_fp8": hbm(t3q, 12 * n),
    }
    for kn, v in gem.items():
        v["quant_frac_hbm"] = round(v["quant_gbps"] * 1e9 / PEAK_HBM, 4)
    return detail


def two_stream_overlap(torch, ops, dev, graph=True, pairs=20):
    """Does a bandwidth-bound row kernel hide under an attention call?  In a single block GELU + quantise of the MLP
    half and the attention call are independent (flux_dit.py:312-317).  Times, at the step's shapes: each kernel
    alone, the pair back to back on one stream, and the pair with the row kernel forked onto a second stream of the
    same priority (events for fork and join), as one recorded sequence of `pairs` pairs."""
    g = torch.Generator(device=dev).manual_seed(0)
    H, S = HEADS, N_IMG + N_TXT
    q, k, v = [torch.randn(1, H, S, HEAD_DIM, generator=g, device=dev, dtype=torch.bfloat16) for _ in range(3)]
    q = torch.nn.functional.normalize(q.float(), dim=-1).mul(HEAD_DIM ** 0.5).bfloat16()
    k = torch.nn.functional.normalize(k.float(), dim=-1).mul(HEAD_DIM ** 0.5).bfloat16()
    out = torch.empty(1, S, H, HEAD_DIM, dtype=torch.bfloat16, device=dev).transpose(1, 2)
    hs = [torch.randn(S, 4 * HIDDEN, generator=g, device=dev, dtype=torch.bfloat16) for _ in range(4)]
    side = torch.cuda.Stream()  # default priority

    def attn():
        ops.attention_bhsd(q, k, v, out=out, score_bound=1.02 * HEAD_DIM ** 0.5)

    def gelu(i):
        ops.gelu_tanh(hs[i % 4], want_bf16=False, want_fp8=True)

    def only_attn(n):
        for _ in range(n):
            attn()

    def only_gelu(n):
        for i in range(n):
            gelu(i)

    def sequential(n):
        for i in range(n):
            attn()
            gelu(i)

    def forked(n):
        main = torch.cuda.current_stream()
        for i in range(n):
            side.wait_stream(main)
            attn()
            with torch.cuda.stream(side):
                gelu(i)
            main.wait_stream(side)

    def timeit(fn):
        fn(3)
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        if graph:
            gr = torch.cuda.CUDAGraph()
            with torch.cuda.graph(gr):
                fn(pairs)
            gr.replay()
            torch.cuda.synchronize()
            e0.record()
            for _ in range(5):
                gr.replay()
            e1.record()
            torch.cuda.synchronize()
            return e0.elapsed_time(e1) * 1e3 / (5 * pairs)
        e0.record()
        fn(pairs)
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) * 1e3 / pairs

    return {"attention_us": round(timeit(only_attn), 1), "gelu_quantise_us": round(timeit(only_gelu), 1),
            "pair_on_one_stream_us": round(timeit(sequential), 1),
            "pair_with_row_kernel_on_second_stream_us": round(timeit(forked), 1),
            "timed_as": "graph replay" if graph else "eager launches"}


def cpu_baseline(num_double, num_single):
    """The oracle (fp32, torch SDPA-equivalent eager attention) on the host cores: ONE double-stream and ONE
    single-stream block at the full 4096+512 tokens, extrapolated to 19 + 38 blocks."""
    import torch

    from oracle import dit_ops as O
    from oracle import flux as oflux

    cores = os.cpu_count() or 1
    torch.set_num_threads(cores)
    sd = oflux.init_params(1, 1, dtype=torch.float32, seed=0)
    P = oflux.Params(sd, "plain")
    g = torch.Generator().manual_seed(0)
    img = torch.randn(1, N_IMG, HIDDEN, generator=g)
    txt = torch.randn(1, N_TXT, HIDDEN, generator=g)
    cond = torch.randn(1, HIDDEN, generator=g)
    ids = torch.cat([torch.zeros(1, N_TXT, 3), oflux.image_ids(128, 128, 1, "cpu", torch.float32)], dim=1)
    freqs = O.rope_table(ids, oflux.AXES_DIM, oflux.THETA)
    sdpa = torch.nn.functional.scaled_dot_product_attention
    reps = 5  # ~10 s of host work in all
    with torch.no_grad():
        a, b = oflux.joint_block(P, 0, img, txt, cond, freqs, attn=sdpa)  # first touch of the weights
        t0 = time.perf_counter()
        for _ in range(reps):
            a, b = oflux.joint_block(P, 0, img, txt, cond, freqs, attn=sdpa)
        t1 = time.perf_counter()
        x = torch.cat([b, a], dim=1)
        for _ in range(reps):
            oflux.single_block(P, 0, x, cond, freqs, attn=sdpa)
        t2 = time.perf_counter()
    td, ts = (t1 - t0) / reps, (t2 - t1) / reps
    ms = (td * num_double + ts * num_single) * 1e3
    return {"value": round(ms, 1), "unit": "ms", "cores": torch.get_num_threads(), "kind": "port",
            "sample": "oracle fp32 on host: 1 double block (%.2f s) + 1 single block (%.2f s) at 4096+512 tokens, "
                      "mean of %d runs each, extrapolated x%d + x%d (embedders and final layer excluded)"
                      % (td, ts, reps, num_double, num_single)}


def _median_time(fn, warm, reps):
    for _ in range(warm):
        fn()
    ts = []
    for _ in range(reps):
        t0 = time.perf_counter()
        fn()
        ts.append(time.perf_counter() - t0)
    return sorted(ts)[len(ts) // 2]


def cpu_config_legs():
    """The CPU torch path of BASELINE configs[0..2] on the host cores, each at its full size:
    configs[0] the fp32 joint block at 1024 image + 256 text tokens with torch SDPA (the configuration IS this CPU
    run; median of 5 after 3 warm-ups); configs[1] the fp32 matmul of the dequantised operands plus bias at
    M = 4608 for the four (K, N); configs[2] fp32 SDPA of (1, 24, 4608, 128) operands (RMSNorm / RoPE are
    negligible beside it)."""
    import torch

    from oracle import dit_ops as O
    from oracle import flux as oflux

    cores = os.cpu_count() or 1
    torch.set_num_threads(cores)
    legs = {"cores": torch.get_num_threads()}
    g = torch.Generator().manual_seed(0)
    with torch.no_grad():
        sd = oflux.init_params(1, 0, dtype=torch.float32, seed=0)
        P = oflux.Params(sd, "plain")
        img, txt, cond = torch.randn(1, 1024, HIDDEN, generator=g), torch.randn(1, 256, HIDDEN, generator=g), \
            torch.randn(1, HIDDEN, generator=g)
        ids = torch.cat([torch.zeros(1, 256, 3), oflux.image_ids(64, 64, 1, "cpu", torch.float32)], dim=1)
        freqs = O.rope_table(ids, oflux.AXES_DIM, oflux.THETA)
        sdpa = torch.nn.functional.scaled_dot_product_attention
        t = _median_time(lambda: oflux.joint_block(P, 0, img, txt, cond, freqs, attn=sdpa), 3, 5)
        gf = (2 * 1280 * HIDDEN * 12 * HIDDEN + 4 * 1280 * 1280 * HIDDEN) / 1e9
        legs["config0_joint_block_1024+256_fp32"] = {"ms": round(t * 1e3, 1), "gflops": round(gf / t, 1),
                                                     "sample": "full size, median of 5 after 3 warm-ups"}
        del sd, P
        mm = {}
        for K, N in ((3072, 9216), (3072, 3072), (3072, 12288), (12288, 3072)):
            a, w, b = torch.randn(N_IMG + N_TXT, K, generator=g), torch.randn(N, K, generator=g), torch.randn(N, generator=g)
            t = _median_time(lambda: torch.addmm(b, a, w.t()), 1, 3)
            mm[f"{K}x{N}"] = {"ms": round(t * 1e3, 1), "gflops": round(2.0 * (N_IMG + N_TXT) * K * N / t / 1e9, 1)}
            del a, w
        legs["config1_fp32_matmul_M4608"] = dict(mm, sample="full size, dequantised-operand fp32 matmul + bias, "
                                                            "median of 3 after 1 warm-up")
        q, k, v = [torch.randn(1, HEADS, N_IMG + N_TXT, HEAD_DIM, generator=g) for _ in range(3)]
        t = _median_time(lambda: sdpa(q, k, v), 1, 3)
        legs["config2_fp32_sdpa_S4608_H24"] = {"ms": round(t * 1e3, 1),
                                               "gflops": round(4.0 * (N_IMG + N_TXT) ** 2 * HEAD_DIM * HEADS / t / 1e9, 1),
                                               "sample": "full size, median of 3 after 1 warm-up"}
    return legs


def wan_cpu_baseline(cfg, S_full, S_sample=2048, reps=2):
    """One Wan2.1-14B DiTBlock (oracle, fp32, torch SDPA) on the host cores at a REDUCED token count, extrapolated:
    the GEMM / row-kernel part scales with S, self-attention with S^2 (measured separately), 512 text tokens kept."""
    import torch

    from oracle import wan as ow

    cores = os.cpu_count() or 1
    torch.set_num_threads(cores)
    c1 = dict(cfg, num_layers=1)
    sd = ow.init_params(c1, dtype=torch.float32, seed=0)
    P = ow.Params(sd, "plain")
    g = torch.Generator().manual_seed(0)
    d, H = cfg["dim"], cfg["num_heads"]
    x, ctx, t_mod = torch.randn(1, S_sample, d, generator=g), torch.randn(1, 512, d, generator=g), \
        torch.randn(1, 6, d, generator=g) * 0.3
    freqs = ow.freqs_cis_3d(d // H, 1, 1, S_sample)
    sdpa = torch.nn.functional.scaled_dot_product_attention
    with torch.no_grad():
        t_block = _median_time(lambda: ow.dit_block(P, 0, x, ctx, t_mod, freqs, c1, attn=sdpa), 1, reps)
        q = torch.randn(1, H, S_sample, d // H, generator=g)
        t_attn = _median_time(lambda: sdpa(q, q, q), 1, reps)
    scale = S_full / S_sample
    per_block = (t_block - t_attn) * scale + t_attn * scale * scale
    return {"value": round(per_block * cfg["num_layers"] * 1e3, 0), "unit": "ms", "cores": torch.get_num_threads(),
            "kind": "port",
            "sample": "oracle fp32 on host: one DiTBlock at %d video + 512 text tokens (%.2f s, of which self-attention "
                      "%.2f s), EXTRAPOLATED to %d tokens (attention x%.0f, the rest x%.1f) and x%d layers"
                      % (S_sample, t_block, t_attn, S_full, scale * scale, scale, cfg["num_layers"])}


# L2-miss bytes per fp8_gemm_kernel launch, averaged over the 152 block-GEMM launches of one 19+38 step (the
# image/text pairs of the joint blocks share a launch): rocprofv3 --pmc FETCH_SIZE (383.0 MB) plus --pmc WRITE_SIZE
# (88.5 MB), each scaled by what the same counter reads for the 256 MiB copy of --calibrate-copy (FETCH_SIZE
# counts half the copied bytes, WRITE_SIZE all of them); profiles/flux_step_hbm_traffic_pmc.txt holds the
# per-shape figures.
GEMM_TRAFFIC_BYTES = 471.5e6
# L2-miss bytes per attention call of the Wan step, averaged over its self- and cross-attention calls (one of each
# per layer): FETCH_SIZE + WRITE_SIZE runs of `--workload wan14b --wan-layers 2 --calibrate-copy`, scaled the same
# way (profiles/wan14b_attention_hbm_traffic_pmc.txt: self-attention 3025 + 335 MB, cross-attention 363 + 335 MB).
WAN_ATTN_TRAFFIC_BYTES = 2029.0e6


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=5)
    ap.add_argument("--warmup", type=int, default=2)
    ap.add_argument("--double", type=int, default=19)
    ap.add_argument("--single", type=int, default=38)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-micro", action="store_true")
    ap.add_argument("--workload", choices=("flux", "wan14b"), default="flux",
                    help="flux (default): the headline Flux-1024 step; wan14b: one Wan2.1-14B step (configs[4])")
    ap.add_argument("--wan-layers", type=int, default=40)
    ap.add_argument("--overlap-probe", action="store_true",
                    help="only run the two-stream overlap probe (attention beside GELU + quantise) with eager "
                         "launches, for a kernel trace of it, and print its figures")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run one 256 MiB device-to-device copy, the known-size dispatch that FETCH_SIZE / "
                         "WRITE_SIZE counter runs are scaled by")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one MI355X; this build has no multi-GPU path (--gpus must be 1)")

    import torch

    from diffsynth_engine_amd import _lib, ops
    from diffsynth_engine_amd.flux_dit import FluxDiTRunner

    if not torch.cuda.is_available():
        sys.exit("bench.py needs an MI355X (no GPU visible)")
    rc = _lib.load().dsx_check_device()
    if rc:
        sys.exit("bench.py: " + _lib.strerror(rc))
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    if args.calibrate_copy:
        src = torch.empty(256 << 20, dtype=torch.uint8, device=dev).random_(0, 255)
        dst = torch.empty_like(src)
        dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst
    if args.overlap_probe:
        print(json.dumps({"two_stream_overlap": two_stream_overlap(torch, ops, dev, graph=False)}))
        return
    if args.workload == "wan14b":
        print(json.dumps(run_wan(torch, dev, args.wan_layers, args.steps, args.warmup, not args.no_cpu_baseline)))
        return

    runner = FluxDiTRunner(flux_state_dict_stream(args.double, args.single, dev), args.double, args.single,
                           scaled=True, device=dev)
    g = torch.Generator(device=dev).manual_seed(0)
    inp = dict(
        hidden_states=torch.randn(1, 16, 128, 128, generator=g, device=dev).to(torch.bfloat16),
        timestep=torch.tensor([500.0], device=dev),
        prompt_emb=torch.randn(1, N_TXT, 4096, generator=g, device=dev).to(torch.bfloat16),
        pooled_prompt_emb=torch.randn(1, 768, generator=g, device=dev).to(torch.bfloat16),
        guidance=torch.tensor([3.5], device=dev),
        text_ids=torch.zeros(1, N_TXT, 3, device=dev),
    )
    gt = GemmTimer(torch, ops)
    with gt:  # bracketed like the timed steps: says how many events a step takes, and creates the first of them
        for _ in range(args.warmup):
            out = runner(**inp)
    if args.warmup:
        gt.prepare(len(gt.records) // args.warmup * args.steps)
    torch.cuda.synchronize()
    with gt:
        t0 = time.perf_counter()
        for _ in range(args.steps):
            out = runner(**inp)
        torch.cuda.synchronize()
        t1 = time.perf_counter()
        n_gemm, gemm_flops, gemm_secs = gt.summary()
    with AttnTimer(torch, ops) as at:  # a second pass of the same steps, outside the timed region
        for _ in range(args.steps):
            out = runner(**inp)
        n_attn, attn_flops, attn_secs = at.summary()
    assert torch.isfinite(out.float()).all().item(), "non-finite output"
    ms = (t1 - t0) * 1e3 / args.steps

    gemm_fl, attn_fl = step_flops(args.double, args.single)
    t_ideal = gemm_fl / PEAK_FP8 + attn_fl / PEAK_BF16
    achieved = gemm_flops / gemm_secs if gemm_secs > 0 else 0.0
    result = {
        "metric": "flux_1024x1024_fp8_dit_step_ms",
        "value": round(ms, 3),
        "unit": "ms",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms, 3),
        "higher_is_better": False,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "fp8_e4m3 GEMM (fp32 accumulate) + bf16 attention",
        "data": "synthetic",
        "config": {"workload": "BASELINE configs[3]: full Flux.1-dev-architecture DiT, one denoising step, "
                               "%d double + %d single blocks, 4096 image + 512 text tokens, batch 1, "
                               "random init N(0,0.02), e4m3 weights (per-tensor scale), per-token activation scale"
                               % (args.double, args.single)},
        "roofline": {"bound": "mfma", "achieved": round(achieved / 1e12, 1), "peak": PEAK_FP8 / 1e12,
                     "unit": "TFLOP/s", "frac": round(achieved / PEAK_FP8, 4),
                     "traffic": GEMM_TRAFFIC_BYTES if (args.double, args.single) == (19, 38) else None,
                     "kernel": "fp8_gemm_kernel", "launches": n_gemm,
                     "avg_launch_us": round(gemm_secs / max(n_gemm, 1) * 1e6, 1), "timed_with": _EventBrackets.kind},
        "step_roofline": {"algorithmic_tflop": round((gemm_fl + attn_fl) / 1e12, 2),
                          "ideal_ms": round(t_ideal * 1e3, 2), "frac": round(t_ideal * 1e3 / ms, 4)},
    }
    result["detail"] = {"attention_in_step": {
        "launches": n_attn, "avg_call_us": round(attn_secs / max(n_attn, 1) * 1e6, 1),
        "tflops": round(attn_flops / max(attn_secs, 1e-12) / 1e12, 1),
        "frac_bf16_peak": round(attn_flops / max(attn_secs, 1e-12) / PEAK_BF16, 4),
        "ms_per_step": round(attn_secs * 1e3 / args.steps, 2)},
        "fp8_gemm_in_step": {"ms_per_step": round(gemm_secs * 1e3 / args.steps, 2)}}
    if not args.no_micro:
        result["detail"].update(micro_benchmarks(torch, ops, dev))
        result["detail"]["two_stream_overlap"] = two_stream_overlap(torch, ops, dev)
        probe = mfma_ceiling(torch, dev)
        result["detail"]["mfma_ceiling_probe"] = probe
        # The same step against what THIS box's matrix pipes sustain on random operand bits (bare MFMA streams, every
        # compute unit busy, no memory traffic): boxes of the pool differ by several per cent in the clock they hold
        # under load, and this second fraction moves with the box where `frac` (published peaks) does not.
        c_fp8 = max(probe["fp8_32x32x64_random"]["tflops"], probe["fp8_16x16x128_random"]["tflops"]) * 1e12
        c_bf16 = max(probe["bf16_32x32x16_random"]["tflops"], probe["bf16_16x16x32_random"]["tflops"]) * 1e12
        t_box = gemm_fl / c_fp8 + attn_fl / c_bf16
        result["step_roofline"]["box_ceiling"] = {
            "fp8_tflops_random_operands": round(c_fp8 / 1e12, 1), "bf16_tflops_random_operands": round(c_bf16 / 1e12, 1),
            "ideal_ms_at_box_ceiling": round(t_box * 1e3, 2), "frac_of_box_ceiling": round(t_box * 1e3 / ms, 4),
            "gemm_frac_of_box_ceiling": round(achieved / c_fp8, 4),
            "attention_frac_of_box_ceiling": round(attn_flops / max(attn_secs, 1e-12) / c_bf16, 4)}
        # the same model at other image sizes (512 text tokens): two warm-up steps, three timed ones each
        other = {}
        for side in (64, 96, 192):
            inp_o = dict(inp, hidden_states=torch.randn(1, 16, side, side, generator=g, device=dev).to(torch.bfloat16))
            for _ in range(2):
                runner(**inp_o)
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for _ in range(3):
                out_o = runner(**inp_o)
            torch.cuda.synchronize()
            ms_o = (time.perf_counter() - t0) * 1e3 / 3
            assert torch.isfinite(out_o.float()).all().item(), "non-finite output"
            tokens = side * side // 4 + N_TXT
            gemm_o, attn_o = step_flops(args.double, args.single, n_img=side * side // 4)
            ideal_o = gemm_o / PEAK_FP8 + attn_o / PEAK_BF16
            entry = {"tokens": tokens, "ms_per_step": round(ms_o, 2),
                     "step_roofline_frac": round(ideal_o * 1e3 / ms_o, 4)}
            if tokens <= 2816 + N_TXT:
                # where the ~1500 launches of a step are the floor: the same step recorded once as a HIP graph and
                # replayed (diffsynth_engine_amd.graph.GraphedStep: one submission per step)
                from diffsynth_engine_amd.graph import GraphedStep

                gstep = GraphedStep(runner, **inp_o)
                gstep(**inp_o)
                torch.cuda.synchronize()
                t0 = time.perf_counter()
                for _ in range(3):
                    out_g = gstep(**inp_o)
                torch.cuda.synchronize()
                ms_g = (time.perf_counter() - t0) * 1e3 / 3
                assert torch.equal(out_g, out_o), "graph replay differs from the eager step"
                entry["graph_replay_ms_per_step"] = round(ms_g, 2)
                entry["graph_replay_step_roofline_frac"] = round(ideal_o * 1e3 / ms_g, 4)
                del gstep
            other["%dx%d" % (side * 8, side * 8)] = entry
        result["detail"]["flux_other_image_sizes"] = other
        # the same step with an unfused rank-16 LoRA on every one of the 228 block linears (LoRALinear.forward,
        # models/basic/lora.py:137-141): the updates ride the main products as 128 more columns of their reduction
        # axis, one small down-projection launch per linear
        def plain_steps(n=5):  # ms per step without event brackets (the headline's timed region carries them)
            for _ in range(2):
                runner(**inp)
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for _ in range(n):
                o = runner(**inp)
            torch.cuda.synchronize()
            assert torch.isfinite(o.float()).all().item(), "non-finite output"
            return (time.perf_counter() - t0) * 1e3 / n

        ms_plain = plain_steps()
        names = [n for n in runner.lin if n.startswith(("blocks.", "single_blocks."))]
        for n in names:
            L = runner.lin[n]
            L.add_lora((torch.randn(16, L.k, generator=g, device=dev) * 0.01).to(torch.bfloat16),
                       (torch.randn(L.n, 16, generator=g, device=dev) * 0.01).to(torch.bfloat16), 1.0)
        riding = sum(runner.lin[n]._extension() is not None for n in names)
        ms_l = plain_steps()
        result["detail"]["lora_rank16_on_all_block_linears"] = {
            "linears": len(names), "riding_the_main_product": riding, "ms_per_step": round(ms_l, 2),
            "ms_per_step_without_lora_same_timing": round(ms_plain, 2),
            "overhead_frac": round(ms_l / ms_plain - 1.0, 4)}
    del runner
    torch.cuda.empty_cache()
    if not args.no_micro:
        # the same step in the reference's own fp8 arithmetic (utils/fp8_linear.py:28-60: bare e4m3 casts, unit
        # scales), weights drawn N(0, 1/fan_in) so that no activation comes near e4m3's 448, next to the scaled
        # mode on the same weights: what the per-token scales of the headline mode cost
        unit = {}
        for mode, scaled in (("unit_scales", False), ("per_token_scales", True)):
            r2 = FluxDiTRunner(flux_state_dict_stream(args.double, args.single, dev, std=None), args.double,
                               args.single, scaled=scaled, device=dev)
            for _ in range(2):
                out_u = r2(**inp)
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for _ in range(5):
                out_u = r2(**inp)
            torch.cuda.synchronize()
            unit[mode + "_ms_per_step"] = round((time.perf_counter() - t0) * 1e3 / 5, 2)
            assert torch.isfinite(out_u.float()).all().item(), "non-finite output"
            del r2
            torch.cuda.empty_cache()
        unit["weights"] = "N(0, 1/fan_in), AdaLN projections at half that deviation"
        result["detail"]["flux_step_in_the_references_arithmetic"] = unit
        # BASELINE configs[4] beside the headline figure: the whole Wan2.1-14B step, all 40 layers at 32 760 + 512
        # tokens, same code path as `--workload wan14b` (one warm-up step, two timed ones; a step is about a second)
        w = run_wan(torch, dev, 40, 2, 1, not args.no_cpu_baseline)
        result["detail"]["wan14b_step"] = {
            "config": w["config"]["workload"], "ms_per_step": w["ms_per_step"],
            "ms_per_layer": round(w["ms_per_step"] / 40, 2),
            "attention": w["roofline"], "fp8_gemm_in_step": w["detail"]["fp8_gemm_in_step"],
            "ms_per_step_without_device_score_bound": w["detail"]["ms_per_step_without_device_score_bound"],
            "step_roofline": w["step_roofline"], "cpu_baseline": w["cpu_baseline"]}
        torch.cuda.empty_cache()
    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline(args.double, args.single)
        result["detail"]["cpu_config_legs"] = cpu_config_legs()
    print(json.dumps(result))


if __name__ == "__main__":
    main()
