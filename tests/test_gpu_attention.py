"""GPU parity: flash attention (plain, joint two-segment, cross, fused RMSNorm+RoPE) vs the fp32 oracle."""
import math

import pytest
import torch

from conftest import row_rel_err
from oracle import dit_ops as O

pytestmark = pytest.mark.gpu

TOL = 2e-2  # the bar stated for the attention kernel, per query row: max_d |err| / max_d |ref| of that row


_rel_err = row_rel_err


def _qkv(B, H, Sq, Skv, seed):
    g = torch.Generator().manual_seed(seed)
    q = torch.randn(B, H, Sq, 128, generator=g).bfloat16()
    k = torch.randn(B, H, Skv, 128, generator=g).bfloat16()
    v = torch.randn(B, H, Skv, 128, generator=g).bfloat16()
    return q, k, v


@pytest.mark.parametrize("B,H,Sq,Skv", [(1, 2, 256, 64), (1, 1, 64, 256), (2, 3, 300, 300), (1, 2, 1, 1),
                                        (1, 2, 1280, 1280), (1, 1, 520, 77), (1, 4, 33, 512)])
def test_attention_matches_fp32_sdpa(dev, B, H, Sq, Skv):
    from diffsynth_engine_amd import mi355x_attention

    q, k, v = _qkv(B, H, Sq, Skv, seed=Sq * 7 + Skv)
    want = O.sdpa(q.float(), k.float(), v.float())
    got = mi355x_attention(q.to(dev), k.to(dev), v.to(dev)).cpu()
    assert got.shape == want.shape and got.dtype == torch.bfloat16
    assert _rel_err(got, want) <= TOL


def test_attention_against_torch_sdpa_library(dev):
    """Second opinion: torch's own fp32 SDPA (the routine the reference calls)."""
    from diffsynth_engine_amd import mi355x_attention

    q, k, v = _qkv(1, 2, 384, 384, seed=3)
    want = torch.nn.functional.scaled_dot_product_attention(q.float(), k.float(), v.float())
    got = mi355x_attention(q.to(dev), k.to(dev), v.to(dev)).cpu()
    assert _rel_err(got, want) <= TOL


def test_attention_noncontiguous_packed_qkv_views(dev):
    """The views FluxJointAttention hands to the slot: (B,S,3H,D).transpose(1,2).chunk(3,1) (flux_dit.py:165-167)."""
    from diffsynth_engine_amd import mi355x_attention

    B, S, H = 1, 320, 3
    qkv = torch.randn(B, S, 3 * H * 128, generator=torch.Generator().manual_seed(1)).bfloat16()
    q, k, v = qkv.view(B, S, 3 * H, 128).transpose(1, 2).chunk(3, dim=1)
    want = O.sdpa(q.float(), k.float(), v.float())
    qd, kd, vd = qkv.to(dev).view(B, S, 3 * H, 128).transpose(1, 2).chunk(3, dim=1)
    got = mi355x_attention(qd, kd, vd).cpu()
    assert _rel_err(got, want) <= TOL


def test_softmax_invariants(dev):
    """Constant V => output equals that constant; permuting keys together with values changes nothing."""
    from diffsynth_engine_amd import mi355x_attention

    q, k, v = _qkv(1, 2, 200, 333, seed=9)
    vc = torch.full_like(v, 0.75)
    out = mi355x_attention(q.to(dev), k.to(dev), vc.to(dev)).cpu().float()
    assert (out - 0.75).abs().max().item() <= 0.75 * 2 ** -7
    perm = torch.randperm(333, generator=torch.Generator().manual_seed(2))
    a = mi355x_attention(q.to(dev), k.to(dev), v.to(dev)).cpu().float()
    b = mi355x_attention(q.to(dev), k[:, :, perm].contiguous().to(dev), v[:, :, perm].contiguous().to(dev)).cpu().float()
    assert (a - b).abs().max().item() <= 2e-2


def test_joint_two_segment_equals_concat(dev):
    """Text-first joint attention from two base pointers == attention over torch.cat (flux_dit.py:176-178)."""
    from diffsynth_engine_amd import ops

    H, St, Si = 2, 72, 200
    qt, kt, vt = _qkv(1, H, St, St, seed=11)
    qi, ki, vi = _qkv(1, H, Si, Si, seed=12)
    want = O.sdpa(torch.cat([qt, qi], 2).float(), torch.cat([kt, ki], 2).float(), torch.cat([vt, vi], 2).float())
    o1, o2 = ops.attention_bhsd(qt.to(dev), kt.to(dev), vt.to(dev), q2=qi.to(dev), k2=ki.to(dev), v2=vi.to(dev))
    got = torch.cat([o1.cpu(), o2.cpu()], dim=2)
    assert _rel_err(got, want) <= TOL


def _flux_ids(St, side):
    txt = torch.zeros(1, St, 3)
    img = torch.zeros(side, side, 3)
    img[..., 1] += torch.arange(side)[:, None]
    img[..., 2] += torch.arange(side)[None, :]
    return torch.cat([txt, img.reshape(1, -1, 3)], dim=1)


@pytest.mark.parametrize("wstd", [0.0, 0.1])
def test_fused_rmsnorm_rope_joint_attention(dev, wstd):
    """RMSNorm + 3-axis RoPE applied by the attention entry point (q as the kernel loads it, k once into caller
    scratch) == oracle RMSNorm -> concat -> apply_rope -> SDPA (flux_dit.py:161-183)."""
    from diffsynth_engine_amd import ops

    H, St, side = 2, 64, 12
    Si = side * side
    g = torch.Generator().manual_seed(21)
    qt, kt, vt = _qkv(1, H, St, St, seed=13)
    qi, ki, vi = _qkv(1, H, Si, Si, seed=14)
    w = [(1.0 + wstd * torch.randn(128, generator=g)).bfloat16() for _ in range(4)]  # q_a, k_a, q_b, k_b
    freqs = O.rope_table(_flux_ids(St, side), (16, 56, 56), 10000)
    # oracle in bf16 (the reference's dtype) up to the attention inputs, fp32 attention
    q = torch.cat([O.rms_norm(qt, w[2], 1e-6), O.rms_norm(qi, w[0], 1e-6)], dim=2)
    k = torch.cat([O.rms_norm(kt, w[3], 1e-6), O.rms_norm(ki, w[1], 1e-6)], dim=2)
    q, k = O.apply_rope(q, freqs), O.apply_rope(k, freqs)
    want = O.sdpa(q.float(), k.float(), torch.cat([vt, vi], 2).float())
    table = ops.rope_table_from_freqs(freqs).to(dev)
    o1, o2 = ops.attention_bhsd(qt.to(dev), kt.to(dev), vt.to(dev), q2=qi.to(dev), k2=ki.to(dev), v2=vi.to(dev),
                                rope=table, q_norm_w=w[2].to(dev), k_norm_w=w[3].to(dev), q2_norm_w=w[0].to(dev),
                                k2_norm_w=w[1].to(dev))
    got = torch.cat([o1.cpu(), o2.cpu()], dim=2)
    assert _rel_err(got, want) <= TOL
    # the standalone pre-pass must agree with the oracle's bf16 q almost bit for bit
    qn = ops.rmsnorm_rope(qi.to(dev), w[0].to(dev), table, pos0=St).cpu()
    ref = q[:, :, St:]
    diff = (qn.float() - ref.float()).abs()
    assert (diff > 0).float().mean().item() < 0.01  # rare 1-ulp flips from the rsqrt / sum order
    assert diff.max().item() <= 2 ** -6 * ref.float().abs().max().item()


def test_wan_seam_cross_attention(dev):
    """wan_dit.attention contract (wan_dit.py:18-22): (B,S,H*D), Lq != Lk."""
    from diffsynth_engine_amd import wan_attention

    B, H, Sq, Skv = 1, 3, 250, 64
    q, k, v = _qkv(B, H, Sq, Skv, seed=5)
    want = O.sdpa(q.float(), k.float(), v.float()).transpose(1, 2).reshape(B, Sq, H * 128)
    flat = lambda t: t.transpose(1, 2).reshape(B, t.shape[2], H * 128).contiguous()
    got = wan_attention(flat(q).to(dev), flat(k).to(dev), flat(v).to(dev), H).cpu()
    assert _rel_err(got, want) <= TOL


def test_bshd_attention_entry_and_errors(dev):
    from diffsynth_engine_amd import attention

    q, k, v = _qkv(1, 2, 100, 100, seed=6)
    want = O.sdpa(q.float(), k.float(), v.float()).transpose(1, 2)
    got = attention(q.transpose(1, 2).contiguous().to(dev), k.transpose(1, 2).contiguous().to(dev),
                    v.transpose(1, 2).contiguous().to(dev), attn_impl="mi355x").cpu()
    assert _rel_err(got, want) <= TOL
    with pytest.raises(ValueError):
        attention(q, k, v, attn_impl="flash3")
    with pytest.raises(ValueError):
        bad = torch.zeros(1, 1, 8, 64, dtype=torch.bfloat16, device=dev)
        attention(bad, bad, bad)


@pytest.mark.parametrize("H,S,extra", [(24, 300, 24 * 128), (3, 17, 0), (5, 64, 128)])
def test_rmsnorm_rope_qk_in_place_equals_per_tensor_kernel(dev, H, S, extra):
    """One pass over the packed (B,S,[q heads | k heads | rest]) projection == the single-tensor kernel applied to
    q and to k separately (same arithmetic), the rest of the row (v, mlp columns) untouched; and the q half
    agrees with the oracle's RMSNorm -> apply_rope (transformer_helper.py:73-78, flux_dit.py:154-159)."""
    from diffsynth_engine_amd import ops

    g = torch.Generator().manual_seed(H * 100 + S)
    B, pos0 = 2, 5
    x = torch.randn(B, S, 2 * H * 128 + extra, generator=g).bfloat16()
    wq = (1.0 + 0.1 * torch.randn(128, generator=g)).bfloat16()
    wk = (1.0 + 0.1 * torch.randn(128, generator=g)).bfloat16()
    ids = torch.zeros(B, pos0 + S, 3)
    ids[..., 1] = torch.arange(pos0 + S).float() // 7
    ids[..., 2] = torch.arange(pos0 + S).float() % 7
    freqs = O.rope_table(ids, (16, 56, 56), 10000)
    table = ops.rope_table_from_freqs(freqs).to(dev)
    xd = x.to(dev)
    heads = xd[:, :, : 2 * H * 128].view(B, S, 2 * H, 128).transpose(1, 2)
    want_q = ops.rmsnorm_rope(heads[:, :H], wq.to(dev), table, pos0=pos0).cpu()
    want_k = ops.rmsnorm_rope(heads[:, H:], wk.to(dev), table, pos0=pos0).cpu()
    got = ops.rmsnorm_rope_qk(xd.clone(), H, H, wq.to(dev), wk.to(dev), table, pos0=pos0).cpu()
    got_h = got[:, :, : 2 * H * 128].view(B, S, 2 * H, 128).transpose(1, 2)
    assert torch.equal(got_h[:, :H], want_q)
    assert torch.equal(got_h[:, H:], want_k)
    assert torch.equal(got[:, :, 2 * H * 128:], x[:, :, 2 * H * 128:])
    xq = x[:, :, : H * 128].view(B, S, H, 128).transpose(1, 2)
    ref = O.apply_rope(O.rms_norm(xq, wq, 1e-6), freqs[:, :, pos0:])
    diff = (got_h[:, :H].float() - ref.float()).abs()
    assert (diff > 0).float().mean().item() < 0.01
    assert diff.max().item() <= 2 ** -6 * ref.float().abs().max().item()


@pytest.mark.parametrize("Sq,Skv", [(300, 300), (64, 1000), (257, 77)])
def test_score_bound_promise_skips_the_running_maximum(dev, Sq, Skv):
    """Rows of norm sqrt(128) (what q/k RMSNorm with unit weights produces) bound |q.k|/sqrt(128) by sqrt(128);
    with that promise the kernel keeps its softmax reference at 0.  Same result as without the promise (on
    such inputs neither variant ever moves the reference), and both match fp32 SDPA.  A promise too large to
    be of use is ignored."""
    from diffsynth_engine_amd import ops

    g = torch.Generator().manual_seed(Sq + Skv)
    unit = lambda t: (t / t.norm(dim=-1, keepdim=True) * math.sqrt(128)).bfloat16()
    q = unit(torch.randn(1, 3, Sq, 128, generator=g))
    k = unit(torch.randn(1, 3, Skv, 128, generator=g))
    k[0, 0, : min(Sq, Skv)] = q[0, 0, : min(Sq, Skv)]  # some scores right at the bound
    v = torch.randn(1, 3, Skv, 128, generator=g).bfloat16()
    want = O.sdpa(q.float(), k.float(), v.float())
    plain = ops.attention_bhsd(q.to(dev), k.to(dev), v.to(dev)).cpu()
    bounded = ops.attention_bhsd(q.to(dev), k.to(dev), v.to(dev), score_bound=1.02 * math.sqrt(128)).cpu()
    ignored = ops.attention_bhsd(q.to(dev), k.to(dev), v.to(dev), score_bound=1e4).cpu()
    assert torch.equal(plain, bounded) and torch.equal(plain, ignored)
    assert _rel_err(bounded, want) <= TOL


@pytest.mark.parametrize("H,Sq,Skv,qscale,bound", [(3, 2048, 2100, 1.0, 0.0), (2, 700, 4200, 12.0, 0.0),
                                                   (5, 1000, 2048, 1.0, 0.0), (3, 2048, 2100, 0.25, 12.0)])
def test_key_range_split_of_the_last_round(dev, H, Sq, Skv, qscale, bound):
    """Few (head, query block) units and a long key axis: the launcher cuts the key ranges of the units into
    equal pieces over all compute units and merges the partial softmax results.  Pieces end inside units and
    span unit boundaries, the key axis is ragged, and with qscale > 1 the softmax references of the parts of
    a row differ (scores beyond +-64 in the log2 domain), so the merge has to rescale."""
    from diffsynth_engine_amd import _lib, ops

    g = torch.Generator().manual_seed(H * Sq + Skv)
    q = (torch.randn(1, H, Sq, 128, generator=g) * qscale).bfloat16()
    k = torch.randn(1, H, Skv, 128, generator=g).bfloat16()
    v = torch.randn(1, H, Skv, 128, generator=g).bfloat16()
    want = O.sdpa(q.float(), k.float(), v.float())
    P = _lib.AttnParams()
    P.sq[0], P.skv[0], P.batch, P.heads, P.head_dim = Sq, Skv, 1, H, 128
    assert _lib.load().dsx_attn_workspace_bytes(P) > 0  # this shape does take the split path
    got = ops.attention_bhsd(q.to(dev), k.to(dev), v.to(dev), score_bound=bound).cpu()
    # The kernel multiplies q by scale * log2(e) once and rounds the product to bf16 (2^-9 relative), so a score s
    # carries an absolute error of about |s| * 2^-9 in the exponent.  For N(0,1) operands (|s| of a few units) that
    # is far inside the bar; the x12 case is there to force the softmax references of the parts apart (|s| up to
    # ~60, near one-hot rows that flip between two values), and is held to 3 x the bar.
    assert _rel_err(got, want) <= (TOL if qscale <= 1.0 else 3 * TOL)
    # the unsplit kernel (no scratch offered) gives the same rows up to the order of the fp32 sums
    same = ops.attention_bhsd(q.to(dev), k.to(dev), v.to(dev), score_bound=bound, split_keys=False).cpu()
    assert _rel_err(got, same) <= (2 ** -7 if qscale <= 1.0 else 2 ** -6)  # (a moved reference re-rounds P once more)


def test_key_range_split_joint_two_segments(dev):
    """The split also has to honour the two-segment (text + image) addressing of q, k, v and o."""
    from diffsynth_engine_amd import ops

    g = torch.Generator().manual_seed(5)
    H, S1, S2 = 4, 512, 1792
    mk = lambda s: torch.randn(1, H, s, 128, generator=g).bfloat16()
    q1, k1, v1, q2, k2, v2 = mk(S1), mk(S1), mk(S1), mk(S2), mk(S2), mk(S2)
    want = O.sdpa(torch.cat([q1, q2], 2).float(), torch.cat([k1, k2], 2).float(), torch.cat([v1, v2], 2).float())
    o1, o2 = ops.attention_bhsd(q1.to(dev), k1.to(dev), v1.to(dev), q2=q2.to(dev), k2=k2.to(dev), v2=v2.to(dev))
    got = torch.cat([o1, o2], 2).cpu()
    assert _rel_err(got, want) <= TOL


def test_q_only_rmsnorm_needs_no_scratch(dev):
    """RMSNorm requested for q alone: the attention kernel applies it as it loads the query rows, no copy of k
    is made and no scratch is asked for."""
    from diffsynth_engine_amd import _lib, ops

    g = torch.Generator().manual_seed(21)
    q, k, v = [torch.randn(1, 2, 200, 128, generator=g).bfloat16() for _ in range(3)]
    w = (1 + 0.1 * torch.randn(128, generator=g)).bfloat16()
    qn = O.rms_norm(q, w, 1e-6)
    want = O.sdpa(qn.float(), k.float(), v.float())
    P = _lib.AttnParams()
    P.sq[0], P.skv[0], P.batch, P.heads, P.head_dim = 200, 200, 1, 2, 128
    wd = w.to(dev)
    P.q_norm_w[0] = wd.data_ptr()
    assert _lib.load().dsx_attn_workspace_bytes(P) == 0
    got = ops.attention_bhsd(q.to(dev), k.to(dev), v.to(dev), q_norm_w=wd).cpu()
    assert _rel_err(got, want) <= TOL


@pytest.mark.parametrize("H,Sq,Skv", [(4, 520, 777), (3, 2048, 2100)])  # whole units; the key-range split
def test_device_side_score_bound_picks_the_kernel(dev, H, Sq, Skv):
    """qk_norm2_max: the two device floats choose between the kernel with a fixed softmax reference and the one
    with the running maximum without the host ever reading them.  Small norms give bit for bit the output of a
    host-side promise (score_bound), large or non-finite ones the output of the default path; the result is the
    same softmax either way."""
    from diffsynth_engine_amd import ops

    g = torch.Generator().manual_seed(H + Sq)
    q, k, v = [torch.randn(1, H, s, 128, generator=g).bfloat16().to(dev) for s in (Sq, Skv, Skv)]
    n2 = lambda t: t.float().square().sum(-1).max()
    scale = 128 ** -0.5

    def bound_of(a, b):
        return float((n2(a) * n2(b)).sqrt()) * scale

    # N(0,1) rows: |q||k| * scale ~ 128 / 11.3 -> log2 domain ~ 18: bounded
    nm = torch.stack([n2(q), n2(k)])
    assert bound_of(q, k) * 1.4427 * 1.02 < 64
    promised = ops.attention_bhsd(q, k, v, score_bound=bound_of(q, k))
    default = ops.attention_bhsd(q, k, v)
    assert torch.equal(ops.attention_bhsd(q, k, v, qk_norm2_max=nm), promised)
    assert _rel_err(promised.cpu(), O.sdpa(q.float().cpu(), k.float().cpu(), v.float().cpu())) <= TOL
    # the same rows, but a bound that does not allow it (true for q * 12; here deliberately pessimistic), Inf, NaN
    for bad in (torch.stack([n2(q) * 144, n2(k)]), torch.tensor([float("inf"), 1.0], device=dev),
                torch.tensor([1.0, float("nan")], device=dev)):
        assert torch.equal(ops.attention_bhsd(q, k, v, qk_norm2_max=bad), default)
    # rows that need the running maximum, with their true norms
    q12 = (q.float() * 12).bfloat16()
    nm12 = torch.stack([n2(q12), n2(k)])
    assert bound_of(q12, k) * 1.4427 > 64
    assert torch.equal(ops.attention_bhsd(q12, k, v, qk_norm2_max=nm12), ops.attention_bhsd(q12, k, v))
    # a host-side promise wins over the device floats
    assert torch.equal(ops.attention_bhsd(q, k, v, score_bound=bound_of(q, k), qk_norm2_max=bad), promised)


def test_device_side_score_bound_not_with_fused_preprocessing(dev):
    from diffsynth_engine_amd import ops

    q, k, v = [torch.randn(1, 2, 64, 128).bfloat16().to(dev) for _ in range(3)]
    w = torch.ones(128).bfloat16().to(dev)
    with pytest.raises(ValueError):
        ops.attention_bhsd(q, k, v, q_norm_w=w, qk_norm2_max=torch.ones(2, device=dev))
    with pytest.raises(ValueError):
        ops.attention_bhsd(q, k, v, qk_norm2_max=torch.ones(3, device=dev))


@pytest.mark.parametrize("variant", ["scan", "score_bound", "device_bound", "far_reference", "two_segments"])
def test_many_round_launches_take_the_16x16_form_and_agree(dev, variant):
    """Launches of three full rounds of workgroups and more (>= 768 units of 256 queries on 256 compute units) run
    on the 16x16x32 form of the kernel (attn_plain16.hip); fewer units run on the 32x32x16 form.  Same operation:
    the rows of a many-round call agree with torch's fp32 SDPA on the device to the bar, and with the same heads
    computed in a small launch (the other form) to a few bf16 roundings.  Ragged query and key counts; the running
    maximum, a caller's score bound, the device-side bound, a softmax reference that has to move (scores far from
    zero), and the two-segment (joint) form each take their own path through the kernel."""
    from diffsynth_engine_amd import ops

    B, H, Sq, Skv = 2, 24, 4200, 1111  # 17 query blocks x 24 heads x 2 = 816 units; 1111 = 17 x 64 + 23 keys
    g = torch.Generator(device=dev).manual_seed(5)
    q, k, v = [torch.randn(B, H, n, 128, generator=g, device=dev).bfloat16() for n in (Sq, Skv, Skv)]
    kw = {}
    if variant == "far_reference":
        q = q * 12  # log2-domain scores of std ~17: block maxima beyond 64 move the softmax reference
    elif variant != "scan":
        q = torch.nn.functional.normalize(q.float(), dim=-1).mul(11.3).bfloat16()
        k = torch.nn.functional.normalize(k.float(), dim=-1).mul(11.3).bfloat16()
        if variant == "score_bound":
            kw["score_bound"] = 11.6
        elif variant == "device_bound":
            n2 = lambda t: t.float().square().sum(-1).max()
            kw["qk_norm2_max"] = torch.stack([n2(q), n2(k)])
    if variant == "two_segments":
        out = ops.attention_bhsd(q[:, :, :500], k[:, :, :300], v[:, :, :300], q2=q[:, :, 500:], k2=k[:, :, 300:],
                                 v2=v[:, :, 300:])
        got = torch.cat(out, dim=2)
    else:
        got = ops.attention_bhsd(q, k, v, **kw)
    heads = (0, 13, 23)
    want = torch.nn.functional.scaled_dot_product_attention(q[:, heads, :].float(), k[:, heads, :].float(),
                                                            v[:, heads, :].float())
    # (q is multiplied by scale * log2(e) once and the product rounded to bf16, so a score s carries an absolute error
    # of about |s| * 2^-9 in the exponent: far inside the bar for scores of a few units, and the x12 case, whose rows
    # are nearly one-hot, is held to 3 x the bar, as in test_key_range_split_of_the_last_round)
    assert _rel_err(got[:, heads, :], want) <= (3 * TOL if variant == "far_reference" else TOL)
    small = ops.attention_bhsd(q[:1, :2].contiguous(), k[:1, :2].contiguous(), v[:1, :2].contiguous(),
                               **{n: t for n, t in kw.items() if n == "score_bound"})  # 34 units: the other form
    assert _rel_err(got[:1, :2], small) <= 1e-2
