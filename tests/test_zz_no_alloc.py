"""The allocation-free attention entry point (dsx_attn_fwd_static: scratch in a static device array of the
library) against dsx_attn_fwd with caller scratch, through the C ABI: bit-equal outputs on two calls in a row,
the second smaller than the first, for both uses of the scratch (the k copy of a fused RMSNorm + RoPE call and
the partial results of the key-range split)."""
import ctypes

import pytest
import torch

from oracle import dit_ops as O

pytestmark = pytest.mark.gpu


def _params(_lib, q, k, v, o, rope=None, wq=None, wk=None):
    B, H, Sq, D = q.shape
    P = _lib.AttnParams()
    for name, t in (("q", q), ("k", k), ("v", v), ("o", o)):
        getattr(P, name)[0] = t.data_ptr()
        getattr(P, name + "_sb")[0], getattr(P, name + "_sh")[0], getattr(P, name + "_ss")[0] = t.stride()[:3]
    P.sq[0], P.skv[0], P.batch, P.heads, P.head_dim = Sq, k.shape[2], B, H, D
    P.softmax_scale = D ** -0.5
    P.norm_eps = 1e-6
    if rope is not None:
        P.rope, P.rope_sb, P.rope_rows = rope.data_ptr(), 0, rope.shape[1]
    if wq is not None:
        P.q_norm_w[0] = wq.data_ptr()
    if wk is not None:
        P.k_norm_w[0] = wk.data_ptr()
    return P


def _both(dev, H, S, fused, seed):
    """Runs one call through each entry point on the same operands; returns (static output, workspace output, q, k, v
    as the kernel saw them)."""
    from diffsynth_engine_amd import _lib, ops

    lib = _lib.load()
    g = torch.Generator().manual_seed(seed)
    q, k, v = [torch.randn(1, H, S, 128, generator=g).bfloat16().to(dev) for _ in range(3)]
    rope = wq = wk = None
    if fused == "k_only":  # only k is normalised: a k copy, no q work, and a unit count that would take the key split
        wk = (1 + 0.1 * torch.randn(128, generator=g)).bfloat16().to(dev)
    elif fused:
        ids = torch.zeros(1, S, 3)
        ids[0, :, 1] = torch.arange(S) // 16
        ids[0, :, 2] = torch.arange(S) % 16
        rope = ops.rope_table_from_freqs(O.rope_table(ids, (16, 56, 56), 10000)).to(dev)
        wq = (1 + 0.1 * torch.randn(128, generator=g)).bfloat16().to(dev)
        wk = (1 + 0.1 * torch.randn(128, generator=g)).bfloat16().to(dev)
    stream = torch.cuda.current_stream().cuda_stream
    o_static = torch.zeros(1, H, S, 128, dtype=torch.bfloat16, device=dev)
    o_ws = torch.zeros_like(o_static)
    P = _params(_lib, q, k, v, o_ws, rope, wq, wk)
    need = lib.dsx_attn_workspace_bytes(P)
    assert 0 < need <= lib.dsx_attn_static_scratch_bytes()
    ws = torch.empty(need, dtype=torch.uint8, device=dev)
    P.workspace, P.workspace_bytes = ws.data_ptr(), need
    assert lib.dsx_attn_fwd(P, stream) == 0
    Ps = _params(_lib, q, k, v, o_static, rope, wq, wk)
    # nothing is allocated during the call: neither through torch (its cumulative allocation counter stands still;
    # the bytes in use may only fall, when the collector frees an earlier test's garbage) nor behind its back
    # (the device's free memory does not shrink)
    torch.cuda.synchronize()
    count = lambda: torch.cuda.memory_stats(dev)["allocation.all.allocated"]
    before, free_before = count(), torch.cuda.mem_get_info(dev)[0]
    assert lib.dsx_attn_fwd_static(Ps, stream) == 0
    torch.cuda.synchronize()
    assert count() == before and torch.cuda.mem_get_info(dev)[0] >= free_before
    return o_static, o_ws


@pytest.mark.parametrize("fused", [True, False])
def test_static_scratch_entry_point_equals_the_workspace_one_on_two_calls_in_a_row(dev, fused):
    # fused: the scratch holds the normalised / rotated copy of k.  Not fused: 3 heads x 8 query blocks = 24 units
    # on 256 compute units, which takes the key-range split (partial results in the scratch).
    shapes = [(4, 1536), (2, 520)] if fused else [(3, 2048), (1, 2048)]
    for i, (H, S) in enumerate(shapes):
        o_static, o_ws = _both(dev, H, S, fused, seed=40 + i)
        assert torch.isfinite(o_static.float()).all().item()
        assert o_static.float().abs().max().item() > 0
        assert torch.equal(o_static, o_ws), (fused, H, S)


def test_a_call_that_copies_k_asks_for_the_copy_only(dev):
    """With a k copy the attention kernel runs without scratch of its own, so the copy is all the call needs: the
    size query must not add the key-range split's bytes (which a plain call of this shape does ask for), and both
    entry points agree on two calls in a row."""
    from diffsynth_engine_amd import _lib

    lib = _lib.load()
    for i, (H, S) in enumerate([(3, 2048), (1, 2048)]):
        z = torch.zeros(1, H, S, 128, dtype=torch.bfloat16, device=dev)
        w = torch.ones(128, dtype=torch.bfloat16, device=dev)
        assert lib.dsx_attn_workspace_bytes(_params(_lib, z, z, z, z)) > 0          # plain: the split's scratch
        assert lib.dsx_attn_workspace_bytes(_params(_lib, z, z, z, z, wk=w)) == 2 * H * S * 128
        o_static, o_ws = _both(dev, H, S, "k_only", seed=50 + i)
        assert o_static.float().abs().max().item() > 0
        assert torch.equal(o_static, o_ws), (H, S)


def test_static_scratch_entry_point_refuses_what_does_not_fit(dev):
    from diffsynth_engine_amd import _lib

    lib = _lib.load()
    H, S = 40, 8192  # k copy: 40 * 8192 * 256 B = 80 MiB > 64 MiB
    q = torch.zeros(1, H, S, 128, dtype=torch.bfloat16, device=dev)
    rope = torch.zeros(1, S, 64, 2, device=dev)
    P = _params(_lib, q, q, q, torch.empty_like(q), rope)
    assert lib.dsx_attn_workspace_bytes(P) > lib.dsx_attn_static_scratch_bytes()
    assert lib.dsx_attn_fwd_static(P, None) == _lib.DSX_EWORKSPACE
    P.workspace, P.workspace_bytes = q.data_ptr(), 16
    assert lib.dsx_attn_fwd_static(P, None) == _lib.DSX_EBADSHAPE  # a caller's buffer belongs to dsx_attn_fwd
