"""The matrix-pipe microbenchmark behind the roofline denominators (dsx_mfma_ceiling_probe): every kind runs,
reports the flops of its launch, and leaves its sink untouched for finite operands."""
import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu


def test_every_probe_kind_runs_and_counts_its_flops(dev):
    from diffsynth_engine_amd import _lib

    lib = _lib.load()
    sink = torch.zeros(1, device=dev)
    stream = torch.cuda.current_stream().cuda_stream
    per_mfma = {0: 2 * 32 * 32 * 16, 1: 2 * 32 * 32 * 64, 2: 2 * 16 * 16 * 32, 3: 2 * 16 * 16 * 128}
    g = torch.Generator(device=dev).manual_seed(0)
    for kind in range(8):
        if kind & 1:
            bits = torch.randn(16 * 256 * 4, generator=g, device=dev).to(torch.float8_e4m3fn).view(torch.int32)
        else:
            bits = torch.randn(16 * 256 * 2, generator=g, device=dev).bfloat16().view(torch.int32)
        assert bits.numel() == 16 * 256
        flops = ctypes.c_int64(0)
        rc = lib.dsx_mfma_ceiling_probe(kind, bits.data_ptr(), 50, 7, sink.data_ptr(), ctypes.byref(flops), stream)
        assert rc == _lib.DSX_OK, (kind, rc)
        # 7 workgroups x 4 wavefronts x 50 rounds x (4 MFMAs of a 32x32 shape, 8 of a 16x16 shape)
        assert flops.value == 7 * 4 * 50 * (8 if (kind & 3) >= 2 else 4) * per_mfma[kind & 3]
    torch.cuda.synchronize()
    assert sink.item() == 0.0
    # the caps that keep one call from occupying the device for minutes
    assert lib.dsx_mfma_ceiling_probe(0, bits.data_ptr(), (1 << 22) + 1, 7, sink.data_ptr(), None, stream) == _lib.DSX_EBADSHAPE
    assert lib.dsx_mfma_ceiling_probe(0, bits.data_ptr(), 50, (1 << 14) + 1, sink.data_ptr(), None, stream) == _lib.DSX_EBADSHAPE
