"""arhip_sage_quant_static (the entry point that allocates nothing) against arhip_sage_quant:
bit-identical int8 tensor, scales and mean, on two calls in a row, the second on a smaller
input so that stale partial sums of the first call lie behind the part the second one uses."""
import ctypes

import numpy as np
import pytest

from autorust_amd import _lib, synth
from autorust_amd.device import BF16, F32
from gpu_util import Bufs

pytestmark = pytest.mark.gpu


def _both(dev, x, B, H, N, D, block, dtype):
    nblk = (N + block - 1) // block
    host = synth.to_bf16_bits(x) if dtype == BF16 else x
    out = []
    with Bufs(dev) as bufs:
        dx = bufs.put(host)
        for static in (False, True):
            x8, sc, mean = bufs.new(x.size), bufs.new(B * H * nblk * 4), bufs.new(B * H * D * 4)
            if static:
                dev.sage_quant_static(dx, x8, sc, B, H, N, D, block, dtype, mean=mean, smooth=True)
            else:
                ws = bufs.new(dev.sage_quant_workspace(B, H, N, D), zero=False)
                dev.sage_quant(dx, x8, sc, B, H, N, D, block, dtype, mean=mean, workspace=ws, smooth=True)
            out.append((x8.copyout(np.int8, x.shape), sc.copyout(np.float32, (B, H, nblk)),
                        mean.copyout(np.float32, (B, H, D))))
    return out


def test_static_scratch_matches_workspace_entry_point(dev):
    shapes = [(2, 8, 1500, 128, 64, BF16), (1, 3, 197, 64, 64, F32)]     # the second is smaller
    for i, (B, H, N, D, block, dtype) in enumerate(shapes):
        x = synth.normal(7100 + i, (B, H, N, D)) + np.float32(3.0) * synth.normal(7110 + i, (1, H, 1, D))
        (a8, asc, amean), (b8, bsc, bmean) = _both(dev, x, B, H, N, D, block, dtype)
        assert np.array_equal(amean, bmean), "mean differs on call %d" % i
        assert np.array_equal(asc, bsc), "scales differ on call %d" % i
        assert np.array_equal(a8, b8), "int8 tensor differs on call %d" % i
        assert np.abs(amean).max() > 0.5 and np.abs(a8).max() == 127   # not vacuous


def test_static_scratch_rejects_oversized_shapes(dev):
    limit = _lib.load().arhip_sage_quant_static_limit()
    assert limit == 16 << 20
    B, H, N, D = 1, 64, 32768 + 64, 128              # one chunk past the limit
    assert dev.sage_quant_workspace(B, H, N, D) > limit
    with Bufs(dev) as bufs:
        tiny = bufs.new(4096)
        with pytest.raises(_lib.ArhipError) as e:
            dev.sage_quant_static(tiny, tiny, tiny, B, H, N, D, 64, BF16, mean=tiny, smooth=True)
    assert e.value.code == _lib.EINVAL and "exceed" in str(e.value)
    # without smoothing there are no partial sums and no limit
    assert _lib.load().arhip_sage_quant_static(None, 16, 16, 16, None, 1, 1, 8, 64, 64, 0, 0, 1, None) == _lib.EINVAL
