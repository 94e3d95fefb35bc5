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


def test_static_entry_point_allocates_nothing_and_can_be_captured(dev):
    """Free device memory is the same before and after two calls, and the call can be recorded into
    a launch graph (a capture refuses allocations) whose replays give the eager result."""
    B, H, N, D, block = 2, 4, 900, 128, 64
    nblk = (N + block - 1) // block
    with Bufs(dev) as bufs:
        dx = bufs.new(B * H * N * D * 2)
        x8, sc, mean = bufs.new(B * H * N * D), bufs.new(B * H * nblk * 4), bufs.new(B * H * D * 4)
        dx.copyin(synth.to_bf16_bits(synth.normal(7201, (B, H, N, D)) + np.float32(2.0)))
        dev.sync()
        free0 = dev.mem_info()[0]
        for _ in range(2):
            dev.sage_quant_static(dx, x8, sc, B, H, N, D, block, BF16, mean=mean, smooth=True)
        assert dev.mem_info()[0] == free0
        eager = [t.copyout(dt, shp) for t, dt, shp in ((x8, np.int8, (B, H, N, D)), (sc, np.float32, (B, H, nblk)),
                                                       (mean, np.float32, (B, H, D)))]
        dev.graph_begin()
        dev.sage_quant_static(dx, x8, sc, B, H, N, D, block, BF16, mean=mean, smooth=True, wait=False)
        graph = dev.graph_end()
        try:
            for rep in range(3):
                for t in (x8, sc, mean):
                    t.zero()
                dev.graph_launch(graph)
                got = [t.copyout(dt, shp) for t, dt, shp in ((x8, np.int8, (B, H, N, D)), (sc, np.float32, (B, H, nblk)),
                                                             (mean, np.float32, (B, H, D)))]
                for a, b_ in zip(eager, got):
                    assert np.array_equal(a, b_), rep
                # eager work and a synchronisation between the replays
                dev.sage_quant_static(dx, x8, sc, B, H, N, D, block, BF16, mean=mean, smooth=True)
                dev.sync()
        finally:
            dev.graph_destroy(graph)


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
        # without smoothing there are no partial sums, hence no limit: the same oversized shape runs
        # and matches the workspace entry point (Q of the long causal configuration, one batch of heads)
        x = synth.normal(7301, (B, H, N, D))
        dx = bufs.put(synth.to_bf16_bits(x))
        nblk = (N + 127) // 128
        a8, asc, b8, bsc = bufs.new(x.size), bufs.new(B * H * nblk * 4), bufs.new(x.size), bufs.new(B * H * nblk * 4)
        dev.sage_quant_static(dx, a8, asc, B, H, N, D, 128, BF16, smooth=False)
        dev.sage_quant(dx, b8, bsc, B, H, N, D, 128, BF16)
        assert np.array_equal(a8.copyout(np.int8, x.shape), b8.copyout(np.int8, x.shape))
        assert np.array_equal(asc.copyout(np.float32, (B, H, nblk)), bsc.copyout(np.float32, (B, H, nblk)))
        assert np.abs(a8.copyout(np.int8, x.shape)).max() == 127
