"""Launch graphs: a recorded sequence of typed launches replays as one submission and gives,
on every replay, what the same calls give eagerly on the buffers' current contents.  Eager work
and synchronisations sit between the replays."""
import numpy as np
import pytest

from autorust_amd import _lib, synth
from autorust_amd.device import BF16, F32
from gpu_util import Bufs

pytestmark = pytest.mark.gpu


def _eager(dev, b, B, H, N, D):
    dev.flash_fwd(b["q"], b["k"], b["v"], b["o1"], B, H, H, N, D, BF16, causal=True, wait=False)
    dev.sage_quant(b["q"], b["q8"], b["sq"], B, H, N, D, 128, BF16, wait=False)
    dev.sage_quant(b["k"], b["k8"], b["sk"], B, H, N, D, 64, BF16, mean=b["mean"], workspace=b["ws"], smooth=True,
                   wait=False)
    dev.sage_fwd(b["q8"], b["k8"], b["sq"], b["sk"], b["v"], b["o2"], B, H, H, N, D, 128, 64, out_dtype=F32,
                 wait=False)


def test_graph_replay_matches_eager(dev):
    B, H, N, D = 2, 4, 640, 128
    n = B * H * N * D
    with Bufs(dev) as bufs:
        b = {k: bufs.new(n * 2) for k in ("q", "k", "v", "o1")}
        b.update(q8=bufs.new(n), k8=bufs.new(n), sq=bufs.new(B * H * 5 * 4), sk=bufs.new(B * H * 10 * 4),
                 mean=bufs.new(B * H * D * 4), ws=bufs.new(dev.sage_quant_workspace(B, H, N, D)), o2=bufs.new(n * 4))
        other = {k: bufs.new(n * 2) for k in ("q", "k", "v", "o1")}

        def fill(seed):
            for i, name in enumerate(("q", "k", "v")):
                b[name].copyin(synth.to_bf16_bits(synth.normal(seed + i, (B, H, N, D))))

        fill(10)
        dev.graph_begin()
        _eager(dev, b, B, H, N, D)
        graph = dev.graph_end()
        try:
            with pytest.raises(_lib.ArhipError):      # nothing ran during the capture; waiting calls are refused in one
                dev.graph_begin()
                try:
                    dev.flash_fwd(b["q"], b["k"], b["v"], b["o1"], B, H, H, N, D, BF16, wait=True)
                finally:
                    dev.graph_destroy(dev.graph_end())
            for rep, seed in enumerate((10, 20, 30, 20)):
                fill(seed)
                b["o1"].zero()
                b["o2"].zero()
                dev.graph_launch(graph)
                g1 = b["o1"].copyout(np.uint16, (n,))
                g2 = b["o2"].copyout(np.float32, (n,))
                gq8 = b["q8"].copyout(np.int8, (n,))
                # eager work on other buffers and a sync between the replays
                for name in ("q", "k", "v"):
                    other[name].copyin(synth.to_bf16_bits(synth.normal(99 + rep, (B, H, N, D))))
                dev.flash_fwd(other["q"], other["k"], other["v"], other["o1"], B, H, H, N, D, BF16)
                dev.sync()
                # the same calls, eagerly, on the same inputs
                b["o1"].zero()
                b["o2"].zero()
                _eager(dev, b, B, H, N, D)
                dev.sync()
                assert np.array_equal(g1, b["o1"].copyout(np.uint16, (n,))), rep
                assert np.array_equal(g2, b["o2"].copyout(np.float32, (n,))), rep
                assert np.array_equal(gq8, b["q8"].copyout(np.int8, (n,))), rep
                assert g1.any() and np.isfinite(g2).all()
        finally:
            dev.graph_destroy(graph)
