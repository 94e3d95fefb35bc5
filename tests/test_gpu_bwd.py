"""fp32 FlashAttention backward on the GPU (arhip_flash_bwd = ar_fl_prep + ar_fl_bwd_dq +
ar_fl_bwd_dkv, src/runtime/cuda_flash_train.rs:145-309) against the float64 oracle, on the
reference's own cases and tolerance (tests/flash_train_cuda.rs:84-123: max |diff| < 2e-3 for the
forward output and each gradient) and on N(0,1) data at a tighter relative bound."""
import numpy as np
import pytest

import oracle
from autorust_amd import synth
from autorust_amd.device import F32
from gpu_util import Bufs

pytestmark = pytest.mark.gpu


def _train_data(n, seed):
    return (np.sin(np.arange(n, dtype=np.float32) * np.float32(0.0137) + np.float32(seed)) * np.float32(0.6)).astype(np.float32)


def run_fwd_bwd(dev, q, k, v, do, mask=None, kv_len=None, causal=False, scale=None):
    B, Hq, N, D = q.shape
    Hkv = k.shape[1]
    with Bufs(dev) as bufs:
        dq_, dk_, dv_, ddo = bufs.put(q), bufs.put(k), bufs.put(v), bufs.put(do)
        o, lse = bufs.new(q.nbytes), bufs.new(B * Hq * N * 4)
        gq, gk, gv = bufs.new(q.nbytes, zero=False), bufs.new(k.nbytes, zero=False), bufs.new(v.nbytes, zero=False)
        delta = bufs.new(B * Hq * N * 4, zero=False)
        dm = bufs.put(np.ascontiguousarray(mask, np.float32)) if mask is not None else None
        dl = bufs.put(np.ascontiguousarray(kv_len, np.int32)) if kv_len is not None else None
        dev.flash_fwd_lse(dq_, dk_, dv_, o, lse, B, Hq, Hkv, N, D, F32, mask=dm, kv_len=dl, causal=causal, scale=scale)
        dev.flash_bwd(dq_, dk_, dv_, o, lse, ddo, gq, gk, gv, delta, B, Hq, Hkv, N, D, mask=dm, kv_len=dl,
                      causal=causal, scale=scale)
        return (o.copyout(np.float32, q.shape), lse.copyout(np.float32, (B, Hq, N)), gq.copyout(np.float32, q.shape),
                gk.copyout(np.float32, k.shape), gv.copyout(np.float32, v.shape))


CASES = [  # tests/flash_train_cuda.rs:108-123: b, h, hk, n, causal, with_mask
    (2, 4, 4, 37, False, False), (1, 2, 2, 197, False, False), (2, 4, 4, 37, True, False),
    (2, 4, 4, 37, False, True), (2, 4, 2, 37, False, False), (2, 4, 2, 37, True, False), (2, 4, 1, 37, False, True),
]


@pytest.mark.parametrize("case", CASES, ids=str)
def test_backward_on_the_reference_cases(dev, case):
    b, h, hk, n, causal, with_mask = case
    d = 64
    q = _train_data(b * h * n * d, 0.0).reshape(b, h, n, d)
    k = _train_data(b * hk * n * d, 1.3).reshape(b, hk, n, d)
    v = _train_data(b * hk * n * d, 2.7).reshape(b, hk, n, d)
    do = _train_data(b * h * n * d, 4.1).reshape(b, h, n, d)
    mask = _train_data(n * n, 5.3).reshape(n, n) if with_mask else None
    want = oracle.attention_backward_f64(q, k, v, do, mask=mask, causal=causal, scale=0.125)
    got = run_fwd_bwd(dev, q, k, v, do, mask=mask, causal=causal, scale=0.125)
    for name, g, w in zip(("o", "lse", "dq", "dk", "dv"), got, want):
        err = np.abs(g - w).max()
        assert err < 2e-3, (name, err)                       # the reference's bound
        assert err <= 2e-5 * max(1.0, np.abs(w).max()), (name, err)   # what fp32 arithmetic gives


@pytest.mark.parametrize("D", [64, 128])
@pytest.mark.parametrize("causal,use_len,hkv", [(False, False, 4), (True, False, 4), (True, True, 2), (False, True, 1)])
def test_backward_random_inputs(dev, D, causal, use_len, hkv):
    B, Hq, N = 2, 4, 333
    q, k, v, do = (synth.normal(s, (B, H, N, D)) for s, H in ((51, Hq), (52, hkv), (53, hkv), (54, Hq)))
    kv_len = np.array([N, 200], np.int32) if use_len else None
    want = oracle.attention_backward_f64(q, k, v, do, kv_len=kv_len, causal=causal)
    got = run_fwd_bwd(dev, q, k, v, do, kv_len=kv_len, causal=causal)
    for name, g, w in zip(("o", "lse", "dq", "dk", "dv"), got, want):
        err = np.abs(g - w).max()
        assert err <= 3e-5 * max(1.0, np.abs(w).max()), (name, err)


@pytest.mark.parametrize("causal", [False, True])
def test_backward_on_a_shape_that_fills_the_chip(dev, causal):
    """B * Hkv * ceil(N / 128) = 512 workgroups: the variant with 128 queries / keys per workgroup
    (shorter shapes deal the tiles of 32 queries / keys out between the four waves instead)."""
    B, Hq, Hkv, N, D = 16, 8, 8, 512, 64
    q, k, v, do = (synth.normal(s, (B, H, N, D)) for s, H in ((71, Hq), (72, Hkv), (73, Hkv), (74, Hq)))
    want = oracle.attention_backward_f64(q, k, v, do, causal=causal)
    got = run_fwd_bwd(dev, q, k, v, do, causal=causal)
    for name, g, w in zip(("o", "lse", "dq", "dk", "dv"), got, want):
        err = np.abs(g - w).max()
        assert err <= 3e-5 * max(1.0, np.abs(w).max()), (name, err)


def test_backward_is_deterministic_and_linear_in_dout(dev):
    B, Hq, Hkv, N, D = 1, 4, 2, 300, 64
    q, k, v, do = (synth.normal(s, (B, H, N, D)) for s, H in ((61, Hq), (62, Hkv), (63, Hkv), (64, Hq)))
    a = run_fwd_bwd(dev, q, k, v, do, causal=True)
    b = run_fwd_bwd(dev, q, k, v, do, causal=True)
    for x, y in zip(a, b):
        assert np.array_equal(x, y)            # no atomics: bit-identical across launches
    c = run_fwd_bwd(dev, q, k, v, np.float32(2.0) * do, causal=True)
    for x, y in zip(a[2:], c[2:]):
        assert np.array_equal(np.float32(2.0) * x, y)   # scaling dO by 2 is exact in binary arithmetic


def test_backward_rejects_what_it_does_not_cover(dev):
    from autorust_amd import _lib
    x = dev.alloc(64 * 4 * 64)
    with pytest.raises(_lib.ArhipError):
        dev.flash_bwd(x, x, x, x, x, x, x, x, x, x, 1, 1, 1, 8, 32)      # head_dim 32
    with pytest.raises(_lib.ArhipError):
        dev.flash_bwd(x, x, x, x, None, x, x, x, x, x, 1, 1, 1, 8, 64)   # no lse
    x.free()


@pytest.mark.parametrize("causal", [False, True])
def test_forward_and_backward_on_a_grid_of_many_workgroups(dev, causal):
    """Large grids (5120 workgroups in the query grids, 2560 in the dK/dV grid with two query heads per K/V head) in
    both orders the fp32 kernels use: head by head with every eighth of the grid (one XCD's share) a contiguous range
    of heads, and, under the causal mask, longest tile first over all heads.  Heads are independent, so a sample of
    them is checked against the float64 oracle on their own slices."""
    B, Hq, Hkv, N, D = 8, 80, 40, 1024, 64
    q, k, v, do = (synth.normal(s, (B, H, N, D)) for s, H in ((81, Hq), (82, Hkv), (83, Hkv), (84, Hq)))
    kv_len = np.array([N, 1000, 513, N, 77, N, 900, 1], np.int32)
    got = run_fwd_bwd(dev, q, k, v, do, kv_len=kv_len, causal=causal)
    for b, hk in ((0, 0), (1, 39), (2, 17), (4, 5), (7, 39), (7, 0)):
        sl = (slice(b, b + 1), slice(2 * hk, 2 * hk + 2))
        slk = (slice(b, b + 1), slice(hk, hk + 1))
        want = oracle.attention_backward_f64(q[sl], k[slk], v[slk], do[sl], kv_len=kv_len[b:b + 1], causal=causal)
        mine = (got[0][sl], got[1][sl], got[2][sl], got[3][slk], got[4][slk])
        for name, g, w in zip(("o", "lse", "dq", "dk", "dv"), mine, want):
            err = np.abs(g - w).max()
            assert err <= 3e-5 * max(1.0, np.abs(w).max()), (b, hk, name, err)
