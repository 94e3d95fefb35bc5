"""Tensors whose batch and head strides put elements beyond 2^31 (and bytes beyond 2^32) from the base
pointer: the [B, H, N, D] indices of the reference's kernels are 32-bit inside a head and 64-bit for
the head's base (src/runtime/cuda_flash_bf16.rs:243-250); here the strides come from the caller, so
every base offset must be carried in 64 bits.  The heads are scattered through buffers of several GB
that are otherwise untouched, and the result must equal the dense call bit for bit."""
import ctypes

import numpy as np
import pytest

import oracle
from autorust_amd import synth
from autorust_amd.device import BF16, F32
from gpu_util import Bufs, run_flash, run_sage

pytestmark = pytest.mark.gpu

HEAD_STRIDE = (1 << 30) + (1 << 21) + 512     # elements; a head of these tests has at most 2^20
BATCH_STRIDE = 3 * HEAD_STRIDE + 4096          # three heads per batch entry at most


def _scatter(dev, buf, host, es):
    """host [B, H, N, D] -> buf at element offset b * BATCH_STRIDE + h * HEAD_STRIDE, rows dense."""
    B, H = host.shape[:2]
    assert H <= 3 and host[0, 0].size <= 1 << 20
    for b in range(B):
        for h in range(H):
            a = np.ascontiguousarray(host[b, h])
            off = (b * BATCH_STRIDE + h * HEAD_STRIDE) * es
            assert off + a.nbytes <= buf.nbytes
            rc = dev.lib.arhip_copyin(dev.handle, ctypes.c_void_p(buf.ptr + off), a.ctypes.data, a.nbytes)
            assert rc == 0


def _gather(dev, buf, shape, dtype):
    B, H, N, D = shape
    out = np.empty(shape, dtype)
    es = out.itemsize
    for b in range(B):
        for h in range(H):
            a = np.empty((N, D), dtype)
            off = (b * BATCH_STRIDE + h * HEAD_STRIDE) * es
            rc = dev.lib.arhip_copyout(dev.handle, a.ctypes.data, ctypes.c_void_p(buf.ptr + off), a.nbytes)
            assert rc == 0
            out[b, h] = a
    return out


def _extent(B, H, N, D, es):
    return ((B - 1) * BATCH_STRIDE + (H - 1) * HEAD_STRIDE + N * D) * es


@pytest.mark.parametrize("dtype,N,D,Hq,Hkv,causal", [
    (BF16, 300, 64, 3, 3, True),        # general kernel, one wave or four
    (BF16, 1100, 128, 3, 1, False),     # grouped heads
    (BF16, 8192, 128, 3, 3, True),      # enough 256-query workgroups for the pipelined kernel
    (F32, 300, 64, 3, 3, True),         # byte offsets beyond 2^34
])
def test_flash_heads_beyond_32_bit_offsets(dev, dtype, N, D, Hq, Hkv, causal):
    B = 2
    if dev.mem_info()[0] < 100 * (1 << 30):
        pytest.skip("needs ~90 GB of free device memory")
    q, k, v = synth.normal(41, (B, Hq, N, D)), synth.normal(42, (B, Hkv, N, D)), synth.normal(43, (B, Hkv, N, D))
    if dtype == BF16 and N >= 8192:
        # make sure this shape is one the pipelined kernel takes: 2 * B * Hq * N / 256 >= compute units
        assert 2 * B * Hq * ((N + 255) // 256) >= dev.compute_units
    dense = run_flash(dev, q, k, v, dtype, causal=causal)
    es = 2 if dtype == BF16 else 4
    conv = synth.to_bf16_bits if dtype == BF16 else (lambda t: t.astype(np.float32))
    with Bufs(dev) as bufs:
        tq, to = bufs.new(_extent(B, Hq, N, D, es), zero=False), bufs.new(_extent(B, Hq, N, D, es), zero=False)
        tk, tv = bufs.new(_extent(B, Hkv, N, D, es), zero=False), bufs.new(_extent(B, Hkv, N, D, es), zero=False)
        for buf, host in ((tq, q), (tk, k), (tv, v)):
            _scatter(dev, buf, conv(host), es)
        st = (BATCH_STRIDE, HEAD_STRIDE, D)
        dev.flash_fwd_strided(tq, tk, tv, to, st, st, st, B, Hq, Hkv, N, D, dtype, causal=causal)
        raw = _gather(dev, to, (B, Hq, N, D), np.uint16 if dtype == BF16 else np.float32)
    got = synth.from_bf16_bits(raw) if dtype == BF16 else raw
    assert np.array_equal(got, dense)
    rows = np.array([0, 1, N // 2, N - 1], np.int32)
    truth = oracle.sdpa_f64(q, k, v, causal=causal, rows=rows)
    assert np.abs(got[:, :, rows] - truth).max() <= (2e-2 if dtype == BF16 else 1e-5 * max(1.0, np.abs(truth).max()))


def test_sage_value_and_output_heads_beyond_32_bit_offsets(dev):
    """The quantised path takes strides for V and the output (Q and K are the quantiser's dense codes)."""
    B, H, N, D = 2, 3, 8192, 128
    if dev.mem_info()[0] < 40 * (1 << 30):
        pytest.skip("needs ~25 GB of free device memory")
    q, k, v = synth.normal(51, (B, H, N, D)), synth.normal(52, (B, H, N, D)), synth.normal(53, (B, H, N, D))
    dense = run_sage(dev, q, k, v, 128, 64, in_dtype=BF16, out_dtype=BF16)
    nqb, nkb = N // 128, N // 64
    with Bufs(dev) as bufs:
        q8, k8 = bufs.put(dense["q8"]), bufs.put(dense["k8"])
        sq, sk = bufs.put(dense["sq"]), bufs.put(dense["sk"])
        tv, to = bufs.new(_extent(B, H, N, D, 2), zero=False), bufs.new(_extent(B, H, N, D, 2), zero=False)
        _scatter(dev, tv, synth.to_bf16_bits(v), 2)
        st = (BATCH_STRIDE, HEAD_STRIDE, D)
        dev.sage_fwd(q8, k8, sq, sk, tv, to, B, H, H, N, D, 128, 64, out_dtype=BF16, v_strides=st, o_strides=st)
        got = synth.from_bf16_bits(_gather(dev, to, (B, H, N, D), np.uint16))
    assert sq.nbytes == B * H * nqb * 4 and sk.nbytes == B * H * nkb * 4
    assert np.array_equal(got, dense["out"])
