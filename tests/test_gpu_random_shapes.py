"""Seeded random sweep over shapes, head groupings, masks and tiling variants: every case is
compared with the float64 oracle.  The tiling variant does not change the function, so the
same case is also run with the tiling forced (the general kernel with 1 and 4 waves, the pipelined one with
8 and, "40", 4 waves): ARHIP_ATTN_WAVES is read
when a device is opened, so those runs open a device handle of their own."""
import contextlib

import numpy as np
import pytest

import oracle
from autorust_amd import synth
from autorust_amd.device import BF16, F32
from gpu_util import run_flash, run_sage

pytestmark = pytest.mark.gpu


@contextlib.contextmanager
def _device_with_waves(dev, waves, monkeypatch):
    """The session's device when nothing is forced, else a second handle opened under the override."""
    if waves is None:
        yield dev
        return
    from autorust_amd.device import Device
    monkeypatch.setenv("ARHIP_ATTN_WAVES", waves)
    forced = Device(0)
    try:
        yield forced
    finally:
        forced.close()


def _cases(seed, count):
    rng = np.random.default_rng(seed)
    out = []
    for _ in range(count):
        D = int(rng.choice([64, 128]))
        N = int(rng.choice([1, 2, 31, 32, 33, 63, 64, 65, 127, 128, 129, 191, 255, 256, 257, 300, 511, 640, 777]))
        Hkv = int(rng.choice([1, 2, 3]))
        group = int(rng.choice([1, 2, 4]))
        B = int(rng.choice([1, 2, 3]))
        causal = bool(rng.integers(0, 2))
        use_len = bool(rng.integers(0, 2))
        kv_len = rng.integers(0, N + 1, size=B).astype(np.int32) if use_len else None
        out.append((B, Hkv * group, Hkv, N, D, causal, kv_len, int(rng.integers(1, 1 << 30))))
    return out


@pytest.mark.parametrize("waves", [None, "1", "4", "8", "40"])
def test_flash_random_shapes(dev, waves, monkeypatch):
    with _device_with_waves(dev, waves, monkeypatch) as d:
        _flash_random_shapes(d)


def _flash_random_shapes(dev):
    worst = {BF16: 0.0, F32: 0.0}
    for (B, Hq, Hkv, N, D, causal, kv_len, seed) in _cases(1234, 24):
        q, k, v = (synth.normal(seed + i, s) for i, s in enumerate(((B, Hq, N, D), (B, Hkv, N, D), (B, Hkv, N, D))))
        truth = oracle.sdpa_f64(q, k, v, kv_len=kv_len, causal=causal)
        # rows without any visible key: the kernels give zeros where the general path gives NaN
        dead = ~np.isfinite(truth)
        truth = np.where(dead, 0.0, truth)
        for dtype, tol in ((BF16, 2e-2), (F32, 1e-5)):
            got = run_flash(dev, q, k, v, dtype, kv_len=kv_len, causal=causal)
            assert np.isfinite(got).all(), (B, Hq, Hkv, N, D, causal, kv_len)
            err = float((np.abs(got - truth) / np.maximum(np.abs(truth), 1.0)).max())
            worst[dtype] = max(worst[dtype], err)
            assert err <= tol, (B, Hq, Hkv, N, D, causal, None if kv_len is None else kv_len.tolist(), dtype, err)
    assert worst[F32] <= 1e-5 and worst[BF16] <= 2e-2


@pytest.mark.parametrize("waves", [None, "4", "8", "40"])
def test_sage_random_shapes(dev, waves, monkeypatch):
    with _device_with_waves(dev, waves, monkeypatch) as d:
        _sage_random_shapes(d)


def _sage_random_shapes(dev):
    for (B, Hq, Hkv, N, D, causal, kv_len, seed) in _cases(4321, 12):
        q, k, v = (synth.normal(seed + i, s) for i, s in enumerate(((B, Hq, N, D), (B, Hkv, N, D), (B, Hkv, N, D))))
        k = (k + np.float32(2.0) * synth.normal(seed + 9, (1, Hkv, 1, D))).astype(np.float32)
        for bq, bk in ((128, 64), (1, 1), (64, 128)):
            r = run_sage(dev, q, k, v, bq, bk, smooth=True, kv_len=kv_len, causal=causal)
            mu = oracle.k_mean(k)
            q8, sq = oracle.quant_blocks(q, bq)
            k8, sk = oracle.quant_blocks(k, bk, sub=mu)
            bits = (np.array_equal(r["q8"], q8), np.array_equal(r["k8"], k8), np.array_equal(r["sq"], sq),
                    np.array_equal(r["sk"], sk), np.array_equal(r["mean"], mu))
            assert all(bits), (B, Hq, Hkv, N, D, bq, bk, bits)
            want = oracle.sage(q8, k8, sq, sk, v, bq, bk, kv_len=kv_len, causal=causal)
            want = np.where(np.isfinite(want), want, 0.0)
            err = float(np.abs(r["out"] - want).max())
            # kernel and emulation round P to bf16 at different points (the running exponent reference
            # against the final maximum) and both sum the unrounded values: up to 2 * 2^-9 * max|v| where
            # a few keys carry a row (short key lengths, first causal rows); measured worst over other
            # seeds: 8e-3
            bound = 2.0 ** -8 * float(np.abs(v).max())
            assert np.isfinite(r["out"]).all() and err < bound, (B, Hq, Hkv, N, D, causal, bq, bk, err, bound)


@pytest.mark.parametrize("waves", [None, "8", "40"])
def test_in_kernel_q_quantiser_random_shapes(dev, waves, monkeypatch):
    """The attention entries that quantise their queries in the prologue (bf16 blocks of 128, int8 and FP8; f32 rows)
    on the random shapes, with the 8- and the 4-wave form forced: scales, codes and output bit for bit those of the
    quantiser launch followed by the plain entry."""
    from gpu_util import Bufs
    with _device_with_waves(dev, waves, monkeypatch) as d:
        for (B, Hq, Hkv, N, D, causal, kv_len, seed) in _cases(9876, 10):
            q, k, v = (synth.normal(seed + i, s) for i, s in enumerate(((B, Hq, N, D), (B, Hkv, N, D), (B, Hkv, N, D))))
            qb, kb = oracle.bf16_round(q), oracle.bf16_round(k)
            case = (B, Hq, Hkv, N, D, causal, None if kv_len is None else kv_len.tolist())
            # bf16 queries, blocks of 128: int8
            r = run_sage(d, qb, kb, v, 128, 64, smooth=True, in_dtype=BF16, out_dtype=BF16, kv_len=kv_len, causal=causal)
            # f32 queries, a scale per query and per key
            rr = run_sage(d, q, k, v, 1, 1, smooth=False, kv_len=kv_len, causal=causal)
            with Bufs(d) as bufs:
                dl = bufs.put(kv_len) if kv_len is not None else None
                dv = bufs.put(synth.to_bf16_bits(v))
                nqb = (N + 127) // 128
                dq = bufs.put(synth.to_bf16_bits(qb))
                k8, sk = bufs.put(r["k8"]), bufs.put(r["sk"])
                do, sq_out, q8_out = bufs.new(q.size * 2), bufs.new(B * Hq * nqb * 4), bufs.new(q.size)
                d.sage_fwd_qfused(dq, k8, sk, dv, do, B, Hq, Hkv, N, D, 64, out_dtype=BF16, sq_out=sq_out, q8_out=q8_out,
                                  kv_len=dl, causal=causal)
                assert np.array_equal(sq_out.copyout(np.float32, (B, Hq, nqb)), r["sq"]), case
                assert np.array_equal(q8_out.copyout(np.int8, q.shape), r["q8"]), case
                assert np.array_equal(synth.from_bf16_bits(do.copyout(np.uint16, q.shape)), r["out"]), case
                dqf = bufs.put(q)
                k8r, skr = bufs.put(rr["k8"]), bufs.put(rr["sk"])
                dor, sqr = bufs.new(q.size * 4), bufs.new(B * Hq * N * 4)
                d.sage_fwd_qfused_rows(dqf, k8r, skr, dv, dor, B, Hq, Hkv, N, D, 1, sq_out=sqr, kv_len=dl, causal=causal)
                assert np.array_equal(sqr.copyout(np.float32, (B, Hq, N)), rr["sq"]), case
                assert np.array_equal(dor.copyout(np.float32, q.shape), rr["out"]), case
