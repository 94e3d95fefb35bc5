"""FlashAttention forward on the GPU (through the C ABI) against the CPU oracle.

Mirrors the reference's kernel tests: tests/flash_cuda.rs (fp32 exact, < 2e-5),
tests/flash_cuda_bf16.rs (bf16 vs the bf16-emulating reference, < 5e-3, for
n in {1,7,8,31,32,33,63,64,65,100,224,789}) and tests/flash_cuda_masks.rs
(causal / additive mask / GQA, 2e-4 fp32 and 5e-3 bf16), at D = 64 as there and
at D = 128, plus the per-batch key lengths of the decoder configuration.
"""
import numpy as np
import pytest

import oracle
from autorust_amd import _lib, synth
from autorust_amd.device import BF16, F32, selections
from gpu_util import bf16_ulps, fill_qkv, ref_mask, run_flash

pytestmark = pytest.mark.gpu

N_LIST = [1, 7, 8, 31, 32, 33, 63, 64, 65, 100, 224, 789]  # tests/flash_cuda_bf16.rs:120
MASK_CASES = [  # tests/flash_cuda_masks.rs:237-244: label, b, hq, hkv, n, causal, has_mask
    ("causal", 1, 2, 2, 100, True, False),
    ("mask", 1, 2, 2, 64, False, True),
    ("causal+mask", 1, 2, 2, 100, True, True),
    ("gqa", 2, 4, 2, 64, False, False),
    ("gqa+causal", 2, 4, 2, 100, True, False),
    ("gqa+mask", 2, 4, 1, 64, False, True),
]


@pytest.mark.parametrize("D", [64, 128])
@pytest.mark.parametrize("N", N_LIST)
def test_bf16_matches_reference(dev, N, D):
    q, k, v = fill_qkv(1, 6, 6, N, D)
    before = selections(_lib.K_FLASH_BF16)
    got = run_flash(dev, q, k, v, BF16)
    assert selections(_lib.K_FLASH_BF16) == before + 1
    want = oracle.attn_bf16(q, k, v)
    assert np.abs(got - want).max() < 5e-3          # tests/flash_cuda_bf16.rs:131


@pytest.mark.parametrize("D", [64, 128])
@pytest.mark.parametrize("N", [1, 33, 64, 197, 789])
def test_f32_exact_matches_reference(dev, N, D):
    q, k, v = fill_qkv(1, 6, 6, N, D)               # tests/flash_cuda.rs: (1,6,789,64)
    got = run_flash(dev, q, k, v, F32)
    want = oracle.flash_f32(q, k, v)
    assert np.abs(got - want).max() < 2e-5          # tests/flash_cuda.rs:74
    truth = oracle.sdpa_f64(q, k, v)
    assert (np.abs(got - truth) / np.maximum(np.abs(truth), 1)).max() <= 1e-5


@pytest.mark.parametrize("D", [64, 128])
@pytest.mark.parametrize("case", MASK_CASES, ids=lambda c: c[0])
def test_causal_mask_gqa(dev, case, D):
    _, B, Hq, Hkv, N, causal, has_mask = case
    q, k, v = fill_qkv(B, Hq, Hkv, N, D)
    mask = ref_mask(N).reshape(N, N) if has_mask else None
    got = run_flash(dev, q, k, v, BF16, mask=mask, causal=causal)
    want = oracle.attn_bf16(q, k, v, mask=mask, causal=causal)
    assert np.abs(got - want).max() < 5e-3          # tests/flash_cuda_masks.rs:289 (bf16)
    got = run_flash(dev, q, k, v, F32, mask=mask, causal=causal)
    want = oracle.flash_f32(q, k, v, mask=mask, causal=causal)
    assert np.abs(got - want).max() < 2e-4          # tests/flash_cuda_masks.rs:289 (f32)


@pytest.mark.parametrize("D", [64, 128])
@pytest.mark.parametrize("dtype", [BF16, F32])
def test_random_inputs_causal_and_key_lengths(dev, dtype, D):
    B, Hq, Hkv, N = 3, 4, 2, 300
    q, k, v = synth.normal(101, (B, Hq, N, D)), synth.normal(102, (B, Hkv, N, D)), synth.normal(103, (B, Hkv, N, D))
    kv_len = np.array([150, 300, 1], np.int32)
    got = run_flash(dev, q, k, v, dtype, kv_len=kv_len, causal=True)
    truth = oracle.sdpa_f64(q, k, v, kv_len=kv_len, causal=True)
    if dtype == F32:
        assert (np.abs(got - truth) / np.maximum(np.abs(truth), 1)).max() <= 1e-5
    else:
        want = oracle.attn_bf16(q, k, v, kv_len=kv_len, causal=True)
        assert np.abs(got - want).max() < 1.6e-2     # two bf16 steps at |o| ~ 2..4
        assert np.abs(got - truth).max() <= 2e-2 * max(1.0, np.abs(truth).max())
    # non-causal with key lengths
    got = run_flash(dev, q, k, v, dtype, kv_len=kv_len)
    truth = oracle.sdpa_f64(q, k, v, kv_len=kv_len)
    tol = 1e-5 if dtype == F32 else 2e-2
    assert (np.abs(got - truth) / np.maximum(np.abs(truth), 1)).max() <= tol


def test_edge_cases(dev):
    D = 64
    q, k, v = synth.normal(111, (1, 2, 40, D)), synth.normal(112, (1, 2, 40, D)), synth.normal(113, (1, 2, 40, D))
    # kv_len == 0: no key contributes, l == 0, output is zero (acc * (l > 0 ? 1/l : 0))
    for dtype in (BF16, F32):
        got = run_flash(dev, q, k, v, dtype, kv_len=np.array([0], np.int32))
        assert not got.any()
    # a row masked with -inf everywhere yields zeros (not NaN), the others are untouched
    mask = np.zeros((40, 40), np.float32)
    mask[5, :] = -np.inf
    for dtype, tol in ((BF16, 2e-2), (F32, 1e-5)):
        got = run_flash(dev, q, k, v, dtype, mask=mask)
        assert not got[:, :, 5].any()
        truth = oracle.sdpa_f64(q, k, v)
        assert np.abs(np.delete(got, 5, 2) - np.delete(truth, 5, 2)).max() <= tol * 4
    # scale is a parameter
    got = run_flash(dev, q, k, v, F32, scale=0.3)
    truth = oracle.sdpa_f64(q, k, v, scale=0.3)
    assert np.abs(got - truth).max() < 1e-5


@pytest.mark.parametrize("N", [70, 333])
def test_f32_scale_signs_wide_logits_and_additive_mask(dev, N):
    """The fp32 kernel takes the row maximum before scaling on plain tiles, which only holds for a
    scale >= 0: negative and zero scales, logits tens of units wide, and an additive mask (with -inf
    entries) on top of the causal mask and key lengths all have to give the float64 result."""
    B, Hq, Hkv, D = 2, 4, 2, 64
    q, k, v = (synth.normal(s, (B, H, N, D)) for s, H in ((301, Hq), (302, Hkv), (303, Hkv)))
    for scale, tol in ((-0.125, 1e-5), (0.0, 1e-5), (-1.5, 5e-5), (3.0, 5e-5)):
        got = run_flash(dev, q, k, v, F32, scale=scale)
        truth = oracle.sdpa_f64(q, k, v, scale=scale)
        assert np.isfinite(got).all()
        assert (np.abs(got - truth) / np.maximum(np.abs(truth), 1)).max() <= tol, scale
    mask = (synth.normal(304, (N, N)) * np.float32(3.0)).astype(np.float32)
    mask[::7, 1::3] = -np.inf          # every row keeps visible keys (column 0 is never masked)
    kv_len = np.array([N, max(1, N // 2)], np.int32)
    for causal in (False, True):
        got = run_flash(dev, q, k, v, F32, mask=mask, kv_len=kv_len, causal=causal, scale=0.2)
        truth = oracle.sdpa_f64(q, k, v, mask=mask, kv_len=kv_len, causal=causal, scale=0.2)
        assert (np.abs(got - truth) / np.maximum(np.abs(truth), 1)).max() <= 1e-5, causal


@pytest.mark.parametrize("causal", [False, True])
def test_f32_tiling_variants_by_workgroup_count(dev, causal):
    """The fp32 kernel picks its tiling from the number of workgroups: 32 queries with the key tiles
    dealt out over four waves (few workgroups), over two waves (more than two and at most four
    workgroups per CU: B8 H12 S197 gives 672 on 256 CUs), or 128 queries per workgroup (many).  All
    are the same function."""
    D = 64
    for B, H, N in ((1, 12, 197), (8, 12, 197), (8, 24, 640)):
        q, k, v = (synth.normal(s, (B, H, N, D)) for s in (311, 312, 313))
        kv_len = np.full(B, N, np.int32)
        kv_len[-1] = N - 37
        got = run_flash(dev, q, k, v, F32, kv_len=kv_len, causal=causal)
        truth = oracle.sdpa_f64(q, k, v, kv_len=kv_len, causal=causal)
        assert (np.abs(got - truth) / np.maximum(np.abs(truth), 1)).max() <= 1e-5, (B, H, N)


def test_unsupported_shapes_are_declined_not_faked(dev):
    # head_dim 32: the dispatcher's cue to use the general path (flash_attention.rs:470-472)
    q = dev.alloc(4096)
    with pytest.raises(_lib.Unsupported):
        dev.flash_fwd(q, q, q, q, 1, 1, 1, 8, 32, BF16)
    with pytest.raises(_lib.ArhipError):
        dev.flash_fwd(q, q, q, q, 1, 3, 2, 8, 64, BF16)      # Hq % Hkv != 0
    with pytest.raises(_lib.ArhipError):
        dev.flash_fwd(q.ptr + 2, q, q, q, 1, 1, 1, 8, 64, BF16)  # misaligned
    q.free()


def test_bf16_is_deterministic(dev):
    # tests/flash_cuda_bf16.rs:181-268 asserts bit-identical outputs across launches
    q, k, v = synth.normal(121, (2, 6, 789, 64)), synth.normal(122, (2, 6, 789, 64)), synth.normal(123, (2, 6, 789, 64))
    a = run_flash(dev, q, k, v, BF16)
    b = run_flash(dev, q, k, v, BF16)
    assert np.array_equal(a, b)


@pytest.mark.parametrize("kind", ["bf16", "int8"])
@pytest.mark.parametrize("causal", [False, True])
def test_long_sequence_kernels_are_deterministic(dev, kind, causal):
    """Same assertion at a shape the software-pipelined kernels take (two waves per SIMD, so a
    result read one instruction too early shows up as a run-to-run difference)."""
    shape = (1, 32, 4096, 128)
    q, k, v = synth.normal(931, shape), synth.normal(932, shape), synth.normal(933, shape)
    if kind == "bf16":
        runs = [run_flash(dev, q, k, v, BF16, causal=causal) for _ in range(3)]
    else:
        from gpu_util import run_sage
        runs = [run_sage(dev, q, k, v, 128, 64, out_dtype=BF16, causal=causal)["out"] for _ in range(3)]
    assert np.array_equal(runs[0], runs[1]) and np.array_equal(runs[0], runs[2])


@pytest.mark.parametrize("dtype", [BF16, F32])
@pytest.mark.parametrize("D,N", [(64, 197), (128, 300), (128, 1100)])
def test_token_major_layout_is_the_same_function(dev, dtype, D, N):
    """Strided entry point: q/k/v as the projections produce them, [B, N, H, D], and the output
    written as [B, N, H*D] (what src/models/transformer.rs:286-299 reaches with two copies)
    must equal the dense [B, H, N, D] call bit for bit."""
    from gpu_util import Bufs
    B, Hq, Hkv = 2, 4, 2
    q, k, v = synth.normal(901, (B, Hq, N, D)), synth.normal(902, (B, Hkv, N, D)), synth.normal(903, (B, Hkv, N, D))
    dense = run_flash(dev, q, k, v, dtype, causal=True)
    conv = (lambda t: synth.to_bf16_bits(t)) if dtype == BF16 else (lambda t: t.astype(np.float32))
    es = 2 if dtype == BF16 else 4
    with Bufs(dev) as bufs:
        tq, tk, tv = (bufs.put(conv(np.ascontiguousarray(t.transpose(0, 2, 1, 3)))) for t in (q, k, v))
        to = bufs.new(q.size * es)
        dev.flash_fwd_strided(tq, tk, tv, to, (N * Hq * D, D, Hq * D), (N * Hkv * D, D, Hkv * D), (N * Hq * D, D, Hq * D),
                              B, Hq, Hkv, N, D, dtype, causal=True)
        raw = to.copyout(np.uint16 if dtype == BF16 else np.float32, (B, N, Hq, D))
    got = (synth.from_bf16_bits(raw) if dtype == BF16 else raw).transpose(0, 2, 1, 3)
    assert np.array_equal(got, dense)
    # and it is the right function, not merely the same one: against the oracle on the same inputs
    if dtype == BF16:
        assert bf16_ulps(got, oracle.attn_bf16(q, k, v, causal=True)) <= 3
    else:
        assert np.abs(got - oracle.flash_f32(q, k, v, causal=True)).max() < 2e-5
    # strides that would misalign rows are rejected
    with pytest.raises(_lib.ArhipError):
        d = dev.alloc(64)
        try:
            dev.flash_fwd_strided(d, d, d, d, (N * D, D, D + 4), (N * D, D, D), (N * D, D, D), 1, 1, 1, N, D, dtype)
        finally:
            d.free()


@pytest.mark.parametrize("dtype,tol", [(F32, 2e-5), (BF16, 2e-2)])
@pytest.mark.parametrize("D,N", [(64, 197), (128, 700)])
def test_log_sum_exp_output(dev, dtype, tol, D, N):
    """The statistic of the reference's training forward (LSE = m + log l,
    src/runtime/cuda_flash_train.rs:141) against the float64 log-sum-exp; the attention
    output itself must be unchanged by asking for it."""
    from gpu_util import Bufs
    B, Hq, Hkv = 2, 4, 2
    q, k, v = synth.normal(911, (B, Hq, N, D)), synth.normal(912, (B, Hkv, N, D)), synth.normal(913, (B, Hkv, N, D))
    kv_len = np.array([N, N // 3], np.int32)
    plain = run_flash(dev, q, k, v, dtype, kv_len=kv_len, causal=True)
    conv = (lambda t: synth.to_bf16_bits(t)) if dtype == BF16 else (lambda t: t.astype(np.float32))
    es = 2 if dtype == BF16 else 4
    with Bufs(dev) as bufs:
        dq, dk, dv = (bufs.put(conv(t)) for t in (q, k, v))
        do, dl, dk_len = bufs.new(q.size * es), bufs.new(B * Hq * N * 4), bufs.put(kv_len)
        dev.flash_fwd_lse(dq, dk, dv, do, dl, B, Hq, Hkv, N, D, dtype, kv_len=dk_len, causal=True)
        raw = do.copyout(np.uint16 if dtype == BF16 else np.float32, q.shape)
        lse = dl.copyout(np.float32, (B, Hq, N))
    got = synth.from_bf16_bits(raw) if dtype == BF16 else raw
    assert np.array_equal(got, plain)
    qq, kk = (oracle.bf16_round(q), oracle.bf16_round(k)) if dtype == BF16 else (q, k)
    want = oracle.lse_f64(qq, kk, kv_len=kv_len, causal=True)
    err = float(np.abs(lse - want).max())
    assert err <= tol


@pytest.mark.parametrize("causal", [False, True])
def test_token_major_layout_long_sequences(dev, causal):
    """The same through the software-pipelined kernel (enough workgroups of 256 queries to be
    chosen): [B, N, H, D] in, [B, N, H*D] out, with per-batch key lengths, against the oracle on
    sampled rows and bit for bit against the dense call."""
    from gpu_util import Bufs
    B, Hq, Hkv, N, D = 2, 16, 8, 4096 + 40, 128
    q, k, v = synth.normal(931, (B, Hq, N, D)), synth.normal(932, (B, Hkv, N, D)), synth.normal(933, (B, Hkv, N, D))
    kv_len = np.array([N, N - 1000], np.int32)
    dense = run_flash(dev, q, k, v, BF16, kv_len=kv_len, causal=causal)
    with Bufs(dev) as bufs:
        tq, tk, tv = (bufs.put(synth.to_bf16_bits(np.ascontiguousarray(t.transpose(0, 2, 1, 3)))) for t in (q, k, v))
        to = bufs.new(q.size * 2)
        dl = bufs.put(kv_len)
        dev.flash_fwd_strided(tq, tk, tv, to, (N * Hq * D, D, Hq * D), (N * Hkv * D, D, Hkv * D), (N * Hq * D, D, Hq * D),
                              B, Hq, Hkv, N, D, BF16, kv_len=dl, causal=causal)
        got = synth.from_bf16_bits(to.copyout(np.uint16, (B, N, Hq, D))).transpose(0, 2, 1, 3)
    assert np.array_equal(got, dense)
    rows = np.array([0, 1, 63, 64, 255, 256, 257, 2047, 3095, 3096, 4095, 4096, N - 1], np.int32)
    want = oracle.attn_bf16(q, k, v, kv_len=kv_len, causal=causal, rows=rows)
    assert bf16_ulps(got[:, :, rows], want) <= 3
    truth = oracle.sdpa_f64(q, k, v, kv_len=kv_len, causal=causal, rows=rows)
    assert np.abs(got[:, :, rows] - truth).max() <= 2e-2
