"""Pins the CPU oracle (oracle/) before anything is compared against it.

Sources of truth used here, none of which is the oracle's own formula retyped:
  - the reference's six SDPA vectors (tests/golden/sdpa_golden.json, from the
    reference's tests/attention_golden.rs; tolerance of tests/nn_attention.rs:20)
  - torch's CPU scaled_dot_product_attention and torch.bfloat16 casts (library)
  - float64 evaluation, exact integer arithmetic, and special cases with a
    known closed-form answer
"""
import json
import os

import numpy as np
import pytest

import oracle
from autorust_amd import synth

GOLDEN = os.path.join(os.path.dirname(__file__), "golden", "sdpa_golden.json")


def _golden_cases():
    with open(GOLDEN) as fh:
        return json.load(fh)["cases"]


def _as4d(c):
    """3-D inputs are [batch, n, d]: give them a head axis of one."""
    def arr(key):
        a = np.array(c[key], np.float32).reshape(c[key + "_shape"])
        return a[:, None] if a.ndim == 3 else a
    q, k, v = arr("q"), arr("k"), arr("v")
    mask = None
    if c["mask_shape"]:
        m = np.array(c["mask"], np.float32).reshape(c["mask_shape"])
        if c["mask_bool"]:
            m = np.where(m != 0, np.float32(0), np.float32(-np.inf))
        mask = m[:, None] if (m.ndim == 3 and len(c["q_shape"]) == 3) else m
    want = np.array(c["out"], np.float32).reshape(c["out_shape"])
    want = want[:, None] if want.ndim == 3 else want
    return q, k, v, mask, want


def _close_ref(got, want, rtol=1e-5):
    # tests/nn_attention.rs:11-24
    return np.all(np.abs(got - want) <= rtol * np.maximum(np.abs(want), 1.0))


@pytest.mark.parametrize("case", _golden_cases(), ids=lambda c: c["name"])
@pytest.mark.parametrize("fn", ["sdpa_f32", "sdpa_f64", "flash_f32"])
def test_reference_golden_vectors(case, fn):
    q, k, v, mask, want = _as4d(case)
    got = getattr(oracle, fn)(q, k, v, mask=mask, causal=case["is_causal"])
    assert got.shape == want.shape
    assert _close_ref(got, want), (case["name"], fn, np.abs(got - want).max())


@pytest.mark.parametrize("causal,use_mask,hkv", [(False, False, 4), (True, False, 4), (False, True, 4),
                                                 (False, False, 2), (True, False, 1)])
def test_against_torch_cpu_sdpa(causal, use_mask, hkv):
    torch = pytest.importorskip("torch")
    B, Hq, N, D = 2, 4, 37, 64
    q, k, v = synth.normal(11, (B, Hq, N, D)), synth.normal(12, (B, hkv, N, D)), synth.normal(13, (B, hkv, N, D))
    mask = (synth.normal(14, (N, N)) * 2).astype(np.float32) if use_mask else None
    rep = Hq // hkv
    tq, tk, tv = (torch.from_numpy(x).double() for x in (q, np.repeat(k, rep, 1), np.repeat(v, rep, 1)))
    tm = None if mask is None else torch.from_numpy(mask).double()
    want = torch.nn.functional.scaled_dot_product_attention(tq, tk, tv, attn_mask=tm, is_causal=causal).numpy()
    for fn, tol in (("sdpa_f64", 2e-7), ("sdpa_f32", 1e-5), ("flash_f32", 1e-5)):
        got = getattr(oracle, fn)(q, k, v, mask=mask, causal=causal)
        err = np.abs(got - want) / np.maximum(np.abs(want), 1.0)
        assert err.max() <= tol, (fn, err.max())


def test_kv_len_is_a_key_padding_mask():
    # keys >= kv_len[b] excluded == attention over the truncated K/V (closed form)
    B, H, N, D = 2, 2, 50, 64
    q, k, v = synth.normal(1, (B, H, N, D)), synth.normal(2, (B, H, N, D)), synth.normal(3, (B, H, N, D))
    kv = np.array([17, 50], np.int32)
    for fn in ("sdpa_f32", "sdpa_f64", "flash_f32", "attn_bf16"):
        got = getattr(oracle, fn)(q, k, v, kv_len=kv)
        for b in range(B):
            L = kv[b]
            # truncated problem: same queries, first L keys; take matching rows
            kt, vt = np.zeros_like(k[b:b + 1]), np.zeros_like(v[b:b + 1])
            sub = getattr(oracle, fn)(np.ascontiguousarray(q[b:b + 1, :, :L]), np.ascontiguousarray(k[b:b + 1, :, :L]),
                                      np.ascontiguousarray(v[b:b + 1, :, :L]))
            assert np.abs(got[b, :, :L] - sub[0]).max() <= (1e-2 if fn == "attn_bf16" else 2e-6), fn


def test_rows_subset_matches_full():
    B, H, N, D = 1, 2, 70, 64
    q, k, v = synth.normal(4, (B, H, N, D)), synth.normal(5, (B, H, N, D)), synth.normal(6, (B, H, N, D))
    rows = np.array([0, 3, 69, 31], np.int32)
    for fn in ("sdpa_f32", "sdpa_f64", "flash_f32", "attn_bf16"):
        full = getattr(oracle, fn)(q, k, v, causal=True)
        part = getattr(oracle, fn)(q, k, v, causal=True, rows=rows)
        assert np.array_equal(part, full[:, :, rows]), fn


def test_flash_sentinel_semantics():
    """A row whose visited keys are all masked with the finite sentinel averages the
    visited V rows (src/runtime/cuda_flash.rs:105-125); an additive -inf mask on every
    key gives l == 0 and therefore zeros (cuda_flash.rs:138)."""
    N, D = 40, 64
    q, k, v = synth.normal(7, (1, 1, N, D)), synth.normal(8, (1, 1, N, D)), synth.normal(9, (1, 1, N, D))
    mask = np.zeros((N, N), np.float32)
    mask[5, :] = -np.inf
    got = oracle.flash_f32(q, k, v, mask=mask)
    assert np.array_equal(got[0, 0, 5], np.zeros(D, np.float32))
    ok = oracle.sdpa_f64(q, k, v)
    assert np.abs(np.delete(got, 5, 2) - np.delete(ok, 5, 2)).max() < 1e-5
    # a constant finite mask on every key of a row == plain softmax of that row (shift invariance)
    mask2 = np.zeros((N, N), np.float32)
    mask2[7, :] = -32.0
    got2 = oracle.flash_f32(q, k, v, mask=mask2)
    assert np.abs(got2 - ok).max() < 1e-4


def test_bf16_rounding_matches_torch():
    torch = pytest.importorskip("torch")
    x = np.concatenate([synth.normal(21, (4096,)) * 100, synth.normal(22, (4096,)) * 1e-3,
                        np.array([0.0, -0.0, 1.0, 1.00390625, 1.01171875, 3.3895314e38, np.inf, -np.inf], np.float32)])
    want = torch.from_numpy(x).to(torch.bfloat16).to(torch.float32).numpy()
    assert np.array_equal(oracle.bf16_round(x), want)
    assert np.array_equal(oracle.bf16_from_bits(oracle.bf16_bits(x)), want)
    assert np.array_equal(synth.to_bf16_bits(x), oracle.bf16_bits(x))
    assert np.array_equal(synth.from_bf16_bits(synth.to_bf16_bits(x)), want)
    # ties go to even: 1 + 2^-8 is halfway between 1 and 1 + 2^-7
    assert oracle.bf16_round(np.array([1.00390625], np.float32))[0] == 1.0
    assert oracle.bf16_round(np.array([1.01171875], np.float32))[0] == np.float32(1.015625)


@pytest.mark.parametrize("causal,use_mask,hkv", [(False, False, 2), (True, False, 2), (True, True, 1)])
def test_bf16_reference_against_torch_casts(causal, use_mask, hkv):
    """Rounding points of the bf16-emulating reference (tests/flash_cuda_masks.rs:41-104),
    re-derived with torch tensor ops and torch's own bf16 casts."""
    torch = pytest.importorskip("torch")
    B, Hq, N, D = 1, 2, 45, 64
    q, k, v = synth.normal(31, (B, Hq, N, D)), synth.normal(32, (B, hkv, N, D)), synth.normal(33, (B, hkv, N, D))
    mask = (synth.normal(34, (N, N))).astype(np.float32) if use_mask else None
    bf = lambda t: t.to(torch.bfloat16).to(torch.float32)
    rep = Hq // hkv
    tq = bf(torch.from_numpy(q))
    tk = bf(torch.from_numpy(np.repeat(k, rep, 1)))
    tv = bf(torch.from_numpy(np.repeat(v, rep, 1)))
    s = (tq.double() @ tk.double().transpose(-1, -2)).float() * np.float32(1.0 / np.sqrt(np.float32(D)))
    if mask is not None:
        s = s + torch.from_numpy(mask)
    if causal:
        s = s.masked_fill(torch.ones(N, N, dtype=torch.bool).triu(1), float("-inf"))
    p = torch.exp(s - s.max(-1, keepdim=True).values)
    want = bf((bf(p).double() @ tv.double()).float() / p.sum(-1, keepdim=True)).numpy()
    got = oracle.attn_bf16(q, k, v, mask=mask, causal=causal)
    # one bf16 ulp of slack for fp32 summation-order differences that land on a rounding boundary
    assert np.abs(got - want).max() <= 2.0 ** -7 * np.abs(want).max()
    assert np.mean(got != want) < 0.02


def test_quantiser_known_values():
    """Closed-form cases of the rule of src/runtime/cuda_flash_sage.rs:124-137,209-222."""
    D = 64
    x = np.zeros((1, 1, 3, D), np.float32)
    # row 0: absmax 127 -> scale exactly 1 -> q = rint(x), ties to even, clamp at +-127
    x[0, 0, 0, :8] = [127.0, -127.0, 0.5, 1.5, 2.5, -0.5, -1.5, 63.49]
    # row 1: all zero -> scale 1 (guard), q 0
    # row 2: absmax 2.54 -> scale 0.02 -> 1.27 -> 63.5 -> 64 (tie to even) or 63 depending on fp32 rounding
    x[0, 0, 2, :3] = [2.54, -2.54, 1.27]
    q, s = oracle.quant_blocks(x, 1)
    assert s[0, 0, 0] == 1.0 and s[0, 0, 1] == 1.0
    assert q[0, 0, 0, :8].tolist() == [127, -127, 0, 2, 2, 0, -2, 63]
    assert not q[0, 0, 1].any()
    assert q[0, 0, 2, 0] == 127 and q[0, 0, 2, 1] == -127
    sc = np.float32(2.54) / np.float32(127.0)
    assert s[0, 0, 2] == sc
    assert q[0, 0, 2, 2] == int(np.rint(np.float32(1.27) * (np.float32(1.0) / sc)))


def test_quantiser_block_reduces_to_row_rule_and_max():
    B, H, N, D = 1, 2, 200, 64
    x = synth.normal(41, (B, H, N, D)) * 3
    q1, s1 = oracle.quant_blocks(x, 1)
    # per-row rule evaluated independently with numpy float32 scalars
    mx = np.abs(x).max(-1)
    sc = np.where(mx > 0, mx / np.float32(127.0), np.float32(1.0)).astype(np.float32)
    inv = (np.float32(1.0) / sc).astype(np.float32)
    want = np.clip(np.rint((x * inv[..., None]).astype(np.float32)), -127, 127).astype(np.int8)
    assert np.array_equal(s1, sc) and np.array_equal(q1, want)
    # block scale == max of the row scales' absmax / 127 (max is order independent), ragged tail block
    for blk in (64, 128):
        qb, sb = oracle.quant_blocks(x, blk)
        nb = (N + blk - 1) // blk
        assert sb.shape == (B, H, nb)
        for b in range(nb):
            m = mx[:, :, b * blk:(b + 1) * blk].max(-1)
            assert np.array_equal(sb[:, :, b], (m / np.float32(127.0)).astype(np.float32))
        assert np.abs(qb.astype(np.int32)).max() == 127
    # the two rounding variants inside the reference (kernel: x*(1/s); its test: x/s) differ by at most one step
    qd, _ = oracle.quant_blocks(x, 1, use_div=True)
    assert np.abs(qd.astype(np.int32) - q1.astype(np.int32)).max() <= 1


def test_int32_logits_known_answer():
    # tests/sage_layout_probe.rs:73-84: A[16x32] = (i*7)%19 - 9, B[32x8] = (i*5)%13 - 6, C brute force
    a = [((i * 7) % 19) - 9 for i in range(512)]
    b = [((i * 5) % 13) - 6 for i in range(256)]
    want = [[sum(a[i * 32 + t] * b[t * 8 + j] for t in range(32)) for j in range(8)] for i in range(16)]
    A = np.array(a, np.int8).reshape(16, 32)
    Bt = np.ascontiguousarray(np.array(b, np.int8).reshape(32, 8).T)  # keys as rows
    got = oracle.logits_i32(A, Bt, 0, 16, 0, 8)
    assert got.tolist() == want
    # extreme values do not overflow: 128 * 127 * 127
    q8 = np.full((4, 128), 127, np.int8)
    k8 = np.full((4, 128), -127, np.int8)
    assert (oracle.logits_i32(q8, k8, 0, 4, 0, 4) == -128 * 127 * 127).all()


def test_k_mean_order_and_value():
    """K smoothing is not in the reference (parity unpinned there): the mean is pinned by
    its value (float64 mean within fp32 rounding) and by its defined summation order."""
    B, H, N, D = 1, 2, 333, 64
    k = synth.normal(51, (B, H, N, D)) + 3 * synth.normal(52, (1, H, 1, D))
    got = oracle.k_mean(k)
    assert np.abs(got - k.astype(np.float64).mean(2)).max() < 5e-6
    # the defined order, spelled out with numpy float32 adds
    want = np.zeros((B, H, D), np.float32)
    for c0 in range(0, N, 64):
        part = np.zeros((B, H, D), np.float32)
        for j in range(c0, min(N, c0 + 64)):
            part = part + k[:, :, j]
        want = want + part
    want = want / np.float32(N)
    assert np.array_equal(got, want)


def test_sage_reference_properties():
    B, H, N, D = 1, 2, 256, 64
    q = synth.normal(61, (B, H, N, D))
    k = synth.normal(62, (B, H, N, D)) + 3 * synth.normal(64, (1, H, 1, D))
    v = synth.normal(63, (B, H, N, D))
    truth = oracle.sdpa_f64(q, k, v)
    q8, sq = oracle.quant_blocks(q, 128)
    # without smoothing the channel bias eats the int8 range
    k8n, skn = oracle.quant_blocks(k, 64)
    err_plain = np.abs(oracle.sage(q8, k8n, sq, skn, v, 128, 64) - truth).max()
    # with smoothing: softmax(q.(k - mu)) == softmax(q.k) exactly, and the quantisation error drops
    mu = oracle.k_mean(k)
    k8s, sks = oracle.quant_blocks(k, 64, sub=mu)
    err_smooth = np.abs(oracle.sage(q8, k8s, sq, sks, v, 128, 64) - truth).max()
    assert err_smooth < 2e-2
    assert err_smooth < err_plain
    # block size 1 == the reference's per-row/per-key kernel; its own test bound is 2e-3
    # against its emulation (tests/sage_int8.rs:148); against the truth int8 costs ~1e-2
    q81, sq1 = oracle.quant_blocks(q, 1)
    k81, sk1 = oracle.quant_blocks(k, 1, sub=mu)
    err_row = np.abs(oracle.sage(q81, k81, sq1, sk1, v, 1, 1) - truth).max()
    assert err_row < 2e-2
    # dequantised logits reproduce q.k up to quantisation error
    lg = oracle.logits_i32(q81[0, 0], k81[0, 0], 0, N, 0, N).astype(np.float64)
    approx = lg * sq1[0, 0][:, None] * sk1[0, 0][None, :]
    exact = q[0, 0].astype(np.float64) @ (k[0, 0] - mu[0, 0]).astype(np.float64).T
    assert np.abs(approx - exact).max() < 0.5


def _sage_inputs(seed, B, Hq, Hkv, N, D, bq, bk):
    q = synth.normal(seed, (B, Hq, N, D))
    k = synth.normal(seed + 1, (B, Hkv, N, D)) + 3 * synth.normal(seed + 3, (1, Hkv, 1, D))
    v = synth.normal(seed + 2, (B, Hkv, N, D))
    q8, sq = oracle.quant_blocks(q, bq)
    k8, sk = oracle.quant_blocks(k, bk, sub=oracle.k_mean(k))
    return q8, k8, sq, sk, v


@pytest.mark.parametrize("bq,bk", [(1, 1), (128, 64), (32, 16)])
@pytest.mark.parametrize("causal,use_mask,kv_len,hkv", [
    (False, False, None, 2), (True, False, None, 2), (False, True, None, 2), (False, False, 100, 2),
    (True, True, 77, 1), (True, False, 131, 4)])
def test_sage_reference_against_torch_ops(bq, bk, causal, use_mask, kv_len, hkv):
    """Every branch and rounding point of the quantised-attention emulation
    (tests/sage_int8.rs:33-76, src/runtime/cuda_flash_sage.rs:315-340), re-derived with torch
    tensor ops: integer matmul, the dequantisation factor in the kernel's order, additive mask,
    causal triangle, key length, fp32 softmax numerator, bf16 P and V, division by the sum of the
    unrounded probabilities."""
    torch = pytest.importorskip("torch")
    B, Hq, N, D = 1, 4, 150, 64
    q8, k8, sq, sk, v = _sage_inputs(91, B, Hq, hkv, N, D, bq, bk)
    mask = synth.normal(95, (N, N)).astype(np.float32) if use_mask else None
    scale = np.float32(1.0) / np.sqrt(np.float32(D))
    rep = Hq // hkv
    bf = lambda t: t.to(torch.bfloat16).to(torch.float32)
    tq = torch.from_numpy(q8).to(torch.int64)
    tk = torch.from_numpy(np.repeat(k8, rep, 1)).to(torch.int64)
    acc = tq @ tk.transpose(-1, -2)                                   # exact integers
    fq = torch.from_numpy(np.repeat(sq, bq, -1)[..., :N])             # scale of row i: sq[i // bq]
    fk = torch.from_numpy(np.repeat(np.repeat(sk, rep, 1), bk, -1)[..., :N])
    a = (fq[..., :, None] * fk[..., None, :]) * torch.tensor(scale)   # (sq * sk) * scale, fp32
    s = acc.to(torch.float32) * a
    if mask is not None:
        s = s + torch.from_numpy(mask)
    dead = torch.zeros(N, N, dtype=torch.bool)
    if causal:
        dead |= torch.ones(N, N, dtype=torch.bool).triu(1)
    if kv_len is not None:
        dead[:, kv_len:] = True
    s = s.masked_fill(dead, float("-inf"))
    p = torch.exp(s - s.max(-1, keepdim=True).values)
    tv = bf(torch.from_numpy(np.repeat(v, rep, 1)))
    want = ((bf(p).double() @ tv.double()).float() / p.sum(-1, keepdim=True)).numpy()
    kl = None if kv_len is None else np.array([kv_len], np.int32)
    got = oracle.sage(q8, k8, sq, sk, v, bq, bk, mask=mask, causal=causal, kv_len=kl)
    # fp32 output: only summation order and libm-vs-torch exp differ (a dropped bf16 rounding of P
    # or V moves the result by ~1e-3, a wrong mask edge by O(0.1))
    assert np.abs(got - want).max() <= 2e-5 * max(1.0, np.abs(want).max())
    got_b = oracle.sage(q8, k8, sq, sk, v, bq, bk, mask=mask, causal=causal, kv_len=kl, round_out=True)
    assert np.array_equal(got_b, oracle.bf16_round(got))


def test_sage_reference_closed_forms():
    B, Hq, Hkv, N, D, bq, bk = 1, 2, 2, 96, 64, 32, 16
    q8, k8, sq, sk, v = _sage_inputs(101, B, Hq, Hkv, N, D, bq, bk)
    full = oracle.sage(q8, k8, sq, sk, v, bq, bk, causal=True)
    # a key length is the truncated problem (L a multiple of both block sizes keeps the scale
    # indices aligned); rows at or past L still attend to keys < L only
    L = 64
    cut = oracle.sage(q8[:, :, :L], k8[:, :, :L], sq[:, :, :L // bq], sk[:, :, :L // bk], v[:, :, :L], bq, bk)
    got = oracle.sage(q8, k8, sq, sk, v, bq, bk, kv_len=np.array([L], np.int32))
    assert np.array_equal(got[:, :, :L], cut)
    # a row subset is the same rows of the full result
    rows = np.array([0, 1, 31, 32, 63, 95], np.int32)
    assert np.array_equal(oracle.sage(q8, k8, sq, sk, v, bq, bk, causal=True, rows=rows), full[:, :, rows])
    # causal row 0 sees key 0 only: the output is bf16(v[0]) whatever the logits are
    assert np.array_equal(full[:, :, 0], oracle.bf16_round(v[:, :, 0]))
    # a mask of -inf above the diagonal is the causal flag
    tri = np.where(np.triu(np.ones((N, N), bool), 1), -np.inf, 0).astype(np.float32)
    assert np.array_equal(oracle.sage(q8, k8, sq, sk, v, bq, bk, mask=tri), full)
    # a constant added to every logit of a row cancels (up to fp32 rounding of s + c)
    shifted = oracle.sage(q8, k8, sq, sk, v, bq, bk, causal=True, mask=np.full((N, N), 0.5, np.float32))
    assert np.abs(shifted - full).max() < 1e-4


def test_cpu_baseline_matches_oracle():
    B, H, N, D = 1, 3, 197, 64
    q, k, v = synth.normal(71, (B, H, N, D)), synth.normal(72, (B, H, N, D)), synth.normal(73, (B, H, N, D))
    for causal in (False, True):
        out, threads = oracle.cpu_sdpa(q, k, v, causal=causal)
        want = oracle.sdpa_f64(q, k, v, causal=causal)
        assert threads >= 1
        assert (np.abs(out - want) / np.maximum(np.abs(want), 1)).max() <= 1e-5


def test_log_sum_exp_against_scipy():
    import scipy.special as sp
    B, Hq, Hkv, N, D = 1, 4, 2, 45, 64
    q, k = synth.normal(81, (B, Hq, N, D)), synth.normal(82, (B, Hkv, N, D))
    s = np.einsum("bhid,bhjd->bhij", q.astype(np.float64), np.repeat(k, 2, 1).astype(np.float64)) / np.sqrt(D)
    s = np.where(np.tril(np.ones((N, N), bool)), s, -np.inf)
    s[:, :, :, 30:] = -np.inf                      # kv_len = 30
    want = sp.logsumexp(s, axis=-1)
    got = oracle.lse_f64(q, k, causal=True, kv_len=np.array([30], np.int32))
    assert np.abs(got - want).max() < 1e-5


def _train_data(n, seed):
    """The generator of the reference's training test (tests/flash_train_cuda.rs:18-22)."""
    return (np.sin(np.arange(n, dtype=np.float32) * np.float32(0.0137) + np.float32(seed)) * np.float32(0.6)).astype(np.float32)


TRAIN_CASES = [  # tests/flash_train_cuda.rs:108-123: b, h, hk, n, causal, with_mask
    (2, 4, 4, 37, False, False), (1, 2, 2, 197, False, False), (2, 4, 4, 37, True, False),
    (2, 4, 4, 37, False, True), (2, 4, 2, 37, False, False), (2, 4, 2, 37, True, False), (2, 4, 1, 37, False, True),
]


@pytest.mark.parametrize("case", TRAIN_CASES, ids=str)
def test_backward_reference_against_torch_autograd(case):
    """The reference checks its fused backward against the autograd of its graph SDPA
    (tests/flash_train_cuda.rs:62-70: loss = sum(out * dO)); torch's autograd in float64 is the
    library stand-in for that here."""
    import torch
    b, h, hk, n, causal, with_mask = case
    d = 64
    q = _train_data(b * h * n * d, 0.0).reshape(b, h, n, d)
    k = _train_data(b * hk * n * d, 1.3).reshape(b, hk, n, d)
    v = _train_data(b * hk * n * d, 2.7).reshape(b, hk, n, d)
    do = _train_data(b * h * n * d, 4.1).reshape(b, h, n, d)
    mask = _train_data(n * n, 5.3).reshape(n, n) if with_mask else None
    o, lse, dq, dk, dv = oracle.attention_backward_f64(q, k, v, do, mask=mask, causal=causal, scale=0.125)

    tq, tk, tv = (torch.tensor(t, dtype=torch.float64, requires_grad=True) for t in (q, k, v))
    g = h // hk
    s = (tq @ tk.repeat_interleave(g, dim=1).transpose(-1, -2)) * 0.125
    if with_mask:
        s = s + torch.tensor(mask, dtype=torch.float64)
    if causal:
        s = s.masked_fill(torch.ones(n, n, dtype=torch.bool).triu(1), float("-inf"))
    out = torch.softmax(s, dim=-1) @ tv.repeat_interleave(g, dim=1)
    (out * torch.tensor(do, dtype=torch.float64)).sum().backward()
    assert np.abs(o - out.detach().numpy()).max() < 1e-6
    assert np.abs(lse - torch.logsumexp(s, dim=-1).detach().numpy()).max() < 1e-5
    for got, want in ((dq, tq.grad), (dk, tk.grad), (dv, tv.grad)):
        want = want.numpy()
        assert np.abs(got - want).max() <= 1e-6 * max(1.0, np.abs(want).max())


def test_backward_reference_closed_forms():
    """What the mathematics fixes: with one visible key p = 1, so dQ = 0, dK = 0 and dV_0 = sum of
    the dO rows; a key-length mask equals the truncated problem; gradients are linear in dO."""
    q, k, v, do = (synth.normal(s, (1, 2, 9, 64)) for s in (41, 42, 43, 44))
    o, lse, dq, dk, dv = oracle.attention_backward_f64(q, k, v, do, kv_len=np.array([1]))
    assert np.abs(dq).max() == 0 and np.abs(dk).max() == 0
    assert np.abs(dv[:, :, 0] - do.sum(axis=2)).max() < 1e-5 and np.abs(dv[:, :, 1:]).max() == 0
    full = oracle.attention_backward_f64(q, k, v, do, kv_len=np.array([5]), causal=True)
    # truncated problem, evaluated directly: rows i see keys j <= min(i, 4)
    qq, kk, vv, dd = (np.asarray(t, np.float64) for t in (q, k, v, do))
    for h in range(2):
        s = (qq[0, h] @ kk[0, h, :5].T) / 8.0
        s = np.where(np.arange(5)[None, :] > np.arange(9)[:, None], -np.inf, s)
        p = np.exp(s - s.max(axis=1, keepdims=True))
        p /= p.sum(axis=1, keepdims=True)
        oo = p @ vv[0, h, :5]
        ds = p * (dd[0, h] @ vv[0, h, :5].T - (oo * dd[0, h]).sum(axis=1, keepdims=True)) / 8.0
        assert np.abs(full[2][0, h] - ds @ kk[0, h, :5]).max() < 1e-5
        assert np.abs(full[3][0, h, :5] - ds.T @ qq[0, h]).max() < 1e-5 and np.abs(full[3][0, h, 5:]).max() == 0
        assert np.abs(full[4][0, h, :5] - p.T @ dd[0, h]).max() < 1e-5 and np.abs(full[4][0, h, 5:]).max() == 0
    a = oracle.attention_backward_f64(q, k, v, do)
    b2 = oracle.attention_backward_f64(q, k, v, 3.0 * do)
    for x, y in zip(a[2:], b2[2:]):
        assert np.abs(3.0 * x - y).max() < 1e-4


def test_fp8_e4m3_against_torch_and_closed_forms():
    """oracle.fp8_e4m3_bits against torch.float8_e4m3fn casts on every representable value, on the
    midpoints between neighbours (ties to even), on subnormals and on random data; saturation and
    the known code points by hand (OCP FP8 specification: 448 = 0x7e, 2^-9 = 0x01, 1.0 = 0x38)."""
    import torch
    codes = np.arange(256, dtype=np.uint8)
    vals = oracle.fp8_e4m3_value(codes)
    finite = ~np.isnan(vals)
    tv = torch.tensor(codes).view(torch.float8_e4m3fn).to(torch.float32).numpy()
    assert np.array_equal(vals[finite], tv[finite]) and np.isnan(tv[~finite]).all()
    assert np.array_equal(oracle.fp8_e4m3_bits(vals[finite]), codes[finite])
    pos = np.sort(vals[finite & (vals >= 0)])
    mids = ((pos[:-1].astype(np.float64) + pos[1:].astype(np.float64)) / 2).astype(np.float32)
    rnd = synth.normal(5, (4096,)) * np.float32(100.0)
    for x in (mids, -mids, np.nextafter(mids, np.float32(0)), np.nextafter(mids, np.float32(1e9)), rnd[np.abs(rnd) <= 448],
              synth.normal(6, (4096,)) * np.float32(0.01)):
        want = torch.tensor(x).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
        assert np.array_equal(oracle.fp8_e4m3_bits(x), want)
    assert oracle.fp8_e4m3_bits(np.float32([448, 460, 1e9, -1e9, 1.0, 2.0 ** -9, 2.0 ** -10, 0.0])).tolist() == \
        [0x7e, 0x7e, 0x7e, 0xfe, 0x38, 0x01, 0x00, 0x00]
    # the quantiser: the block maximum maps to +-448 exactly, a zero block gets scale 1
    x = synth.normal(7, (1, 2, 64, 64))
    x[0, 1] = 0
    c, sc = oracle.quant_blocks_fp8(x, 32)
    assert np.abs(oracle.fp8_e4m3_value(c[0, 0, :32])).max() == 448 and sc[0, 1].tolist() == [1.0, 1.0]
    assert np.abs(oracle.fp8_e4m3_value(c[0, 0]) * np.repeat(sc[0, 0], 32)[:, None] - x[0, 0]).max() <= np.abs(x[0, 0]).max() / 16


def _sage_fp8_inputs(seed, B, Hq, Hkv, N, D, bq, bk):
    q = synth.normal(seed, (B, Hq, N, D))
    k = synth.normal(seed + 1, (B, Hkv, N, D)) + 3 * synth.normal(seed + 3, (1, Hkv, 1, D))
    v = synth.normal(seed + 2, (B, Hkv, N, D))
    qc, sq = oracle.quant_blocks_fp8(q, bq)
    kc, sk = oracle.quant_blocks_fp8(k, bk, sub=oracle.k_mean(k))
    return qc, kc, sq, sk, v


@pytest.mark.parametrize("bq,bk", [(1, 1), (128, 64), (32, 16)])
@pytest.mark.parametrize("causal,use_mask,kv_len,hkv", [
    (False, False, None, 2), (True, False, None, 2), (False, True, None, 2), (False, False, 100, 2),
    (True, True, 77, 1), (True, False, 131, 4)])
def test_sage_fp8_reference_against_torch_ops(bq, bk, causal, use_mask, kv_len, hkv):
    """Every branch and rounding point of the FP8 attention emulation (the AR_FP8 branch of
    src/runtime/cuda_flash_sage.rs:92-147,280-412), re-derived with torch tensor ops: operands are
    torch's own float8_e4m3fn view of the codes (exact in float64, as are their products and sums),
    the dequantisation factor in the kernel's order, additive mask, causal triangle, key length,
    fp32 softmax numerator, bf16 P and V, division by the sum of the unrounded probabilities."""
    torch = pytest.importorskip("torch")
    B, Hq, N, D = 1, 4, 150, 64
    qc, kc, sq, sk, v = _sage_fp8_inputs(191, B, Hq, hkv, N, D, bq, bk)
    mask = synth.normal(195, (N, N)).astype(np.float32) if use_mask else None
    scale = np.float32(1.0) / np.sqrt(np.float32(D))
    rep = Hq // hkv
    bf = lambda t: t.to(torch.bfloat16).to(torch.float32)
    tq = torch.from_numpy(qc).view(torch.float8_e4m3fn).double()
    tk = torch.from_numpy(np.repeat(kc, rep, 1)).view(torch.float8_e4m3fn).double()
    acc = (tq @ tk.transpose(-1, -2)).float()                         # exact in float64, one rounding
    fq = torch.from_numpy(np.repeat(sq, bq, -1)[..., :N])             # scale of row i: sq[i // bq]
    fk = torch.from_numpy(np.repeat(np.repeat(sk, rep, 1), bk, -1)[..., :N])
    a = (fq[..., :, None] * fk[..., None, :]) * torch.tensor(scale)   # (sq * sk) * scale, fp32
    s = acc * a
    if mask is not None:
        s = s + torch.from_numpy(mask)
    dead = torch.zeros(N, N, dtype=torch.bool)
    if causal:
        dead |= torch.ones(N, N, dtype=torch.bool).triu(1)
    if kv_len is not None:
        dead[:, kv_len:] = True
    s = s.masked_fill(dead, float("-inf"))
    # the fp32 exponential correctly rounded (float64 exp of the fp32 argument, rounded once): a last-place
    # difference between two exp routines would flip bf16 roundings of P (2^-9 of a probability each)
    p = torch.exp((s - s.max(-1, keepdim=True).values).double()).float()
    tv = bf(torch.from_numpy(np.repeat(v, rep, 1)))
    want = ((bf(p).double() @ tv.double()).float() / p.sum(-1, keepdim=True)).numpy()
    kl = None if kv_len is None else np.array([kv_len], np.int32)
    got = oracle.sage_fp8(qc, kc, sq, sk, v, bq, bk, mask=mask, causal=causal, kv_len=kl)
    # only summation order and libm-vs-torch exp differ (a dropped bf16 rounding of P or V moves the
    # result by ~1e-3, a wrong mask edge or scale index by O(0.1))
    assert np.abs(got - want).max() <= 2e-5 * max(1.0, np.abs(want).max())
    got_b = oracle.sage_fp8(qc, kc, sq, sk, v, bq, bk, mask=mask, causal=causal, kv_len=kl, round_out=True)
    assert np.array_equal(got_b, oracle.bf16_round(got))


def test_sage_fp8_reference_closed_forms():
    B, Hq, Hkv, N, D, bq, bk = 1, 2, 2, 96, 64, 32, 16
    qc, kc, sq, sk, v = _sage_fp8_inputs(201, B, Hq, Hkv, N, D, bq, bk)
    full = oracle.sage_fp8(qc, kc, sq, sk, v, bq, bk, causal=True)
    # a key length is the truncated problem (L a multiple of both block sizes keeps the scale
    # indices aligned); rows at or past L still attend to keys < L only
    L = 64
    cut = oracle.sage_fp8(qc[:, :, :L], kc[:, :, :L], sq[:, :, :L // bq], sk[:, :, :L // bk], v[:, :, :L], bq, bk)
    got = oracle.sage_fp8(qc, kc, sq, sk, v, bq, bk, kv_len=np.array([L], np.int32))
    assert np.array_equal(got[:, :, :L], cut)
    # causal row 0 sees key 0 only: the output is bf16(v[0]) whatever the logits are
    assert np.array_equal(full[:, :, 0], oracle.bf16_round(v[:, :, 0]))
    # a mask of -inf above the diagonal is the causal flag
    tri = np.where(np.triu(np.ones((N, N), bool), 1), -np.inf, 0).astype(np.float32)
    assert np.array_equal(oracle.sage_fp8(qc, kc, sq, sk, v, bq, bk, mask=tri), full)
    # a constant added to every logit of a row cancels (up to fp32 rounding of s + c)
    shifted = oracle.sage_fp8(qc, kc, sq, sk, v, bq, bk, causal=True, mask=np.full((N, N), 0.5, np.float32))
    assert np.abs(shifted - full).max() < 1e-4
    # codes that are small integers: the FP8 emulation must agree with the (pinned) int8 emulation
    # on the same integers, scales and values
    ints = np.clip(np.rint(synth.normal(205, (B, Hq, N, D)) * 3), -8, 8).astype(np.int8)
    ints_k = np.clip(np.rint(synth.normal(206, (B, Hkv, N, D)) * 3), -8, 8).astype(np.int8)
    as_fp8 = lambda t: oracle.fp8_e4m3_bits(t.astype(np.float32))
    for kw in (dict(causal=True), dict(kv_len=np.array([50], np.int32)), dict(mask=synth.normal(207, (N, N)))):
        a = oracle.sage_fp8(as_fp8(ints), as_fp8(ints_k), sq, sk, v, bq, bk, **kw)
        b = oracle.sage(ints, ints_k, sq, sk, v, bq, bk, **kw)
        assert np.abs(a - b).max() <= 2e-6 * max(1.0, np.abs(b).max())


def test_quant_blocks_fp8_subtracts_the_mean_first():
    """quant_blocks_fp8(x, sub=mu) is quant_blocks_fp8(x - mu) with the subtraction done once in
    fp32 (K smoothing before the FP8 quantiser), and its scale is absmax / 448 of the shifted block
    (src/runtime/cuda_flash_sage.rs:9,209-222), checked with torch's cast."""
    torch = pytest.importorskip("torch")
    B, H, N, D, blk = 2, 3, 100, 64, 32
    x = synth.normal(211, (B, H, N, D)) + 3 * synth.normal(212, (1, H, 1, D))
    mu = oracle.k_mean(x)
    c1, s1 = oracle.quant_blocks_fp8(x, blk, sub=mu)
    shifted = (x - mu[:, :, None, :]).astype(np.float32)
    c2, s2 = oracle.quant_blocks_fp8(shifted, blk)
    assert np.array_equal(c1, c2) and np.array_equal(s1, s2)
    # the mean matters: without it the codes differ
    c3, _ = oracle.quant_blocks_fp8(x, blk)
    assert not np.array_equal(c1, c3)
    # independent evaluation of one ragged block (the last: rows 96..99) with torch
    seg = torch.from_numpy(shifted[1, 2, 96:])
    sc = seg.abs().max() / torch.tensor(np.float32(448.0))
    want = (seg * (torch.tensor(np.float32(1.0)) / sc)).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    assert np.array_equal(c1[1, 2, 96:], want) and s1[1, 2, 3] == sc.numpy()
