"""The C++ mirror of the reference's attention interface (csrc/host/): policy and gates on the
CPU, the Tensor / Session path on the GPU.  The GPU cases follow the reference's dispatch tests
(tests/flash_cuda_masks.rs:298-362, tests/flash_cuda_bf16.rs `bf16_gate_and_dispatch`,
tests/sage_int8.rs:152-250)."""
import os

import numpy as np
import pytest

import oracle
from autorust_amd import host, synth
from autorust_amd.host import (BFLOAT16, FLOAT32, K_FLASH_BF16, K_FLASH_F32, K_NONE, K_SAGE, OTHER, AttentionKind,
                               Session, Settings, Tensor)

# ------------------------------------------------------------------ CPU: policy and gates ---


def test_attention_kind_names_and_env(monkeypatch):
    assert [AttentionKind.name(k) for k in (0, 1, 2)] == ["sdpa", "flash", "sage"]   # flash_attention.rs:731-737
    assert AttentionKind.from_str("sdpa") == AttentionKind.Sdpa
    assert AttentionKind.from_str("sage") == AttentionKind.Sage
    assert AttentionKind.from_str("anything") == AttentionKind.Flash                 # default (settings.rs:209-213)
    monkeypatch.setenv("AUTORUST_ATTN", "sage")
    monkeypatch.setenv("AUTORUST_MATH", "exact")
    s = Settings.from_env()
    assert s.attention == AttentionKind.Sage and s.math_exact == 1 and s.tensor_cores == 0   # settings.rs:202-208
    monkeypatch.delenv("AUTORUST_MATH")
    monkeypatch.setenv("AUTORUST_TENSOR_CORES", "0")
    assert Settings.from_env().tensor_cores == 0
    d = Settings.default()
    assert d.attention == AttentionKind.Flash and d.tensor_cores == 1
    assert (d.sage_block_q, d.sage_block_k, d.sage_smooth_k) == (128, 64, 1)


def test_policy_matches_attention_kind():
    # tensor/mod.rs:2198-2207: fused iff kind != Sdpa and dropout_p == 0 and a session is given
    d = Settings.default()
    assert host.wants_fused(None, d, 0.0, True) == (True, False)
    assert host.wants_fused(None, d, 0.0, False) == (False, False)       # sessionless entry points always run SDPA
    assert host.wants_fused(None, d, 0.1, True) == (False, False)        # dropout
    assert host.wants_fused(AttentionKind.Sage, d, 0.0, True) == (True, True)
    s = Settings.default()
    s.attention = AttentionKind.Sdpa
    assert host.wants_fused(None, s, 0.0, True) == (False, False)        # configured sdpa
    assert host.wants_fused(AttentionKind.Flash, s, 0.0, True) == (True, False)   # explicit calls are never overridden


def test_gates_of_fused_attention_ex():
    q = [2, 4, 100, 64]
    assert host.plan_fused(q, q, q)[0] == K_FLASH_F32
    assert host.plan_fused(q, q, q, qd=BFLOAT16)[0] == K_FLASH_BF16
    assert host.plan_fused(q, q, q, quantized=True) == (K_SAGE, False)
    assert host.plan_fused([2, 4, 100, 128], [2, 4, 100, 128], [2, 4, 100, 128], qd=BFLOAT16)[0] == K_FLASH_BF16
    # flash_attention.rs:358-396
    assert host.plan_fused([4, 100, 64], [4, 100, 64], [4, 100, 64])[0] == K_NONE            # not 4-D
    assert host.plan_fused(q, [2, 4, 99, 64], [2, 4, 99, 64])[0] == K_NONE                   # nk != n
    assert host.plan_fused(q, q, [2, 4, 100, 32])[0] == K_NONE                               # dv != d
    assert host.plan_fused(q, [2, 2, 100, 64], [2, 2, 100, 64])[0] == K_NONE                 # GQA not announced
    assert host.plan_fused(q, [2, 2, 100, 64], [2, 2, 100, 64], enable_gqa=True)[0] == K_FLASH_F32
    assert host.plan_fused(q, [2, 3, 100, 64], [2, 3, 100, 64], enable_gqa=True)[0] == K_NONE  # 4 % 3
    assert host.plan_fused(q, q, q, qd=OTHER)[0] == K_NONE
    assert host.plan_fused(q, q, q, qd=FLOAT32, kd=BFLOAT16)[0] == K_NONE                    # mixed dtypes
    assert host.plan_fused(q, q, q, mask=[100, 100])[0] == K_FLASH_F32
    assert host.plan_fused(q, q, q, mask=[1, 100, 100])[0] == K_NONE                         # broadcast mask -> SDPA
    assert host.plan_fused(q, q, q, mask=[100, 100], mask_dtype=OTHER)[0] == K_NONE          # bool mask -> SDPA
    # head_dim the kernels do not cover (tests/flash_cuda_bf16.rs:144 analogue)
    assert host.plan_fused([1, 2, 64, 32], [1, 2, 64, 32], [1, 2, 64, 32], qd=BFLOAT16)[0] == K_NONE
    # tensor cores off: bf16 has no fused kernel, f32 keeps the exact one, sage is declined with a notice
    s = Settings.default()
    s.tensor_cores = 0
    assert host.plan_fused(q, q, q, qd=BFLOAT16, settings=s)[0] == K_NONE
    assert host.plan_fused(q, q, q, settings=s)[0] == K_FLASH_F32
    assert host.plan_fused(q, q, q, quantized=True, settings=s) == (K_FLASH_F32, True)


# ------------------------------------------------------------------ GPU: Tensor / Session ---

gpu = pytest.mark.gpu


@pytest.fixture(scope="module")
def hdev():
    d = host.HipDevice(0)
    yield d
    d.close()


def _fill(shape, seed):
    return synth.fill(int(np.prod(shape)), seed).reshape(shape)


@gpu
def test_dispatch_handles_mask_and_causal(hdev):
    """tests/flash_cuda_masks.rs:298-362: attention_with takes the fused kernel for causal + mask and GQA."""
    n, d = 100, 64
    sess = Session()
    for (b, hq, hkv, causal, has_mask) in [(1, 2, 2, True, True), (2, 4, 2, False, False), (2, 4, 1, True, False)]:
        q, k, v = _fill((b, hq, n, d), 3), _fill((b, hkv, n, d), 11), _fill((b, hkv, n, d), 19)
        mask = (((np.arange(n * n) * 7) % 23).astype(np.float32) - 11.0).reshape(n, n) * np.float32(0.05) if has_mask else None
        tq, tk, tv = (Tensor.from_slice(hdev, a, a.shape) for a in (q, k, v))
        tm = Tensor.from_slice(hdev, mask, mask.shape) if has_mask else None
        before = host.selections(K_FLASH_F32)
        out = tq.attention_with(tk, tv, tm, 0.0, causal, sess)
        assert host.selections(K_FLASH_F32) == before + 1
        assert out.shape == (b, hq, n, d) and out.dtype == FLOAT32
        want = oracle.sdpa_f64(q, k, v, mask=mask, causal=causal)
        err = float(np.abs(out.to_list() - want).max())
        assert err < 2e-4                                   # tests/flash_cuda_masks.rs:289


@gpu
def test_bf16_gate_and_dispatch(hdev):
    n, d = 197, 64
    q, k, v = _fill((1, 6, n, d), 3), _fill((1, 6, n, d), 11), _fill((1, 6, n, d), 19)
    tq, tk, tv = (Tensor.from_slice(hdev, a, a.shape, BFLOAT16) for a in (q, k, v))
    sess = Session()
    before = host.selections(K_FLASH_BF16)
    out = tq.flash_attention_with(tk, tv, None, 0.0, False, sess)
    assert host.selections(K_FLASH_BF16) == before + 1
    assert out.dtype == BFLOAT16                             # bf16 tensors give a bf16 result (flash_attention.rs:514-521)
    err = float(np.abs(out.to_list() - oracle.attn_bf16(q, k, v)).max())
    assert err < 5e-3
    # tensor cores off: the bf16 kernel is not selected and the caller is told to take SDPA
    s = Settings.default()
    s.tensor_cores = 0
    with pytest.raises(host.HostError, match="general SDPA path"):
        tq.flash_attention_with(tk, tv, None, 0.0, False, sess, s)


@gpu
def test_sage_attention_with_selects_the_quantised_kernel(hdev):
    """tests/sage_int8.rs:152-250; with the reference's per-row quantiser (block 1, no smoothing)
    and with this build's defaults (128/64 blocks, K smoothing)."""
    b, h, n, d = 1, 2, 64, 64
    q, k, v = _fill((b, h, n, d), 3), _fill((b, h, n, d), 11), _fill((b, h, n, d), 19)
    tq, tk, tv = (Tensor.from_slice(hdev, a, a.shape) for a in (q, k, v))
    sess = Session()
    ref = Settings.default()
    ref.sage_block_q = ref.sage_block_k = 1
    ref.sage_smooth_k = 0
    before = host.selections(K_SAGE)
    out = tq.sage_attention_with(tk, tv, None, 0.0, False, sess, ref)
    assert host.selections(K_SAGE) == before + 1
    assert out.dtype == FLOAT32                              # the reference's Sage kernel stores f32
    q8, sq = oracle.quant_blocks(q, 1)
    k8, sk = oracle.quant_blocks(k, 1)
    err = float(np.abs(out.to_list() - oracle.sage(q8, k8, sq, sk, v, 1, 1)).max())
    assert err < 2e-3                                        # tests/sage_int8.rs:148
    # that convention is two launches: K's per-key quantiser together with V's cast, then the attention kernel,
    # which quantises the f32 queries row by row itself (as the reference's kernel does, cuda_flash_sage.rs:201-223)
    sess.begin_capture()
    again = tq.sage_attention_with(tk, tv, None, 0.0, False, sess, ref)
    ncalls = sess.end_capture()
    assert [sess.step(i)[0] for i in range(ncalls)] == ["ar_sage_quant_rows_cast_f32", "ar_flash_sage_qr_mid"]
    assert sess.step_detail(1)[4][0] == (0, FLOAT32) and np.array_equal(again.to_list(), out.to_list())
    sess.replay()
    assert np.array_equal(again.to_list(), out.to_list())
    out2 = tq.sage_attention_with(tk, tv, None, 0.0, False, sess)
    err2 = float(np.abs(out2.to_list() - oracle.sdpa_f64(q, k, v)).max())
    assert err2 < 2e-2


@gpu
def test_fallback_is_reported_not_faked(hdev):
    q = _fill((1, 2, 16, 32), 3)                             # head_dim 32: no fused kernel
    t = Tensor.from_slice(hdev, q, q.shape)
    sess = Session()
    with pytest.raises(host.HostError, match="TGERR"):
        t.attention_with(t, t, None, 0.0, False, sess)
    q = _fill((1, 2, 16, 64), 3)
    t = Tensor.from_slice(hdev, q, q.shape)
    with pytest.raises(host.HostError, match="general SDPA path"):
        t.attention(t, t)                                    # no session -> SDPA (tensor/mod.rs:2043-2054)
    with pytest.raises(host.HostError, match="general SDPA path"):
        t.attention_with(t, t, None, 0.5, False, sess)       # dropout -> SDPA


@gpu
def test_fused_attention_wrappers(hdev):
    """fused_attention / fused_attention_kind (src/models/flash_attention.rs:292-320): no mask, not
    causal, no GQA; a Tensor when a fused kernel runs, None when the kernels decline."""
    b, h, n, d = 2, 3, 130, 64
    q, k, v = _fill((b, h, n, d), 3), _fill((b, h, n, d), 11), _fill((b, h, n, d), 19)
    tq, tk, tv = (Tensor.from_slice(hdev, a, a.shape) for a in (q, k, v))
    sess = Session()
    before = host.selections(K_FLASH_F32)
    out = host.fused_attention(tq, tk, tv, sess)
    assert out is not None and host.selections(K_FLASH_F32) == before + 1
    assert float(np.abs(out.to_list() - oracle.flash_f32(q, k, v)).max()) < 2e-5      # tests/flash_cuda.rs:74
    before = host.selections(K_SAGE)
    out = host.fused_attention(tq, tk, tv, sess, kind=AttentionKind.Sage)
    assert out is not None and host.selections(K_SAGE) == before + 1
    assert float(np.abs(out.to_list() - oracle.sdpa_f64(q, k, v)).max()) < 2e-2
    out = host.fused_attention(tq, tk, tv, sess, kind=AttentionKind.Flash)
    assert float(np.abs(out.to_list() - oracle.flash_f32(q, k, v)).max()) < 2e-5
    # head_dim 32 has no fused kernel: None, not an error (flash_attention.rs:470-472)
    q32 = _fill((1, 2, 16, 32), 3)
    t32 = Tensor.from_slice(hdev, q32, q32.shape)
    assert host.fused_attention(t32, t32, t32, sess) is None
    # fewer K/V heads without enable_gqa: the wrappers pass enable_gqa = false, so they decline
    tk2 = Tensor.from_slice(hdev, k[:, :1], (b, 1, n, d))
    assert host.fused_attention(tq, tk2, tk2, sess) is None


@gpu
def test_sage_fp8_setting(hdev):
    """Settings.sage_fp8 (the reference's `Options::fp8`, cuda_flash_sage.rs:53-54) routes the quantised
    path through the FP8 entries."""
    b, h, n, d = 1, 4, 300, 128
    q, k, v = _fill((b, h, n, d), 3), _fill((b, h, n, d), 11), _fill((b, h, n, d), 19)
    tq, tk, tv = (Tensor.from_slice(hdev, a, a.shape) for a in (q, k, v))
    st = Settings.default()
    st.sage_fp8 = 1
    sess = Session()
    sess.begin_capture()
    out = tq.sage_attention_with(tk, tv, None, 0.0, True, sess, st)
    n_calls = sess.end_capture()
    names = [sess.step(i)[0] for i in range(n_calls)]
    assert names[0] == "ar_sage_quant_blocks_fp8_f32" and "ar_flash_sage_fp8_mid" in names
    assert float(np.abs(out.to_list() - oracle.sdpa_f64(q, k, v, causal=True)).max()) < 6e-2
    # bf16 tensors: the FP8 attention kernel quantises the queries itself, as the int8 one does
    bq_, bk_, bv_ = (Tensor.from_slice(hdev, a, a.shape, BFLOAT16) for a in (q, k, v))
    sess.begin_capture()
    outb = bq_.sage_attention_with(bk_, bv_, None, 0.0, True, sess, st)
    n_calls = sess.end_capture()
    names = [sess.step(i)[0] for i in range(n_calls)]
    assert names == ["ar_sage_kmean_partial_bf16", "ar_sage_kmean_final", "ar_sage_quant_blocks_fp8_bf16", "ar_flash_sage_fp8_qf_mid"]
    assert float(np.abs(outb.to_list() - oracle.sdpa_f64(q, k, v, causal=True)).max()) < 6e-2
    # enough long 256-query workgroups: the 8-wave pipelined FP8 entry, as for int8
    b, h, n = 2, 32, 2048
    q, k, v = _fill((b, h, n, d), 3), _fill((b, h, n, d), 11), _fill((b, h, n, d), 19)
    tq, tk, tv = (Tensor.from_slice(hdev, a, a.shape) for a in (q, k, v))
    sess.begin_capture()
    out = tq.sage_attention_with(tk, tv, None, 0.0, False, sess, st)
    n_calls = sess.end_capture()
    assert "ar_flash_sage_fp8_long" in [sess.step(i)[0] for i in range(n_calls)]
    rows = np.array([0, 255, 256, 777, 2047])
    assert float(np.abs(out.to_list()[:, :, rows] - oracle.sdpa_f64(q, k, v, rows=rows)).max()) < 6e-2


@gpu
def test_fused_attention_train_and_backward(hdev):
    """The reference's own differential test of the training path (tests/flash_train_cuda.rs:40-106):
    fused forward (out, lse) then fused backward (dq, dk, dv) within 2e-3 of the gradients of SDPA
    under loss = sum(out * dO), through the host API and a captured replay."""
    def data(n, seed):
        return (np.sin(np.arange(n, dtype=np.float32) * np.float32(0.0137) + np.float32(seed)) * np.float32(0.6)).astype(np.float32)
    b, h, hk, n, d, causal = 2, 4, 2, 37, 64, True
    q, k, v, do = (data(b * hh * n * d, s).reshape(b, hh, n, d) for hh, s in ((h, 0.0), (hk, 1.3), (hk, 2.7), (h, 4.1)))
    tq, tk, tv, tdo = (Tensor.from_slice(hdev, a, a.shape) for a in (q, k, v, do))
    sess = Session()
    sess.begin_capture()
    out, lse = host.fused_attention_train(tq, tk, tv, sess, is_causal=causal)
    dq, dk, dv = host.fused_attention_backward(tq, tk, tv, out, lse, tdo, sess, is_causal=causal)
    assert sess.end_capture() == 4
    # few, short heads: the 32-row entries, grid.x = ceil(n / 32)
    assert [sess.step(i)[0] for i in range(4)] == ["ar_fl_fwd_short", "ar_fl_prep", "ar_fl_bwd_dq_short", "ar_fl_bwd_dkv_short"]
    assert sess.step(0)[1] == [2, b * h, 1] and sess.step(2)[1] == [2, b * h, 1] and sess.step(3)[1] == [2, b * hk, 1]
    want = oracle.attention_backward_f64(q, k, v, do, causal=causal, scale=0.125)
    for name, got, w in zip(("out", "lse", "dq", "dk", "dv"), (out, lse, dq, dk, dv), want):
        assert float(np.abs(got.to_list().reshape(w.shape) - w).max()) < 2e-3, name
    sess.replay()                                         # same buffers, same results
    assert float(np.abs(dq.to_list() - want[2]).max()) < 2e-3
    # bf16 tensors keep the graph path: None (flash_attention.rs:802-807)
    tb = Tensor.from_slice(hdev, q, q.shape, BFLOAT16)
    assert host.fused_attention_train(tb, tb, tb, sess) is None
    # enough 128-row workgroups to fill the chip: the reference's own grid and names
    b, h, hk = 72, 8, 8
    q, k, v, do = (data(b * hh * n * d, s).reshape(b, hh, n, d) for hh, s in ((h, 0.0), (hk, 1.3), (hk, 2.7), (h, 4.1)))
    tq, tk, tv, tdo = (Tensor.from_slice(hdev, a, a.shape) for a in (q, k, v, do))
    sess = Session()
    sess.begin_capture()
    out, lse = host.fused_attention_train(tq, tk, tv, sess, is_causal=causal)
    dq, dk, dv = host.fused_attention_backward(tq, tk, tv, out, lse, tdo, sess, is_causal=causal)
    assert sess.end_capture() == 4
    assert [sess.step(i)[0] for i in range(4)] == ["ar_fl_fwd", "ar_fl_prep", "ar_fl_bwd_dq", "ar_fl_bwd_dkv"]
    assert sess.step(0)[1] == [1, b * h, 1]
    want = oracle.attention_backward_f64(q, k, v, do, causal=causal, scale=0.125)
    for name, got, w in zip(("out", "lse", "dq", "dk", "dv"), (out, lse, dq, dk, dv), want):
        assert float(np.abs(got.to_list().reshape(w.shape) - w).max()) < 2e-3, name


@gpu
def test_attention_debug_line_and_kernel_info(hdev, capfd, monkeypatch):
    """AUTORUST_ATTN_DEBUG prints one line per kernel on its first dispatch
    (src/runtime/cuda_flash_bf16.rs:446-456)."""
    monkeypatch.setenv("AUTORUST_ATTN_DEBUG", "1")
    q = _fill((1, 2, 64, 64), 3)
    t = Tensor.from_slice(hdev, q, q.shape, BFLOAT16)
    sess = Session()
    t.flash_attention_with(t, t, None, 0.0, False, sess)
    t.flash_attention_with(t, t, None, 0.0, False, sess)
    err = capfd.readouterr().err
    assert err.count("[attention] flash: bf16 MFMA") <= 1      # at most once per process


@gpu
def test_short_sequences_take_the_pipelined_kernel(hdev):
    """ViT-B/16's sequence length through the host API: the dispatcher's HostCall names the 4-wave form of
    the software-pipelined kernel (128 queries per workgroup, two workgroups per compute unit)."""
    b, h, n, d = 2, 12, 197, 64
    q, k, v = (synth.normal(710 + i, (b, h, n, d)) for i in range(3))
    tq, tk, tv = (Tensor.from_slice(hdev, a, a.shape, BFLOAT16) for a in (q, k, v))
    sess = Session()
    sess.begin_capture()
    out = tq.attention_with(tk, tv, None, 0.0, False, sess)
    assert sess.end_capture() == 1
    name, grid, vals = sess.step(0)
    assert name == "ar_flash_bf16_mid" and grid == [2, b * h, 1] and sess.step_detail(0)[1] == [256, 1, 1]
    assert float(np.abs(out.to_list() - oracle.sdpa_f64(q, k, v)).max()) < 2e-2


@gpu
def test_fp32_exact_mode_picks_its_tiling_from_the_shape(hdev):
    """Float32 tensors take the fp32 exact kernel: the 32-query entry for few, short heads (ViT-B/16 at
    batch 1), the reference's 128-query grid when that fills the chip."""
    d = 64
    for (b, h, n), want_name, per_wg in (((1, 12, 197), "ar_flash_f32_short", 32), ((48, 12, 197), "ar_flash_f32", 128)):
        q, k, v = (synth.normal(720 + i, (b, h, n, d)) for i in range(3))
        tq, tk, tv = (Tensor.from_slice(hdev, a, a.shape) for a in (q, k, v))
        sess = Session()
        sess.begin_capture()
        out = tq.flash_attention_with(tk, tv, None, 0.0, True, sess)
        assert sess.end_capture() == 1
        name, grid, vals = sess.step(0)
        assert name == want_name and grid == [(n + per_wg - 1) // per_wg, b * h, 1] and vals == [n, d, 1, 0, h, h]
        assert float(np.abs(out.to_list() - oracle.sdpa_f64(q, k, v, causal=True)).max()) < 2e-5


@gpu
def test_capture_and_replay(hdev):
    """Session::capture_host + Jit replay (session.rs:138-146, jit.rs:186-195): the captured launch
    re-runs on the same buffers and reproduces the result; the allocator serves repeats from its
    free list."""
    b, h, n, d = 1, 4, 300, 128
    q, k, v = (synth.normal(700 + i, (b, h, n, d)) for i in range(3))
    tq, tk, tv = (Tensor.from_slice(hdev, a, a.shape, BFLOAT16) for a in (q, k, v))
    sess = Session()
    sess.begin_capture()
    out = tq.attention_with(tk, tv, None, 0.0, True, sess)
    o2 = tq.sage_attention_with(tk, tv, None, 0.0, True, sess)
    nsteps = sess.end_capture()
    # one launch for flash; for Sage the pre-pass launches (K mean in two steps, quantise K) and the
    # attention kernel, which quantises the bf16 queries itself and stores bf16, each a HostCall of its own
    names = [sess.step(i)[0] for i in range(nsteps)]
    assert names == ["ar_flash_bf16_mid", "ar_sage_kmean_partial_bf16", "ar_sage_kmean_final",
                     "ar_sage_quant_blocks_bf16", "ar_flash_sage_qf_mid"]
    name, grid, vals = sess.step(0)
    # grid [query tiles of 128, b*h, 1], vals [n, head_dim, causal, has_mask, hq, hkv] (cuda_flash_bf16.rs:550-599)
    assert grid == [(n + 127) // 128, b * h, 1] and vals == [n, d, 1, 0, h, h]
    src, local, nbufs, nvals, sig = sess.step_detail(0)
    assert src.endswith("attn_kernels.hsaco") and local == [256, 1, 1] and (nbufs, nvals) == (5, 6)
    BF, F, I32 = 1, 0, 4
    assert sig == [(0, BF), (1, BF), (2, BF), (3, BF), (4, F)] + [(5 + i, I32) for i in range(6)]   # cuda_flash_bf16.rs:563-578
    assert sess.step(4)[2] == [n, d, 1, 0, h, h] and sess.step_detail(4)[2:4] == (7, 9)   # the six common scalars; then bq, bk, out_f32
    assert sess.step_detail(4)[4][0] == (0, BF)               # the queries themselves, not their codes
    first = out.to_list().copy()
    first2 = o2.to_list().copy()
    allocs = hdev.raw_allocs
    sess.replay()
    sess.replay()
    assert hdev.raw_allocs == allocs                         # scratch came from the free list
    assert np.array_equal(out.to_list(), first) and np.array_equal(o2.to_list(), first2)
    err = float(np.abs(first - oracle.attn_bf16(q, k, v, causal=True)).max())
    assert err < 1.6e-2


@gpu
@pytest.mark.parametrize("api,dtype", [("attention_with", BFLOAT16), ("flash_attention_with", FLOAT32),
                                       ("sage_attention_with", FLOAT32), ("sage_attention_with", BFLOAT16)])
def test_key_lengths_through_the_tensor_api(hdev, api, dtype):
    """A key-padding mask as per-batch key lengths through Tensor::*_with: the captured HostCall
    names the `_lens` entry point, carries the lengths after the mask slot, and the result matches
    the oracle with the same lengths (the reference sends such masks to its general path,
    src/tensor/mod.rs:2405-2447, src/models/flash_attention.rs:389-396)."""
    b, h, hk, n, d = 2, 4, 2, 300, 64
    q, k, v = synth.normal(801, (b, h, n, d)), synth.normal(802, (b, hk, n, d)), synth.normal(803, (b, hk, n, d))
    lens = np.array([123, 300], np.int32)
    tq, tk, tv = (Tensor.from_slice(hdev, a, a.shape, dtype) for a in (q, k, v))
    tl = Tensor.from_i32(hdev, lens)
    sess = Session()
    sess.begin_capture()
    out = getattr(tq, api)(tk, tv, None, 0.0, True, sess, None, tl)
    nsteps = sess.end_capture()
    at = [i for i in range(nsteps) if sess.step(i)[0].startswith("ar_fl")]     # the attention kernel among the pre-passes
    assert len(at) == 1 and sess.step(at[0])[0].endswith("_lens"), [sess.step(i)[0] for i in range(nsteps)]
    src, local, nbufs, nvals, sig = sess.step_detail(at[0])
    assert sig[5][1] == 4                                # DType::Int32 in the slot after the mask
    got = out.to_list()
    if api == "sage_attention_with":
        qr, kr = (oracle.bf16_round(q), oracle.bf16_round(k)) if dtype == BFLOAT16 else (q, k)
        q8, sq = oracle.quant_blocks(qr, 128)
        k8, sk = oracle.quant_blocks(kr, 64, sub=oracle.k_mean(kr))
        want = oracle.sage(q8, k8, sq, sk, v, 128, 64, causal=True, kv_len=lens, round_out=dtype == BFLOAT16)
        # P is rounded to bf16 on both sides (2^-9 relative each), at different rounding points
        assert np.abs(got - want).max() <= (2.0 ** -6 if dtype == BFLOAT16 else 2.0 ** -8 * float(np.abs(v).max()))
    elif dtype == BFLOAT16:
        assert np.abs(got - oracle.attn_bf16(q, k, v, causal=True, kv_len=lens)).max() <= 2.0 ** -6
    else:
        assert np.abs(got - oracle.flash_f32(q, k, v, causal=True, kv_len=lens)).max() < 2e-5
    # replay finds the lengths again
    sess.replay()
    assert np.array_equal(out.to_list(), got)
    # lengths of the wrong shape: the fused kernels decline (the reference's None -> general path)
    with pytest.raises(host.HostError, match="general SDPA path"):
        getattr(tq, api)(tk, tv, None, 0.0, True, sess, None, Tensor.from_i32(hdev, np.array([1, 2, 3], np.int32)))


@gpu
def test_decoder_configuration_through_the_tensor_api(hdev):
    """Causal decoder attention, B4 H32 S2048 D128 bf16 with key lengths uniform in [S/2, S], from
    Tensor::attention_with: the pipelined `_lens` entry, sampled rows within three bf16 steps of the bf16
    emulation."""
    from gpu_util import bf16_ulps
    b, h, n, d = 4, 32, 2048, 128
    q, k, v = (synth.normal(3001 + i, (b, h, n, d)) for i in range(3))
    lens = synth.randint(3005, b, n // 2, n)
    tq, tk, tv = (Tensor.from_slice(hdev, a, a.shape, BFLOAT16) for a in (q, k, v))
    sess = Session()
    sess.begin_capture()
    out = tq.attention_with(tk, tv, None, 0.0, True, sess, None, Tensor.from_i32(hdev, lens))
    assert sess.end_capture() == 1 and sess.step(0)[0] == "ar_flash_bf16_long_lens" and sess.step_detail(0)[1] == [512, 1, 1]
    # without key lengths the same shape takes the 4-wave form (two workgroups per compute unit)
    sess.begin_capture()
    out2 = tq.attention_with(tk, tv, None, 0.0, True, sess)
    assert sess.end_capture() == 1 and sess.step(0)[0] == "ar_flash_bf16_mid" and sess.step_detail(0)[1] == [256, 1, 1]
    full = out2.to_list()
    bi, hi = 3, 9
    rr = np.array([0, 127, 128, 1000, 2047], np.int32)
    want = oracle.attn_bf16(q[bi:bi + 1, hi:hi + 1], k[bi:bi + 1, hi:hi + 1], v[bi:bi + 1, hi:hi + 1], causal=True, rows=rr)
    assert bf16_ulps(full[bi:bi + 1, hi:hi + 1][:, :, rr], want) <= 3.0
    got = out.to_list()
    rows = np.array([0, 63, 64, 255, 256, 1023, 1024, 1500, 2047], np.int32)
    for bi, hi in ((0, 3), (2, 30)):
        rr = np.unique(np.concatenate([rows, [lens[bi] - 1, min(lens[bi], n - 1)]])).astype(np.int32)
        want = oracle.attn_bf16(q[bi:bi + 1, hi:hi + 1], k[bi:bi + 1, hi:hi + 1], v[bi:bi + 1, hi:hi + 1], causal=True,
                                kv_len=lens[bi:bi + 1], rows=rr)
        assert bf16_ulps(got[bi:bi + 1, hi:hi + 1][:, :, rr], want) <= 3.0


@gpu
def test_kprof_line_of_run_host_kernel(hdev, capfd, monkeypatch):
    """AUTORUST_KPROF: a launch that would not wait is synchronised and reported as
    `KPROF\\t<name>\\t<secs>\\t<content key>` (src/runtime/ops_cuda.rs:879-885, 1004-1012)."""
    import re
    from autorust_amd import _lib
    x = synth.normal(5, (1000,))
    tx, ty = Tensor.from_slice(hdev, x, x.shape), Tensor.from_slice(hdev, np.zeros_like(x), x.shape)
    capfd.readouterr()
    assert hdev.run_host_kernel(_lib.PROBES_PATH, "probe_axpb", [tx, ty], [1000], [4, 1, 1], [256, 1, 1], wait=False) is None
    assert "KPROF" not in capfd.readouterr().err
    monkeypatch.setenv("AUTORUST_KPROF", "1")
    secs = hdev.run_host_kernel(_lib.PROBES_PATH, "probe_axpb", [tx, ty], [1000], [4, 1, 1], [256, 1, 1], wait=False)
    err = capfd.readouterr().err
    m = re.search(r"^KPROF\tprobe_axpb\t(\d+\.\d{6})\t([0-9a-f]{16})$", err, re.M)
    assert m and secs is not None and abs(float(m.group(1)) - secs) < 1e-6
    assert np.abs(ty.to_list() - (x * np.float32(3.0) + np.float32(1.0))).max() < 1e-5   # the kernel may contract x * 3 + 1
    # a launch that waits anyway prints nothing (the reference's `kprof_enabled() && !wait`)
    assert hdev.run_host_kernel(_lib.PROBES_PATH, "probe_axpb", [tx, ty], [1000], [4, 1, 1], [256, 1, 1], wait=True) is not None
    assert "KPROF" not in capfd.readouterr().err
