"""The pipelined kernels (int8, bf16) against a numpy restatement of THEIR OWN order of operations
(autorust_amd/csrc/attn_pipe.h), wave by wave: 32-key blocks in sequence, the biased-float logits
(12582912 + sum) * c' - m_bias with c' cut to 21 bits, the lazy exponent reference on its grid, the
rescue path (row maximum, reference moved up to the grid, accumulators rescaled, block redone with
converted logits), row sums per lane half in the kernel's tree order, P rounded to bf16 for the
matrix product, fp32 accumulators.

The tolerance tests against the reference's emulation (tests/test_gpu_sage.py) cannot see anything
below the rounding of P (2^-9 of |v|); this one can: what is left between kernel and restatement is
the last bit of v_exp_f32 and the summation order inside a matrix instruction.  It pins the kernel's
arithmetic (a slip in the bias, the cut, the grid or the rescue shows up as 1e-4 .. 1e-2), not the
reference's: the oracle stays the judge of that."""
import numpy as np
import pytest

import oracle
from autorust_amd import synth
from autorust_amd.device import BF16, F32
from gpu_util import run_flash, run_sage

pytestmark = pytest.mark.gpu

F = np.float32
BIAS = 12582912.0
LOG2E = F(1.4426950408889634)
LIMIT = F(16.0) * F(2.0 ** 60)


def _cut21(c):
    u = np.asarray(c, F).view(np.uint32)
    return ((u + np.uint32(4)) & np.uint32(0xFFFFFFF8)).view(F)


def _fl32(x):
    return np.asarray(x, np.float64).astype(F)


def _tree(x):
    """((x0+x1)+(x2+x3))+((x4+x5)+(x6+x7)) in fp32 along the last axis (8 values)."""
    a = [F(x[..., 2 * i] + x[..., 2 * i + 1]) for i in range(4)]
    return F(F(a[0] + a[1]) + F(a[2] + a[3]))


def _lane_keys(h):
    """keys of a 32-key block held by lane half h, in register order r = 0..15"""
    return np.array([8 * (r // 4) + 4 * h + (r % 4) for r in range(16)])


def _wave(q8, k8, sq_rows, sk_tiles, vb, scale, grid):
    """One wave of the int8 kernel: q8 [32, D] int8, k8 [N, D] int8, sq_rows [32], sk_tiles [N/64], vb [N, D]
    (bf16 values).  With sq_rows None: the bf16 kernel on bf16 values q8, k8 (fp32 logits, factor
    scale * log2(e), no bias, no grid)."""
    if sq_rows is None:
        return _wave_bf16(q8, k8, vb, scale)
    N, D = k8.shape
    m = np.full(32, -1e30, F)
    l = np.zeros((32, 2), F)                       # per lane half
    o = np.zeros((32, D), F)
    inv_grid = F(1.0) / F(grid)
    moves = 0
    for blk in range(N // 32):
        kb0 = blk * 32
        acc = q8.astype(np.int64) @ k8[kb0:kb0 + 32].astype(np.int64).T          # [32, 32] exact
        c = _cut21(F(F(F(sq_rows * sk_tiles[kb0 // 64]) * F(scale)) * LOG2E))    # [32]
        c64 = c.astype(np.float64)
        m_bias = _fl32(BIAS * c64 + m)                                            # one fused multiply-add
        t = _fl32((BIAS + acc) * c64[:, None] - m_bias[:, None].astype(np.float64))
        with np.errstate(over="ignore"):
            p = np.exp2(t.astype(np.float64)).astype(F)
        rs = np.stack([F(_tree(p[:, _lane_keys(h)[:8]]) + _tree(p[:, _lane_keys(h)[8:]])) for h in (0, 1)], axis=1)
        if not np.all(rs <= LIMIT):
            moves += 1
            x = F(acc.astype(F) * c[:, None])
            m_new = np.maximum(m, x.max(axis=1))
            on = m_new > F(-1e29)
            m_new = np.where(on, F(np.ceil(F(m_new * inv_grid)) * F(grid)), m_new).astype(F)
            with np.errstate(under="ignore"):
                alpha = np.exp2((m - m_new).astype(np.float64)).astype(F)
            m = m_new
            l = F(l * alpha[:, None])
            o = F(o * alpha[:, None])
            t = _fl32(acc.astype(np.float64) * c64[:, None] - m[:, None].astype(np.float64))
            p = np.exp2(t.astype(np.float64)).astype(F)
            rs = np.stack([F(_tree(p[:, _lane_keys(h)[:8]]) + _tree(p[:, _lane_keys(h)[8:]])) for h in (0, 1)], axis=1)
        l = F(l + rs)
        pb = oracle.bf16_round(p).astype(np.float64)
        for ks in (0, 1):                                                         # two 16-key matrix steps
            o = (o.astype(np.float64) + pb[:, 16 * ks:16 * ks + 16] @ vb[kb0 + 16 * ks:kb0 + 16 * ks + 16].astype(np.float64)).astype(F)
    l_tot = F(l[:, 0] + l[:, 1])
    inv = np.where(l_tot > 0, F(1.0) / l_tot, F(0.0)).astype(F)
    return F(o * inv[:, None]), moves


def _wave_bf16(qb, kb, vb, scale):
    N, D = kb.shape
    m = np.full(32, -1e30, F)
    l = np.zeros((32, 2), F)
    o = np.zeros((32, D), F)
    c = F(F(scale) * LOG2E)
    sums = lambda p: np.stack([F(_tree(p[:, _lane_keys(h)[:8]]) + _tree(p[:, _lane_keys(h)[8:]])) for h in (0, 1)], axis=1)
    for blk in range(N // 32):
        kb0 = blk * 32
        s = (qb.astype(np.float64) @ kb[kb0:kb0 + 32].astype(np.float64).T).astype(F)     # fp32 accumulators
        t = _fl32(s.astype(np.float64) * np.float64(c) - m[:, None].astype(np.float64))
        with np.errstate(over="ignore"):
            p = np.exp2(t.astype(np.float64)).astype(F)
        rs = sums(p)
        if not np.all(rs <= LIMIT):
            m_new = np.maximum(m, F(s * c).max(axis=1))
            with np.errstate(under="ignore"):
                alpha = np.exp2((m - m_new).astype(np.float64)).astype(F)
            m = m_new
            l = F(l * alpha[:, None])
            o = F(o * alpha[:, None])
            t = _fl32(s.astype(np.float64) * np.float64(c) - m[:, None].astype(np.float64))
            p = np.exp2(t.astype(np.float64)).astype(F)
            rs = sums(p)
        l = F(l + rs)
        pb = oracle.bf16_round(p).astype(np.float64)
        for ks in (0, 1):
            o = (o.astype(np.float64) + pb[:, 16 * ks:16 * ks + 16] @ vb[kb0 + 16 * ks:kb0 + 16 * ks + 16].astype(np.float64)).astype(F)
    l_tot = F(l[:, 0] + l[:, 1])
    inv = np.where(l_tot > 0, F(1.0) / l_tot, F(0.0)).astype(F)
    return F(o * inv[:, None]), 0


def test_bf16_pipelined_kernel_matches_its_own_order_of_operations(dev):
    """The same for the bf16 kernel, whose output is rounded to bf16: almost every sampled output has the
    bits of the rounded restatement, the rest sit one bf16 step away (a value near a rounding boundary
    and the last bits of the logits, which depend on the summation order inside a matrix instruction)."""
    B, H, N, D = 1, 32, 1024, 128
    q, k, v = synth.normal(711, (B, H, N, D)), synth.normal(712, (B, H, N, D)), synth.normal(713, (B, H, N, D))
    gain = F(2.0) ** np.linspace(-3.0, 2.0, H, dtype=F)
    q = q * gain[None, :, None, None]
    got_all = run_flash(dev, q, k, v, BF16)
    qb, kb, vb = oracle.bf16_round(q), oracle.bf16_round(k), oracle.bf16_round(v)
    scale = F(1.0) / np.sqrt(F(D))
    same = total = 0
    for h in (0, 9, 18, 31):
        for wave in (0, 7, 20, 31):
            rows = np.arange(32 * wave, 32 * wave + 32)
            want, _ = _wave(qb[0, h, rows], kb[0, h], None, None, vb[0, h], scale, None)
            wb = oracle.bf16_round(want)
            got = got_all[0, h, rows]
            big = np.maximum(np.maximum(np.abs(got), np.abs(wb)), F(2.0 ** -100)).astype(np.float64)
            step = np.exp2(np.floor(np.log2(big)) - 7.0)                       # one bf16 step at the larger of the two
            # (plus the noise floor of the fp32 result itself, which matters for outputs near zero)
            floor = 1e-5 + 1e-4 * float(np.abs(want).max())
            assert np.all(np.abs(got.astype(np.float64) - wb) <= step + floor), float(np.abs(got - wb).max())
            same += int((got == wb).sum())
            total += got.size
    assert same >= 0.995 * total, (same, total)            # measured: 0.9992


def test_int8_pipelined_kernel_matches_its_own_order_of_operations(dev):
    B, H, N, D, bq, bk = 1, 32, 1024, 128, 128, 64
    q, k, v = synth.normal(701, (B, H, N, D)), synth.normal(702, (B, H, N, D)), synth.normal(703, (B, H, N, D))
    gain = F(2.0) ** np.linspace(-8.0, 5.0, H, dtype=F)           # steps c from ~4e-7 to ~3e-3
    q = q * gain[None, :, None, None]
    k = (k + F(2.0) * synth.normal(709, (1, H, 1, D))).astype(F)
    r = run_sage(dev, q, k, v, bq, bk, smooth=True, out_dtype=F32)
    q8, sq, k8, sk, vb = r["q8"], r["sq"], r["k8"], r["sk"], r["vb"]
    scale = F(1.0) / np.sqrt(F(D))
    worst, medians, total_moves = 0.0, [], 0
    for h in (0, 5, 13, 22, 27, 31):
        for wave in (0, 3, 13, 31):                                # waves of 32 queries; a workgroup holds 8
            wg = wave // 8
            rows = np.arange(32 * wave, 32 * wave + 32)
            qb = np.arange((wg * 256) // bq, (wg * 256 + 255) // bq + 1)
            x = F(BIAS) * F(F(F(np.abs(sq[0, h, qb]).max() * np.abs(sk[0, h]).max()) * scale) * LOG2E)
            e = int((np.asarray(x, F).view(np.uint32) >> 23) & 0xFF) - 127
            grid = 2.0 ** (e - 21)
            want, moves = _wave(q8[0, h, rows], k8[0, h], sq[0, h, rows // bq], sk[0, h], vb[0, h], scale, grid)
            got = r["out"][0, h, rows]
            err = np.abs(got - want)
            worst = max(worst, float(err.max()))
            medians.append(float(np.median(err)))
            total_moves += moves
            assert moves >= 1                                       # the first block always moves the reference
    # measured: worst 1.6e-5, largest median 3e-8 (outputs of magnitude ~1).  Restating the kernel with the
    # uncut c, with the reference off its grid, or with row sums over the rounded P each gives worst
    # > 1e-2 and medians of 7e-4 .. 1e-3.
    assert worst < 1e-4 and max(medians) < 1e-6, (worst, medians)
    assert total_moves >= 24
