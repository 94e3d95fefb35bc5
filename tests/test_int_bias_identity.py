"""CPU check of the arithmetic the pipelined int8 kernel relies on when it reads its int32 logit
accumulators as biased floats (autorust_amd/csrc/attn_pipe.h, s_init / set_bias / the grid set in the prologue):

    accumulators start at 0x4B400000, so their bits read as the float B + acc, B = 12582912;
    c' = c cut to 21 significant bits (round to nearest);
    m_run only takes multiples of grid = 2^(floor(log2(B c_max)) - 21);
    m_bias = fl32(B c' + m_run);   t = fl32((B + acc) c' - m_bias)   (one fused multiply-add)

and claims t == fl32(acc c' - m_run), i.e. exactly what the converting kernel computes with the same
c', whenever the bias outweighs the reference; otherwise the two differ by at most half a unit in
the last place of m_run.  float64 holds every intermediate exactly (24 x 21-bit products, sums of
nearly equal numbers), so numpy can evaluate both sides with a single rounding to float32 each.
The reference computes s = (float)acc * ((sq*sk)*scale) (src/runtime/cuda_flash_sage.rs:315-322);
cutting c to 21 bits changes a logit by a relative 2^-21 at most, which the last test bounds."""
import numpy as np

B = 12582912.0


def cut21(c):
    u = np.asarray(c, np.float32).view(np.uint32)
    return ((u + np.uint32(4)) & np.uint32(0xFFFFFFF8)).view(np.float32)


def grid_for(c_max):
    x = np.float32(B) * np.float32(c_max)
    e = int((np.float32(x).view(np.uint32) >> 23) & 0xFF) - 127
    return 2.0 ** (e - 21)


def biased_and_direct(acc, c, m_run):
    """fl32 of the kernel's biased evaluation and of the converting evaluation (float64 is exact here)."""
    c = c.astype(np.float64)
    m_bias = (B * c + m_run).astype(np.float32).astype(np.float64)     # one rounding: the fused multiply-add
    t_biased = ((B + acc) * c - m_bias).astype(np.float32)
    t_direct = (acc * c - m_run).astype(np.float32)
    return t_biased, t_direct


def _cases(rng, n, c_max):
    acc = rng.integers(-(1 << 21), (1 << 21) + 1, n).astype(np.float64)
    # per-tile factors anywhere from c_max down to a 256th of it
    c = cut21((c_max * 2.0 ** -rng.uniform(0.0, 8.0, n)).astype(np.float32))
    return acc, c


def test_bias_is_exact_on_the_grid_when_it_outweighs_the_reference():
    rng = np.random.default_rng(7)
    for c_max in [2.0 ** -14, 7.1e-5, 2.0 ** -10, 1.3e-3, 2.5e-3, 0.04, 0.7, 3.0]:
        grid = grid_for(c_max)
        acc, c = _cases(rng, 200000, c_max)
        # references on the grid, of either sign, below the bias
        m_run = np.ceil(rng.uniform(-1.0, 1.0, acc.size) * np.minimum(B * c.astype(np.float64), 300.0) / grid) * grid
        t_b, t_d = biased_and_direct(acc, c, m_run)
        assert np.array_equal(t_b, t_d), (c_max, np.abs(t_b - t_d).max())


def test_without_the_cut_or_the_grid_the_bias_rounds():
    """The test above has teeth: drop either device and the two evaluations differ."""
    rng = np.random.default_rng(8)
    c_max = 2.5e-3
    grid = grid_for(c_max)
    acc = rng.integers(-(1 << 21), (1 << 21) + 1, 200000).astype(np.float64)
    c_full = (c_max * 2.0 ** -rng.uniform(0.0, 2.0, acc.size)).astype(np.float32)          # 24 significant bits
    m_grid = np.ceil(rng.uniform(-100.0, 100.0, acc.size) / grid) * grid
    t_b, t_d = biased_and_direct(acc, c_full, m_grid)
    assert (t_b != t_d).mean() > 0.2
    m_free = rng.uniform(-100.0, 100.0, acc.size).astype(np.float32).astype(np.float64)   # off the grid
    t_b, t_d = biased_and_direct(acc, cut21(c_full), m_free)
    assert (t_b != t_d).mean() > 0.2
    # and the size of what is avoided: up to ~0.75 c in the exponent
    assert np.abs(t_b.astype(np.float64) - t_d).max() > 0.25 * c_max


def test_reference_outweighing_the_bias_costs_half_an_ulp_of_the_reference():
    rng = np.random.default_rng(9)
    c_max = 2.0 ** -12
    grid = grid_for(c_max)
    acc = rng.integers(-(1 << 21), (1 << 21) + 1, 200000).astype(np.float64)
    c = cut21((c_max * 2.0 ** -rng.uniform(6.0, 12.0, acc.size)).astype(np.float32))   # B c from 12 down to 0.2
    m_run = np.ceil(rng.uniform(-250.0, 250.0, acc.size) / grid) * grid
    t_b, t_d = biased_and_direct(acc, c, m_run)
    assert np.abs(t_b.astype(np.float64) - t_d).max() <= 2.0 ** -16 + 2.0 ** -24 * 512


def test_cutting_c_moves_a_logit_by_2_to_the_minus_21_relative():
    rng = np.random.default_rng(10)
    c = (2.0 ** rng.uniform(-20.0, 2.0, 100000)).astype(np.float32)
    rel = np.abs(cut21(c).astype(np.float64) - c) / c
    assert rel.max() <= 2.0 ** -21
    assert np.all((cut21(c).view(np.uint32) & 7) == 0)
