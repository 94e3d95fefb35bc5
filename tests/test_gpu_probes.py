"""Generic host-kernel seam and MFMA layout known answers (the counterparts of the
reference's tests/host_kernel.rs and tests/sage_layout_probe.rs)."""
import numpy as np
import pytest

from autorust_amd import _lib, synth

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def probes(dev):
    return dev.module_load(open(_lib.PROBES_PATH, "rb").read())


def test_device_identity(dev):
    assert dev.arch == "gfx950"
    assert dev.compute_units >= 200
    free, total = dev.mem_info()
    assert 0 < free <= total and total > 200 * 2 ** 30


def test_host_kernel_seam(dev, probes):
    # tests/host_kernel.rs:28-61: [1,2,3,4] * 3 + 1
    x = dev.from_numpy(np.array([1, 2, 3, 4], np.float32))
    y = dev.alloc(16)
    secs = dev.launch(probes, "probe_axpb", (1, 1, 1), (64, 1, 1), [x, y], [4], [32])
    assert secs >= 0
    assert y.copyout(np.float32, 4).tolist() == [4.0, 7.0, 10.0, 13.0]
    # module cache: same image -> same handle
    assert dev.module_load(open(_lib.PROBES_PATH, "rb").read()) == probes
    # a zero-sized grid is a no-op
    assert dev.launch(probes, "probe_axpb", (0, 1, 1), (64, 1, 1), [x, y], [4], [32]) == 0.0
    with pytest.raises(_lib.ArhipError):
        dev.launch(probes, "no_such_kernel", (1, 1, 1), (64, 1, 1), [x, y], [4], [32])
    x.free(); y.free()


def test_copy_roundtrip_and_fill(dev):
    a = synth.normal(5, (1000,))
    b = dev.from_numpy(a)
    c = dev.alloc(a.nbytes)
    dev.lib.arhip_copy_d2d(dev.handle, c.ptr, b.ptr, a.nbytes)
    assert np.array_equal(c.copyout(np.float32, a.shape), a)
    c.zero()
    assert not c.copyout(np.float32, a.shape).any()
    b.free(); c.free()


def test_int8_mfma_layout(dev, probes):
    A = (((np.arange(1024) * 7) % 19) - 9).astype(np.int8).reshape(32, 32)
    B = (((np.arange(1024) * 5) % 13) - 6).astype(np.int8).reshape(32, 32)
    a, b, c = dev.from_numpy(A), dev.from_numpy(B), dev.alloc(4096).zero()
    dev.launch(probes, "probe_i8_32x32x32", (1, 1, 1), (64, 1, 1), [a, b, c])
    assert np.array_equal(c.copyout(np.int32, (32, 32)), A.astype(np.int32) @ B.astype(np.int32))
    for t in (a, b, c):
        t.free()


def test_int8_reference_known_answer(dev, probes):
    # tests/sage_layout_probe.rs:73-84
    a = (((np.arange(512) * 7) % 19) - 9).astype(np.int8)
    b = (((np.arange(256) * 5) % 13) - 6).astype(np.int8)
    want = a.reshape(16, 32).astype(np.int32) @ b.reshape(32, 8).astype(np.int32)
    da, db, dc = dev.from_numpy(a), dev.from_numpy(b), dev.alloc(512).zero()
    dev.launch(probes, "probe_i8_16x8_padded", (1, 1, 1), (64, 1, 1), [da, db, dc])
    assert np.array_equal(dc.copyout(np.int32, (16, 8)), want)
    for t in (da, db, dc):
        t.free()


def test_bf16_mfma_layout(dev, probes):
    A = ((np.arange(512) * 7) % 19 - 9).astype(np.float32).reshape(32, 16)
    B = ((np.arange(512) * 5) % 13 - 6).astype(np.float32).reshape(16, 32)
    a, b, c = dev.from_numpy(synth.to_bf16_bits(A)), dev.from_numpy(synth.to_bf16_bits(B)), dev.alloc(4096).zero()
    dev.launch(probes, "probe_bf16_32x32x16", (1, 1, 1), (64, 1, 1), [a, b, c])
    assert np.array_equal(c.copyout(np.float32, (32, 32)), A @ B)
    for t in (a, b, c):
        t.free()


def test_fp8_matrix_instructions_add_their_products_with_about_14_bits(dev, probes):
    """The E4M3 matrix instructions (64-deep scaled and 16-deep) do not add their exact products in
    fp32: against the exact dot product of 64 random codes they are off by up to ~6e-5 of the sum of
    the absolute products (both instructions identically), where an fp32 accumulation would be within
    1e-7.  This is why the FP8 attention follows a restatement of its own arithmetic only to the
    extent the logits do (tests/test_gpu_kernel_order.py); the int8 instruction is exact and the
    bf16 one is accurate to fp32 rounding (the layout tests above, the kernel-order tests)."""
    import oracle
    rng = np.random.default_rng(11)
    out = dev.alloc(8)
    worst = 0.0
    for trial in range(20):
        codes = rng.integers(0, 256, size=(2, 64)).astype(np.uint8)
        codes[(codes & 0x7F) == 0x7F] = 0x38                      # no NaN codes
        if trial >= 10:
            codes &= 0x7F                                          # all positive: no cancellation
        a, b = dev.from_numpy(codes[0]), dev.from_numpy(codes[1])
        dev.launch(probes, "probe_fp8_dot64", (1, 1, 1), (64, 1, 1), [a, b, out])
        got = out.copyout(np.float32, (2,)).astype(np.float64)
        prod = oracle.fp8_e4m3_value(codes[0]).astype(np.float64) * oracle.fp8_e4m3_value(codes[1]).astype(np.float64)
        rel = np.abs(got - prod.sum()) / np.abs(prod).sum()
        assert got[0] == got[1]                                    # the two instructions agree bit for bit
        worst = max(worst, float(rel.max()))
        a.free(); b.free()
    out.free()
    assert 1e-6 < worst < 2e-4, worst                              # measured: 6e-5
