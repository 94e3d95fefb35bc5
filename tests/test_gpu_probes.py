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
