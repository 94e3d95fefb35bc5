"""The C-ABI library: loads, exports what include/arhip.h declares, and fails
loudly (never silently falls back) when there is no device.  No GPU needed."""
import ctypes
import os
import re

import pytest

from autorust_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared():
    text = open(os.path.join(ROOT, "include", "arhip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(arhip_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    lib = _lib.load()
    names = _declared()
    assert len(names) >= 25
    for n in names:
        assert hasattr(lib, n), n
    # and the binding table covers exactly the header
    assert sorted(_lib.SIGNATURES) == names


def test_supported_gates():
    lib = _lib.load()
    # src/runtime/cuda_flash_bf16.rs:431-433 accepts d == 64, n > 0; this build adds d == 128
    assert lib.arhip_attn_supported(_lib.ATTN_FLASH, 197, 64, _lib.BF16) == 1
    assert lib.arhip_attn_supported(_lib.ATTN_FLASH, 2048, 128, _lib.BF16) == 1
    assert lib.arhip_attn_supported(_lib.ATTN_FLASH, 197, 64, _lib.F32) == 1
    assert lib.arhip_attn_supported(_lib.ATTN_SAGE, 8192, 128, _lib.F32) == 1
    assert lib.arhip_attn_supported(_lib.ATTN_FLASH, 64, 32, _lib.BF16) == 0   # tests/flash_cuda_bf16.rs:144 analogue
    assert lib.arhip_attn_supported(_lib.ATTN_FLASH, 0, 64, _lib.BF16) == 0
    assert lib.arhip_attn_supported(_lib.ATTN_FLASH, 64, 64, 7) == 0
    assert lib.arhip_attn_supported(_lib.ATTN_SDPA, 64, 64, _lib.F32) == 0


def test_null_device_is_an_error_not_a_fallback():
    lib = _lib.load()
    rc = lib.arhip_flash_fwd(None, 16, 16, 16, 16, None, None, 1, 1, 1, 8, 64, 0, _lib.BF16, 0.125, 1, None)
    assert rc == _lib.EINVAL
    assert b"null device" in lib.arhip_last_error()
    rc = lib.arhip_sage_fwd(None, 16, 16, 16, 16, 16, 16, None, None, 1, 1, 1, 8, 64, 128, 64, 0, 0, 0.125,
                            None, None, 1, None)
    assert rc == _lib.EINVAL
    rc = lib.arhip_sage_quant(None, 16, 16, 16, None, None, 1, 1, 8, 64, 64, 0, 0, 1, None)
    assert rc == _lib.EINVAL
    with pytest.raises(_lib.ArhipError) as e:
        _lib.check(rc)
    assert "TGERR" in str(e.value)   # the reference's error convention (AGENTS.md principle 2)


def test_open_without_device_reports_no_device():
    lib = _lib.load()
    n = ctypes.c_int(-1)
    assert lib.arhip_device_count(ctypes.byref(n)) == 0
    if n.value > 0:
        pytest.skip("a GPU is visible here")
    h = ctypes.c_void_p()
    assert lib.arhip_open(0, ctypes.byref(h)) == _lib.ENODEVICE
    assert h.value is None
    assert b"no HIP device" in lib.arhip_last_error()
    from autorust_amd.device import Device
    with pytest.raises(_lib.ArhipError):
        Device(0)


def test_workspace_size():
    lib = _lib.load()
    assert lib.arhip_sage_quant_workspace(4, 32, 8192, 128) == 4 * 32 * 128 * 128 * 4
    assert lib.arhip_sage_quant_workspace(1, 1, 65, 64) == 2 * 64 * 4
    assert lib.arhip_sage_quant_workspace(0, 1, 65, 64) == 0


def test_code_object_is_built_and_names_every_entry_point():
    """The named kernels (include/arhip_kernels.h) are all in the code object (no launch here)."""
    text = open(os.path.join(ROOT, "include", "arhip_kernels.h")).read()
    names = re.findall(r'#define ARHIP_KERNEL_\w+ "(\w+)"', text)
    assert len(names) == 53
    image = open(_lib.KERNELS_PATH, "rb").read()
    for n in names:
        assert n.encode() + b"\0" in image or n.encode() in image, n


def test_code_object_file_is_a_container_of_elf_parts():
    """attn_kernels.hsaco holds the entry points as several code objects (they compile side by side): "ARHIPKO1",
    count, then per part its size and bytes padded to 16; arhip_module_load takes the file as a whole.  Every part
    is a gfx950 code object and every named kernel lives in exactly one of them."""
    import struct
    image = open(_lib.KERNELS_PATH, "rb").read()
    assert image[:8] == b"ARHIPKO1"
    count, zero = struct.unpack_from("<II", image, 8)
    assert count == 15 and zero == 0
    at, parts = 16, []
    for _ in range(count):
        (size,) = struct.unpack_from("<Q", image, at)
        at += 8
        parts.append(image[at:at + size])
        # hipcc --genco writes an offload bundle around the ELF image; hipModuleLoadData takes either
        assert parts[-1].startswith((b"\x7fELF", b"__CLANG_OFFLOAD_BUNDLE__")) and len(parts[-1]) == size
        at += (size + 15) & ~15
    assert at == len(image)
    text = open(os.path.join(ROOT, "include", "arhip_kernels.h")).read()
    for n in re.findall(r'#define ARHIP_KERNEL_\w+ "(\w+)"', text):
        homes = [i for i, part in enumerate(parts) if n.encode() + b".kd\0" in part]
        assert len(homes) == 1, (n, homes)
