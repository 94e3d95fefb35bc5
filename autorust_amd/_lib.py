"""ctypes binding of libarhip.so (declared in include/arhip.h).

The library is the product; this module only loads it and gives the entry
points their argument types.  There is no CPU fallback: if the library is
missing or no gfx950 device opens, the caller gets an exception.
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libarhip.so")
PROBES_PATH = os.path.join(_HERE, "probes.hsaco")
KERNELS_PATH = os.path.join(_HERE, "attn_kernels.hsaco")

OK, EINVAL, EUNSUPPORTED, EHIP, ENODEVICE = 0, -1, -2, -3, -4
F32, BF16 = 0, 1
ATTN_SDPA, ATTN_FLASH, ATTN_SAGE = 0, 1, 2
K_FLASH_F32, K_FLASH_BF16, K_SAGE, K_SAGE_QUANT, K_FLASH_BWD = 0, 1, 2, 3, 4

c_void_p, c_int, c_int64, c_size_t = ctypes.c_void_p, ctypes.c_int, ctypes.c_int64, ctypes.c_size_t
c_float, c_double, c_char_p = ctypes.c_float, ctypes.c_double, ctypes.c_char_p
_pd = ctypes.POINTER(c_double)

# name -> (restype, argtypes); every symbol include/arhip.h declares
SIGNATURES = {
    "arhip_last_error": (c_char_p, []),
    "arhip_device_count": (c_int, [ctypes.POINTER(c_int)]),
    "arhip_open": (c_int, [c_int, ctypes.POINTER(c_void_p)]),
    "arhip_close": (c_int, [c_void_p]),
    "arhip_arch": (c_char_p, [c_void_p]),
    "arhip_compute_units": (c_int, [c_void_p]),
    "arhip_alloc": (c_int, [c_void_p, c_size_t, ctypes.POINTER(c_void_p)]),
    "arhip_free": (c_int, [c_void_p, c_void_p]),
    "arhip_copyin": (c_int, [c_void_p, c_void_p, c_void_p, c_size_t]),
    "arhip_copyout": (c_int, [c_void_p, c_void_p, c_void_p, c_size_t]),
    "arhip_copy_d2d": (c_int, [c_void_p, c_void_p, c_void_p, c_size_t]),
    "arhip_fill_zero": (c_int, [c_void_p, c_void_p, c_size_t]),
    "arhip_mem_info": (c_int, [c_void_p, ctypes.POINTER(c_size_t), ctypes.POINTER(c_size_t)]),
    "arhip_sync": (c_int, [c_void_p]),
    "arhip_stream": (c_void_p, [c_void_p]),
    "arhip_timer_start": (c_int, [c_void_p]),
    "arhip_timer_stop": (c_int, [c_void_p, _pd]),
    "arhip_kprof_enable": (c_int, [c_void_p, c_int]),
    "arhip_kprof_collect": (c_int, [c_void_p, c_int, _pd, ctypes.POINTER(ctypes.c_uint64)]),
    "arhip_kprof_collect_stats": (c_int, [c_void_p, c_int, _pd, ctypes.POINTER(ctypes.c_uint64), _pd, _pd]),
    "arhip_graph_begin": (c_int, [c_void_p]),
    "arhip_graph_end": (c_int, [c_void_p, ctypes.POINTER(c_void_p)]),
    "arhip_graph_launch": (c_int, [c_void_p, c_void_p, c_int, _pd]),
    "arhip_graph_destroy": (c_int, [c_void_p, c_void_p]),
    "arhip_module_load": (c_int, [c_void_p, c_void_p, c_size_t, ctypes.POINTER(c_void_p)]),
    "arhip_launch": (c_int, [c_void_p, c_void_p, c_char_p, ctypes.POINTER(ctypes.c_uint), ctypes.POINTER(ctypes.c_uint),
                             ctypes.POINTER(c_void_p), c_int, ctypes.POINTER(c_int64), ctypes.POINTER(c_int), c_int,
                             c_int, _pd]),
    "arhip_attn_supported": (c_int, [c_int, c_int64, c_int64, c_int]),
    "arhip_flash_fwd": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                c_int64, c_int64, c_int64, c_int64, c_int64, c_int, c_int, c_float, c_int, _pd]),
    "arhip_flash_fwd_strided": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                        ctypes.POINTER(c_int64), ctypes.POINTER(c_int64), ctypes.POINTER(c_int64),
                                        c_void_p, c_void_p, c_int64, c_int64, c_int64, c_int64, c_int64,
                                        c_int, c_int, c_float, c_int, _pd]),
    "arhip_flash_fwd_lse": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                    ctypes.POINTER(c_int64), ctypes.POINTER(c_int64), ctypes.POINTER(c_int64),
                                    c_void_p, c_void_p, c_int64, c_int64, c_int64, c_int64, c_int64,
                                    c_int, c_int, c_float, c_int, _pd]),
    "arhip_flash_bwd": (c_int, [c_void_p] * 13 + [c_int64] * 5 + [c_int, c_float, c_int, _pd]),
    "arhip_sage_quant_workspace": (c_size_t, [c_int64, c_int64, c_int64, c_int64]),
    "arhip_sage_quant": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                 c_int64, c_int64, c_int64, c_int64, c_int64, c_int, c_int, c_int, _pd]),
    "arhip_sage_quant_strided": (c_int, [c_void_p, c_void_p, ctypes.POINTER(c_int64), c_void_p, c_void_p, c_void_p, c_void_p,
                                         c_int64, c_int64, c_int64, c_int64, c_int64, c_int, c_int, c_int, _pd]),
    "arhip_sage_quant_static_limit": (c_size_t, []),
    "arhip_sage_quant_static": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                        c_int64, c_int64, c_int64, c_int64, c_int64, c_int, c_int, c_int, _pd]),
    "arhip_cast_bf16": (c_int, [c_void_p, c_void_p, c_void_p, c_int64, c_int, _pd]),
    "arhip_sage_prep_kv_rows": (c_int, [c_void_p] * 6 + [c_int64] * 4 + [c_int, _pd]),
    "arhip_sage_quant_fp8": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                     c_int64, c_int64, c_int64, c_int64, c_int64, c_int, c_int, c_int, _pd]),
    "arhip_sage_fwd_fp8": (c_int, [c_void_p] * 9 + [c_int64] * 7 + [c_int, c_int, c_float, c_int, _pd]),
    "arhip_sage_fwd_qfused": (c_int, [c_void_p] * 9 + [c_int64] * 6 + [c_int, c_int, c_float, c_int, _pd]),
    "arhip_sage_fwd_fp8_qfused": (c_int, [c_void_p] * 9 + [c_int64] * 6 + [c_int, c_int, c_float, c_int, _pd]),
    "arhip_sage_fwd_qfused_rows": (c_int, [c_void_p] * 9 + [c_int64] * 6 + [c_int, c_int, c_float, c_int, _pd]),
    "arhip_sage_fwd": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                               c_int64, c_int64, c_int64, c_int64, c_int64, c_int64, c_int64, c_int, c_int, c_float,
                               c_void_p, ctypes.POINTER(ctypes.c_int32), c_int, _pd]),
    "arhip_sage_fwd_strided": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                       ctypes.POINTER(c_int64), ctypes.POINTER(c_int64), c_void_p, c_void_p,
                                       c_int64, c_int64, c_int64, c_int64, c_int64, c_int64, c_int64, c_int, c_int, c_float,
                                       c_void_p, ctypes.POINTER(ctypes.c_int32), c_int, _pd]),
    "arhip_selections": (ctypes.c_uint64, [c_int]),
}

_lib = None


class ArhipError(RuntimeError):
    def __init__(self, code, message):
        super().__init__("TGERR: arhip %d: %s" % (code, message))
        self.code = code


class Unsupported(ArhipError):
    """The fused kernels do not cover this shape/dtype (the caller's cue to use the general path)."""


def load():
    """Load libarhip.so; raises if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise FileNotFoundError(
                "%s is missing: build it with `python -m autorust_amd.build` (needs hipcc)" % LIB_PATH)
        lib = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(lib, name)
            fn.restype = res
            fn.argtypes = args
        _lib = lib
    return _lib


def check(rc):
    if rc == OK:
        return
    msg = load().arhip_last_error().decode("utf-8", "replace")
    if rc == EUNSUPPORTED:
        raise Unsupported(rc, msg)
    raise ArhipError(rc, msg)
