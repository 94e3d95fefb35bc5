"""Python view of the C++ host layer (csrc/host/autorust_host.h): Tensor, Session,
AttentionKind and the attention entry points with the reference's names
(src/tensor/mod.rs:2045-2161, src/models/flash_attention.rs:292-747).  Thin ctypes calls;
the logic lives in C++ and computes through libarhip.so.
"""
import ctypes
import os

import numpy as np

from . import _lib

_HERE = os.path.dirname(os.path.abspath(__file__))
HOST_LIB_PATH = os.path.join(_HERE, "libautorust_host.so")
_host = None

FLOAT32, BFLOAT16, OTHER = 0, 1, 2
K_NONE, K_FLASH_F32, K_FLASH_BF16, K_SAGE = -1, 0, 1, 2


class AttentionKind:
    Sdpa, Flash, Sage = 0, 1, 2

    @staticmethod
    def name(k):
        return host().arh_attention_kind_name(k).decode()

    @staticmethod
    def from_str(s):
        return host().arh_attention_kind_from_str(s.encode())


class Settings(ctypes.Structure):
    _fields_ = [("attention", ctypes.c_int), ("tensor_cores", ctypes.c_int), ("async_pipeline", ctypes.c_int),
                ("math_exact", ctypes.c_int), ("sage_block_q", ctypes.c_int64), ("sage_block_k", ctypes.c_int64),
                ("sage_smooth_k", ctypes.c_int), ("sage_fp8", ctypes.c_int)]

    @staticmethod
    def default():
        s = Settings()
        host().arh_settings_default(ctypes.byref(s))
        return s

    @staticmethod
    def from_env():
        s = Settings()
        host().arh_settings_from_env(ctypes.byref(s))
        return s


def host():
    global _host
    if _host is None:
        _lib.load()  # libarhip.so first (the host library links against it)
        if not os.path.exists(HOST_LIB_PATH):
            raise FileNotFoundError("%s is missing: build it with `python -m autorust_amd.build`" % HOST_LIB_PATH)
        h = ctypes.CDLL(HOST_LIB_PATH)
        vp, ci, i64p = ctypes.c_void_p, ctypes.c_int, ctypes.POINTER(ctypes.c_int64)
        h.arh_last_error.restype = ctypes.c_char_p
        h.arh_attention_kind_name.restype = ctypes.c_char_p
        h.arh_attention_kind_name.argtypes = [ci]
        h.arh_attention_kind_from_str.argtypes = [ctypes.c_char_p]
        h.arh_device_open.restype = vp
        h.arh_device_open.argtypes = [ci]
        h.arh_device_close.argtypes = [vp]
        h.arh_device_raw_allocs.restype = ctypes.c_uint64
        h.arh_device_raw_allocs.argtypes = [vp]
        h.arh_tensor_from_slice.restype = vp
        h.arh_tensor_from_slice.argtypes = [vp, ctypes.c_void_p, i64p, ci, ci]
        h.arh_tensor_from_i32.restype = vp
        h.arh_tensor_from_i32.argtypes = [vp, ctypes.c_void_p, i64p, ci]
        h.arh_tensor_ptr.restype = vp
        h.arh_tensor_ptr.argtypes = [vp]
        h.arh_run_host_kernel.argtypes = [vp, ctypes.c_char_p, ctypes.c_char_p, ctypes.POINTER(vp), ci, i64p, ci, i64p, i64p, ci,
                                          ctypes.POINTER(ctypes.c_double)]
        h.arh_tensor_free.argtypes = [vp]
        h.arh_tensor_numel.restype = ctypes.c_int64
        h.arh_tensor_numel.argtypes = [vp]
        h.arh_tensor_dtype.argtypes = [vp]
        h.arh_tensor_shape.argtypes = [vp, i64p, ci]
        h.arh_tensor_to_list.argtypes = [vp, ctypes.c_void_p]
        h.arh_session_new.restype = vp
        for f in ("arh_session_free", "arh_session_begin_capture", "arh_session_end_capture", "arh_session_replay"):
            getattr(h, f).argtypes = [vp]
        h.arh_session_step_info.argtypes = [vp, ci, ctypes.c_char_p, ci, i64p, i64p]
        h.arh_session_step_detail.argtypes = [vp, ci, ctypes.c_char_p, ci, i64p, ctypes.POINTER(ci), ctypes.POINTER(ci),
                                              i64p, ci]
        h.arh_fused_attention.restype = vp
        h.arh_fused_attention.argtypes = [vp, vp, vp, ci, vp, ctypes.POINTER(Settings)]
        pvp = ctypes.POINTER(vp)
        h.arh_fused_attention_train.argtypes = [vp, vp, vp, vp, ci, vp, pvp, pvp]
        h.arh_fused_attention_backward.argtypes = [vp, vp, vp, vp, vp, vp, vp, ci, vp, pvp, pvp, pvp]
        h.arh_attention.restype = vp
        h.arh_attention.argtypes = [vp, vp, vp, vp, ctypes.c_double, ci, ci, vp, ctypes.POINTER(Settings), vp]
        h.arh_plan_fused.argtypes = [i64p, ci, i64p, ci, i64p, ci, ci, ci, ci, i64p, ci, ci, ci, ci,
                                     ctypes.POINTER(Settings), ctypes.POINTER(ci)]
        h.arh_wants_fused.argtypes = [ci, ctypes.POINTER(Settings), ctypes.c_double, ci, ctypes.POINTER(ci)]
        h.arh_selections.restype = ctypes.c_uint64
        h.arh_selections.argtypes = [ci]
        _host = h
    return _host


class HostError(RuntimeError):
    pass


def _err():
    return HostError(host().arh_last_error().decode("utf-8", "replace"))


def _i64(seq):
    return (ctypes.c_int64 * max(len(seq), 1))(*seq)


class HipDevice:
    """`device("HIP")` with the reference's free-list allocator."""

    def __init__(self, ordinal=0):
        self.h = host().arh_device_open(ordinal)
        if not self.h:
            raise _err()

    def close(self):
        if self.h:
            host().arh_device_close(self.h)
            self.h = None

    @property
    def raw_allocs(self):
        return int(host().arh_device_raw_allocs(self.h))

    def run_host_kernel(self, src, name, bufs, vals, global_, local, wait=True):
        """`Compiled::run_host_kernel` (src/runtime/device.rs:383-402) on Tensor buffers and 32-bit
        scalars; returns the elapsed device seconds, or None for a launch that did not wait."""
        ptrs = (ctypes.c_void_p * max(len(bufs), 1))(*[host().arh_tensor_ptr(b.h) for b in bufs])
        secs = ctypes.c_double(-1.0)
        if host().arh_run_host_kernel(self.h, src.encode(), name.encode(), ptrs, len(bufs), _i64(list(vals)), len(vals),
                                      _i64(list(global_)), _i64(list(local)), int(wait), ctypes.byref(secs)) != 0:
            raise _err()
        return None if secs.value < 0 else secs.value


class Session:
    def __init__(self):
        self.h = host().arh_session_new()

    def __del__(self):
        if getattr(self, "h", None):
            host().arh_session_free(self.h)
            self.h = None

    def begin_capture(self):
        host().arh_session_begin_capture(self.h)

    def end_capture(self):
        """Number of captured host launches (kept inside the session for replay)."""
        return host().arh_session_end_capture(self.h)

    def step(self, i):
        name = ctypes.create_string_buffer(64)
        g, v = (ctypes.c_int64 * 3)(), (ctypes.c_int64 * 6)()
        if host().arh_session_step_info(self.h, i, name, 64, g, v) != 0:
            raise IndexError(i)
        return name.value.decode(), list(g), list(v)

    def step_detail(self, i):
        """(code object path, local[3], number of buffers, number of scalars, [(slot, dtype), ...])."""
        src = ctypes.create_string_buffer(1024)
        loc, nb, nv = (ctypes.c_int64 * 3)(), ctypes.c_int(), ctypes.c_int()
        sig = (ctypes.c_int64 * 64)()
        n = host().arh_session_step_detail(self.h, i, src, 1024, loc, ctypes.byref(nb), ctypes.byref(nv), sig, 64)
        if n < 0:
            raise IndexError(i)
        return src.value.decode(), list(loc), nb.value, nv.value, [(sig[2 * j], sig[2 * j + 1]) for j in range(n)]

    def replay(self):
        if host().arh_session_replay(self.h) != 0:
            raise _err()


class Tensor:
    def __init__(self, h):
        self.h = h

    def __del__(self):
        if getattr(self, "h", None):
            host().arh_tensor_free(self.h)
            self.h = None

    @staticmethod
    def from_slice(dev, data, shape, dtype=FLOAT32):
        data = np.ascontiguousarray(data, dtype=np.float32)
        h = host().arh_tensor_from_slice(dev.h, data.ctypes.data, _i64(list(shape)), len(shape), dtype)
        if not h:
            raise _err()
        return Tensor(h)

    @staticmethod
    def from_i32(dev, data, shape=None):
        """An Int32 tensor (per-batch key lengths)."""
        data = np.ascontiguousarray(data, dtype=np.int32)
        shape = data.shape if shape is None else shape
        h = host().arh_tensor_from_i32(dev.h, data.ctypes.data, _i64(list(shape)), len(shape))
        if not h:
            raise _err()
        return Tensor(h)

    @property
    def shape(self):
        out = (ctypes.c_int64 * 8)()
        n = host().arh_tensor_shape(self.h, out, 8)
        return tuple(out[:n])

    @property
    def dtype(self):
        return host().arh_tensor_dtype(self.h)

    def to_list(self):
        out = np.empty(host().arh_tensor_numel(self.h), dtype=np.float32)
        if host().arh_tensor_to_list(self.h, out.ctypes.data) != 0:
            raise _err()
        return out.reshape(self.shape)

    def _call(self, api, k, v, mask, dropout_p, is_causal, sess, settings, key_lengths=None):
        st = settings if settings is not None else Settings.default()
        h = host().arh_attention(self.h, k.h, v.h, mask.h if mask is not None else None, float(dropout_p),
                                 int(is_causal), api, sess.h if sess is not None else None, ctypes.byref(st),
                                 key_lengths.h if key_lengths is not None else None)
        if not h:
            raise _err()
        return Tensor(h)

    def attention(self, k, v, mask=None, dropout_p=0.0, is_causal=False):
        return self._call(0, k, v, mask, dropout_p, is_causal, None, None)

    def attention_with(self, k, v, mask, dropout_p, is_causal, sess, settings=None, key_lengths=None):
        return self._call(1, k, v, mask, dropout_p, is_causal, sess, settings, key_lengths)

    def flash_attention_with(self, k, v, mask, dropout_p, is_causal, sess, settings=None, key_lengths=None):
        return self._call(2, k, v, mask, dropout_p, is_causal, sess, settings, key_lengths)

    def sage_attention_with(self, k, v, mask, dropout_p, is_causal, sess, settings=None, key_lengths=None):
        return self._call(3, k, v, mask, dropout_p, is_causal, sess, settings, key_lengths)


def fused_attention(q, k, v, sess, kind=None, settings=None):
    """`fused_attention` (kind None) / `fused_attention_kind`: a Tensor, or None when the fused
    kernels decline (src/models/flash_attention.rs:292-320)."""
    st = settings if settings is not None else Settings.default()
    h = host().arh_fused_attention(q.h, k.h, v.h, -1 if kind is None else int(kind), sess.h, ctypes.byref(st))
    if not h:
        msg = host().arh_last_error()
        if msg:
            raise HostError(msg.decode("utf-8", "replace"))
        return None
    return Tensor(h)


def _declined_or_raise(rc):
    if rc < 0:
        raise HostError(host().arh_last_error().decode("utf-8", "replace"))
    return rc == 0


def fused_attention_train(q, k, v, sess, mask=None, is_causal=False):
    """`fused_attention_train` (src/models/flash_attention.rs:789-870): (out, lse) or None."""
    out, lse = ctypes.c_void_p(), ctypes.c_void_p()
    rc = host().arh_fused_attention_train(q.h, k.h, v.h, mask.h if mask is not None else None, int(is_causal), sess.h,
                                          ctypes.byref(out), ctypes.byref(lse))
    if _declined_or_raise(rc):
        return None
    return Tensor(out.value), Tensor(lse.value)


def fused_attention_backward(q, k, v, out, lse, dout, sess, mask=None, is_causal=False):
    """`fused_attention_backward` (src/models/flash_attention.rs:872-977): (dq, dk, dv) or None."""
    dq, dk, dv = ctypes.c_void_p(), ctypes.c_void_p(), ctypes.c_void_p()
    rc = host().arh_fused_attention_backward(q.h, k.h, v.h, out.h, lse.h, dout.h, mask.h if mask is not None else None,
                                             int(is_causal), sess.h, ctypes.byref(dq), ctypes.byref(dk), ctypes.byref(dv))
    if _declined_or_raise(rc):
        return None
    return Tensor(dq.value), Tensor(dk.value), Tensor(dv.value)


def plan_fused(q, k, v, qd=FLOAT32, kd=None, vd=None, mask=None, mask_dtype=FLOAT32, enable_gqa=False, quantized=False,
               settings=None):
    """(kernel id, sage_declined): the gates of fused_attention_ex without a device."""
    kd = qd if kd is None else kd
    vd = qd if vd is None else vd
    st = settings if settings is not None else Settings.default()
    declined = ctypes.c_int()
    kern = host().arh_plan_fused(_i64(q), len(q), _i64(k), len(k), _i64(v), len(v), qd, kd, vd,
                                 _i64(mask) if mask is not None else None, len(mask) if mask is not None else 0,
                                 mask_dtype, int(enable_gqa), int(quantized), ctypes.byref(st), ctypes.byref(declined))
    return kern, bool(declined.value)


def wants_fused(force, settings, dropout_p, has_session):
    """(fused?, quantized?): the policy of Tensor::attention_kind."""
    st = settings if settings is not None else Settings.default()
    qz = ctypes.c_int()
    w = host().arh_wants_fused(-1 if force is None else force, ctypes.byref(st), float(dropout_p), int(has_session),
                               ctypes.byref(qz))
    return bool(w), bool(qz.value)


def selections(kernel):
    return int(host().arh_selections(kernel))
