"""Thin Python view of the C ABI: a device handle, device buffers and the typed
attention entry points.  Everything here calls libarhip.so; nothing computes on
the host.
"""
import ctypes

import numpy as np

from . import _lib
from ._lib import BF16, F32, check


class Buffer:
    """Caller-owned device memory (`OpaqueT`: base pointer + size, src/runtime/buffer.rs:32-39)."""

    def __init__(self, dev, nbytes):
        self.dev = dev
        self.nbytes = int(nbytes)
        p = ctypes.c_void_p()
        check(dev.lib.arhip_alloc(dev.handle, self.nbytes, ctypes.byref(p)))
        self.ptr = p.value or 0

    def free(self):
        if self.ptr and self.dev.handle:
            check(self.dev.lib.arhip_free(self.dev.handle, self.ptr))
        self.ptr = 0

    def copyin(self, arr):
        arr = np.ascontiguousarray(arr)
        assert arr.nbytes <= self.nbytes, (arr.nbytes, self.nbytes)
        check(self.dev.lib.arhip_copyin(self.dev.handle, self.ptr, arr.ctypes.data, arr.nbytes))
        return self

    def copyout(self, dtype, shape):
        out = np.empty(shape, dtype=dtype)
        assert out.nbytes <= self.nbytes, (out.nbytes, self.nbytes)
        check(self.dev.lib.arhip_copyout(self.dev.handle, out.ctypes.data, self.ptr, out.nbytes))
        return out

    def zero(self):
        check(self.dev.lib.arhip_fill_zero(self.dev.handle, self.ptr, self.nbytes))
        return self


class Device:
    """One MI355X (`device("HIP:n")`; the reference's registry is src/runtime/device.rs:635-689)."""

    def __init__(self, ordinal=0):
        self.lib = _lib.load()
        h = ctypes.c_void_p()
        check(self.lib.arhip_open(int(ordinal), ctypes.byref(h)))
        self.handle = h.value
        self.ordinal = int(ordinal)

    def close(self):
        if self.handle:
            check(self.lib.arhip_close(self.handle))
            self.handle = None

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()

    @property
    def arch(self):
        return self.lib.arhip_arch(self.handle).decode()

    @property
    def compute_units(self):
        return self.lib.arhip_compute_units(self.handle)

    def mem_info(self):
        f, t = ctypes.c_size_t(), ctypes.c_size_t()
        check(self.lib.arhip_mem_info(self.handle, ctypes.byref(f), ctypes.byref(t)))
        return f.value, t.value

    def alloc(self, nbytes):
        return Buffer(self, nbytes)

    def from_numpy(self, arr):
        arr = np.ascontiguousarray(arr)
        return Buffer(self, max(arr.nbytes, 1)).copyin(arr)

    def sync(self):
        check(self.lib.arhip_sync(self.handle))

    def timer_start(self):
        check(self.lib.arhip_timer_start(self.handle))

    def timer_stop(self):
        s = ctypes.c_double()
        check(self.lib.arhip_timer_stop(self.handle, ctypes.byref(s)))
        return s.value

    def kprof_enable(self, on=True):
        check(self.lib.arhip_kprof_enable(self.handle, int(on)))

    def kprof_collect_stats(self, kernel):
        """(total seconds, launches, shortest, median) of `kernel` since the last collect."""
        s, n, lo, med = ctypes.c_double(), ctypes.c_uint64(), ctypes.c_double(), ctypes.c_double()
        check(self.lib.arhip_kprof_collect_stats(self.handle, kernel, ctypes.byref(s), ctypes.byref(n), ctypes.byref(lo),
                                                 ctypes.byref(med)))
        return s.value, n.value, lo.value, med.value

    def kprof_collect(self, kernel):
        """(total seconds, launches) of `kernel` since the last collect."""
        s, n = ctypes.c_double(), ctypes.c_uint64()
        check(self.lib.arhip_kprof_collect(self.handle, kernel, ctypes.byref(s), ctypes.byref(n)))
        return s.value, n.value

    # ---- launch graphs ----
    def graph_begin(self):
        check(self.lib.arhip_graph_begin(self.handle))

    def graph_end(self):
        g = ctypes.c_void_p()
        check(self.lib.arhip_graph_end(self.handle, ctypes.byref(g)))
        return g.value

    def graph_launch(self, graph, wait=True):
        s = ctypes.c_double()
        check(self.lib.arhip_graph_launch(self.handle, graph, int(wait), ctypes.byref(s)))
        return s.value if wait else None

    def graph_destroy(self, graph):
        check(self.lib.arhip_graph_destroy(self.handle, graph))

    # ---- generic launch (run_host_kernel) ----
    def module_load(self, image):
        m = ctypes.c_void_p()
        buf = ctypes.create_string_buffer(image, len(image))
        check(self.lib.arhip_module_load(self.handle, buf, len(image), ctypes.byref(m)))
        return m.value

    def launch(self, module, name, grid, block, bufs, vals=(), val_bits=None, wait=True):
        g = (ctypes.c_uint * 3)(*grid)
        b = (ctypes.c_uint * 3)(*block)
        bp = (ctypes.c_void_p * max(len(bufs), 1))(*[x.ptr if isinstance(x, Buffer) else x for x in bufs])
        vals = list(vals)
        val_bits = [32] * len(vals) if val_bits is None else list(val_bits)
        va = (ctypes.c_int64 * max(len(vals), 1))(*vals)
        vb = (ctypes.c_int * max(len(vals), 1))(*val_bits)
        s = ctypes.c_double()
        check(self.lib.arhip_launch(self.handle, module, name.encode(), g, b, bp, len(bufs), va, vb, len(vals),
                                    int(wait), ctypes.byref(s)))
        return s.value if wait else None

    # ---- typed attention entry points ----
    @staticmethod
    def _ptr(x):
        if x is None:
            return None
        return x.ptr if isinstance(x, Buffer) else int(x)

    def flash_fwd(self, q, k, v, o, B, Hq, Hkv, N, D, dtype, mask=None, kv_len=None, causal=False, scale=None,
                  wait=True):
        scale = float(1.0 / np.sqrt(np.float32(D))) if scale is None else float(scale)
        s = ctypes.c_double()
        check(self.lib.arhip_flash_fwd(self.handle, self._ptr(q), self._ptr(k), self._ptr(v), self._ptr(o),
                                       self._ptr(mask), self._ptr(kv_len), B, Hq, Hkv, N, D, int(causal), dtype,
                                       scale, int(wait), ctypes.byref(s)))
        return s.value if wait else None

    def flash_fwd_strided(self, q, k, v, o, q_strides, kv_strides, o_strides, B, Hq, Hkv, N, D, dtype, mask=None,
                          kv_len=None, causal=False, scale=None, wait=True):
        """Element strides {batch, head, token} per tensor; see include/arhip.h."""
        scale = float(1.0 / np.sqrt(np.float32(D))) if scale is None else float(scale)
        arr = lambda t: (ctypes.c_int64 * 3)(*[int(x) for x in t])
        s = ctypes.c_double()
        check(self.lib.arhip_flash_fwd_strided(self.handle, self._ptr(q), self._ptr(k), self._ptr(v), self._ptr(o),
                                               arr(q_strides), arr(kv_strides), arr(o_strides), self._ptr(mask),
                                               self._ptr(kv_len), B, Hq, Hkv, N, D, int(causal), dtype, scale,
                                               int(wait), ctypes.byref(s)))
        return s.value if wait else None

    def flash_bwd(self, q, k, v, o, lse, dout, dq, dk, dv, delta, B, Hq, Hkv, N, D, mask=None, kv_len=None,
                  causal=False, scale=None, wait=True):
        """f32 dense [B,H,N,D]; o and lse from flash_fwd_lse of the same call; delta: B*Hq*N floats of scratch."""
        scale = float(1.0 / np.sqrt(np.float32(D))) if scale is None else float(scale)
        s = ctypes.c_double()
        check(self.lib.arhip_flash_bwd(self.handle, self._ptr(q), self._ptr(k), self._ptr(v), self._ptr(o),
                                       self._ptr(lse), self._ptr(dout), self._ptr(dq), self._ptr(dk), self._ptr(dv),
                                       self._ptr(delta), self._ptr(mask), self._ptr(kv_len), B, Hq, Hkv, N, D,
                                       int(causal), scale, int(wait), ctypes.byref(s)))
        return s.value if wait else None

    def flash_fwd_lse(self, q, k, v, o, lse, B, Hq, Hkv, N, D, dtype, mask=None, kv_len=None, causal=False,
                      scale=None, wait=True):
        """Dense [B,H,N,D] tensors; also writes lse [B,Hq,N] (f32)."""
        scale = float(1.0 / np.sqrt(np.float32(D))) if scale is None else float(scale)
        arr = lambda t: (ctypes.c_int64 * 3)(*[int(x) for x in t])
        qs, ks = (Hq * N * D, N * D, D), (Hkv * N * D, N * D, D)
        s = ctypes.c_double()
        check(self.lib.arhip_flash_fwd_lse(self.handle, self._ptr(q), self._ptr(k), self._ptr(v), self._ptr(o),
                                           self._ptr(lse), arr(qs), arr(ks), arr(qs), self._ptr(mask),
                                           self._ptr(kv_len), B, Hq, Hkv, N, D, int(causal), dtype, scale,
                                           int(wait), ctypes.byref(s)))
        return s.value if wait else None

    def sage_quant_workspace(self, B, H, N, D):
        return self.lib.arhip_sage_quant_workspace(B, H, N, D)

    def sage_quant(self, x, x8, scales, B, H, N, D, block, dtype, mean=None, workspace=None, smooth=False, wait=True,
                   x_strides=None):
        """x_strides: element strides {batch, head, token} of x (None = dense [B,H,N,D])."""
        s = ctypes.c_double()
        if x_strides is None:
            check(self.lib.arhip_sage_quant(self.handle, self._ptr(x), self._ptr(x8), self._ptr(scales), self._ptr(mean),
                                            self._ptr(workspace), B, H, N, D, block, dtype, int(smooth), int(wait),
                                            ctypes.byref(s)))
        else:
            xs = (ctypes.c_int64 * 3)(*[int(t) for t in x_strides])
            check(self.lib.arhip_sage_quant_strided(self.handle, self._ptr(x), xs, self._ptr(x8), self._ptr(scales),
                                                    self._ptr(mean), self._ptr(workspace), B, H, N, D, block, dtype,
                                                    int(smooth), int(wait), ctypes.byref(s)))
        return s.value if wait else None

    def sage_quant_fp8(self, x, x8, scales, B, H, N, D, block, dtype, mean=None, workspace=None, smooth=False, wait=True):
        """sage_quant with FP8 E4M3 codes (scale = absmax / 448) instead of int8 values."""
        s = ctypes.c_double()
        check(self.lib.arhip_sage_quant_fp8(self.handle, self._ptr(x), self._ptr(x8), self._ptr(scales), self._ptr(mean),
                                            self._ptr(workspace), B, H, N, D, block, dtype, int(smooth), int(wait),
                                            ctypes.byref(s)))
        return s.value if wait else None

    def sage_fwd_fp8(self, q8, k8, sq, sk, v, o, B, Hq, Hkv, N, D, bq, bk, out_dtype=F32, mask=None, kv_len=None,
                     causal=False, scale=None, wait=True):
        scale = float(1.0 / np.sqrt(np.float32(D))) if scale is None else float(scale)
        s = ctypes.c_double()
        check(self.lib.arhip_sage_fwd_fp8(self.handle, self._ptr(q8), self._ptr(k8), self._ptr(sq), self._ptr(sk),
                                          self._ptr(v), self._ptr(o), self._ptr(mask), self._ptr(kv_len),
                                          B, Hq, Hkv, N, D, bq, bk, int(causal), out_dtype, scale, int(wait),
                                          ctypes.byref(s)))
        return s.value if wait else None

    def sage_fwd_qfused(self, q, k8, sk, v, o, B, Hq, Hkv, N, D, bk, out_dtype=BF16, sq_out=None, q8_out=None, kv_len=None,
                        causal=False, scale=None, wait=True, fp8=False):
        """sage_quant of Q (bf16, blocks of 128 queries) inside the attention kernel; sq_out / q8_out receive the
        scales and codes it derived.  fp8: E4M3 codes (k8 from sage_quant_fp8)."""
        scale = float(1.0 / np.sqrt(np.float32(D))) if scale is None else float(scale)
        s = ctypes.c_double()
        fn = self.lib.arhip_sage_fwd_fp8_qfused if fp8 else self.lib.arhip_sage_fwd_qfused
        check(fn(self.handle, self._ptr(q), self._ptr(k8), self._ptr(sk), self._ptr(v), self._ptr(o),
                 self._ptr(sq_out), self._ptr(q8_out), self._ptr(kv_len), B, Hq, Hkv, N, D, bk,
                 int(causal), out_dtype, scale, int(wait), ctypes.byref(s)))
        return s.value if wait else None

    def sage_prep_kv_rows(self, k, k8, sk, v, vb, B, Hkv, N, D, wait=True):
        """K quantised row by row (no smoothing) and V cast to bf16 in one launch (f32 tensors)."""
        s = ctypes.c_double()
        check(self.lib.arhip_sage_prep_kv_rows(self.handle, self._ptr(k), self._ptr(k8), self._ptr(sk), self._ptr(v), self._ptr(vb),
                                               B, Hkv, N, D, int(wait), ctypes.byref(s)))
        return s.value if wait else None

    def sage_fwd_qfused_rows(self, q, k8, sk, v, o, B, Hq, Hkv, N, D, bk, out_dtype=F32, sq_out=None, q8_out=None, kv_len=None,
                             causal=False, scale=None, wait=True):
        """The reference's convention in one attention launch: f32 q quantised row by row inside the kernel, K scales
        per key (bk a power of two below 64)."""
        scale = float(1.0 / np.sqrt(np.float32(D))) if scale is None else float(scale)
        s = ctypes.c_double()
        check(self.lib.arhip_sage_fwd_qfused_rows(self.handle, self._ptr(q), self._ptr(k8), self._ptr(sk), self._ptr(v),
                                                  self._ptr(o), self._ptr(sq_out), self._ptr(q8_out), self._ptr(kv_len),
                                                  B, Hq, Hkv, N, D, bk, int(causal), out_dtype, scale, int(wait), ctypes.byref(s)))
        return s.value if wait else None

    def sage_quant_static(self, x, x8, scales, B, H, N, D, block, dtype, mean=None, smooth=False, wait=True):
        """sage_quant with the partial sums in the library's own device array (no allocation)."""
        s = ctypes.c_double()
        check(self.lib.arhip_sage_quant_static(self.handle, self._ptr(x), self._ptr(x8), self._ptr(scales),
                                               self._ptr(mean), B, H, N, D, block, dtype, int(smooth), int(wait),
                                               ctypes.byref(s)))
        return s.value if wait else None

    def cast_bf16(self, x, y, n, wait=True):
        s = ctypes.c_double()
        check(self.lib.arhip_cast_bf16(self.handle, self._ptr(x), self._ptr(y), n, int(wait), ctypes.byref(s)))
        return s.value if wait else None

    def sage_fwd(self, q8, k8, sq, sk, v, o, B, Hq, Hkv, N, D, bq, bk, out_dtype=F32, mask=None, kv_len=None,
                 causal=False, scale=None, dbg_logits=None, dbg_sel=None, wait=True, v_strides=None, o_strides=None):
        scale = float(1.0 / np.sqrt(np.float32(D))) if scale is None else float(scale)
        sel = None
        if dbg_sel is not None:
            sel = (ctypes.c_int32 * 3)(*dbg_sel)
        s = ctypes.c_double()
        arr = lambda t: None if t is None else (ctypes.c_int64 * 3)(*[int(x) for x in t])
        check(self.lib.arhip_sage_fwd_strided(self.handle, self._ptr(q8), self._ptr(k8), self._ptr(sq), self._ptr(sk),
                                              self._ptr(v), self._ptr(o), arr(v_strides), arr(o_strides),
                                              self._ptr(mask), self._ptr(kv_len),
                                              B, Hq, Hkv, N, D, bq, bk, int(causal), out_dtype, scale,
                                              self._ptr(dbg_logits), sel, int(wait), ctypes.byref(s)))
        return s.value if wait else None


def selections(kernel):
    return int(_lib.load().arhip_selections(kernel))


def attn_supported(kind, n, d, dtype):
    return bool(_lib.load().arhip_attn_supported(kind, n, d, dtype))
