"""Helpers shared by the GPU parity tests: move arrays through the C ABI and run
the typed entry points on them.  No computation happens here."""
import numpy as np

from autorust_amd import synth
from autorust_amd.device import BF16, F32


class Bufs:
    """Frees every device buffer it handed out."""

    def __init__(self, dev):
        self.dev = dev
        self.items = []

    def put(self, arr):
        b = self.dev.from_numpy(arr)
        self.items.append(b)
        return b

    def new(self, nbytes, zero=True):
        b = self.dev.alloc(max(int(nbytes), 4))
        if zero:
            b.zero()
        self.items.append(b)
        return b

    def free(self):
        for b in self.items:
            b.free()
        self.items = []

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.free()


def fill_qkv(B, Hq, Hkv, N, D):
    """The reference tests' inputs: fill(n, 3 / 11 / 19) (tests/flash_cuda_bf16.rs:125-127)."""
    q = synth.fill(B * Hq * N * D, 3).reshape(B, Hq, N, D)
    k = synth.fill(B * Hkv * N * D, 11).reshape(B, Hkv, N, D)
    v = synth.fill(B * Hkv * N * D, 19).reshape(B, Hkv, N, D)
    return q, k, v


def ref_mask(N):
    """tests/flash_cuda_masks.rs:249-253: ((i*7) % 23 - 11) * 0.05."""
    i = np.arange(N * N, dtype=np.int64)
    return (((i * 7) % 23).astype(np.float32) - np.float32(11.0)) * np.float32(0.05)


def run_flash(dev, q, k, v, dtype, mask=None, kv_len=None, causal=False, scale=None):
    B, Hq, N, D = q.shape
    Hkv = k.shape[1]
    with Bufs(dev) as bufs:
        if dtype == BF16:
            dq, dk, dv = (bufs.put(synth.to_bf16_bits(t)) for t in (q, k, v))
            do = bufs.new(q.size * 2)
        else:
            dq, dk, dv = (bufs.put(t.astype(np.float32)) for t in (q, k, v))
            do = bufs.new(q.size * 4)
        dm = bufs.put(np.ascontiguousarray(mask, np.float32)) if mask is not None else None
        dl = bufs.put(np.ascontiguousarray(kv_len, np.int32)) if kv_len is not None else None
        dev.flash_fwd(dq, dk, dv, do, B, Hq, Hkv, N, D, dtype, mask=dm, kv_len=dl, causal=causal, scale=scale)
        if dtype == BF16:
            return synth.from_bf16_bits(do.copyout(np.uint16, q.shape))
        return do.copyout(np.float32, q.shape)


def run_sage(dev, q, k, v, bq, bk, smooth=True, in_dtype=F32, out_dtype=F32, mask=None, kv_len=None, causal=False,
             dbg_sel=None, scale=None):
    """Quantise Q and K, cast V, run the int8 kernel; returns everything the checks need."""
    B, Hq, N, D = q.shape
    Hkv = k.shape[1]
    nqb, nkb = (N + bq - 1) // bq, (N + bk - 1) // bk
    with Bufs(dev) as bufs:
        if in_dtype == BF16:
            dq, dk = bufs.put(synth.to_bf16_bits(q)), bufs.put(synth.to_bf16_bits(k))
        else:
            dq, dk = bufs.put(q), bufs.put(k)
        dvf = bufs.put(v)
        dv = bufs.new(v.size * 2)
        dev.cast_bf16(dvf, dv, v.size)
        q8, k8 = bufs.new(q.size), bufs.new(k.size)
        sq, sk = bufs.new(B * Hq * nqb * 4), bufs.new(B * Hkv * nkb * 4)
        mean = bufs.new(B * Hkv * D * 4)
        ws = bufs.new(dev.sage_quant_workspace(B, Hkv, N, D))
        dev.sage_quant(dq, q8, sq, B, Hq, N, D, bq, in_dtype)
        dev.sage_quant(dk, k8, sk, B, Hkv, N, D, bk, in_dtype, mean=mean, workspace=ws, smooth=smooth)
        do = bufs.new(q.size * (4 if out_dtype == F32 else 2))
        dm = bufs.put(np.ascontiguousarray(mask, np.float32)) if mask is not None else None
        dl = bufs.put(np.ascontiguousarray(kv_len, np.int32)) if kv_len is not None else None
        dbg = bufs.new(32 * 64 * 4) if dbg_sel is not None else None
        dev.sage_fwd(q8, k8, sq, sk, dv, do, B, Hq, Hkv, N, D, bq, bk, out_dtype=out_dtype, mask=dm, kv_len=dl,
                     causal=causal, dbg_logits=dbg, dbg_sel=dbg_sel, scale=scale)
        res = {
            "q8": q8.copyout(np.int8, q.shape), "k8": k8.copyout(np.int8, k.shape),
            "sq": sq.copyout(np.float32, (B, Hq, nqb)), "sk": sk.copyout(np.float32, (B, Hkv, nkb)),
            "mean": mean.copyout(np.float32, (B, Hkv, D)),
            "vb": synth.from_bf16_bits(dv.copyout(np.uint16, v.shape)),
        }
        if out_dtype == F32:
            res["out"] = do.copyout(np.float32, q.shape)
        else:
            res["out"] = synth.from_bf16_bits(do.copyout(np.uint16, q.shape))
        if dbg is not None:
            res["logits"] = dbg.copyout(np.int32, (32, 64))
        return res


def bf16_ulps(got, want, floor=0.5):
    """Largest |got - want| in units of the bf16 step at max(|want|, floor), the step being
    2^(floor(log2 m) - 7).  A bf16-stored output that differs from the emulation only through
    rounding points is a couple of steps away at most; below `floor` the error is governed by
    the rounding of the probabilities (relative to sum p|v|, not to |o|), hence the floor.
    Three steps at the floor are 5.9e-3, the reference's 5e-3 (tests/flash_cuda_bf16.rs:131)."""
    mag = np.maximum(np.abs(want), floor)
    step = 2.0 ** (np.floor(np.log2(mag)) - 7)
    return float((np.abs(got - want) / step).max())


def max_abs(a, b):
    return float(np.abs(a - b).max())


def max_rel1(a, b):
    """max |a-b| / max(|b|, 1): the reference's closeness measure (tests/nn_attention.rs:11-24)."""
    return float((np.abs(a - b) / np.maximum(np.abs(b), 1.0)).max())
