#!/usr/bin/env python3
"""Benchmark of the fused attention forward on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME] [--no-secondary] [--no-cpu]

A "step" is one pass of the hot path over one batch of synthetic input that is
already resident in HBM.  The headline workload is the Sage INT8 forward at
B=4, H=32, S=8192, D=128 (the shape the metric and the target are quoted on):
quantise Q per 128 tokens, smooth + quantise K per 64 tokens, then the int8
attention kernel.  One JSON line is printed; the other single-GPU
configurations are reported in its "secondary" array.

Work model: ops = 4*B*H*S^2*D (half for causal); bytes = Q, K, V read once and
O written once at their storage types.
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

from autorust_amd import _lib, synth  # noqa: E402
from autorust_amd.device import BF16, F32, Device  # noqa: E402

PEAK_BF16 = 2500.0   # TFLOP/s, MI355X dense bf16 MFMA
PEAK_F32 = 157.3     # TFLOP/s, MI355X dense fp32 MFMA
PEAK_INT8 = 5000.0   # TOP/s, MI355X dense int8 MFMA (dense fp8 MFMA: the same 5000 TFLOP/s)
PEAK_HBM = 8000.0    # GB/s, MI355X HBM3E

# HBM bytes per launch of the dominant kernel, measured with rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE
# and calibrated against a 1 GiB copy kernel (profiles/attn_pipe_s8192_hbm_traffic.md).
MEASURED_TRAFFIC = {"sage_int8_b4_h32_s8192_d128": 940.0e6}


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def attn_ops(B, H, S, D, causal):
    return 4.0 * B * H * S * S * D / (2.0 if causal else 1.0)


class SageWorkload:
    """SageAttention INT8 forward: Q ~ N(0,1), K = N(0,1) + per-(head,channel) bias ~ N(0, sigma),
    V ~ N(0,1); all three stored as bf16; O bf16."""

    def __init__(self, dev, B, H, S, D, causal, sigma, outliers, cfg, bq=128, bk=64, f32_io=False, fp8=False):
        self.dev, self.B, self.H, self.S, self.D, self.causal = dev, B, H, S, D, causal
        self.bq, self.bk = bq, bk
        self.fp8 = fp8  # E4M3 codes instead of int8 (the reference's AR_FP8 build of the same kernel)
        # f32_io: the reference's own convention (f32 tensors in, f32 out, per-row scales, no smoothing)
        self.f32_io = f32_io
        self.name = "sage_%s_b%d_h%d_s%d_d%d%s%s" % ("fp8" if fp8 else "int8", B, H, S, D, "_causal" if causal else "",
                                                      "_f32io_rowscales" if f32_io else "")
        n = B * H * S * D
        base = 1000 * cfg
        q = synth.normal(base + 1, (B, H, S, D))
        k = synth.normal(base + 2, (B, H, S, D))
        k += np.float32(sigma) * synth.normal(base + 4, (1, H, 1, D))
        if outliers:
            for t, seed in ((q, base + 6), (k, base + 7)):
                flat = t.reshape(-1)
                for o in range(0, n, 1 << 24):
                    m = min(1 << 24, n - o)
                    hit = synth.uniform(seed, m, o) < outliers
                    flat[o:o + m][hit] *= np.float32(20.0)
        self.host = {"q": q, "k": k}
        v = synth.normal(base + 3, (B, H, S, D))
        self.host["v"] = v
        if f32_io:
            self.dq, self.dk, self.dvf = dev.from_numpy(q), dev.from_numpy(k), dev.from_numpy(v)
            self.dv = dev.alloc(n * 2)
            self.do = dev.alloc(n * 4)
        else:
            self.dq = dev.from_numpy(synth.to_bf16_bits(q))
            self.dk = dev.from_numpy(synth.to_bf16_bits(k))
            self.dvf = None
            self.dv = dev.from_numpy(synth.to_bf16_bits(v))
            self.do = dev.alloc(n * 2)
        self.q8, self.k8 = dev.alloc(n), dev.alloc(n)
        self.sq = dev.alloc(B * H * ((S + bq - 1) // bq) * 4)
        self.sk = dev.alloc(B * H * ((S + bk - 1) // bk) * 4)
        self.mean = dev.alloc(B * H * D * 4)
        self.ws = dev.alloc(dev.sage_quant_workspace(B, H, S, D))
        self.ops = attn_ops(B, H, S, D, causal)
        self.kernel = _lib.K_SAGE
        # dominant kernel: int8 K (1 B), Q as int8 codes (1 B) or, quantised in its prologue, bf16 (2 B), bf16 V and O
        # (2 B), block scales
        q_bytes = 2 if (not f32_io and bq == 128 and bk % 64 == 0) else 4 if (f32_io and bq == 1 and bk == 1) else 1
        self.kernel_bytes = n * (q_bytes + 1 + 2 + 2) + 4 * B * H * (S // bq + S // bk)
        self.dtype = "fp8" if fp8 else "int8"

    def step(self):
        d, B, H, S, D = self.dev, self.B, self.H, self.S, self.D
        io = F32 if self.f32_io else BF16
        if self.fp8:
            d.sage_quant_fp8(self.dk, self.k8, self.sk, B, H, S, D, self.bk, io, mean=self.mean, workspace=self.ws,
                             smooth=True, wait=False)
            if not self.f32_io and self.bq == 128 and self.bk % 64 == 0:
                d.sage_fwd_qfused(self.dq, self.k8, self.sk, self.dv, self.do, B, H, H, S, D, self.bk, out_dtype=io,
                                  sq_out=self.sq, causal=self.causal, wait=False, fp8=True)
                return
            d.sage_quant_fp8(self.dq, self.q8, self.sq, B, H, S, D, self.bq, io, wait=False)
            d.sage_fwd_fp8(self.q8, self.k8, self.sq, self.sk, self.dv, self.do, B, H, H, S, D, self.bq, self.bk,
                           out_dtype=io, causal=self.causal, wait=False)
            return
        # bf16 queries with scales over blocks of 128: the attention kernel quantises Q itself (as the host mirror's
        # Tensor::sage_attention_with does); otherwise the Q quantiser is a launch of its own
        q_fused = not self.f32_io and self.bq == 128 and self.bk % 64 == 0 and not self.fp8
        if self.f32_io and self.bq == 1 and self.bk == 1:
            # the reference's convention in two launches: K's per-key quantiser together with V's cast, then the
            # attention kernel, which quantises the f32 queries row by row in its prologue
            d.sage_prep_kv_rows(self.dk, self.k8, self.sk, self.dvf, self.dv, B, H, S, D, wait=False)
            d.sage_fwd_qfused_rows(self.dq, self.k8, self.sk, self.dv, self.do, B, H, H, S, D, self.bk, out_dtype=io,
                                   sq_out=self.sq, causal=self.causal, wait=False)
            return
        if not q_fused:
            d.sage_quant(self.dq, self.q8, self.sq, B, H, S, D, self.bq, io, wait=False)
        d.sage_quant(self.dk, self.k8, self.sk, B, H, S, D, self.bk, io, mean=self.mean, workspace=self.ws,
                     smooth=not self.f32_io, wait=False)
        if self.f32_io:
            d.cast_bf16(self.dvf, self.dv, B * H * S * D, wait=False)
        if q_fused:
            d.sage_fwd_qfused(self.dq, self.k8, self.sk, self.dv, self.do, B, H, H, S, D, self.bk, out_dtype=io,
                              sq_out=self.sq, causal=self.causal, wait=False)
        else:
            d.sage_fwd(self.q8, self.k8, self.sq, self.sk, self.dv, self.do, B, H, H, S, D, self.bq, self.bk,
                       out_dtype=io, causal=self.causal, wait=False)

    def roofline(self, secs):
        half = self.ops / 2.0
        t_min = half / (PEAK_INT8 * 1e12) + half / (PEAK_BF16 * 1e12)
        ach = self.ops / secs / 1e12
        return {"bound": "mfma", "achieved": ach, "peak": PEAK_INT8, "unit": "TOP/s", "frac": ach / PEAK_INT8,
                "traffic": MEASURED_TRAFFIC.get(self.name), "traffic_source": "rocprofv3 --pmc profile (profiles/), not this run",
                "kernel": "attn_pipe_kernel<int8, per-key scales>" if self.bk == 1 else "attn_pipe_kernel<%s>" % self.dtype, "launch_ms": secs * 1e3,
                "ops_per_launch": self.ops, "peak_note": "dense %s MFMA; half of the ops are bf16 (P.V)" % self.dtype,
                "frac_of_mixed_int8_bf16_bound": t_min / secs}

    def free(self):
        for b in (self.dq, self.dk, self.dv, self.dvf, self.do, self.q8, self.k8, self.sq, self.sk, self.mean, self.ws):
            if b is not None:
                b.free()


class FlashWorkload:
    """FlashAttention forward, bf16 or fp32 tensors, Q/K/V ~ N(0,1)."""

    def __init__(self, dev, B, H, S, D, causal, dtype, cfg, kv_lens=False):
        self.dev, self.B, self.H, self.S, self.D, self.causal, self.dt = dev, B, H, S, D, causal, dtype
        tag = "bf16" if dtype == BF16 else "f32"
        self.name = "flash_%s_b%d_h%d_s%d_d%d%s%s" % (tag, B, H, S, D, "_causal" if causal else "",
                                                       "_kvlen" if kv_lens else "")
        n = B * H * S * D
        base = 1000 * cfg
        arrs = [synth.normal(base + i, (B, H, S, D)) for i in (1, 2, 3)]
        self.host = dict(zip("qkv", arrs))
        if dtype == BF16:
            self.dq, self.dk, self.dv = (dev.from_numpy(synth.to_bf16_bits(a)) for a in arrs)
        else:
            self.dq, self.dk, self.dv = (dev.from_numpy(a) for a in arrs)
        es = 2 if dtype == BF16 else 4
        self.do = dev.alloc(n * es)
        self.kv = None
        if kv_lens:
            self.kv_host = synth.randint(base + 5, B, S // 2, S)
            self.kv = dev.from_numpy(self.kv_host)
        self.ops = attn_ops(B, H, S, D, causal)
        if kv_lens:
            # visible (query, key) pairs: key j < L[b] and, under the causal mask, j <= i
            q = np.arange(S, dtype=np.int64)
            pairs = sum(int(np.minimum(q + 1, int(L)).sum()) if causal else S * int(L) for L in self.kv_host)
            self.ops = 4.0 * H * D * pairs
        self.kernel = _lib.K_FLASH_BF16 if dtype == BF16 else _lib.K_FLASH_F32
        self.kernel_bytes = 4 * n * es
        self.dtype = tag

    def step(self):
        self.dev.flash_fwd(self.dq, self.dk, self.dv, self.do, self.B, self.H, self.H, self.S, self.D, self.dt,
                           kv_len=self.kv, causal=self.causal, wait=False)

    def roofline(self, secs):
        # the bound is the larger of ops / matrix peak and bytes / HBM rate (fp32 tensors: fp32 MFMA peak)
        ai = self.ops / self.kernel_bytes
        peak = PEAK_BF16 if self.dt == BF16 else PEAK_F32
        if ai > peak * 1e12 / (PEAK_HBM * 1e9):
            ach = self.ops / secs / 1e12
            kern = "flash_f32_kernel" if self.dt != BF16 else "attn_pipe_kernel<bf16>"
            return {"bound": "mfma", "achieved": ach, "peak": peak, "unit": "TFLOP/s", "frac": ach / peak,
                    "traffic": None, "kernel": kern, "launch_ms": secs * 1e3, "ops_per_launch": self.ops,
                    "peak_note": "dense %s MFMA" % self.dtype}
        ach = self.kernel_bytes / secs / 1e9
        return {"bound": "hbm", "achieved": ach, "peak": PEAK_HBM, "unit": "GB/s", "frac": ach / PEAK_HBM,
                "traffic": None, "kernel": "attn_pipe_kernel<bf16>" if self.dt == BF16 else "flash_f32_kernel",
                "launch_ms": secs * 1e3, "bytes_per_launch": self.kernel_bytes,
                "tflops": self.ops / secs / 1e12}

    def free(self):
        for b in (self.dq, self.dk, self.dv, self.do, self.kv):
            if b is not None:
                b.free()


class TrainWorkload:
    """fp32 training step of one attention layer: forward with the saved log-sum-exp, then the
    backward (prep + dQ + dK/dV): src/runtime/cuda_flash_train.rs.  14 B H S^2 D flops per step:
    2 products forward, 5 backward (S and dP are each computed by both backward kernels)."""

    def __init__(self, dev, B, H, S, D, causal, cfg):
        self.dev, self.B, self.H, self.S, self.D, self.causal = dev, B, H, S, D, causal
        self.name = "train_f32_b%d_h%d_s%d_d%d%s" % (B, H, S, D, "_causal" if causal else "")
        n = B * H * S * D
        arrs = [synth.normal(1000 * cfg + i, (B, H, S, D)) for i in (1, 2, 3, 8)]
        self.host = dict(zip("qkv", arrs[:3]))
        self.dq, self.dk, self.dv, self.ddo = (dev.from_numpy(a) for a in arrs)
        self.o, self.gq, self.gk, self.gv = (dev.alloc(n * 4) for _ in range(4))
        self.lse, self.delta = dev.alloc(B * H * S * 4), dev.alloc(B * H * S * 4)
        self.ops = 14.0 * B * H * S * S * D * (0.5 if causal else 1.0)
        self.kernel = _lib.K_FLASH_BWD
        self.kernel_bytes = 8 * n * 4   # backward: q, k, v, o, dO in; dq, dk, dv out
        self.dtype = "f32"

    def step(self):
        d, B, H, S, D = self.dev, self.B, self.H, self.S, self.D
        d.flash_fwd_lse(self.dq, self.dk, self.dv, self.o, self.lse, B, H, H, S, D, F32, causal=self.causal, wait=False)
        d.flash_bwd(self.dq, self.dk, self.dv, self.o, self.lse, self.ddo, self.gq, self.gk, self.gv, self.delta,
                    B, H, H, S, D, causal=self.causal, wait=False)

    def roofline(self, secs):
        bwd_ops = self.ops * 10.0 / 14.0
        ach = bwd_ops / secs / 1e12
        return {"bound": "mfma", "achieved": ach, "peak": PEAK_F32, "unit": "TFLOP/s", "frac": ach / PEAK_F32,
                "traffic": None, "kernel": "bwd_prep + bwd_dq + bwd_dkv (f32)", "launch_ms": secs * 1e3,
                "ops_per_launch": bwd_ops, "peak_note": "dense fp32 MFMA"}

    def free(self):
        for b in (self.dq, self.dk, self.dv, self.ddo, self.o, self.gq, self.gk, self.gv, self.lse, self.delta):
            b.free()


def measure(dev, w, steps, warmup):
    for _ in range(warmup):
        w.step()
    dev.sync()
    dev.kprof_enable(True)
    for k in range(_lib.K_FLASH_BWD + 1):
        dev.kprof_collect(k)
    dev.timer_start()
    for _ in range(steps):
        w.step()
    total = dev.timer_stop()
    ksecs, kn, kmin, kmed = dev.kprof_collect_stats(w.kernel)
    qsecs, qn = dev.kprof_collect(_lib.K_SAGE_QUANT)
    dev.kprof_enable(False)
    ms = total / steps * 1e3
    res = {"workload": w.name, "ms_per_step": ms, "ops_per_step": w.ops,
           "tops": w.ops / (total / steps) / 1e12,
           "roofline": w.roofline(ksecs / max(kn, 1))}
    res["roofline"]["launch_ms_min"] = kmin * 1e3
    res["roofline"]["launch_ms_median"] = kmed * 1e3
    if qn:
        res["prepass_ms_per_step"] = qsecs / steps * 1e3
    if w.S < 1024:
        # launch-bound shapes: the same steps recorded once into a HIP graph and replayed as one
        # submission (the reference's captured replay, src/engine/jit.rs:186-195), so that the
        # per-launch host overhead drops out of the step time
        dev.graph_begin()
        for _ in range(steps):
            w.step()
        g = dev.graph_end()
        dev.graph_launch(g)
        reps = 5
        secs = min(dev.graph_launch(g) for _ in range(reps))
        dev.graph_destroy(g)
        res["ms_per_step_graph_replay"] = secs / steps * 1e3
    return res


def _probes(dev):
    return dev.module_load(open(_lib.PROBES_PATH, "rb").read())


def sustained_mfma(dev):
    """Dense bf16 MFMA rate and shader clock of a loop of nothing but matrix instructions, on
    constant and on random operands (probe_mfma_rate in csrc/probes.hip): what the power limit
    leaves of the published peak."""
    mod = _probes(dev)
    out, ticks = dev.alloc(256 * 512 * 4), dev.alloc(256 * 16)
    res = {}
    for name, data in (("constant", np.full(8192 * 8, 0x3F80, np.uint16)),
                       ("random", synth.to_bf16_bits(synth.normal(99, (8192 * 8,))))):
        src = dev.from_numpy(data)
        iters = 100000
        dev.launch(mod, "probe_mfma_rate", (256, 1, 1), (512, 1, 1), [src, out, ticks], [iters])
        t = dev.launch(mod, "probe_mfma_rate", (256, 1, 1), (512, 1, 1), [src, out, ticks], [iters])
        c = ticks.copyout(np.int64, (256, 2))
        res[name] = {"tflops": 256 * 8 * iters * 8 * 32768 / t / 1e12,
                     "shader_clock_mhz": float((c[:, 0] / c[:, 1]).mean() * 100.0)}
        src.free()
    out.free()
    ticks.free()
    return res


def issue_mix(dev):
    """Cost per matrix instruction of a loop of { 1 MFMA ; K vector instructions } for K = 0..18
    (probe_mix_* in csrc/probes.hip) with one, two (the attention kernels) and three waves per SIMD,
    operands with random mantissas: how much vector work fits beside the matrix pipe before the loop
    slows down.  Every entry is [shader-clock cycles, nanoseconds, shader clock in MHz] per matrix
    instruction per SIMD: the cycles tell an issue limit from a clock (power) limit."""
    mod = _probes(dev)
    rng = np.random.default_rng(5)
    bits = (rng.integers(0, 1 << 16, 8192 * 8, dtype=np.uint32) & 0x007F) | 0x3C00     # bf16 values in [0.0078, 0.0156)
    src = dev.from_numpy(bits.astype(np.uint16))
    out, ticks = dev.alloc(256 * 768 * 4), dev.alloc(256 * 12 * 16)
    iters = 2000
    res = {}
    for waves in (2, 1, 3):
        for mat in ("bf16", "i8"):
            for op in ("fma", "exp"):
                row = {}
                for k in (0, 2, 4, 6, 8, 10, 14, 18):
                    name = "probe_mix_%s_%s_k%d" % (mat, op, k)
                    for _ in range(2):
                        dev.launch(mod, name, (256, 1, 1), (256 * waves, 1, 1), [src, out, ticks], [iters])
                    t = ticks.copyout(np.int64, (256 * 4 * waves, 2)).astype(np.float64).mean(axis=0)
                    # 4 matrix instructions per iteration; `waves` waves share a SIMD; real-time ticks are 10 ns
                    cyc, ns = t[0] / (iters * 4) / waves, t[1] * 10.0 / (iters * 4) / waves
                    row["K=%d" % k] = [round(float(cyc), 1), round(float(ns), 2), round(float(t[0] / t[1] * 100.0))]
                res["%s_mfma+%s_%dwaves" % (mat, op, waves)] = row
    # scalar instructions: bf16 MFMA + 8 v_fma_f32 + S s_add_u32 per matrix instruction, two waves per SIMD
    row = {}
    for sc in (0, 2, 4, 8):
        for _ in range(2):
            dev.launch(mod, "probe_mix_salu_s%d" % sc, (256, 1, 1), (512, 1, 1), [src, out, ticks], [iters])
        t = ticks.copyout(np.int64, (256 * 8, 2)).astype(np.float64).mean(axis=0)
        row["S=%d" % sc] = [round(float(t[0] / (iters * 4) / 2), 1), round(float(t[1] * 10.0 / (iters * 4) / 2), 2),
                            round(float(t[0] / t[1] * 100.0))]
    res["bf16_mfma+8fma+S_salu_2waves"] = row
    src.free()
    out.free()
    ticks.free()
    return res


def shader_clock_during(dev, w, steps):
    """Median shader clock (MHz) while `steps` steps of the workload run: a one-wave sampler
    (probe_clock_sampler) on a second stream beside them.  Not part of the timed region."""
    side = Device(dev.ordinal)
    try:
        mod = _probes(side)
        samples = 64
        ticks = side.alloc(samples * 16)
        ticks.zero()
        side.sync()
        w.step()
        dev.sync()
        side.launch(mod, "probe_clock_sampler", (1, 1, 1), (64, 1, 1), [ticks], [samples, 40], wait=False)
        for _ in range(steps):
            w.step()
        dev.sync()
        side.sync()
        c = ticks.copyout(np.int64, (samples, 2)).astype(np.float64)
        ticks.free()
        mhz = c[:, 0] / np.maximum(c[:, 1], 1.0) * 100.0
        return float(np.median(mhz[: max(4, samples // 2)]))
    finally:
        side.close()


def cpu_baseline(w, budget_heads):
    """The reference CPU backend's attention (oracle/cpu_sdpa_baseline.c) on a head subset of the same inputs."""
    import oracle
    oracle.build()
    heads = max(1, min(budget_heads, w.B * w.H))
    q = w.host["q"].reshape(-1, w.S, w.D)[:heads][None]
    k = w.host["k"].reshape(-1, w.S, w.D)[:heads][None]
    v = w.host["v"].reshape(-1, w.S, w.D)[:heads][None]
    oracle.cpu_sdpa(q[:, :1], k[:, :1], v[:, :1], causal=w.causal)   # warm-up
    ts = []
    threads = 1
    for _ in range(3):
        t0 = time.perf_counter()
        _, threads = oracle.cpu_sdpa(q, k, v, causal=w.causal)
        ts.append(time.perf_counter() - t0)
    t = sorted(ts)[1]
    ops = attn_ops(1, heads, w.S, w.D, w.causal)
    return {"value": ops / t / 1e12, "unit": "TFLOP/s", "cores": int(threads), "kind": "port",
            "sample": "%d of %d (batch,head) slices of the same inputs, fp32 packed-GEMM SDPA "
                      "(restated RUST/RAYON-equivalent CPU path), median of 3, %.2f s each" % (heads, w.B * w.H, t)}


def build_workload(dev, name):
    if name == "sage":
        return SageWorkload(dev, 4, 32, 8192, 128, False, 3.0, 0.0, cfg=4)
    if name == "sage_causal_long":
        return SageWorkload(dev, 1, 64, 32768, 128, True, 5.0, 0.01, cfg=5)
    if name == "sage_fp8":   # the headline shape on E4M3 codes
        return SageWorkload(dev, 4, 32, 8192, 128, False, 3.0, 0.0, cfg=4, fp8=True)
    if name == "vit":
        return FlashWorkload(dev, 8, 12, 197, 64, False, BF16, cfg=2)
    if name == "flash_long":
        return FlashWorkload(dev, 4, 32, 8192, 128, False, BF16, cfg=6)
    if name == "decoder":
        return FlashWorkload(dev, 4, 32, 2048, 128, True, BF16, cfg=3, kv_lens=True)
    if name == "vit_f32":
        return FlashWorkload(dev, 1, 12, 197, 64, False, F32, cfg=1)
    # the shape the reference publishes its own kernel times on (B8 H6 N789 D64, PERFORMANCE.md:314-317)
    if name == "train_f32":   # the ViT-B/16 layer shape at batch 8, fp32 (the reference's training kernels are f32 only)
        return TrainWorkload(dev, 8, 12, 197, 64, False, cfg=8)
    if name == "train_f32_causal":   # a decoder layer's shape, fp32, causal: forward with lse + backward
        return TrainWorkload(dev, 2, 16, 2048, 128, True, cfg=9)
    if name == "ref_bf16":
        return FlashWorkload(dev, 8, 6, 789, 64, False, BF16, cfg=7)
    if name == "ref_f32":
        return FlashWorkload(dev, 8, 6, 789, 64, False, F32, cfg=7)
    if name == "ref_sage":
        return SageWorkload(dev, 8, 6, 789, 64, False, 0.0, 0.0, cfg=7, bq=1, bk=1, f32_io=True)
    raise SystemExit("unknown workload %r" % name)


# The reference's published kernel times for that shape, on an RTX 3060 (not comparable hardware;
# reported next to ours for orientation only): PERFORMANCE.md:314-317.
REFERENCE_RTX3060_MS = {"ref_f32": 7.0, "ref_bf16": 0.53, "ref_sage": 1.26}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default="sage",
                    choices=["sage", "sage_causal_long", "vit", "decoder", "vit_f32", "flash_long", "ref_bf16",
                             "ref_f32", "ref_sage", "train_f32", "train_f32_causal", "sage_fp8"])
    ap.add_argument("--no-secondary", action="store_true")
    ap.add_argument("--traffic-probe", action="store_true",
                    help="one step of the workload plus one plain 1 GiB copy kernel and nothing else: "
                         "the run to put under `rocprofv3 --pmc FETCH_SIZE` / `WRITE_SIZE`")
    ap.add_argument("--issue-probe", action="store_true",
                    help="time loops of one matrix instruction plus K vector instructions (no workload)")
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--no-clock", action="store_true", help="skip the shader-clock and sustained-MFMA probes")
    args = ap.parse_args()
    if args.gpus != 1:
        raise SystemExit("bench.py measures one GPU: this build has no multi-GPU path (--gpus must be 1)")

    if args.issue_probe:
        dev = Device(0)
        print(json.dumps({"issue_mix_per_mfma_per_simd": issue_mix(dev),
                          "note": "loop of {1 MFMA (32x32x16 bf16 or 32x32x32 int8); K v_fma_f32 or v_exp_f32}; entries are "
                                  "[shader-clock cycles, ns, MHz] per matrix instruction per SIMD; 256 workgroups of "
                                  "256 / 512 / 768 threads = 1 / 2 / 3 waves per SIMD"}))
        dev.close()
        return
    dev = Device(0)
    log("device", dev.arch, dev.compute_units, "CUs")
    t0 = time.time()
    w = build_workload(dev, args.workload)
    log("inputs for %s ready in %.1f s" % (w.name, time.time() - t0))
    if args.traffic_probe:
        w.step()
        dev.sync()
        n16 = (1 << 30) // 16
        src, dst = dev.alloc(n16 * 16), dev.alloc(n16 * 16)
        src.zero()
        mod = dev.module_load(open(_lib.PROBES_PATH, "rb").read())
        dev.launch(mod, "probe_copy", (4096, 1, 1), (256, 1, 1), [src, dst], [n16], [64])
        print(json.dumps({"traffic_probe": w.name, "kernel_bytes_algorithmic": w.kernel_bytes,
                          "copy_bytes_read": n16 * 16, "copy_bytes_written": n16 * 16}))
        return
    res = measure(dev, w, args.steps, args.warmup)
    if w.S >= 1024 and not args.no_clock:
        res["roofline"]["shader_clock_mhz_under_load"] = shader_clock_during(dev, w, max(4, args.steps // 2))
    log(json.dumps(res))
    cpu = None
    if not args.no_cpu:
        heads = {"sage": 32, "sage_causal_long": 2, "decoder": 128, "vit": 96, "vit_f32": 12, "flash_long": 32}.get(
            args.workload, 48)
        cpu = cpu_baseline(w, heads)
        log(json.dumps(cpu))
    w.free()

    secondary = []
    if not args.no_secondary:
        for name in ("vit", "decoder", "flash_long", "vit_f32", "sage", "sage_causal_long", "ref_bf16", "ref_f32",
                     "ref_sage", "train_f32", "train_f32_causal", "sage_fp8"):
            if name == args.workload:
                continue
            sw = build_workload(dev, name)
            r = measure(dev, sw, max(args.steps, 20) if sw.S < 1024 else args.steps, args.warmup)
            if sw.S >= 1024 and not args.no_clock:
                r["roofline"]["shader_clock_mhz_under_load"] = shader_clock_during(dev, sw, max(4, args.steps // 2))
            if name in REFERENCE_RTX3060_MS:
                r["reference_kernel_ms_rtx3060"] = REFERENCE_RTX3060_MS[name]
            sw.free()
            log(json.dumps(r))
            secondary.append(r)
    power = None if args.no_clock else sustained_mfma(dev)
    dev.close()

    line = {
        "metric": "attention fwd TFLOPS/TOPS + % MFMA peak, ViT-B/16 and S=8192 D=128 shapes",
        "value": res["tops"], "unit": "TOP/s" if w.dtype in ("int8", "fp8") else "TFLOP/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": res["ms_per_step"],
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": w.dtype, "data": "synthetic",
        "config": {"workload": w.name, "B": w.B, "H": w.H, "S": w.S, "D": w.D, "causal": bool(w.causal),
                   "step": "smooth and quantise K (64-token blocks) + %s attention with the Q quantiser (128-token blocks) "
                           "in its prologue" % w.dtype if w.dtype in ("int8", "fp8") else "attention forward"},
        "roofline": res["roofline"],
        "cpu_baseline": cpu,
    }
    if "prepass_ms_per_step" in res:
        line["prepass_ms_per_step"] = res["prepass_ms_per_step"]
    if power is not None:
        # the published peaks assume 2.4 GHz; under a matrix load on random data the chip clocks down
        line["power_limit_probe"] = {"kernel": "probe_mfma_rate (bf16 32x32x16 MFMAs only, 2 waves per SIMD)",
                                     "constant_operands": power["constant"], "random_operands": power["random"]}
        line["roofline"]["frac_of_sustained_bf16_mfma_rate"] = (
            (res["ops_per_step"] / 2 / (PEAK_INT8 / PEAK_BF16) + res["ops_per_step"] / 2) if w.dtype in ("int8", "fp8")
            else res["ops_per_step"]) / (line["roofline"]["launch_ms"] * 1e-3) / 1e12 / power["random"]["tflops"]
    if "ms_per_step_graph_replay" in res:
        line["ms_per_step_graph_replay"] = res["ms_per_step_graph_replay"]
    if secondary:
        line["secondary"] = secondary
    print(json.dumps(line), flush=True)


if __name__ == "__main__":
    main()
