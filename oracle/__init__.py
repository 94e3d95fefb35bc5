"""NumPy front-end of the CPU oracle (oracle/attn_oracle.c, oracle/cpu_sdpa_baseline.c).

TEST INFRASTRUCTURE ONLY: imported by tests/, by __graft_entry__.smoke() and by
bench.py's cpu_baseline leg as the checker / the reported CPU baseline.  The
product package (autorust_amd) never imports it.

Every function takes [B, H, N, D] float32 arrays (K/V may have fewer heads than
Q: grouped-query attention with the reference's head mapping
`kv_head = head // (Hq // Hkv)`, src/runtime/cuda_flash.rs:67-72) and loops the
C head functions over (batch, head).  `rows` restricts the evaluated query rows
(the same subset for every head) so that the large configurations can be
spot-checked in bounded time; the result then has shape [B, H, len(rows), D].
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle.so")
_lib = None

_f32p = ctypes.POINTER(ctypes.c_float)
_i32p = ctypes.POINTER(ctypes.c_int32)
_i8p = ctypes.POINTER(ctypes.c_int8)
_u16p = ctypes.POINTER(ctypes.c_uint16)


def build(force=False):
    """Compile liboracle.so with gcc (seconds)."""
    srcs = [os.path.join(_HERE, f) for f in ("attn_oracle.c", "cpu_sdpa_baseline.c", "Makefile")]
    if (not force and os.path.exists(_LIB_PATH)
            and all(os.path.getmtime(_LIB_PATH) >= os.path.getmtime(s) for s in srcs)):
        return _LIB_PATH
    subprocess.run(["make", "-C", _HERE, "-B", "liboracle.so"], check=True, capture_output=True)
    return _LIB_PATH


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        _lib = ctypes.CDLL(_LIB_PATH)
        _lib.ar_bf16_round.restype = ctypes.c_float
        _lib.ar_bf16_round.argtypes = [ctypes.c_float]
        _lib.ar_cpu_sdpa.restype = ctypes.c_int
    return _lib


def _p(a, typ):
    return None if a is None else a.ctypes.data_as(typ)


def _f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


# ------------------------------------------------------------------ bf16 ---

def bf16_round(x):
    x = _f32(x)
    y = np.empty_like(x)
    lib().ar_bf16_round_array(_p(x, _f32p), _p(y, _f32p), ctypes.c_int64(x.size))
    return y


def bf16_bits(x):
    x = _f32(x)
    y = np.empty(x.shape, dtype=np.uint16)
    lib().ar_bf16_bits_array(_p(x, _f32p), _p(y, _u16p), ctypes.c_int64(x.size))
    return y


def bf16_from_bits(b):
    return (np.ascontiguousarray(b, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)


# ------------------------------------------------------------ attention ---

def _prep(q, k, v, mask, kv_len, rows):
    q, k, v = _f32(q), _f32(k), _f32(v)
    assert q.ndim == 4 and k.ndim == 4 and v.ndim == 4
    B, Hq, N, D = q.shape
    Hkv = k.shape[1]
    assert k.shape == (B, Hkv, N, D) and v.shape == (B, Hkv, N, D) and Hq % Hkv == 0
    if mask is not None:
        mask = np.ascontiguousarray(np.broadcast_to(_f32(mask), (B, Hq, N, N)))
    if kv_len is None:
        kv_len = np.full(B, -1, dtype=np.int32)
    kv_len = np.ascontiguousarray(kv_len, dtype=np.int32)
    assert kv_len.shape == (B,)
    if rows is not None:
        rows = np.ascontiguousarray(rows, dtype=np.int32)
        assert rows.ndim == 1 and (rows >= 0).all() and (rows < N).all()
    nrows = N if rows is None else len(rows)
    out = np.empty((B, Hq, nrows, D), dtype=np.float32)
    return q, k, v, mask, kv_len, rows, nrows, out, (B, Hq, Hkv, N, D)


def _heads(fn, q, k, v, mask, causal, kv_len, rows, extra):
    q, k, v, mask, kv_len, rows, nrows, out, (B, Hq, Hkv, N, D) = _prep(q, k, v, mask, kv_len, rows)
    group = Hq // Hkv
    for b in range(B):
        for h in range(Hq):
            kh = h // group
            m = None if mask is None else mask[b, h]
            fn(_p(q[b, h], _f32p), _p(k[b, kh], _f32p), _p(v[b, kh], _f32p), _p(m, _f32p),
               N, D, int(causal), int(kv_len[b]), *extra,
               _p(rows, _i32p), nrows, _p(out[b, h], _f32p))
    return out


def sdpa_f32(q, k, v, mask=None, causal=False, kv_len=None, rows=None):
    """General path, fp32, reference op order (src/tensor/mod.rs:2395-2446)."""
    return _heads(lib().ar_head_sdpa_f32, q, k, v, mask, causal, kv_len, rows, ())


def sdpa_f64(q, k, v, mask=None, causal=False, kv_len=None, rows=None, scale=None):
    """Same function in binary64, rounded once."""
    scale = 1.0 / np.sqrt(q.shape[-1]) if scale is None else scale
    return _heads(lib().ar_head_sdpa_f64, q, k, v, mask, causal, kv_len, rows, (ctypes.c_double(scale),))


def lse_f64(q, k, mask=None, causal=False, kv_len=None, rows=None, scale=None):
    """log-sum-exp of the scaled, masked logits per query row: [B, H, rows] (float64 inside)."""
    q, k = _f32(q), _f32(k)
    B, Hq, N, D = q.shape
    Hkv = k.shape[1]
    group = Hq // Hkv
    scale = 1.0 / np.sqrt(D) if scale is None else scale
    if mask is not None:
        mask = np.ascontiguousarray(np.broadcast_to(_f32(mask), (B, Hq, N, N)))
    kv_len = np.full(B, -1, np.int32) if kv_len is None else np.ascontiguousarray(kv_len, np.int32)
    if rows is not None:
        rows = np.ascontiguousarray(rows, dtype=np.int32)
    nrows = N if rows is None else len(rows)
    out = np.empty((B, Hq, nrows), dtype=np.float32)
    for b in range(B):
        for h in range(Hq):
            m = None if mask is None else mask[b, h]
            lib().ar_head_lse_f64(_p(q[b, h], _f32p), _p(k[b, h // group], _f32p), _p(m, _f32p), N, D, int(causal),
                                  int(kv_len[b]), ctypes.c_double(scale), _p(rows, _i32p), nrows, _p(out[b, h], _f32p))
    return out


def attention_backward_f64(q, k, v, dout, mask=None, causal=False, kv_len=None, scale=None):
    """Training forward + backward in binary64, by the reference's formulas
    (src/runtime/cuda_flash_train.rs:145-309): lse = log sum exp(s), o = softmax(s) v,
    D_i = o_i . dO_i, p = exp(s - lse), dp = dO v^T, ds = p (dp - D) scale, dQ = ds K,
    dK = sum over the GQA group of ds^T Q, dV = sum over the group of p^T dO; masked keys
    (causal: j > i, key length: j >= kv_len[b]) have p = 0.  Returns (o, lse, dq, dk, dv) as
    float32 arrays.  Pinned against torch.autograd in tests/test_oracle.py."""
    q, k, v, dout = (np.asarray(t, np.float64) for t in (q, k, v, dout))
    B, Hq, N, D = q.shape
    Hkv = k.shape[1]
    group = Hq // Hkv
    scale = 1.0 / np.sqrt(D) if scale is None else float(scale)
    o = np.zeros((B, Hq, N, D)); lse = np.full((B, Hq, N), -1e30)
    dq = np.zeros((B, Hq, N, D)); dk = np.zeros((B, Hkv, N, D)); dv = np.zeros((B, Hkv, N, D))
    i, j = np.arange(N)[:, None], np.arange(N)[None, :]
    for b in range(B):
        dead = np.zeros((N, N), bool)
        if causal:
            dead |= j > i
        if kv_len is not None:
            dead |= j >= int(kv_len[b])
        for h in range(Hq):
            kh = h // group
            s = (q[b, h] @ k[b, kh].T) * scale
            if mask is not None:
                s = s + np.broadcast_to(np.asarray(mask, np.float64), (B, Hq, N, N))[b, h]
            s = np.where(dead, -np.inf, s)
            m = s.max(axis=1, keepdims=True)
            live = np.isfinite(m[:, 0])
            e = np.where(live[:, None], np.exp(s - np.where(live[:, None], m, 0.0)), 0.0)
            l = e.sum(axis=1, keepdims=True)
            pr = np.where(live[:, None], e / np.where(l > 0, l, 1.0), 0.0)
            lse[b, h] = np.where(live, (m + np.log(np.where(l > 0, l, 1.0)))[:, 0], -1e30)
            o[b, h] = pr @ v[b, kh]
            delta = (o[b, h] * dout[b, h]).sum(axis=1, keepdims=True)
            dp = dout[b, h] @ v[b, kh].T
            ds = pr * (dp - delta) * scale
            dq[b, h] = ds @ k[b, kh]
            dk[b, kh] += ds.T @ q[b, h]
            dv[b, kh] += pr.T @ dout[b, h]
    return tuple(t.astype(np.float32) for t in (o, lse, dq, dk, dv))


def flash_f32(q, k, v, mask=None, causal=False, kv_len=None, rows=None, scale=None, bq=64, bk=32):
    """fp32 exact-mode FA2 kernel restated (src/runtime/cuda_flash.rs:53-141)."""
    scale = np.float32(1.0) / np.sqrt(np.float32(q.shape[-1])) if scale is None else scale
    return _heads(lib().ar_head_flash_f32, q, k, v, mask, causal, kv_len, rows,
                  (ctypes.c_float(scale), bq, bk))


def attn_bf16(q, k, v, mask=None, causal=False, kv_len=None, rows=None, scale=None, round_out=True):
    """bf16-emulating reference (tests/flash_cuda_masks.rs:41-104, round=true)."""
    scale = np.float32(1.0) / np.sqrt(np.float32(q.shape[-1])) if scale is None else scale
    return _heads(lib().ar_head_bf16, q, k, v, mask, causal, kv_len, rows,
                  (ctypes.c_float(scale), int(round_out)))


# ----------------------------------------------------------------- Sage ---

def k_mean(k):
    """mean over tokens per (batch, kv-head, channel), fixed fp32 order. [B,H,D]."""
    k = _f32(k)
    B, H, N, D = k.shape
    out = np.empty((B, H, D), dtype=np.float32)
    for b in range(B):
        for h in range(H):
            lib().ar_k_mean(_p(k[b, h], _f32p), N, D, _p(out[b, h], _f32p))
    return out


def quant_blocks(x, blk, sub=None, use_div=False):
    """Per-block symmetric int8. Returns (int8 [B,H,N,D], scales f32 [B,H,ceil(N/blk)])."""
    x = _f32(x)
    B, H, N, D = x.shape
    nblk = (N + blk - 1) // blk
    q = np.empty((B, H, N, D), dtype=np.int8)
    s = np.empty((B, H, nblk), dtype=np.float32)
    if sub is not None:
        sub = _f32(sub)
        assert sub.shape == (B, H, D)
    for b in range(B):
        for h in range(H):
            lib().ar_quant_blocks(_p(x[b, h], _f32p), N, D, blk,
                                  _p(None if sub is None else sub[b, h], _f32p), int(use_div),
                                  _p(q[b, h], _i8p), _p(s[b, h], _f32p))
    return q, s


def fp8_e4m3_bits(x):
    """float32 -> FP8 E4M3 codes (OCP "FN": bias 7, subnormal step 2^-9, largest finite 448, no
    infinities), round to nearest even, saturating: the reference's
    `__nv_cvt_float2_to_fp8x2(..., __NV_SATFINITE, __NV_E4M3)` (src/runtime/cuda_flash_sage.rs:125-128)."""
    x = np.asarray(x, np.float32)
    sign = (np.signbit(x).astype(np.uint8) << 7)
    a = np.minimum(np.abs(x).astype(np.float64), 448.0)   # SATFINITE; (448, 464) rounds to 448 anyway
    e = np.floor(np.log2(np.where(a > 0, a, 1.0))).astype(np.int64)
    e = np.maximum(e, -6)
    q = np.rint(a / np.exp2(e - 3.0))                      # numpy rint is half-to-even; 0..16
    up = q >= 16                                           # rounded up into the next binade
    e = np.where(up, e + 1, e)
    q = np.where(up, 8.0, q)
    normal = q >= 8
    code = np.where(normal, ((e + 7) << 3) | (q.astype(np.int64) - 8), q.astype(np.int64))
    code = np.where(np.isnan(x), 0x7f, code)
    return (sign | code.astype(np.uint8)).astype(np.uint8)


def fp8_e4m3_value(bits):
    """FP8 E4M3 codes -> float32 values (exact)."""
    b = np.asarray(bits, np.uint8).astype(np.int64)
    e, m = (b >> 3) & 15, b & 7
    v = np.where(e == 0, m * 2.0 ** -9, (8 + m) * np.exp2(e - 10.0))
    v = np.where((b & 0x7f) == 0x7f, np.nan, v)
    return np.where(b & 0x80, -v, v).astype(np.float32)


def quant_blocks_fp8(x, blk, sub=None):
    """quant_blocks with FP8 E4M3 codes and scale = absmax / 448 (cuda_flash_sage.rs:9, 209-222):
    returns (codes uint8 [B,H,N,D], scales f32 [B,H,ceil(N/blk)])."""
    x = _f32(x)
    B, H, N, D = x.shape
    if sub is not None:
        x = (x - _f32(sub)[:, :, None, :]).astype(np.float32)
    nblk = (N + blk - 1) // blk
    codes = np.empty(x.shape, np.uint8)
    scales = np.empty((B, H, nblk), np.float32)
    for i in range(nblk):
        seg = x[:, :, i * blk:(i + 1) * blk]
        mx = np.abs(seg).max(axis=(2, 3)).astype(np.float32)
        sc = np.where(mx > 0, mx / np.float32(448.0), np.float32(1.0)).astype(np.float32)
        inv = (np.float32(1.0) / sc).astype(np.float32)
        scales[:, :, i] = sc
        codes[:, :, i * blk:(i + 1) * blk] = fp8_e4m3_bits((seg * inv[:, :, None, None]).astype(np.float32))
    return codes, scales


def sage_fp8(qc, kc, sq, sk, v, bq, bk, mask=None, causal=False, kv_len=None, scale=None, round_out=False):
    """The quantised kernel's arithmetic with FP8 operands (the AR_FP8 branch of
    src/runtime/cuda_flash_sage.rs:280-412): logits = sum of exact FP8 products, accumulated here in
    binary64 and rounded to f32 once (the matrix instruction's f32 accumulation can differ in the last
    place), s = logits * ((sq*sk)*scale), masks, f32 softmax, P and V rounded to bf16, f32 accumulate."""
    qv, kv = fp8_e4m3_value(qc).astype(np.float64), fp8_e4m3_value(kc).astype(np.float64)
    v = _f32(v)
    B, Hq, N, D = qv.shape
    Hkv = kv.shape[1]
    group = Hq // Hkv
    scale = np.float32(1.0 / np.sqrt(np.float32(D))) if scale is None else np.float32(scale)
    out = np.zeros((B, Hq, N, D), np.float32)
    i, j = np.arange(N)[:, None], np.arange(N)[None, :]
    vb = bf16_round(v)
    for b in range(B):
        dead = np.zeros((N, N), bool)
        if causal:
            dead |= j > i
        if kv_len is not None:
            dead |= j >= int(kv_len[b])
        for h in range(Hq):
            kh = h // group
            acc = (qv[b, h] @ kv[b, kh].T).astype(np.float32)
            f = ((_f32(sq)[b, h][np.arange(N) // bq][:, None] * _f32(sk)[b, kh][np.arange(N) // bk][None, :]) * scale).astype(np.float32)
            s = (acc * f).astype(np.float32)
            if mask is not None:
                s = (s + np.broadcast_to(_f32(mask), (N, N))).astype(np.float32)
            s = np.where(dead, np.float32(-1e30), s)
            m = s.max(axis=1, keepdims=True)
            # the fp32 exponential, correctly rounded (float64 evaluation of the fp32 argument, one rounding):
            # numpy's own fp32 exp is a vector routine that may be 1 ulp off, which moves bf16 roundings of P
            p = np.exp((s - m).astype(np.float32).astype(np.float64)).astype(np.float32)
            p = np.where(dead, np.float32(0), p) if (causal or kv_len is not None) else p
            l = p.sum(axis=1, keepdims=True, dtype=np.float32)
            o = (bf16_round(p).astype(np.float64) @ vb[b, kh].astype(np.float64)).astype(np.float32)
            o = np.where(l > 0, o / np.where(l > 0, l, 1), 0).astype(np.float32)
            out[b, h] = bf16_round(o) if round_out else o
    return out


def logits_i32(q8_head, k8_head, i0, i1, j0, j1):
    """int32 QK^T of one head for rows [i0,i1) x keys [j0,j1)."""
    q8 = np.ascontiguousarray(q8_head, dtype=np.int8)
    k8 = np.ascontiguousarray(k8_head, dtype=np.int8)
    D = q8.shape[-1]
    out = np.empty((i1 - i0, j1 - j0), dtype=np.int32)
    lib().ar_logits_i32(_p(q8, _i8p), _p(k8, _i8p), D, i0, i1, j0, j1, _p(out, _i32p))
    return out


def sage(q8, k8, sq, sk, v, bq, bk, mask=None, causal=False, kv_len=None, rows=None, scale=None,
         round_out=False):
    """Attention from quantised Q/K (src/runtime/cuda_flash_sage.rs:280-412)."""
    q8 = np.ascontiguousarray(q8, dtype=np.int8)
    k8 = np.ascontiguousarray(k8, dtype=np.int8)
    sq, sk, v = _f32(sq), _f32(sk), _f32(v)
    B, Hq, N, D = q8.shape
    Hkv = k8.shape[1]
    group = Hq // Hkv
    scale = np.float32(1.0) / np.sqrt(np.float32(D)) if scale is None else scale
    if mask is not None:
        mask = np.ascontiguousarray(np.broadcast_to(_f32(mask), (B, Hq, N, N)))
    if kv_len is None:
        kv_len = np.full(B, -1, dtype=np.int32)
    if rows is not None:
        rows = np.ascontiguousarray(rows, dtype=np.int32)
    nrows = N if rows is None else len(rows)
    out = np.empty((B, Hq, nrows, D), dtype=np.float32)
    for b in range(B):
        for h in range(Hq):
            kh = h // group
            m = None if mask is None else mask[b, h]
            lib().ar_head_sage(_p(q8[b, h], _i8p), _p(k8[b, kh], _i8p), _p(sq[b, h], _f32p),
                               _p(sk[b, kh], _f32p), _p(v[b, kh], _f32p), _p(m, _f32p),
                               N, D, bq, bk, int(causal), int(kv_len[b]), ctypes.c_float(scale),
                               int(round_out), _p(rows, _i32p), nrows, _p(out[b, h], _f32p))
    return out


# --------------------------------------------------------- CPU baseline ---

def cpu_sdpa(q, k, v, causal=False):
    """The reference CPU backend's attention (packed GEMM, softmax, packed GEMM).
    q/k/v [B,H,N,D] with equal head counts. Returns (out, threads used)."""
    q, k, v = _f32(q), _f32(k), _f32(v)
    B, H, N, D = q.shape
    out = np.empty_like(q)
    scratch = np.empty(N * N + N * D, dtype=np.float32)
    threads = lib().ar_cpu_sdpa(_p(q, _f32p), _p(k, _f32p), _p(v, _f32p), _p(out, _f32p),
                                B * H, N, D, int(causal), _p(scratch, _f32p))
    return out, threads
