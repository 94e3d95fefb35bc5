/*
 * libarhip — C ABI of the MI355X (gfx950) device and fused-attention kernels.
 *
 * This is the boundary a host in any language binds (Rust `libloading`,
 * ctypes, cgo ...).  It replaces, for the fused attention forward, what the
 * reference reaches through its Rust device traits; each entry point cites the
 * reference interface (path:line under the reference tree) it stands in for.
 *
 * Conventions
 *   - every function returns 0 on success and a negative ARHIP_E* code on
 *     failure; arhip_last_error() returns a thread-local message.  The
 *     reference's convention is `panic!("TGERR: ...")`; a Rust shim reproduces
 *     it by panicking on a non-zero return.
 *   - ARHIP_EUNSUPPORTED is not a failure of the device: it is the typed
 *     kernels' way of saying "this shape/dtype is not covered", on which the
 *     reference's dispatcher returns None and the caller runs the general path
 *     (src/models/flash_attention.rs:470-472).
 *   - tensors are dense row-major [B, H, N, D] (src/runtime/cuda_flash.rs:199-201),
 *     caller-owned device memory, 16-byte aligned; K/V may have Hkv heads with
 *     Hq % Hkv == 0 (grouped-query attention, kv head = head / (Hq/Hkv)).
 *   - one stream per device handle; calls are asynchronous on it unless `wait`
 *     is non-zero, in which case the call returns after the kernel finished and
 *     *secs (if not NULL) receives the elapsed device time in seconds measured
 *     with events on that stream (src/runtime/device.rs:295-311 `Prog::call`).
 *   - a handle is used by one host thread at a time.
 */
#ifndef ARHIP_H
#define ARHIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct arhip_device arhip_device;

enum {
    ARHIP_OK = 0,
    ARHIP_EINVAL = -1,       /* bad argument (shape, alignment, null pointer) */
    ARHIP_EUNSUPPORTED = -2, /* shape/dtype not covered by the fused kernels */
    ARHIP_EHIP = -3,         /* a HIP runtime call failed */
    ARHIP_ENODEVICE = -4     /* no usable gfx950 device */
};

/* element types of q/k/v/o */
enum { ARHIP_F32 = 0, ARHIP_BF16 = 1 };

/* attention kinds: src/models/flash_attention.rs:709-717 `AttentionKind` */
enum { ARHIP_ATTN_SDPA = 0, ARHIP_ATTN_FLASH = 1, ARHIP_ATTN_SAGE = 2 };

/* kernels counted by arhip_selections() */
enum { ARHIP_K_FLASH_F32 = 0, ARHIP_K_FLASH_BF16 = 1, ARHIP_K_SAGE = 2, ARHIP_K_SAGE_QUANT = 3, ARHIP_K_FLASH_BWD = 4, ARHIP_K_COUNT = 5 };

const char *arhip_last_error(void);

/* ---- device: src/runtime/ops_cuda.rs:140-174 (open), :1132-1159 (factory) ---- */
int arhip_device_count(int *count);
int arhip_open(int ordinal, arhip_device **dev);
int arhip_close(arhip_device *dev);
/* "gfx950"; src/runtime/ops_cuda.rs `arch_sm()` */
const char *arhip_arch(arhip_device *dev);
int arhip_compute_units(arhip_device *dev);

/* ---- memory: `BackendAllocator`, src/runtime/device.rs:39-62;
 *      CUDA implementation src/runtime/ops_cuda.rs:595-685 ---- */
int arhip_alloc(arhip_device *dev, size_t bytes, void **dptr);        /* _alloc: uninitialised */
int arhip_free(arhip_device *dev, void *dptr);                        /* _free */
int arhip_copyin(arhip_device *dev, void *dst, const void *host, size_t bytes);  /* _copyin */
int arhip_copyout(arhip_device *dev, void *host, const void *src, size_t bytes); /* _copyout: syncs first */
int arhip_copy_d2d(arhip_device *dev, void *dst, const void *src, size_t bytes); /* _copy_into: async, no sync */
int arhip_fill_zero(arhip_device *dev, void *dst, size_t bytes);      /* fill kernel, async */
int arhip_mem_info(arhip_device *dev, size_t *free_bytes, size_t *total_bytes);  /* memory_info */
int arhip_sync(arhip_device *dev);                                    /* Prog::flush */
/* the handle's stream as a hipStream_t, for callers that order their own work on it */
void *arhip_stream(arhip_device *dev);

/* ---- timing on the handle's stream (HIP events) ---- */
int arhip_timer_start(arhip_device *dev);
int arhip_timer_stop(arhip_device *dev, double *secs); /* records, waits, returns elapsed seconds */

/* ---- per-kernel device time: the reference's AUTORUST_KPROF
 *      (src/runtime/ops_cuda.rs:1004-1016) without a sync per launch.  While
 *      enabled, every typed launch below is bracketed by two events on the
 *      handle's stream; collect() waits for the stream, returns the summed
 *      elapsed time and the number of launches of `kernel` (ARHIP_K_*) since
 *      the last collect, and forgets them. ---- */
int arhip_kprof_enable(arhip_device *dev, int on);
int arhip_kprof_collect(arhip_device *dev, int kernel, double *total_secs, uint64_t *launches);
/* the same, also returning the shortest and the median launch (NULL: not wanted) */
int arhip_kprof_collect_stats(arhip_device *dev, int kernel, double *total_secs, uint64_t *launches,
                              double *min_secs, double *median_secs);

/* ---- launch graphs: captured replay (`Session::capture_host` + `Jit::replay`,
 *      src/engine/session.rs:138-146, src/engine/jit.rs:186-195) as one device submission.
 *      Between begin and end, launches on this handle issued with wait = 0 are recorded, not
 *      run; arhip_graph_launch replays them in order.  Buffers are captured by address: a replay
 *      reads and writes the same memory as the recorded calls.  Allocation, copies and calls
 *      that wait are not allowed inside a capture. ---- */
int arhip_graph_begin(arhip_device *dev);
int arhip_graph_end(arhip_device *dev, void **graph_exec);
int arhip_graph_launch(arhip_device *dev, void *graph_exec, int wait, double *secs);
int arhip_graph_destroy(arhip_device *dev, void *graph_exec);

/* ---- generic host-kernel launch: `Compiled::run_host_kernel`,
 *      src/runtime/device.rs:383-402; argument encoding of
 *      src/runtime/ops_cuda.rs:930-1019 (`CudaProgram::call`) ----
 * image: a gfx950 code object (hipcc --genco), or a container of several that are looked up as
 * one: "ARHIPKO1", uint32 count, uint32 0, then per code object uint64 size and its bytes padded
 * to a multiple of 16 (autorust_amd/attn_kernels.hsaco is such a file: its entry points compile as
 * fifteen code objects side by side).  Modules are cached per device by content hash.  args: nbufs device pointers followed by nvals scalars;
 * val_bits[i] in {32, 64} narrows vals[i] like the reference's signature
 * dtype does.  grid is in blocks. */
int arhip_module_load(arhip_device *dev, const void *image, size_t len, void **module);
int arhip_launch(arhip_device *dev, void *module, const char *name,
                 const unsigned grid[3], const unsigned block[3],
                 void *const *bufs, int nbufs,
                 const int64_t *vals, const int *val_bits, int nvals,
                 int wait, double *secs);

/* ---- fused attention forward ----
 * arhip_attn_supported: the `supports` / `supported` gates
 *   (src/runtime/cuda_flash.rs:145-147, cuda_flash_bf16.rs:431-441,
 *    cuda_flash_sage.rs:69-74).  Returns 1 or 0.
 *   The reference's kernels take D == 64 only; these take D in {64, 128}. */
int arhip_attn_supported(int kind, int64_t n, int64_t d, int dtype);

/* arhip_flash_fwd: `cuda_flash::run_ex` (src/runtime/cuda_flash.rs:203-217,
 *   fp32 exact mode) and `cuda_flash_bf16::run_ex`
 *   (src/runtime/cuda_flash_bf16.rs:495-512), selected by dtype.
 *   o[B,Hq,N,D] = softmax(q.k^T * scale + mask) . v, fp32 accumulate.
 *   mask: optional additive f32 [N,N] shared by every (b,h), or NULL
 *         (the reference passes `o` as a dummy, cuda_flash.rs:233-240).
 *   kv_len: optional device int32[B]; keys j >= kv_len[b] are excluded
 *         (per-batch key-padding mask).  No counterpart in the reference's
 *         kernels, which only bound keys by N; NULL means N for every batch.
 *   causal: keys j > i are excluded (cuda_flash.rs:112).
 *   scale: the reference hard-codes 0.125 = 1/sqrt(64) (cuda_flash.rs:89);
 *         pass 1/sqrt(D). */
int arhip_flash_fwd(arhip_device *dev, const void *q, const void *k, const void *v, void *o,
                    const float *mask, const int32_t *kv_len,
                    int64_t B, int64_t Hq, int64_t Hkv, int64_t N, int64_t D,
                    int causal, int dtype, float scale, int wait, double *secs);

/* arhip_flash_fwd_strided: the same kernels on strided tensors.  Strides are in elements,
 *   {batch, head, token}; the channel stride is 1.  Dense [B,H,N,D] is {H*N*D, N*D, D};
 *   the token-major layout the projections produce, [B,N,H,D], is {N*H*D, D, H*D}.
 *   This is the caller-side fusion the reference lists as missing: its transformer block
 *   copies q/k/v into [B,H,S,hs] before the kernel and the result back
 *   (src/models/transformer.rs:286-299); with strides both copies disappear (pass the
 *   projection output as is, and ask for o in [B,N,H*D]).
 *   Every stride must be a multiple of 8 elements, the token stride >= D. */
int arhip_flash_fwd_strided(arhip_device *dev, const void *q, const void *k, const void *v, void *o,
                            const int64_t q_strides[3], const int64_t kv_strides[3], const int64_t o_strides[3],
                            const float *mask, const int32_t *kv_len,
                            int64_t B, int64_t Hq, int64_t Hkv, int64_t N, int64_t D,
                            int causal, int dtype, float scale, int wait, double *secs);

/* arhip_flash_fwd_lse: arhip_flash_fwd_strided that also writes, when lse != NULL, the
 *   log-sum-exp of the scaled, masked logits of every query row, f32 [B,Hq,N] (natural log;
 *   -1e30 for a row without visible keys): the statistic the reference's training forward
 *   saves as LSE = m + log(l) (src/runtime/cuda_flash_train.rs:5-11,141) for its backward. */
int arhip_flash_fwd_lse(arhip_device *dev, const void *q, const void *k, const void *v, void *o, float *lse,
                        const int64_t q_strides[3], const int64_t kv_strides[3], const int64_t o_strides[3],
                        const float *mask, const int32_t *kv_len,
                        int64_t B, int64_t Hq, int64_t Hkv, int64_t N, int64_t D,
                        int causal, int dtype, float scale, int wait, double *secs);

/* arhip_flash_bwd: `fused_attention_backward` (src/models/flash_attention.rs:789-977) = the three
 *   training kernels of src/runtime/cuda_flash_train.rs:145-309 in one call: ar_fl_prep
 *   (delta[b,h,i] = O_i . dO_i), ar_fl_bwd_dq and ar_fl_bwd_dkv.  f32 only, dense [B,H,N,D] tensors
 *   (the reference: "f32 only; other dtypes keep the graph path"); o and lse are what
 *   arhip_flash_fwd_lse(dtype = ARHIP_F32) produced for the same q, k, v, mask, kv_len, causal and
 *   scale.  dq [B,Hq,N,D], dk and dv [B,Hkv,N,D] are written in full (no zero-fill needed: the
 *   sum over a GQA group happens inside the kernel, in a fixed order, without atomics).  delta is a
 *   caller-provided scratch of B*Hq*N floats.  D is 64 or 128 (the reference: 64). */
int arhip_flash_bwd(arhip_device *dev, const float *q, const float *k, const float *v, const float *o,
                    const float *lse, const float *dout, float *dq, float *dk, float *dv, float *delta,
                    const float *mask, const int32_t *kv_len,
                    int64_t B, int64_t Hq, int64_t Hkv, int64_t N, int64_t D,
                    int causal, float scale, int wait, double *secs);

/* arhip_sage_quant: the quantiser of the Sage kernel hoisted into a pre-pass
 *   (the reference quantises inside the attention kernel, K once per query
 *   block: src/runtime/cuda_flash_sage.rs:201-223, 248-278).
 *   x [B,H,N,D] (f32 or bf16, `dtype`) -> x8 int8 [B,H,N,D] and
 *   scales f32 [B,H,ceil(N/block)], in blocks of `block` tokens:
 *     scale = absmax > 0 ? absmax/127 : 1;  x8 = clamp(rint(x * (1/scale)), +-127)
 *   (cuda_flash_sage.rs:124-137, 209-222; block == 1 is the reference's rule).
 *   smooth != 0 first subtracts the per-(b,h,channel) mean over the N tokens
 *   (K smoothing; not in the reference) and writes that mean to
 *   mean f32 [B,H,D] (required then, else may be NULL).
 *   workspace: device scratch of arhip_sage_quant_workspace(B,H,N,D) bytes
 *   when smooth != 0 (may be NULL otherwise). */
size_t arhip_sage_quant_workspace(int64_t B, int64_t H, int64_t N, int64_t D);
int arhip_sage_quant(arhip_device *dev, const void *x, int8_t *x8, float *scales, float *mean,
                     void *workspace, int64_t B, int64_t H, int64_t N, int64_t D,
                     int64_t block, int dtype, int smooth, int wait, double *secs);

/* arhip_sage_quant_strided: arhip_sage_quant on a strided input (element strides {batch, head,
 *   token}, channel stride 1; every stride a multiple of 8, token stride >= D): the projection
 *   output [B,N,H,D] is quantised in place of the copy to [B,H,N,D] the reference makes
 *   (src/models/transformer.rs:286-299).  x8, scales and mean are dense as for arhip_sage_quant. */
int arhip_sage_quant_strided(arhip_device *dev, const void *x, const int64_t x_strides[3], int8_t *x8,
                             float *scales, float *mean, void *workspace, int64_t B, int64_t H, int64_t N,
                             int64_t D, int64_t block, int dtype, int smooth, int wait, double *secs);

/* arhip_sage_quant_static: arhip_sage_quant without a workspace argument and without any
 *   allocation inside the call.  It has no counterpart in the reference; it is for callers that
 *   cannot allocate device memory: code under HIP graph capture, tight serving loops, harnesses
 *   that forbid hipMalloc.  The partial sums of the K mean go to a device array inside the
 *   library (16 MiB per GPU, resolved when the device is opened), so smoothing is limited to
 *   arhip_sage_quant_workspace(B,H,N,D) <= arhip_sage_quant_static_limit() bytes; larger shapes
 *   are rejected with ARHIP_EINVAL.  Same kernels and bit-identical results as arhip_sage_quant.
 *   All calls on one GPU share the array: calls that overlap in time on one GPU race.  The
 *   launches are not entered in the arhip_kprof_* log. */
size_t arhip_sage_quant_static_limit(void);
int arhip_sage_quant_static(arhip_device *dev, const void *x, int8_t *x8, float *scales, float *mean,
                            int64_t B, int64_t H, int64_t N, int64_t D,
                            int64_t block, int dtype, int smooth, int wait, double *secs);

/* FP8 E4M3 variant of the quantised path: the reference's AR_FP8 branch
 *   (src/runtime/cuda_flash_sage.rs:9, 92-147: `mma ... e4m3.e4m3.f32`, scale = max/448,
 *   `__nv_cvt_float2_to_fp8x2(..., __NV_SATFINITE, __NV_E4M3)`).  Same arguments and semantics as
 *   arhip_sage_quant / arhip_sage_fwd with x8 holding OCP E4M3 codes instead of int8 values; the
 *   logits are accumulated in f32 by v_mfma_f32_32x32x16_fp8_fp8, so there is no int32 export.
 *   Runs on the general kernel (any mask, any block sizes incl. per-row scales). */
int arhip_sage_quant_fp8(arhip_device *dev, const void *x, uint8_t *x8, float *scales, float *mean,
                         void *workspace, int64_t B, int64_t H, int64_t N, int64_t D,
                         int64_t block, int dtype, int smooth, int wait, double *secs);
int arhip_sage_fwd_fp8(arhip_device *dev, const uint8_t *q8, const uint8_t *k8,
                       const float *sq, const float *sk, const uint16_t *v, void *o,
                       const float *mask, const int32_t *kv_len,
                       int64_t B, int64_t Hq, int64_t Hkv, int64_t N, int64_t D,
                       int64_t bq, int64_t bk, int causal, int out_dtype, float scale,
                       int wait, double *secs);

/* arhip_sage_prep_kv_rows: the reference's K and V preparation (cuda_flash_sage.rs:209-222, 257-262: a scale per
 *   key, no smoothing, V to bf16) for f32 tensors in ONE launch: k8 / sk as arhip_sage_quant(block 1, smooth 0)
 *   writes them, vb as arhip_cast_bf16 writes it, bit for bit.  k, v [B,Hkv,N,D] f32. */
int arhip_sage_prep_kv_rows(arhip_device *dev, const float *k, int8_t *k8, float *sk, const float *v, uint16_t *vb,
                            int64_t B, int64_t Hkv, int64_t N, int64_t D, int wait, double *secs);

/* arhip_cast_bf16: f32 -> bf16 round-to-nearest-even of n elements (the V
 *   operand of the Sage kernel: cuda_flash_sage.rs:99-103, 257-262). */
int arhip_cast_bf16(arhip_device *dev, const float *x, uint16_t *y, int64_t n, int wait, double *secs);

/* arhip_sage_fwd: `cuda_flash_sage::run_ex` (src/runtime/cuda_flash_sage.rs:452-485)
 *   on pre-quantised operands: int8 q8/k8 with block scales sq [B,Hq,ceil(N/bq)],
 *   sk [B,Hkv,ceil(N/bk)], v bf16 [B,Hkv,N,D]; logits int32 = q8.k8^T,
 *   s = (float)logit * ((sq*sk)*scale) (cuda_flash_sage.rs:315-322), fp32
 *   softmax, P and V in bf16, fp32 accumulate; o is f32 (out_dtype ARHIP_F32,
 *   the reference's convention) or bf16.
 *   dbg_logits: optional device int32 [32 x 64] receiving the raw logits of the
 *   tile (query rows dbg_sel[1]*32.., keys dbg_sel[2]*64..) of head dbg_sel[0]
 *   (b*Hq+h), row-major [query][key]; pass NULL in production. */
int arhip_sage_fwd(arhip_device *dev, const int8_t *q8, const int8_t *k8,
                   const float *sq, const float *sk, const uint16_t *v, void *o,
                   const float *mask, const int32_t *kv_len,
                   int64_t B, int64_t Hq, int64_t Hkv, int64_t N, int64_t D,
                   int64_t bq, int64_t bk, int causal, int out_dtype, float scale,
                   int32_t *dbg_logits, const int32_t dbg_sel[3],
                   int wait, double *secs);

/* arhip_sage_fwd_qfused: arhip_sage_quant of Q (bf16 input, blocks of 128 queries, no smoothing) and
 *   arhip_sage_fwd in one launch: the reference quantises Q inside its attention kernel
 *   (src/runtime/cuda_flash_sage.rs:201-223), and so does the pipelined kernel's prologue here, with the
 *   quantiser's own operations in its own order, so o is bit for bit what the two calls give.
 *   q bf16 [B,Hq,N,D]; k8 / sk from arhip_sage_quant with bk = 64 * 2^j; v bf16; no additive mask.
 *   sq_out [B,Hq,ceil(N/128)] and q8_out [B,Hq,N,D] receive the scales and codes where not NULL. */
int arhip_sage_fwd_qfused(arhip_device *dev, const uint16_t *q, const int8_t *k8, const float *sk,
                          const uint16_t *v, void *o, float *sq_out, int8_t *q8_out, const int32_t *kv_len,
                          int64_t B, int64_t Hq, int64_t Hkv, int64_t N, int64_t D, int64_t bk,
                          int causal, int out_dtype, float scale, int wait, double *secs);

/* arhip_sage_fwd_fp8_qfused: the same on E4M3 codes (the reference's AR_FP8 branch, src/runtime/cuda_flash_sage.rs:125-128):
 *   k8 / sk from arhip_sage_quant_fp8; the kernel derives the codes of q with scale = absmax / 448; bit for bit
 *   arhip_sage_quant_fp8 on q followed by arhip_sage_fwd_fp8. */
int arhip_sage_fwd_fp8_qfused(arhip_device *dev, const uint16_t *q, const uint8_t *k8, const float *sk,
                              const uint16_t *v, void *o, float *sq_out, uint8_t *q8_out, const int32_t *kv_len,
                              int64_t B, int64_t Hq, int64_t Hkv, int64_t N, int64_t D, int64_t bk,
                              int causal, int out_dtype, float scale, int wait, double *secs);

/* arhip_sage_fwd_qfused_rows: the same for the reference's own convention: q f32 [B,Hq,N,D], a scale
 *   per query (sq_out [B,Hq,N]), k8 / sk from arhip_sage_quant with bk = 1 (or a power of two below
 *   64); bit for bit arhip_sage_quant(block 1) on q followed by arhip_sage_fwd. */
int arhip_sage_fwd_qfused_rows(arhip_device *dev, const float *q, const int8_t *k8, const float *sk,
                               const uint16_t *v, void *o, float *sq_out, int8_t *q8_out, const int32_t *kv_len,
                               int64_t B, int64_t Hq, int64_t Hkv, int64_t N, int64_t D, int64_t bk,
                               int causal, int out_dtype, float scale, int wait, double *secs);

/* arhip_sage_fwd_strided: arhip_sage_fwd with element strides {batch, head, token} for v and o
 *   (NULL = dense): v as the projection produced it ([B,N,Hkv,D]), o written as [B,N,Hq*D].
 *   q8, k8 and the scales are this library's own pre-pass outputs and stay dense. */
int arhip_sage_fwd_strided(arhip_device *dev, const int8_t *q8, const int8_t *k8,
                           const float *sq, const float *sk, const uint16_t *v, void *o,
                           const int64_t v_strides[3], const int64_t o_strides[3],
                           const float *mask, const int32_t *kv_len,
                           int64_t B, int64_t Hq, int64_t Hkv, int64_t N, int64_t D,
                           int64_t bq, int64_t bk, int causal, int out_dtype, float scale,
                           int32_t *dbg_logits, const int32_t dbg_sel[3],
                           int wait, double *secs);

/* dispatch counters: `selections()` (src/runtime/cuda_flash_bf16.rs:443-461,
 *   cuda_flash_sage.rs:417-436) */
uint64_t arhip_selections(int kernel);

#ifdef __cplusplus
}
#endif
#endif /* ARHIP_H */
