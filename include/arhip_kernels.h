/*
 * Entry points of the loadable gfx950 code object autorust_amd/attn_kernels.hsaco
 * (built from autorust_amd/csrc/attn_entry.hip).
 *
 * This is the second face of the boundary: hosts that launch kernels by name, the way the
 * reference's `HostCall{src, name, signature, bufs, global, local, vals}` ->
 * `Compiled::run_host_kernel` -> `Prog::call` does (src/engine/session.rs:210-256,
 * src/runtime/device.rs:383-402), load the file with arhip_module_load and launch these with
 * arhip_launch.  (The file is a container of fifteen code objects, see arhip_module_load in
 * arhip.h; a host that wants hipModuleLoadData / hipModuleLaunchKernel itself loads each part,
 * or builds csrc/attn_entry.hip without -DARHIP_ENTRY_PART as one plain code object.)
 * Arguments are device pointers followed by scalars, in the reference's order
 * (src/runtime/cuda_flash_bf16.rs:226-231, 550-599):
 *
 *     (Q, K, V, O, M,   int N, int head_dim, int causal, int has_mask, int hq, int hkv)
 *     vals = [n, head_dim, causal, has_mask, hq, hkv]
 *
 * Tensors are dense [B, H, N, D]; M (f32 [N, N], additive) is read only when has_mask != 0
 * (pass O again otherwise, as the reference does: src/runtime/cuda_flash.rs:233-240); B follows
 * from the grid (grid.y = B * hq <= 65535); scale = 1/sqrt(head_dim); head_dim is 64 or 128.
 * The grid is in workgroups: [ceil(N / ARHIP_KQ_*), B * hq, 1].
 */
#ifndef ARHIP_KERNELS_H
#define ARHIP_KERNELS_H

/* queries per workgroup and workgroup size of the tilings */
#define ARHIP_KQ_GENERAL 128 /* block [256,1,1] */
#define ARHIP_KQ_LONG 256    /* block [512,1,1] */
#define ARHIP_KQ_MID 128     /* block [256,1,1]: the pipelined kernel with 4 waves, two workgroups per compute unit */

/* fp32 exact mode: replaces `ar_flash_f32`, src/runtime/cuda_flash.rs:53-141.
 * (const float *Q, *K, *V, float *O, const float *M, 6 ints); general tiling. */
#define ARHIP_KERNEL_FLASH_F32 "ar_flash_f32"
/* the variant for few, short heads (B * hq * ceil(N/128) below twice the compute units): same
 * arguments, head_dim 64 only; 32 queries per workgroup, block [256,1,1], grid [ceil(N/32), B*hq, 1]. */
#define ARHIP_KERNEL_FLASH_F32_SHORT "ar_flash_f32_short"

/* Training kernels, f32: replace `ar_fl_fwd`, `ar_fl_prep`, `ar_fl_bwd_dq`, `ar_fl_bwd_dkv`,
 * src/runtime/cuda_flash_train.rs:57-309, with the reference's argument order and head_dim
 * inserted after N; block [256,1,1].
 *   ar_fl_fwd     (Q, K, V, float *O, float *LSE, M, 6 ints)           grid [ceil(N/128), B*hq, 1]
 *   ar_fl_prep    (O, dO, float *D, int N, int head_dim)               grid [ceil(N/4), B*hq, 1]
 *   ar_fl_bwd_dq  (Q, K, V, dO, LSE, D, M, float *dQ, 6 ints)          grid [ceil(N/128), B*hq, 1]
 *   ar_fl_bwd_dkv (Q, K, V, dO, LSE, D, M, float *dK, float *dV, 6 ints)  grid [ceil(N/128), B*hkv, 1]
 * LSE and D are [B, hq, N]; dK and dV are summed over the GQA group inside the kernel. */
#define ARHIP_KERNEL_FL_FWD "ar_fl_fwd"
#define ARHIP_KERNEL_FL_PREP "ar_fl_prep"
#define ARHIP_KERNEL_FL_BWD_DQ "ar_fl_bwd_dq"
#define ARHIP_KERNEL_FL_BWD_DKV "ar_fl_bwd_dkv"
/* the variants for few, short heads (B * hkv * ceil(N/128) below twice the compute units): the same
 * arguments, head_dim 64 only; 32 queries (keys for dK/dV) per workgroup, block [256,1,1], grid.x =
 * ceil(N/32); `ar_fl_prep` is shared. */
#define ARHIP_KERNEL_FL_FWD_SHORT "ar_fl_fwd_short"
#define ARHIP_KERNEL_FL_BWD_DQ_SHORT "ar_fl_bwd_dq_short"
#define ARHIP_KERNEL_FL_BWD_DKV_SHORT "ar_fl_bwd_dkv_short"

/* bf16: replaces `ar_flash_bf16`, src/runtime/cuda_flash_bf16.rs:226-427.
 * (const bf16 *Q, *K, *V, bf16 *O, const float *M, 6 ints); general tiling, any mask. */
#define ARHIP_KERNEL_FLASH_BF16 "ar_flash_bf16"
/* the software-pipelined variant for long sequences: same arguments, has_mask must be 0,
 * (N + 320) * head_dim * 2 < 2^31; long tiling. */
#define ARHIP_KERNEL_FLASH_BF16_LONG "ar_flash_bf16_long"
/* the same kernel with 4 waves and 128 queries per workgroup (mid tiling, two workgroups per compute unit),
 * for launches whose workgroups see few tiles, down to the shortest sequences: same arguments and limits as
 * ar_flash_bf16_long. */
#define ARHIP_KERNEL_FLASH_BF16_MID "ar_flash_bf16_mid"
/* Sage int8: replaces `ar_flash_sage`, src/runtime/cuda_flash_sage.rs:168-414, on pre-quantised
 * operands (the quantiser is the pre-pass below):
 * (const int8 *Q8, *K8, const bf16 *V, float *O, const float *M, const float *SQ, const float *SK,
 *  6 ints, int bq, int bk); SQ [B,hq,ceil(N/bq)], SK [B,hkv,ceil(N/bk)]; any bq, bk >= 1 (1 = the
 * reference's per-row scales); O is f32 like the reference's; general tiling. */
#define ARHIP_KERNEL_FLASH_SAGE "ar_flash_sage"
/* pipelined variant: has_mask 0, bk = 64 * 2^n; one more int `out_f32` (O is f32 when set,
 * bf16 otherwise); long tiling. */
#define ARHIP_KERNEL_FLASH_SAGE_LONG "ar_flash_sage_long"
/* its 4-wave form (mid tiling), chosen like ar_flash_bf16_mid: same arguments as ar_flash_sage_long. */
#define ARHIP_KERNEL_FLASH_SAGE_MID "ar_flash_sage_mid"

/* Sage pre-pass (src/runtime/cuda_flash_sage.rs:124-137, 201-223 hoisted out of the attention
 * kernel; K smoothing is an extension).  x is [B*H, N, D]; block [256,1,1] unless noted.
 *   ar_sage_kmean_partial_{f32,bf16}(x, float *part, int N, int D, int nchunk)
 *        grid [ceil(nchunk / (256 / (D/8))), B*H, 1], nchunk = ceil(N/64); part [B*H, nchunk, D]
 *   ar_sage_kmean_final(const float *part, float *mean, int N, int D, int nchunk)
 *        grid [B*H, 1, 1], block [D, 1, 1]; mean [B*H, D]
 *   ar_sage_quant_blocks_{f32,bf16}(x, int8 *x8, float *scales, const float *mean,
 *                                   int N, int D, int blk, int nblk, int smooth)
 *        grid [nblk, B*H, 1]; scales [B*H, nblk]
 *   ar_sage_quant_rows_{f32,bf16}(x, int8 *x8, float *scales, const float *mean,
 *                                 int N, int D, long rows_total, int smooth)
 *        grid [ceil(rows_total / (256 / (D/8))), 1, 1]; rows_total = B*H*N (a 64-bit scalar)
 *   ar_cast_bf16(const float *x, bf16 *y, long n)
 *        grid [min(ceil(n/256), 16384), 1, 1]
 */
#define ARHIP_KERNEL_SAGE_KMEAN_PARTIAL_F32 "ar_sage_kmean_partial_f32"
#define ARHIP_KERNEL_SAGE_KMEAN_PARTIAL_BF16 "ar_sage_kmean_partial_bf16"
#define ARHIP_KERNEL_SAGE_KMEAN_FINAL "ar_sage_kmean_final"
#define ARHIP_KERNEL_SAGE_QUANT_BLOCKS_F32 "ar_sage_quant_blocks_f32"
#define ARHIP_KERNEL_SAGE_QUANT_BLOCKS_BF16 "ar_sage_quant_blocks_bf16"
#define ARHIP_KERNEL_SAGE_QUANT_ROWS_F32 "ar_sage_quant_rows_f32"
#define ARHIP_KERNEL_SAGE_QUANT_ROWS_BF16 "ar_sage_quant_rows_bf16"
#define ARHIP_KERNEL_CAST_BF16 "ar_cast_bf16"
/* ar_sage_quant_rows_f32 (smooth = 0) on K and ar_cast_bf16 on V in one launch, for the reference's convention:
 *   (K f32, K8, SK, V f32, Vb bf16, int N, int D, long rows_total, long nv, int row_blocks),
 *   grid [row_blocks + min(ceil(nv/256), 16384), 1, 1], row_blocks = ceil(rows_total / (256/(D/8))), block [256,1,1] */
#define ARHIP_KERNEL_SAGE_QUANT_ROWS_CAST_F32 "ar_sage_quant_rows_cast_f32"

/* Key-padding masks on the named-kernel seam.  The reference's fused kernels admit a dense [n, n] mask
 * only (src/models/flash_attention.rs:389-396) and leave per-batch key lengths to its general path
 * (src/tensor/mod.rs:2405-2447); these twins keep padded batches on the fused path.  Each takes the
 * arguments of the entry it is named after with one more pointer directly after M:
 *     const int *L   [B] int32; batch b attends to keys [0, L[b]) only (clamped to [0, N]; 0 => zeros)
 * and the same scalars, grid and block.
 *   ar_flash_f32_lens, ar_flash_bf16_lens, ar_flash_bf16_long_lens, ar_flash_bf16_mid_lens   (Q, K, V, O, M, L, 6 ints)
 *   ar_flash_sage_lens, ar_flash_sage_fp8_lens                           (Q8, K8, V, O, M, L, SQ, SK, 6 ints, bq, bk)
 *   ar_flash_sage_long_lens, ar_flash_sage_mid_lens, ar_flash_sage_fp8_long_lens, ar_flash_sage_fp8_mid_lens   (..., bq, bk, out_f32) */
#define ARHIP_KERNEL_FLASH_F32_LENS "ar_flash_f32_lens"
#define ARHIP_KERNEL_FLASH_BF16_LENS "ar_flash_bf16_lens"
#define ARHIP_KERNEL_FLASH_BF16_LONG_LENS "ar_flash_bf16_long_lens"
#define ARHIP_KERNEL_FLASH_BF16_MID_LENS "ar_flash_bf16_mid_lens"
#define ARHIP_KERNEL_FLASH_SAGE_LENS "ar_flash_sage_lens"
#define ARHIP_KERNEL_FLASH_SAGE_LONG_LENS "ar_flash_sage_long_lens"
#define ARHIP_KERNEL_FLASH_SAGE_MID_LENS "ar_flash_sage_mid_lens"
#define ARHIP_KERNEL_FLASH_SAGE_FP8_LENS "ar_flash_sage_fp8_lens"
#define ARHIP_KERNEL_FLASH_SAGE_FP8_LONG_LENS "ar_flash_sage_fp8_long_lens"
#define ARHIP_KERNEL_FLASH_SAGE_FP8_MID_LENS "ar_flash_sage_fp8_mid_lens"

/* The Q quantiser inside the attention kernel, as in the reference (src/runtime/cuda_flash_sage.rs:201-223), for
 * the pipelined int8 kernel: the argument lists of ar_flash_sage_long / _mid (and their _lens twins) with
 *     Q    bf16 [b*hq, n, head_dim] instead of int8 codes
 *     SQ   [b*hq, ceil(n/128)] f32, WRITTEN: the scales the kernel derived (bq must be 128)
 * K8 / SK as the K quantiser left them, bk = 64 * 2^j.  Bit-identical to ar_sage_quant_blocks_bf16 on Q followed
 * by ar_flash_sage_long / _mid.  The _fp8_ entries do the same on E4M3 codes (scale = absmax / 448): bit-identical to
 * ar_sage_quant_blocks_fp8_bf16 on Q followed by ar_flash_sage_fp8_long / _mid. */
#define ARHIP_KERNEL_FLASH_SAGE_QF_LONG "ar_flash_sage_qf_long"
#define ARHIP_KERNEL_FLASH_SAGE_QF_MID "ar_flash_sage_qf_mid"
#define ARHIP_KERNEL_FLASH_SAGE_QF_LONG_LENS "ar_flash_sage_qf_long_lens"
#define ARHIP_KERNEL_FLASH_SAGE_QF_MID_LENS "ar_flash_sage_qf_mid_lens"
#define ARHIP_KERNEL_FLASH_SAGE_FP8_QF_LONG "ar_flash_sage_fp8_qf_long"
#define ARHIP_KERNEL_FLASH_SAGE_FP8_QF_MID "ar_flash_sage_fp8_qf_mid"
#define ARHIP_KERNEL_FLASH_SAGE_FP8_QF_LONG_LENS "ar_flash_sage_fp8_qf_long_lens"
#define ARHIP_KERNEL_FLASH_SAGE_FP8_QF_MID_LENS "ar_flash_sage_fp8_qf_mid_lens"
/* The reference's own convention in one launch: the argument lists of ar_flash_sage_long / _mid (and _lens) with
 *     Q    f32 [b*hq, n, head_dim], quantised row by row in the kernel's prologue
 *     SQ   [b*hq, n] f32, WRITTEN: one scale per query (bq must be 1)
 * K8 / SK as the K quantiser left them, bk a power of two below 64 (1: a scale per key).  Bit-identical to
 * ar_sage_quant_rows_f32 on Q followed by ar_flash_sage_long / _mid. */
#define ARHIP_KERNEL_FLASH_SAGE_QR_LONG "ar_flash_sage_qr_long"
#define ARHIP_KERNEL_FLASH_SAGE_QR_MID "ar_flash_sage_qr_mid"
#define ARHIP_KERNEL_FLASH_SAGE_QR_LONG_LENS "ar_flash_sage_qr_long_lens"
#define ARHIP_KERNEL_FLASH_SAGE_QR_MID_LENS "ar_flash_sage_qr_mid_lens"

/* FP8 E4M3 variant (the reference's `src(fp8 = true)`, src/runtime/cuda_flash_sage.rs:82-84, 92-147):
 * the same argument lists as ar_flash_sage / ar_sage_quant_{blocks,rows}_*, with E4M3 codes
 * (scale = absmax / 448) in place of int8 values. */
#define ARHIP_KERNEL_FLASH_SAGE_FP8 "ar_flash_sage_fp8"
#define ARHIP_KERNEL_FLASH_SAGE_FP8_LONG "ar_flash_sage_fp8_long"   /* as ar_flash_sage_long */
#define ARHIP_KERNEL_FLASH_SAGE_FP8_MID "ar_flash_sage_fp8_mid"     /* as ar_flash_sage_mid */
#define ARHIP_KERNEL_SAGE_QUANT_BLOCKS_FP8_F32 "ar_sage_quant_blocks_fp8_f32"
#define ARHIP_KERNEL_SAGE_QUANT_BLOCKS_FP8_BF16 "ar_sage_quant_blocks_fp8_bf16"
#define ARHIP_KERNEL_SAGE_QUANT_ROWS_FP8_F32 "ar_sage_quant_rows_fp8_f32"
#define ARHIP_KERNEL_SAGE_QUANT_ROWS_FP8_BF16 "ar_sage_quant_rows_fp8_bf16"

#endif /* ARHIP_KERNELS_H */
