// The fused-attention kernels as a loadable gfx950 code object with named entry points, for hosts
// that launch kernels the way the reference does: `HostCall{src, name, signature, bufs, global,
// local, vals}` -> `Compiled::run_host_kernel` -> `Prog::call` (src/engine/session.rs:210-256,
// src/runtime/device.rs:383-402), i.e. hipModuleLoadData + hipModuleLaunchKernel
// (arhip_module_load + arhip_launch).  Arguments are device pointers followed by 32-bit scalars,
// in the reference's order:
//     (Q, K, V, O, M,  N, head_dim, causal, has_mask, hq, hkv)
//     vals = [n, head_dim, causal, has_mask, hq, hkv]          src/runtime/cuda_flash_bf16.rs:226-231,550-599
// M is read only when has_mask != 0 (the reference passes O as a dummy, cuda_flash.rs:233-240).
// Tensors are dense [B, H, N, D]; B follows from the grid (grid.y = B * hq); the scale is
// 1/sqrt(head_dim) (the reference hard-codes 0.125 for its only head_dim, 64).
//
//   entry               block      grid                      covers
//   ar_flash_f32        [256,1,1]  [ceil(n/128), B*hq, 1]    fp32 exact (cuda_flash.rs)
//   ar_flash_f32_short  [256,1,1]  [ceil(n/32), B*hq, 1]     fp32 exact for few, short heads; head_dim 64
//   ar_flash_bf16       [256,1,1]  [ceil(n/128), B*hq, 1]    bf16 (cuda_flash_bf16.rs), any mask
//   ar_flash_bf16_long  [512,1,1]  [ceil(n/256), B*hq, 1]    bf16 software-pipelined, has_mask must be 0
//   ar_flash_bf16_mid   [256,1,1]  [ceil(n/128), B*hq, 1]    the same with 4 waves (two workgroups per CU): short / causal
//   ar_flash_sage       [256,1,1]  [ceil(n/128), B*hq, 1]    int8 (cuda_flash_sage.rs), any mask, any
//                                                            block sizes incl. per-row scales; O f32
//   ar_flash_sage_long  [512,1,1]  [ceil(n/256), B*hq, 1]    int8 pipelined: has_mask 0, bk = 64 * 2^n
//   ar_flash_sage_mid   [256,1,1]  [ceil(n/128), B*hq, 1]    the same with 4 waves
//   ar_flash_sage_fp8_long, ar_flash_sage_fp8_mid  the same on E4M3 codes
// The Sage entries take pre-quantised operands (the quantiser is the pre-pass below, not part of
// the attention kernel as in the reference):
//     (Q8, K8, V, O, M, SQ, SK,  N, head_dim, causal, has_mask, hq, hkv, bq, bk [, out_f32])
// Training (src/runtime/cuda_flash_train.rs:57-309), f32, dense, the reference's argument order with
// head_dim inserted after N:
//   ar_fl_fwd      [256,1,1]  [ceil(n/128), B*hq, 1]   (Q, K, V, O, LSE, M,  N, head_dim, causal, has_mask, hq, hkv)
//   ar_fl_prep     [256,1,1]  [ceil(n/4), B*hq, 1]     (O, dO, D,  N, head_dim)
//   ar_fl_bwd_dq   [256,1,1]  [ceil(n/128), B*hq, 1]   (Q, K, V, dO, LSE, D, M, dQ,  N, head_dim, causal, has_mask, hq, hkv)
//   ar_fl_bwd_dkv  [256,1,1]  [ceil(n/128), B*hkv, 1]  (Q, K, V, dO, LSE, D, M, dK, dV,  N, head_dim, causal, has_mask, hq, hkv)
//   ar_fl_fwd_short, ar_fl_bwd_dq_short, ar_fl_bwd_dkv_short: the same arguments with grid.x = ceil(n/32), for few,
//   short heads (32 queries / keys per workgroup, the tiles of the other side dealt out between its waves); head_dim 64
// Key-padding masks: every forward entry `X` of the first table has a twin `X_lens` that takes one more
// pointer after M, `const int *L` ([B] int32: batch b attends to keys [0, L[b]) only, clamped to [0, N];
// a batch with L[b] = 0 yields zeros), with the same scalars, grid and block:
//     ar_flash_f32_lens, ar_flash_bf16_lens, ar_flash_bf16_long_lens, ar_flash_bf16_mid_lens   (Q, K, V, O, M, L,  6 ints)
//     ar_flash_sage_lens, ar_flash_sage_long_lens, ar_flash_sage_mid_lens, ar_flash_sage_fp8_lens,
//     ar_flash_sage_fp8_long_lens, ar_flash_sage_fp8_mid_lens                 (Q8, K8, V, O, M, L, SQ, SK,  ints as above)
// (The reference's fused kernels take a dense [n, n] mask only, src/models/flash_attention.rs:389-396; its
// Tensor API reaches key-padding masks through the general path, src/tensor/mod.rs:2405-2447.)
// head_dim must be 64 or 128; any other value makes the kernel return without writing.
// The *_long entries address K and V with 32-bit byte offsets: (N + 320) * head_dim * 2 < 2^31.
#include "attn_fwd.h"
#include "attn_pipe.h"
#include "flash_f32.h"
#include "flash_bwd_f32.h"
// last: it switches floating-point contraction off for the rest of the file
#include "sage_quant_kernels.h"

// The entry points compile as fifteen code objects side by side (-DARHIP_ENTRY_PART=1 ... 15; the build packs them into
// one file that arhip_module_load takes as a whole): the pipelined kernels are several thousand instructions per
// variant, minutes of compilation per entry.  Without the macro this file is one code object with all of them.
#ifndef ARHIP_ENTRY_PART
#define ARHIP_ENTRY_PART 0
#endif
#define ARHIP_PART(k) (ARHIP_ENTRY_PART == 0 || ARHIP_ENTRY_PART == (k))

using namespace arhip;

namespace {

__device__ __forceinline__ int linear_wg() { return (int)(blockIdx.y * gridDim.x + blockIdx.x); }

__device__ __forceinline__ void dense(long s[3], int H, int N, int D)
{
    s[0] = (long)H * N * D;
    s[1] = (long)N * D;
    s[2] = D;
}

// AttnParams of a dense launch whose grid is [query tiles, B * hq, 1]
__device__ __forceinline__ AttnParams dense_params(const void *q, const void *k, const void *v, void *o, const float *m,
                                                   int N, int D, int has_mask, int hq, int hkv, const int *lens = nullptr)
{
    AttnParams p = {};
    p.q = q; p.k = k; p.v = (const uint16_t *)v; p.o = o;
    p.mask = has_mask ? m : nullptr;
    p.kv_len = lens;
    p.Hq = hq; p.Hkv = hkv; p.N = N;
    dense(p.qs, hq, N, D);
    dense(p.ks, hkv, N, D);
    dense(p.vs, hkv, N, D);
    dense(p.os, hq, N, D);
    p.bq = p.bk = 1;
    p.nq = (int)gridDim.x;
    p.total = (int)(gridDim.x * gridDim.y);
    p.lpt = p.total <= 16 * 256;  // few workgroups per compute unit: order them longest first
    p.scale = 1.0f / __builtin_sqrtf((float)D);
    return p;
}

}  // namespace

namespace {
__device__ __forceinline__ void flash_f32_entry(float *lds, const float *Q, const float *K, const float *V, float *O,
                                                const float *M, const int *L, int N, int head_dim, int causal, int has_mask,
                                                int hq, int hkv)
{
    FlashF32Params p = {};
    p.q = Q; p.k = K; p.v = V; p.o = O;
    p.mask = has_mask ? M : nullptr;
    p.kv_len = L;
    p.Hq = hq; p.Hkv = hkv; p.N = N;
    p.nq = (int)gridDim.x;
    p.total = (int)(gridDim.x * gridDim.y);
    p.lpt_heads = (int)gridDim.y;  // causal: longest query tile first over all heads
    dense(p.qs, hq, N, head_dim);
    dense(p.ks, hkv, N, head_dim);
    dense(p.os, hq, N, head_dim);
    p.scale = 1.0f / __builtin_sqrtf((float)head_dim);
    const int wg = linear_wg();
    if (head_dim == 64) {
        if (causal) flash_f32_body<64, 4, true>(p, lds, wg);
        else flash_f32_body<64, 4, false>(p, lds, wg);
    } else if (head_dim == 128) {
        if (causal) flash_f32_body<128, 4, true>(p, lds, wg);
        else flash_f32_body<128, 4, false>(p, lds, wg);
    }
}
}  // namespace

#if ARHIP_PART(1)
extern "C" __global__ void __launch_bounds__(256) ar_flash_f32(const float *Q, const float *K, const float *V, float *O,
                                                                const float *M, int N, int head_dim, int causal,
                                                                int has_mask, int hq, int hkv)
{
    __shared__ __attribute__((aligned(16))) float lds[flash_f32_lds_floats<128>()];
    flash_f32_entry(lds, Q, K, V, O, M, nullptr, N, head_dim, causal, has_mask, hq, hkv);
}

extern "C" __global__ void __launch_bounds__(256) ar_flash_f32_lens(const float *Q, const float *K, const float *V, float *O,
                                                                     const float *M, const int *L, int N, int head_dim,
                                                                     int causal, int has_mask, int hq, int hkv)
{
    __shared__ __attribute__((aligned(16))) float lds[flash_f32_lds_floats<128>()];
    flash_f32_entry(lds, Q, K, V, O, M, L, N, head_dim, causal, has_mask, hq, hkv);
}

extern "C" __global__ void __launch_bounds__(256) ar_fl_fwd(const float *Q, const float *K, const float *V, float *O,
                                                             float *LSE, const float *M, int N, int head_dim, int causal,
                                                             int has_mask, int hq, int hkv)
{
    __shared__ __attribute__((aligned(16))) float lds[flash_f32_lds_floats<128>()];
    FlashF32Params p = {};
    p.q = Q; p.k = K; p.v = V; p.o = O; p.lse = LSE;
    p.mask = has_mask ? M : nullptr;
    p.Hq = hq; p.Hkv = hkv; p.N = N;
    p.nq = (int)gridDim.x;
    p.total = (int)(gridDim.x * gridDim.y);
    p.lpt_heads = (int)gridDim.y;  // causal: longest query tile first over all heads
    dense(p.qs, hq, N, head_dim);
    dense(p.ks, hkv, N, head_dim);
    dense(p.os, hq, N, head_dim);
    p.scale = 1.0f / __builtin_sqrtf((float)head_dim);
    const int wg = linear_wg();
    if (head_dim == 64) {
        if (causal) flash_f32_body<64, 4, true>(p, lds, wg);
        else flash_f32_body<64, 4, false>(p, lds, wg);
    } else if (head_dim == 128) {
        if (causal) flash_f32_body<128, 4, true>(p, lds, wg);
        else flash_f32_body<128, 4, false>(p, lds, wg);
    }
}

#endif
// Short shapes (few workgroups of 128 queries would leave most of the chip idle): 32 queries per
// workgroup, grid [ceil(N/32), B*hq, 1], the key tiles dealt out between the four waves.  head_dim 64
// only (the reference's own head size); any other returns without writing.  LSE may be null.
namespace {
__device__ __forceinline__ void flash_f32_short(const float *Q, const float *K, const float *V, float *O, float *LSE,
                                                const float *M, int N, int causal, int has_mask, int hq, int hkv, float *lds)
{
    FlashF32Params p = {};
    p.q = Q; p.k = K; p.v = V; p.o = O; p.lse = LSE;
    p.mask = has_mask ? M : nullptr;
    p.Hq = hq; p.Hkv = hkv; p.N = N;
    p.nq = (int)gridDim.x;
    p.total = (int)(gridDim.x * gridDim.y);
    p.lpt_heads = (int)gridDim.y;  // causal: longest query tile first over all heads
    dense(p.qs, hq, N, 64);
    dense(p.ks, hkv, N, 64);
    dense(p.os, hq, N, 64);
    p.scale = 0.125f;
    const int wg = linear_wg();
    if (causal) flash_f32_body<64, 4, true, true>(p, lds, wg);
    else flash_f32_body<64, 4, false, true>(p, lds, wg);
}
}  // namespace

#if ARHIP_PART(1)
extern "C" __global__ void __launch_bounds__(256, 2) ar_flash_f32_short(const float *Q, const float *K, const float *V, float *O,
                                                                         const float *M, int N, int head_dim, int causal,
                                                                         int has_mask, int hq, int hkv)
{
    __shared__ __attribute__((aligned(16))) float lds[flash_f32_lds_floats<64, 4, true>()];
    if (head_dim != 64) return;
    flash_f32_short(Q, K, V, O, nullptr, M, N, causal, has_mask, hq, hkv, lds);
}

extern "C" __global__ void __launch_bounds__(256, 2) ar_fl_fwd_short(const float *Q, const float *K, const float *V, float *O,
                                                                      float *LSE, const float *M, int N, int head_dim,
                                                                      int causal, int has_mask, int hq, int hkv)
{
    __shared__ __attribute__((aligned(16))) float lds[flash_f32_lds_floats<64, 4, true>()];
    if (head_dim != 64) return;
    flash_f32_short(Q, K, V, O, LSE, M, N, causal, has_mask, hq, hkv, lds);
}

extern "C" __global__ void __launch_bounds__(256) ar_fl_prep(const float *O, const float *dO, float *D, int N, int head_dim)
{
    const long row0 = (long)blockIdx.y * N + (long)blockIdx.x * 4, rows = ((long)blockIdx.y + 1) * N;
    if (head_dim == 64) bwd_prep_body<64>(O, dO, D, rows, row0);
    else if (head_dim == 128) bwd_prep_body<128>(O, dO, D, rows, row0);
}

#endif
namespace {
__device__ __forceinline__ FlashBwdParams bwd_params(const float *Q, const float *K, const float *V, const float *dO,
                                                     const float *LSE, const float *D, const float *M, int N,
                                                     int head_dim, int has_mask, int hq, int hkv)
{
    FlashBwdParams p = {};
    p.q = Q; p.k = K; p.v = V; p.dout = dO; p.lse = LSE; p.delta = D;
    p.mask = has_mask ? M : nullptr;
    p.Hq = hq; p.Hkv = hkv; p.N = N;
    p.nt = (int)gridDim.x;
    p.total_q = p.total_kv = (int)(gridDim.x * gridDim.y);
    p.lpt_q = p.lpt_kv = (int)gridDim.y;  // causal: longest tile first over all heads
    p.scale = 1.0f / __builtin_sqrtf((float)head_dim);
    return p;
}
}  // namespace

#if ARHIP_PART(1)
extern "C" __global__ void __launch_bounds__(256) ar_fl_bwd_dq(const float *Q, const float *K, const float *V,
                                                                const float *dO, const float *LSE, const float *D,
                                                                const float *M, float *dQ, int N, int head_dim, int causal,
                                                                int has_mask, int hq, int hkv)
{
    __shared__ __attribute__((aligned(16))) float lds[bwd_lds_floats<128>()];
    FlashBwdParams p = bwd_params(Q, K, V, dO, LSE, D, M, N, head_dim, has_mask, hq, hkv);
    p.dq = dQ;
    const int wg = linear_wg();
    if (head_dim == 64) {
        if (causal) bwd_dq_body<64, 4, true>(p, lds, wg);
        else bwd_dq_body<64, 4, false>(p, lds, wg);
    } else if (head_dim == 128) {
        if (causal) bwd_dq_body<128, 4, true>(p, lds, wg);
        else bwd_dq_body<128, 4, false>(p, lds, wg);
    }
}

extern "C" __global__ void __launch_bounds__(256) ar_fl_bwd_dkv(const float *Q, const float *K, const float *V,
                                                                 const float *dO, const float *LSE, const float *D,
                                                                 const float *M, float *dK, float *dV, int N, int head_dim,
                                                                 int causal, int has_mask, int hq, int hkv)
{
    __shared__ __attribute__((aligned(16))) float lds[bwd_lds_floats<128>()];
    FlashBwdParams p = bwd_params(Q, K, V, dO, LSE, D, M, N, head_dim, has_mask, hq, hkv);
    p.dk = dK; p.dv = dV;
    const int wg = linear_wg();
    if (head_dim == 64) {
        if (causal) bwd_dkv_body<64, 4, true>(p, lds, wg);
        else bwd_dkv_body<64, 4, false>(p, lds, wg);
    } else if (head_dim == 128) {
        if (causal) bwd_dkv_body<128, 4, true>(p, lds, wg);
        else bwd_dkv_body<128, 4, false>(p, lds, wg);
    }
}

#endif
// The same for short shapes: 32 queries (dQ) / 32 keys (dK, dV) per workgroup, grid [ceil(N/32), B*hq, 1] /
// [ceil(N/32), B*hkv, 1], the tiles of the other side dealt out between the four waves.  head_dim 64 only.
#if ARHIP_PART(1)
extern "C" __global__ void __launch_bounds__(256, 2) ar_fl_bwd_dq_short(const float *Q, const float *K, const float *V,
                                                                         const float *dO, const float *LSE, const float *D,
                                                                         const float *M, float *dQ, int N, int head_dim,
                                                                         int causal, int has_mask, int hq, int hkv)
{
    __shared__ __attribute__((aligned(16))) float lds[bwd_lds_floats<64, 4, true>()];
    if (head_dim != 64) return;
    FlashBwdParams p = bwd_params(Q, K, V, dO, LSE, D, M, N, head_dim, has_mask, hq, hkv);
    p.dq = dQ;
    const int wg = linear_wg();
    if (causal) bwd_dq_body<64, 4, true, true>(p, lds, wg);
    else bwd_dq_body<64, 4, false, true>(p, lds, wg);
}

extern "C" __global__ void __launch_bounds__(256) ar_fl_bwd_dkv_short(const float *Q, const float *K, const float *V,
                                                                       const float *dO, const float *LSE, const float *D,
                                                                       const float *M, float *dK, float *dV, int N,
                                                                       int head_dim, int causal, int has_mask, int hq, int hkv)
{
    __shared__ __attribute__((aligned(16))) float lds[bwd_lds_floats<64, 4, true>()];
    if (head_dim != 64) return;
    FlashBwdParams p = bwd_params(Q, K, V, dO, LSE, D, M, N, head_dim, has_mask, hq, hkv);
    p.dk = dK; p.dv = dV;
    const int wg = linear_wg();
    if (causal) bwd_dkv_body<64, 4, true, true>(p, lds, wg);
    else bwd_dkv_body<64, 4, false, true>(p, lds, wg);
}

#endif
namespace {
__device__ __forceinline__ void flash_bf16_entry(unsigned char *lds, const uint16_t *Q, const uint16_t *K, const uint16_t *V,
                                                 uint16_t *O, const float *M, const int *L, int N, int head_dim, int causal,
                                                 int has_mask, int hq, int hkv)
{
    AttnParams p = dense_params(Q, K, V, O, M, N, head_dim, has_mask, hq, hkv, L);
    const int wg = linear_wg();
#define AR_BF16(DD)                                                                                       \
    do {                                                                                                  \
        if (has_mask) {                                                                                   \
            if (causal) attn_fwd_body<DD, 4, true, true, MODE_BF16, false, false, false>(p, lds, wg);     \
            else attn_fwd_body<DD, 4, false, true, MODE_BF16, false, false, false>(p, lds, wg);           \
        } else {                                                                                          \
            if (causal) attn_fwd_body<DD, 4, true, false, MODE_BF16, false, false, false>(p, lds, wg);    \
            else attn_fwd_body<DD, 4, false, false, MODE_BF16, false, false, false>(p, lds, wg);          \
        }                                                                                                 \
    } while (0)
    if (head_dim == 64) AR_BF16(64);
    else if (head_dim == 128) AR_BF16(128);
#undef AR_BF16
}
}  // namespace

#if ARHIP_PART(1)
extern "C" __global__ void __launch_bounds__(256) ar_flash_bf16(const uint16_t *Q, const uint16_t *K, const uint16_t *V,
                                                                 uint16_t *O, const float *M, int N, int head_dim, int causal,
                                                                 int has_mask, int hq, int hkv)
{
    __shared__ __attribute__((aligned(16))) unsigned char lds[attn_fwd_lds_bytes<128, 4, MODE_BF16, false>()];
    flash_bf16_entry(lds, Q, K, V, O, M, nullptr, N, head_dim, causal, has_mask, hq, hkv);
}

extern "C" __global__ void __launch_bounds__(256) ar_flash_bf16_lens(const uint16_t *Q, const uint16_t *K, const uint16_t *V,
                                                                      uint16_t *O, const float *M, const int *L, int N,
                                                                      int head_dim, int causal, int has_mask, int hq, int hkv)
{
    __shared__ __attribute__((aligned(16))) unsigned char lds[attn_fwd_lds_bytes<128, 4, MODE_BF16, false>()];
    flash_bf16_entry(lds, Q, K, V, O, M, L, N, head_dim, causal, has_mask, hq, hkv);
}

#endif
namespace {
template <int NW>
__device__ __forceinline__ void flash_bf16_long_entry(unsigned char *lds, const uint16_t *Q, const uint16_t *K, const uint16_t *V,
                                                      uint16_t *O, const float *M, const int *L, int N, int head_dim, int causal,
                                                      int has_mask, int hq, int hkv)
{
    if (has_mask) return;  // this entry has no additive mask: the host picks ar_flash_bf16 for those
    AttnParams p = dense_params(Q, K, V, O, M, N, head_dim, 0, hq, hkv, L);
    const int wg = linear_wg();
    if (head_dim == 64) {
        if (causal) attn_pipe_body<64, true, MODE_BF16, false, NW>(p, lds, wg);
        else attn_pipe_body<64, false, MODE_BF16, false, NW>(p, lds, wg);
    } else if (head_dim == 128) {
        if (causal) attn_pipe_body<128, true, MODE_BF16, false, NW>(p, lds, wg);
        else attn_pipe_body<128, false, MODE_BF16, false, NW>(p, lds, wg);
    }
}
}  // namespace

#if ARHIP_PART(2)
extern "C" __global__ void __launch_bounds__(512) ar_flash_bf16_long(const uint16_t *Q, const uint16_t *K, const uint16_t *V,
                                                                      uint16_t *O, const float *M, int N, int head_dim,
                                                                      int causal, int has_mask, int hq, int hkv)
{
    __shared__ __attribute__((aligned(1024))) unsigned char lds[attn_pipe_lds_bytes<128, MODE_BF16>()];
    flash_bf16_long_entry<8>(lds, Q, K, V, O, M, nullptr, N, head_dim, causal, has_mask, hq, hkv);
}

extern "C" __global__ void __launch_bounds__(512) ar_flash_bf16_long_lens(const uint16_t *Q, const uint16_t *K, const uint16_t *V,
                                                                           uint16_t *O, const float *M, const int *L, int N,
                                                                           int head_dim, int causal, int has_mask, int hq, int hkv)
{
    __shared__ __attribute__((aligned(1024))) unsigned char lds[attn_pipe_lds_bytes<128, MODE_BF16>()];
    flash_bf16_long_entry<8>(lds, Q, K, V, O, M, L, N, head_dim, causal, has_mask, hq, hkv);
}

#endif
// the 4-wave form of the pipelined kernel: 128 queries per workgroup, two workgroups per compute unit
#if ARHIP_PART(3)
extern "C" __global__ void __launch_bounds__(256, 2) ar_flash_bf16_mid(const uint16_t *Q, const uint16_t *K, const uint16_t *V,
                                                                        uint16_t *O, const float *M, int N, int head_dim,
                                                                        int causal, int has_mask, int hq, int hkv)
{
    __shared__ __attribute__((aligned(1024))) unsigned char lds[attn_pipe_lds_bytes<128, MODE_BF16, 4>()];
    flash_bf16_long_entry<4>(lds, Q, K, V, O, M, nullptr, N, head_dim, causal, has_mask, hq, hkv);
}

extern "C" __global__ void __launch_bounds__(256, 2) ar_flash_bf16_mid_lens(const uint16_t *Q, const uint16_t *K, const uint16_t *V,
                                                                             uint16_t *O, const float *M, const int *L, int N,
                                                                             int head_dim, int causal, int has_mask, int hq, int hkv)
{
    __shared__ __attribute__((aligned(1024))) unsigned char lds[attn_pipe_lds_bytes<128, MODE_BF16, 4>()];
    flash_bf16_long_entry<4>(lds, Q, K, V, O, M, L, N, head_dim, causal, has_mask, hq, hkv);
}

#endif
namespace {
// ar_flash_sage / ar_flash_sage_fp8: the general kernel on pre-quantised operands, QMODE = MODE_I8 or MODE_FP8
template <int QMODE>
__device__ __forceinline__ void flash_sage_entry(unsigned char *lds, const void *Q8, const void *K8, const uint16_t *V, float *O,
                                                 const float *M, const int *L, const float *SQ, const float *SK, int N, int head_dim,
                                                 int causal, int has_mask, int hq, int hkv, int bq, int bk)
{
    AttnParams p = dense_params(Q8, K8, V, O, M, N, head_dim, has_mask, hq, hkv, L);
    p.sq = SQ; p.sk = SK;
    p.bq = bq; p.bk = bk;
    // K scales that are uniform over a 64-key tile (bk = 64 * 2^n) are a scalar per tile; any other
    // block size, the reference's per-key scales (bk = 1) included, stages the tile's scales in LDS
    int shift = 0;
    while ((64 << shift) < bk) ++shift;
    const bool per_key = (64 << shift) != bk;
    p.bk_tile_shift = shift;
    const int wg = linear_wg();
#define AR_SAGE(DD, PK)                                                                                 \
    do {                                                                                                \
        if (has_mask) {                                                                                 \
            if (causal) attn_fwd_body<DD, 4, true, true, QMODE, PK, true, false>(p, lds, wg);           \
            else attn_fwd_body<DD, 4, false, true, QMODE, PK, true, false>(p, lds, wg);                 \
        } else {                                                                                        \
            if (causal) attn_fwd_body<DD, 4, true, false, QMODE, PK, true, false>(p, lds, wg);          \
            else attn_fwd_body<DD, 4, false, false, QMODE, PK, true, false>(p, lds, wg);                \
        }                                                                                               \
    } while (0)
    if (head_dim == 64) {
        if (per_key) AR_SAGE(64, true);
        else AR_SAGE(64, false);
    } else if (head_dim == 128) {
        if (per_key) AR_SAGE(128, true);
        else AR_SAGE(128, false);
    }
#undef AR_SAGE
}
}  // namespace

#if ARHIP_PART(4)
extern "C" __global__ void __launch_bounds__(256) ar_flash_sage(const int8_t *Q8, const int8_t *K8, const uint16_t *V, float *O,
                                                                 const float *M, const float *SQ, const float *SK, int N,
                                                                 int head_dim, int causal, int has_mask, int hq, int hkv,
                                                                 int bq, int bk)
{
    __shared__ __attribute__((aligned(16))) unsigned char lds[attn_fwd_lds_bytes<128, 4, MODE_I8, true>()];
    flash_sage_entry<MODE_I8>(lds, Q8, K8, V, O, M, nullptr, SQ, SK, N, head_dim, causal, has_mask, hq, hkv, bq, bk);
}

extern "C" __global__ void __launch_bounds__(256) ar_flash_sage_lens(const int8_t *Q8, const int8_t *K8, const uint16_t *V, float *O,
                                                                      const float *M, const int *L, const float *SQ, const float *SK,
                                                                      int N, int head_dim, int causal, int has_mask, int hq, int hkv,
                                                                      int bq, int bk)
{
    __shared__ __attribute__((aligned(16))) unsigned char lds[attn_fwd_lds_bytes<128, 4, MODE_I8, true>()];
    flash_sage_entry<MODE_I8>(lds, Q8, K8, V, O, M, L, SQ, SK, N, head_dim, causal, has_mask, hq, hkv, bq, bk);
}

#endif
// the FP8 E4M3 variant (the reference's AR_FP8 = 1 source, src/runtime/cuda_flash_sage.rs:82-84): same
// arguments, Q8 / K8 hold E4M3 codes
#if ARHIP_PART(5)
extern "C" __global__ void __launch_bounds__(256) ar_flash_sage_fp8(const uint8_t *Q8, const uint8_t *K8, const uint16_t *V,
                                                                     float *O, const float *M, const float *SQ, const float *SK,
                                                                     int N, int head_dim, int causal, int has_mask, int hq,
                                                                     int hkv, int bq, int bk)
{
    __shared__ __attribute__((aligned(16))) unsigned char lds[attn_fwd_lds_bytes<128, 4, MODE_FP8, true>()];
    flash_sage_entry<MODE_FP8>(lds, Q8, K8, V, O, M, nullptr, SQ, SK, N, head_dim, causal, has_mask, hq, hkv, bq, bk);
}

extern "C" __global__ void __launch_bounds__(256) ar_flash_sage_fp8_lens(const uint8_t *Q8, const uint8_t *K8, const uint16_t *V,
                                                                          float *O, const float *M, const int *L, const float *SQ,
                                                                          const float *SK, int N, int head_dim, int causal,
                                                                          int has_mask, int hq, int hkv, int bq, int bk)
{
    __shared__ __attribute__((aligned(16))) unsigned char lds[attn_fwd_lds_bytes<128, 4, MODE_FP8, true>()];
    flash_sage_entry<MODE_FP8>(lds, Q8, K8, V, O, M, L, SQ, SK, N, head_dim, causal, has_mask, hq, hkv, bq, bk);
}

#endif
// ar_flash_sage_long / ar_flash_sage_fp8_long: the pipelined kernel on pre-quantised operands
template <int QMODE, int NW = 8>
__device__ __forceinline__ void flash_sage_long_entry(unsigned char *lds, const void *Q8, const void *K8, const uint16_t *V, void *O,
                                                      const float *M, const int *L, const float *SQ, const float *SK, int N,
                                                      int head_dim, int causal, int has_mask, int hq, int hkv, int bq, int bk,
                                                      int out_f32)
{
    int shift = 0, key_shift = 0;
    while ((64 << shift) < bk) ++shift;
    while ((1 << key_shift) < bk) ++key_shift;
    // K scales over a power of two of keys below 64 take the per-key form
    const bool keys = bk < 64 && (1 << key_shift) == bk;
    if (has_mask || ((64 << shift) != bk && !keys)) return;  // the general kernels cover those
    AttnParams p = dense_params(Q8, K8, V, O, M, N, head_dim, 0, hq, hkv, L);
    p.sq = SQ; p.sk = SK;
    p.bq = bq; p.bk = bk;
    p.bk_tile_shift = shift;
    p.bk_key_shift = keys ? key_shift : -1;
    p.out_f32 = out_f32;
    const int wg = linear_wg();
#define AR_SAGE_LONG(DD, PK)                                                              \
    do {                                                                                  \
        if (causal) attn_pipe_body<DD, true, QMODE, false, NW, PK>(p, lds, wg);           \
        else attn_pipe_body<DD, false, QMODE, false, NW, PK>(p, lds, wg);                 \
    } while (0)
    if (keys) {
        if (head_dim == 64) AR_SAGE_LONG(64, true);
        else if (head_dim == 128) AR_SAGE_LONG(128, true);
        return;
    }
    if (head_dim == 64) AR_SAGE_LONG(64, false);
    else if (head_dim == 128) AR_SAGE_LONG(128, false);
#undef AR_SAGE_LONG
}

#if ARHIP_PART(6)
extern "C" __global__ void __launch_bounds__(512) ar_flash_sage_long(const int8_t *Q8, const int8_t *K8, const uint16_t *V,
                                                                      void *O, const float *M, const float *SQ, const float *SK,
                                                                      int N, int head_dim, int causal, int has_mask, int hq,
                                                                      int hkv, int bq, int bk, int out_f32)
{
    __shared__ __attribute__((aligned(1024))) unsigned char lds[attn_pipe_lds_bytes<128, MODE_I8, 8, true>()];
    flash_sage_long_entry<MODE_I8>(lds, Q8, K8, V, O, M, nullptr, SQ, SK, N, head_dim, causal, has_mask, hq, hkv, bq, bk, out_f32);
}

extern "C" __global__ void __launch_bounds__(512) ar_flash_sage_long_lens(const int8_t *Q8, const int8_t *K8, const uint16_t *V,
                                                                           void *O, const float *M, const int *L, const float *SQ,
                                                                           const float *SK, int N, int head_dim, int causal,
                                                                           int has_mask, int hq, int hkv, int bq, int bk, int out_f32)
{
    __shared__ __attribute__((aligned(1024))) unsigned char lds[attn_pipe_lds_bytes<128, MODE_I8, 8, true>()];
    flash_sage_long_entry<MODE_I8>(lds, Q8, K8, V, O, M, L, SQ, SK, N, head_dim, causal, has_mask, hq, hkv, bq, bk, out_f32);
}

#endif
// the 4-wave form: 128 queries per workgroup, two workgroups per compute unit
#if ARHIP_PART(7)
extern "C" __global__ void __launch_bounds__(256, 2) ar_flash_sage_mid(const int8_t *Q8, const int8_t *K8, const uint16_t *V,
                                                                        void *O, const float *M, const float *SQ, const float *SK,
                                                                        int N, int head_dim, int causal, int has_mask, int hq,
                                                                        int hkv, int bq, int bk, int out_f32)
{
    __shared__ __attribute__((aligned(1024))) unsigned char lds[attn_pipe_lds_bytes<128, MODE_I8, 4, true>()];
    flash_sage_long_entry<MODE_I8, 4>(lds, Q8, K8, V, O, M, nullptr, SQ, SK, N, head_dim, causal, has_mask, hq, hkv, bq, bk, out_f32);
}

extern "C" __global__ void __launch_bounds__(256, 2) ar_flash_sage_mid_lens(const int8_t *Q8, const int8_t *K8, const uint16_t *V,
                                                                             void *O, const float *M, const int *L, const float *SQ,
                                                                             const float *SK, int N, int head_dim, int causal,
                                                                             int has_mask, int hq, int hkv, int bq, int bk, int out_f32)
{
    __shared__ __attribute__((aligned(1024))) unsigned char lds[attn_pipe_lds_bytes<128, MODE_I8, 4, true>()];
    flash_sage_long_entry<MODE_I8, 4>(lds, Q8, K8, V, O, M, L, SQ, SK, N, head_dim, causal, has_mask, hq, hkv, bq, bk, out_f32);
}

#endif
// ar_flash_sage_qf_long / _mid (and ar_flash_sage_fp8_qf_long / _mid on E4M3 codes): the pipelined 8-bit kernel with the
// Q quantiser in its prologue.  Q holds bf16
// values; SQ [b*hq, ceil(n/128)] RECEIVES the scales (bq must be 128); K8 / SK as from the K quantiser with
// bk = 64 * 2^j.  Same grid and block as ar_flash_sage_long / _mid.
template <int NW, int MODE = MODE_I8>
__device__ __forceinline__ void flash_sage_qf_entry(unsigned char *lds, const uint16_t *Q, const void *K8, const uint16_t *V, void *O,
                                                    const float *M, const int *L, float *SQ, const float *SK, int N, int head_dim,
                                                    int causal, int has_mask, int hq, int hkv, int bq, int bk, int out_f32)
{
    int shift = 0;
    while ((64 << shift) < bk) ++shift;
    if (has_mask || (64 << shift) != bk || bq != 128) return;  // refused on the host
    AttnParams p = dense_params(Q, K8, V, O, M, N, head_dim, 0, hq, hkv, L);
    p.sk = SK;
    p.sq_out = SQ;
    p.bq = bq; p.bk = bk;
    p.bk_tile_shift = shift;
    p.bk_key_shift = -1;
    p.out_f32 = out_f32;
    const int wg = linear_wg();
#define AR_SAGE_QF(DD)                                                                        \
    do {                                                                                      \
        if (causal) attn_pipe_body<DD, true, MODE, false, NW, false, true>(p, lds, wg);       \
        else attn_pipe_body<DD, false, MODE, false, NW, false, true>(p, lds, wg);             \
    } while (0)
    if (head_dim == 64) AR_SAGE_QF(64);
    else if (head_dim == 128) AR_SAGE_QF(128);
#undef AR_SAGE_QF
}

#if ARHIP_PART(8)
extern "C" __global__ void __launch_bounds__(512) ar_flash_sage_qf_long(const uint16_t *Q, const int8_t *K8, const uint16_t *V,
                                                                         void *O, const float *M, float *SQ, const float *SK,
                                                                         int N, int head_dim, int causal, int has_mask, int hq,
                                                                         int hkv, int bq, int bk, int out_f32)
{
    __shared__ __attribute__((aligned(1024))) unsigned char lds[attn_pipe_lds_bytes<128, MODE_I8, 8, false, true>()];
    flash_sage_qf_entry<8>(lds, Q, K8, V, O, M, nullptr, SQ, SK, N, head_dim, causal, has_mask, hq, hkv, bq, bk, out_f32);
}

extern "C" __global__ void __launch_bounds__(512) ar_flash_sage_qf_long_lens(const uint16_t *Q, const int8_t *K8, const uint16_t *V,
                                                                              void *O, const float *M, const int *L, float *SQ,
                                                                              const float *SK, int N, int head_dim, int causal,
                                                                              int has_mask, int hq, int hkv, int bq, int bk,
                                                                              int out_f32)
{
    __shared__ __attribute__((aligned(1024))) unsigned char lds[attn_pipe_lds_bytes<128, MODE_I8, 8, false, true>()];
    flash_sage_qf_entry<8>(lds, Q, K8, V, O, M, L, SQ, SK, N, head_dim, causal, has_mask, hq, hkv, bq, bk, out_f32);
}

#endif
#if ARHIP_PART(9)
extern "C" __global__ void __launch_bounds__(256, 2) ar_flash_sage_qf_mid(const uint16_t *Q, const int8_t *K8, const uint16_t *V,
                                                                           void *O, const float *M, float *SQ, const float *SK,
                                                                           int N, int head_dim, int causal, int has_mask, int hq,
                                                                           int hkv, int bq, int bk, int out_f32)
{
    __shared__ __attribute__((aligned(1024))) unsigned char lds[attn_pipe_lds_bytes<128, MODE_I8, 4, false, true>()];
    flash_sage_qf_entry<4>(lds, Q, K8, V, O, M, nullptr, SQ, SK, N, head_dim, causal, has_mask, hq, hkv, bq, bk, out_f32);
}

extern "C" __global__ void __launch_bounds__(256, 2) ar_flash_sage_qf_mid_lens(const uint16_t *Q, const int8_t *K8, const uint16_t *V,
                                                                                void *O, const float *M, const int *L, float *SQ,
                                                                                const float *SK, int N, int head_dim, int causal,
                                                                                int has_mask, int hq, int hkv, int bq, int bk,
                                                                                int out_f32)
{
    __shared__ __attribute__((aligned(1024))) unsigned char lds[attn_pipe_lds_bytes<128, MODE_I8, 4, false, true>()];
    flash_sage_qf_entry<4>(lds, Q, K8, V, O, M, L, SQ, SK, N, head_dim, causal, has_mask, hq, hkv, bq, bk, out_f32);
}

#endif
#if ARHIP_PART(14)
extern "C" __global__ void __launch_bounds__(512) ar_flash_sage_fp8_qf_long(const uint16_t *Q, const uint8_t *K8, const uint16_t *V,
                                                                             void *O, const float *M, float *SQ, const float *SK,
                                                                             int N, int head_dim, int causal, int has_mask, int hq,
                                                                             int hkv, int bq, int bk, int out_f32)
{
    __shared__ __attribute__((aligned(1024))) unsigned char lds[attn_pipe_lds_bytes<128, MODE_FP8, 8, false, true>()];
    flash_sage_qf_entry<8, MODE_FP8>(lds, Q, K8, V, O, M, nullptr, SQ, SK, N, head_dim, causal, has_mask, hq, hkv, bq, bk, out_f32);
}

extern "C" __global__ void __launch_bounds__(512) ar_flash_sage_fp8_qf_long_lens(const uint16_t *Q, const uint8_t *K8, const uint16_t *V,
                                                                                  void *O, const float *M, const int *L, float *SQ,
                                                                                  const float *SK, int N, int head_dim, int causal,
                                                                                  int has_mask, int hq, int hkv, int bq, int bk,
                                                                                  int out_f32)
{
    __shared__ __attribute__((aligned(1024))) unsigned char lds[attn_pipe_lds_bytes<128, MODE_FP8, 8, false, true>()];
    flash_sage_qf_entry<8, MODE_FP8>(lds, Q, K8, V, O, M, L, SQ, SK, N, head_dim, causal, has_mask, hq, hkv, bq, bk, out_f32);
}

#endif
#if ARHIP_PART(15)
extern "C" __global__ void __launch_bounds__(256, 2) ar_flash_sage_fp8_qf_mid(const uint16_t *Q, const uint8_t *K8, const uint16_t *V,
                                                                               void *O, const float *M, float *SQ, const float *SK,
                                                                               int N, int head_dim, int causal, int has_mask, int hq,
                                                                               int hkv, int bq, int bk, int out_f32)
{
    __shared__ __attribute__((aligned(1024))) unsigned char lds[attn_pipe_lds_bytes<128, MODE_FP8, 4, false, true>()];
    flash_sage_qf_entry<4, MODE_FP8>(lds, Q, K8, V, O, M, nullptr, SQ, SK, N, head_dim, causal, has_mask, hq, hkv, bq, bk, out_f32);
}

extern "C" __global__ void __launch_bounds__(256, 2) ar_flash_sage_fp8_qf_mid_lens(const uint16_t *Q, const uint8_t *K8, const uint16_t *V,
                                                                                    void *O, const float *M, const int *L, float *SQ,
                                                                                    const float *SK, int N, int head_dim, int causal,
                                                                                    int has_mask, int hq, int hkv, int bq, int bk,
                                                                                    int out_f32)
{
    __shared__ __attribute__((aligned(1024))) unsigned char lds[attn_pipe_lds_bytes<128, MODE_FP8, 4, false, true>()];
    flash_sage_qf_entry<4, MODE_FP8>(lds, Q, K8, V, O, M, L, SQ, SK, N, head_dim, causal, has_mask, hq, hkv, bq, bk, out_f32);
}

#endif
// ar_flash_sage_qr_long / _mid: the reference's convention in one launch.  Q holds f32 values and is quantised row by
// row in the prologue; SQ [b*hq, n] RECEIVES the scales (bq must be 1); K8 / SK as from the K quantiser with bk a
// power of two below 64 (bk = 1: a scale per key).  Same grid and block as ar_flash_sage_long / _mid.
template <int NW>
__device__ __forceinline__ void flash_sage_qr_entry(unsigned char *lds, const float *Q, const void *K8, const uint16_t *V, void *O,
                                                    const float *M, const int *L, float *SQ, const float *SK, int N, int head_dim,
                                                    int causal, int has_mask, int hq, int hkv, int bq, int bk, int out_f32)
{
    int key_shift = 0;
    while ((1 << key_shift) < bk) ++key_shift;
    if (has_mask || bk >= 64 || (1 << key_shift) != bk || bq != 1) return;  // refused on the host
    AttnParams p = dense_params(Q, K8, V, O, M, N, head_dim, 0, hq, hkv, L);
    p.sk = SK;
    p.sq_out = SQ;
    p.bq = bq; p.bk = bk;
    p.bk_tile_shift = 0;
    p.bk_key_shift = key_shift;
    p.out_f32 = out_f32;
    const int wg = linear_wg();
#define AR_SAGE_QR(DD)                                                                       \
    do {                                                                                     \
        if (causal) attn_pipe_body<DD, true, MODE_I8, false, NW, true, true>(p, lds, wg);    \
        else attn_pipe_body<DD, false, MODE_I8, false, NW, true, true>(p, lds, wg);          \
    } while (0)
    if (head_dim == 64) AR_SAGE_QR(64);
    else if (head_dim == 128) AR_SAGE_QR(128);
#undef AR_SAGE_QR
}

#if ARHIP_PART(12)
extern "C" __global__ void __launch_bounds__(512) ar_flash_sage_qr_long(const float *Q, const int8_t *K8, const uint16_t *V,
                                                                         void *O, const float *M, float *SQ, const float *SK,
                                                                         int N, int head_dim, int causal, int has_mask, int hq,
                                                                         int hkv, int bq, int bk, int out_f32)
{
    __shared__ __attribute__((aligned(1024))) unsigned char lds[attn_pipe_lds_bytes<128, MODE_I8, 8, true, true>()];
    flash_sage_qr_entry<8>(lds, Q, K8, V, O, M, nullptr, SQ, SK, N, head_dim, causal, has_mask, hq, hkv, bq, bk, out_f32);
}

extern "C" __global__ void __launch_bounds__(512) ar_flash_sage_qr_long_lens(const float *Q, const int8_t *K8, const uint16_t *V,
                                                                              void *O, const float *M, const int *L, float *SQ,
                                                                              const float *SK, int N, int head_dim, int causal,
                                                                              int has_mask, int hq, int hkv, int bq, int bk,
                                                                              int out_f32)
{
    __shared__ __attribute__((aligned(1024))) unsigned char lds[attn_pipe_lds_bytes<128, MODE_I8, 8, true, true>()];
    flash_sage_qr_entry<8>(lds, Q, K8, V, O, M, L, SQ, SK, N, head_dim, causal, has_mask, hq, hkv, bq, bk, out_f32);
}

#endif
#if ARHIP_PART(13)
extern "C" __global__ void __launch_bounds__(256, 2) ar_flash_sage_qr_mid(const float *Q, const int8_t *K8, const uint16_t *V,
                                                                           void *O, const float *M, float *SQ, const float *SK,
                                                                           int N, int head_dim, int causal, int has_mask, int hq,
                                                                           int hkv, int bq, int bk, int out_f32)
{
    __shared__ __attribute__((aligned(1024))) unsigned char lds[attn_pipe_lds_bytes<128, MODE_I8, 4, true, true>()];
    flash_sage_qr_entry<4>(lds, Q, K8, V, O, M, nullptr, SQ, SK, N, head_dim, causal, has_mask, hq, hkv, bq, bk, out_f32);
}

extern "C" __global__ void __launch_bounds__(256, 2) ar_flash_sage_qr_mid_lens(const float *Q, const int8_t *K8, const uint16_t *V,
                                                                                void *O, const float *M, const int *L, float *SQ,
                                                                                const float *SK, int N, int head_dim, int causal,
                                                                                int has_mask, int hq, int hkv, int bq, int bk,
                                                                                int out_f32)
{
    __shared__ __attribute__((aligned(1024))) unsigned char lds[attn_pipe_lds_bytes<128, MODE_I8, 4, true, true>()];
    flash_sage_qr_entry<4>(lds, Q, K8, V, O, M, L, SQ, SK, N, head_dim, causal, has_mask, hq, hkv, bq, bk, out_f32);
}

#endif
#if ARHIP_PART(10)
extern "C" __global__ void __launch_bounds__(512) ar_flash_sage_fp8_long(const uint8_t *Q8, const uint8_t *K8, const uint16_t *V,
                                                                          void *O, const float *M, const float *SQ, const float *SK,
                                                                          int N, int head_dim, int causal, int has_mask, int hq,
                                                                          int hkv, int bq, int bk, int out_f32)
{
    __shared__ __attribute__((aligned(1024))) unsigned char lds[attn_pipe_lds_bytes<128, MODE_FP8, 8, true>()];
    flash_sage_long_entry<MODE_FP8>(lds, Q8, K8, V, O, M, nullptr, SQ, SK, N, head_dim, causal, has_mask, hq, hkv, bq, bk, out_f32);
}

extern "C" __global__ void __launch_bounds__(512) ar_flash_sage_fp8_long_lens(const uint8_t *Q8, const uint8_t *K8, const uint16_t *V,
                                                                               void *O, const float *M, const int *L, const float *SQ,
                                                                               const float *SK, int N, int head_dim, int causal,
                                                                               int has_mask, int hq, int hkv, int bq, int bk,
                                                                               int out_f32)
{
    __shared__ __attribute__((aligned(1024))) unsigned char lds[attn_pipe_lds_bytes<128, MODE_FP8, 8, true>()];
    flash_sage_long_entry<MODE_FP8>(lds, Q8, K8, V, O, M, L, SQ, SK, N, head_dim, causal, has_mask, hq, hkv, bq, bk, out_f32);
}

#endif
#if ARHIP_PART(11)
extern "C" __global__ void __launch_bounds__(256, 2) ar_flash_sage_fp8_mid(const uint8_t *Q8, const uint8_t *K8, const uint16_t *V,
                                                                            void *O, const float *M, const float *SQ, const float *SK,
                                                                            int N, int head_dim, int causal, int has_mask, int hq,
                                                                            int hkv, int bq, int bk, int out_f32)
{
    __shared__ __attribute__((aligned(1024))) unsigned char lds[attn_pipe_lds_bytes<128, MODE_FP8, 4, true>()];
    flash_sage_long_entry<MODE_FP8, 4>(lds, Q8, K8, V, O, M, nullptr, SQ, SK, N, head_dim, causal, has_mask, hq, hkv, bq, bk, out_f32);
}

extern "C" __global__ void __launch_bounds__(256, 2) ar_flash_sage_fp8_mid_lens(const uint8_t *Q8, const uint8_t *K8, const uint16_t *V,
                                                                                 void *O, const float *M, const int *L, const float *SQ,
                                                                                 const float *SK, int N, int head_dim, int causal,
                                                                                 int has_mask, int hq, int hkv, int bq, int bk,
                                                                                 int out_f32)
{
    __shared__ __attribute__((aligned(1024))) unsigned char lds[attn_pipe_lds_bytes<128, MODE_FP8, 4, true>()];
    flash_sage_long_entry<MODE_FP8, 4>(lds, Q8, K8, V, O, M, L, SQ, SK, N, head_dim, causal, has_mask, hq, hkv, bq, bk, out_f32);
}

#endif
// ---- Sage pre-pass (the quantiser the reference runs inside its attention kernel,
// src/runtime/cuda_flash_sage.rs:201-223,248-278, hoisted into passes of its own) ----
// x [B*H, N, D] f32 or bf16; block [256,1,1] for all of them.
//   ar_sage_kmean_partial_*  grid [ceil(ceil(N/64) / (256/(D/8))), B*H, 1]   part [B*H, ceil(N/64), D]
//   ar_sage_kmean_final      grid [B*H, 1, 1], block [D,1,1]                 mean [B*H, D]
//   ar_sage_quant_blocks_*   grid [ceil(N/blk), B*H, 1]                      x8, scales [B*H, ceil(N/blk)]
//   ar_sage_quant_rows_*     grid [ceil(B*H*N / (256/(D/8))), 1, 1]          x8, scales [B*H*N]
//   ar_cast_bf16             grid [min(ceil(n/256), 16384), 1, 1]            y bf16
// smooth != 0 subtracts mean[bh][d] first (K smoothing).
#if ARHIP_PART(1)
extern "C" __global__ void __launch_bounds__(256) ar_sage_kmean_partial_f32(const float *x, float *part, int N, int D, int nchunk)
{
    k_mean_partial_body<float>(x, part, N, D, nchunk, XLayout::dense(1, N, D), blockIdx);
}
extern "C" __global__ void __launch_bounds__(256) ar_sage_kmean_partial_bf16(const uint16_t *x, float *part, int N, int D, int nchunk)
{
    k_mean_partial_body<uint16_t>(x, part, N, D, nchunk, XLayout::dense(1, N, D), blockIdx);
}
extern "C" __global__ void ar_sage_kmean_final(const float *part, float *mean, int N, int D, int nchunk)
{
    k_mean_final_body(part, mean, N, D, nchunk, blockIdx);
}
extern "C" __global__ void __launch_bounds__(256) ar_sage_quant_blocks_f32(const float *x, int8_t *x8, float *scales,
                                                                            const float *mean, int N, int D, int blk, int nblk,
                                                                            int smooth)
{
    if (smooth) quant_blocks_body<float, true>(x, x8, scales, mean, N, D, blk, nblk, XLayout::dense(1, N, D), blockIdx);
    else quant_blocks_body<float, false>(x, x8, scales, mean, N, D, blk, nblk, XLayout::dense(1, N, D), blockIdx);
}
extern "C" __global__ void __launch_bounds__(256) ar_sage_quant_blocks_bf16(const uint16_t *x, int8_t *x8, float *scales,
                                                                             const float *mean, int N, int D, int blk, int nblk,
                                                                             int smooth)
{
    if (smooth) quant_blocks_body<uint16_t, true>(x, x8, scales, mean, N, D, blk, nblk, XLayout::dense(1, N, D), blockIdx);
    else quant_blocks_body<uint16_t, false>(x, x8, scales, mean, N, D, blk, nblk, XLayout::dense(1, N, D), blockIdx);
}
extern "C" __global__ void __launch_bounds__(256) ar_sage_quant_rows_f32(const float *x, int8_t *x8, float *scales,
                                                                          const float *mean, int N, int D, long rows_total,
                                                                          int smooth)
{
    if (smooth) quant_rows_body<float, true>(x, x8, scales, mean, N, D, rows_total, XLayout::dense(1, N, D), blockIdx);
    else quant_rows_body<float, false>(x, x8, scales, mean, N, D, rows_total, XLayout::dense(1, N, D), blockIdx);
}
extern "C" __global__ void __launch_bounds__(256) ar_sage_quant_rows_bf16(const uint16_t *x, int8_t *x8, float *scales,
                                                                           const float *mean, int N, int D, long rows_total,
                                                                           int smooth)
{
    if (smooth) quant_rows_body<uint16_t, true>(x, x8, scales, mean, N, D, rows_total, XLayout::dense(1, N, D), blockIdx);
    else quant_rows_body<uint16_t, false>(x, x8, scales, mean, N, D, rows_total, XLayout::dense(1, N, D), blockIdx);
}
#endif
// FP8 E4M3 quantiser entries: same arguments, x8 receives E4M3 codes, scale = absmax / 448
#define AR_QUANT_FP8(SUFFIX, T)                                                                                              \
    extern "C" __global__ void __launch_bounds__(256) ar_sage_quant_blocks_fp8_##SUFFIX(                                     \
        const T *x, uint8_t *x8, float *scales, const float *mean, int N, int D, int blk, int nblk, int smooth)              \
    {                                                                                                                        \
        if (smooth) quant_blocks_body<T, true, true>(x, (int8_t *)x8, scales, mean, N, D, blk, nblk, XLayout::dense(1, N, D), blockIdx);  \
        else quant_blocks_body<T, false, true>(x, (int8_t *)x8, scales, mean, N, D, blk, nblk, XLayout::dense(1, N, D), blockIdx);        \
    }                                                                                                                        \
    extern "C" __global__ void __launch_bounds__(256) ar_sage_quant_rows_fp8_##SUFFIX(                                       \
        const T *x, uint8_t *x8, float *scales, const float *mean, int N, int D, long rows_total, int smooth)                \
    {                                                                                                                        \
        if (smooth) quant_rows_body<T, true, true>(x, (int8_t *)x8, scales, mean, N, D, rows_total, XLayout::dense(1, N, D), blockIdx);   \
        else quant_rows_body<T, false, true>(x, (int8_t *)x8, scales, mean, N, D, rows_total, XLayout::dense(1, N, D), blockIdx);         \
    }
#if ARHIP_PART(1)
AR_QUANT_FP8(f32, float)
AR_QUANT_FP8(bf16, uint16_t)
#endif
#undef AR_QUANT_FP8

#if ARHIP_PART(1)
extern "C" __global__ void __launch_bounds__(256) ar_cast_bf16(const float *x, uint16_t *y, long n)
{
    cast_bf16_body(x, y, (size_t)n, blockIdx);
}

// ar_sage_quant_rows_cast_f32: ar_sage_quant_rows_f32 (smooth = 0) on K and ar_cast_bf16 on V in one launch.
//   grid [row_blocks + cast_blocks, 1, 1] with row_blocks = ceil(B*Hkv*N / (256/(D/8))), cast_blocks = min(ceil(nv/256), 16384)
extern "C" __global__ void __launch_bounds__(256) ar_sage_quant_rows_cast_f32(const float *k, int8_t *k8, float *scales,
                                                                               const float *v, uint16_t *vb, int N, int D,
                                                                               long rows_total, long nv, int row_blocks)
{
    quant_rows_cast_body(k, k8, scales, v, vb, N, D, rows_total, nv, row_blocks, blockIdx);
}

#endif