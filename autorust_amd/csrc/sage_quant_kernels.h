// Kernels of the Sage pre-pass: K mean (smoothing), per-block / per-row symmetric int8
// quantisation, f32 -> bf16 cast.  All of it is HBM-bound streaming work.
//
// The quantisation rule is the reference's (src/runtime/cuda_flash_sage.rs):
//   scale = absmax > 0 ? absmax / 127 : 1      (:209-213, :264-268)
//   inv   = 1 / scale                          (:218, :273)
//   x8    = clamp(rint(x * inv), -127, 127)    (:124-137), rint = nearest-even
// hoisted out of the attention kernel (the reference re-quantises K for every query block,
// :248-278) and applied to blocks of tokens instead of single rows.  Every fp32 operation is a
// single IEEE operation in a fixed order, so the int8 tensors and scales are bit-reproducible on
// the CPU.  Each kernel is a __device__ body plus a __global__ template; the loadable code
// object wraps the same bodies in named entry points.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#pragma clang fp contract(off)

namespace arhip {

constexpr int MEAN_CHUNK = 64;  // tokens per partial sum

// Where the input tensor's rows are: element strides of batch / head / token (the channel stride
// is 1).  Dense [B, H, N, D] is {H*N*D, N*D, D}; the token-major layout a projection produces,
// [B, N, H, D], is {N*H*D, D, H*D}.  Outputs of the pre-pass are always dense.
struct XLayout {
    long sb, sh, st;
    int H;
    __host__ __device__ static XLayout dense(int H, int N, int D) { return {(long)H * N * D, (long)N * D, (long)D, H}; }
    __device__ __forceinline__ size_t head(int bh) const { return (size_t)(bh / H) * sb + (size_t)(bh % H) * sh; }
};


__device__ __forceinline__ void ld8(const float *x, size_t e, float v[8])
{
    const float4 a = *(const float4 *)(x + e), b = *(const float4 *)(x + e + 4);
    v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w; v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
}
__device__ __forceinline__ void ld8(const uint16_t *x, size_t e, float v[8])
{
    const uint4 a = *(const uint4 *)(x + e);
    v[0] = __uint_as_float(a.x << 16); v[1] = __uint_as_float(a.x & 0xffff0000u);
    v[2] = __uint_as_float(a.y << 16); v[3] = __uint_as_float(a.y & 0xffff0000u);
    v[4] = __uint_as_float(a.z << 16); v[5] = __uint_as_float(a.z & 0xffff0000u);
    v[6] = __uint_as_float(a.w << 16); v[7] = __uint_as_float(a.w & 0xffff0000u);
}

// part[bh][c][d] = k[64c][d] + k[64c+1][d] + ... in token order.
// One thread owns 8 adjacent channels of one 64-token chunk: D/8 threads read a whole row
// (coalesced), 256/(D/8) chunks per workgroup.
template <typename T>
__device__ __forceinline__ void k_mean_partial_body(const T *x, float *part, int N, int D, int nchunk, const XLayout lay, const dim3 bid)
{
    const int gpr = D / 8;                       // 8-channel groups per row
    const int cpb = 256 / gpr;                   // chunks per workgroup
    const int c = bid.x * cpb + threadIdx.x / gpr;
    const int g = threadIdx.x % gpr, bh = bid.y;
    if (c >= nchunk) return;
    const int j0 = c * MEAN_CHUNK;
    const int j1 = min(N, j0 + MEAN_CHUNK);
    const size_t base = lay.head(bh) + g * 8;
    float s[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    // eight rows in flight per thread (the loads of a group are issued together), added in token order
    int j = j0;
    for (; j + 8 <= j1; j += 8) {
        float v[8][8];
#pragma unroll
        for (int u = 0; u < 8; ++u) ld8(x, base + (size_t)(j + u) * lay.st, v[u]);
#pragma unroll
        for (int u = 0; u < 8; ++u)
#pragma unroll
            for (int i = 0; i < 8; ++i) s[i] += v[u][i];
    }
    for (; j < j1; ++j) {
        float v[8];
        ld8(x, base + (size_t)j * lay.st, v);
#pragma unroll
        for (int i = 0; i < 8; ++i) s[i] += v[i];
    }
    float *o = part + ((size_t)bh * nchunk + c) * D + g * 8;
    *(float4 *)o = make_float4(s[0], s[1], s[2], s[3]);
    *(float4 *)(o + 4) = make_float4(s[4], s[5], s[6], s[7]);
}

template <typename T>
__global__ void __launch_bounds__(256) k_mean_partial_kernel(const T *x, float *part, int N, int D, int nchunk, const XLayout lay)
{
    k_mean_partial_body<T>(x, part, N, D, nchunk, lay, blockIdx);
}

// mean[bh][d] = (part[0] + part[1] + ...) / N in chunk order (loads batched, adds in order)
__device__ __forceinline__ void k_mean_final_body(const float *part, float *mean, int N, int D, int nchunk, const dim3 bid)
{
    const int bh = bid.x, d = threadIdx.x;
    const float *p = part + (size_t)bh * nchunk * D + d;
    float tot = 0.f;
    int c = 0;
    // few waves run this kernel (one per 64 channels of a head), so its time is the number of load round trips
    for (; c + 32 <= nchunk; c += 32) {
        float v[32];
#pragma unroll
        for (int i = 0; i < 32; ++i) v[i] = p[(size_t)(c + i) * D];
#pragma unroll
        for (int i = 0; i < 32; ++i) tot += v[i];
    }
    for (; c + 8 <= nchunk; c += 8) {
        float v[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) v[i] = p[(size_t)(c + i) * D];
#pragma unroll
        for (int i = 0; i < 8; ++i) tot += v[i];
    }
    for (; c < nchunk; ++c) tot += p[(size_t)c * D];
    mean[(size_t)bh * D + d] = tot / (float)N;
}

__global__ void k_mean_final_kernel(const float *part, float *mean, int N, int D, int nchunk)
{
    k_mean_final_body(part, mean, N, D, nchunk, blockIdx);
}

// FP8 E4M3 (OCP "FN" flavour: bias 7, no infinities, largest finite 448) of the reference's AR_FP8
// branch: `__nv_cvt_float2_to_fp8x2(..., __NV_SATFINITE, __NV_E4M3)`, src/runtime/cuda_flash_sage.rs:125-128,
// with scale = absmax / 448 (:9).  The hardware conversion rounds to nearest even; the operands
// are clamped to +-448 first, which is what SATFINITE does to anything larger (values in
// (448, 464) round down to 448 either way).
template <bool FP8>
struct QFormat {
    static constexpr float QMAX = FP8 ? 448.0f : 127.0f;
};
template <bool FP8>
__device__ __forceinline__ uint2 quantise8(const float (&v)[8], float inv)
{
    uint32_t w[2] = {0u, 0u};
    if constexpr (FP8) {
        float c[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) c[i] = fminf(fmaxf(v[i] * inv, -448.0f), 448.0f);
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            int r = 0;
            r = __builtin_amdgcn_cvt_pk_fp8_f32(c[4 * j + 0], c[4 * j + 1], r, false);
            r = __builtin_amdgcn_cvt_pk_fp8_f32(c[4 * j + 2], c[4 * j + 3], r, true);
            w[j] = (uint32_t)r;
        }
    } else {
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            int iv = (int)rintf(v[i] * inv);
            iv = iv < -127 ? -127 : (iv > 127 ? 127 : iv);
            w[i >> 2] |= ((uint32_t)iv & 0xffu) << ((i & 3) * 8);
        }
    }
    return make_uint2(w[0], w[1]);
}

// One workgroup per (block of `blk` tokens, head).  Blocks of up to 256*64 elements are kept
// in registers between the absmax pass and the quantising pass (one trip to memory); larger
// ones are read twice.
template <typename T, bool SMOOTH, bool FP8 = false>
__device__ __forceinline__ void quant_blocks_body(const T *x, int8_t *x8, float *scales, const float *mean,
                                                  int N, int D, int blk, int nblk, const XLayout lay, const dim3 bid)
{
    constexpr int KEEP = 8;  // 8-element groups a thread can hold
    __shared__ float red[4];  // one instance per kernel that inlines this body
    const int bi = bid.x, bh = bid.y, tid = threadIdx.x;
    const int r0 = bi * blk;
    const int r1 = min(N, r0 + blk);
    const size_t base = ((size_t)bh * N + r0) * D;  // of the dense output
    const size_t xbase = lay.head(bh) + (size_t)r0 * lay.st;
    // element e of the block (row e / D, channel e % D) in the input
    auto xin = [&](int e) __attribute__((always_inline)) { return xbase + (size_t)(e / D) * lay.st + (e % D); };
    const int nelem = (r1 - r0) * D;  // multiple of 8
    const float *mu = SMOOTH ? mean + (size_t)bh * D : nullptr;
    const bool keep = nelem <= 256 * 8 * KEEP;

    float held[KEEP][8];
    float mx = 0.f;
    if (keep) {
#pragma unroll
        for (int it = 0; it < KEEP; ++it) {
            const int e = (it * 256 + tid) * 8;
            if (e < nelem) {
                ld8(x, xin(e), held[it]);
                const int d = e % D;
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    if (SMOOTH) held[it][i] = held[it][i] - mu[d + i];
                    mx = fmaxf(mx, fabsf(held[it][i]));
                }
            }
        }
    } else {
        for (int e = tid * 8; e < nelem; e += 256 * 8) {
            float v[8];
            ld8(x, xin(e), v);
            const int d = e % D;
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                float xv = v[i];
                if (SMOOTH) xv = xv - mu[d + i];
                mx = fmaxf(mx, fabsf(xv));
            }
        }
    }
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) mx = fmaxf(mx, __shfl_xor(mx, off));
    if ((tid & 63) == 0) red[tid >> 6] = mx;
    __syncthreads();
    mx = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));

    const float scale = (mx > 0.f) ? mx / QFormat<FP8>::QMAX : 1.f;
    const float inv = 1.f / scale;
    if (tid == 0) scales[(size_t)bh * nblk + bi] = scale;

    auto quant8 = [&](const float (&v)[8]) { return quantise8<FP8>(v, inv); };
    if (keep) {
#pragma unroll
        for (int it = 0; it < KEEP; ++it) {
            const int e = (it * 256 + tid) * 8;
            if (e < nelem) *(uint2 *)(x8 + base + e) = quant8(held[it]);
        }
    } else {
        for (int e = tid * 8; e < nelem; e += 256 * 8) {
            float v[8];
            ld8(x, xin(e), v);
            const int d = e % D;
            if (SMOOTH) {
#pragma unroll
                for (int i = 0; i < 8; ++i) v[i] = v[i] - mu[d + i];
            }
            *(uint2 *)(x8 + base + e) = quant8(v);
        }
    }
}

template <typename T, bool SMOOTH, bool FP8 = false>
__global__ void __launch_bounds__(256) quant_blocks_kernel(const T *x, int8_t *x8, float *scales, const float *mean,
                                                           int N, int D, int blk, int nblk, const XLayout lay)
{
    quant_blocks_body<T, SMOOTH, FP8>(x, x8, scales, mean, N, D, blk, nblk, lay, blockIdx);
}

// The reference's own granularity, one scale per token row (block == 1): D/8 lanes share a row,
// so a workgroup of 256 threads quantises 256/(D/8) rows and the absmax is a shuffle reduction
// inside the lane group.  Same arithmetic, same order of operations per element.
template <typename T, bool SMOOTH, bool FP8 = false>
__device__ __forceinline__ void quant_rows_body(const T *x, int8_t *x8, float *scales, const float *mean,
                                                int N, int D, long rows_total, const XLayout lay, const dim3 bid)
{
    const int gpr = D / 8;                                   // lanes per row (8 or 16)
    const long row = (long)bid.x * (256 / gpr) + threadIdx.x / gpr;   // global row over [B*H*N]
    const int g = threadIdx.x % gpr;
    const bool live = row < rows_total;
    float v[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    if (live) {
        ld8(x, lay.head((int)(row / N)) + (size_t)(row % N) * lay.st + g * 8, v);
        if (SMOOTH) {
            const float *mu = mean + (size_t)(row / N) * D + g * 8;
#pragma unroll
            for (int i = 0; i < 8; ++i) v[i] = v[i] - mu[i];
        }
    }
    float mx = 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i) mx = fmaxf(mx, fabsf(v[i]));
    for (int off = gpr >> 1; off >= 1; off >>= 1) mx = fmaxf(mx, __shfl_xor(mx, off));
    const float scale = (mx > 0.f) ? mx / QFormat<FP8>::QMAX : 1.f;
    const float inv = 1.f / scale;
    if (live) {
        if (g == 0) scales[row] = scale;
        *(uint2 *)(x8 + (size_t)row * D + g * 8) = quantise8<FP8>(v, inv);
    }
}

template <typename T, bool SMOOTH, bool FP8 = false>
__global__ void __launch_bounds__(256) quant_rows_kernel(const T *x, int8_t *x8, float *scales, const float *mean,
                                                         int N, int D, long rows_total, const XLayout lay)
{
    quant_rows_body<T, SMOOTH, FP8>(x, x8, scales, mean, N, D, rows_total, lay, blockIdx);
}

__device__ __forceinline__ void cast_bf16_body(const float *x, uint16_t *y, size_t n, const dim3 bid)
{
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (size_t i = (size_t)bid.x * blockDim.x + threadIdx.x; i < n; i += stride) {
        const __bf16 b = (__bf16)x[i];  // round-to-nearest-even
        y[i] = __builtin_bit_cast(uint16_t, b);
    }
}

__global__ void __launch_bounds__(256) cast_bf16_kernel(const float *x, uint16_t *y, size_t n)
{
    cast_bf16_body(x, y, n, blockIdx);
}

// The reference's pre-pass for K and V in one launch (f32 tensors, a scale per key, no smoothing): workgroups
// [0, row_blocks) quantise rows of K as quant_rows does, the rest cast V to bf16 as cast_bf16 does.  Two launches of a
// few microseconds each become one; results are those of the two kernels bit for bit.
__device__ __forceinline__ void quant_rows_cast_body(const float *k, int8_t *k8, float *scales, const float *v, uint16_t *vb,
                                                     int N, int D, long rows_total, long nv, int row_blocks, const dim3 bid)
{
    if ((int)bid.x < row_blocks) {
        quant_rows_body<float, false>(k, k8, scales, nullptr, N, D, rows_total, XLayout::dense(1, N, D), bid);
    } else {
        const size_t stride = (size_t)(gridDim.x - row_blocks) * blockDim.x;
        for (size_t i = (size_t)(bid.x - row_blocks) * blockDim.x + threadIdx.x; i < (size_t)nv; i += stride) {
            const __bf16 b = (__bf16)v[i];  // round-to-nearest-even
            vb[i] = __builtin_bit_cast(uint16_t, b);
        }
    }
}

__global__ void __launch_bounds__(256) quant_rows_cast_kernel(const float *k, int8_t *k8, float *scales, const float *v,
                                                              uint16_t *vb, int N, int D, long rows_total, long nv, int row_blocks)
{
    quant_rows_cast_body(k, k8, scales, v, vb, N, D, rows_total, nv, row_blocks, blockIdx);
}


}  // namespace arhip
