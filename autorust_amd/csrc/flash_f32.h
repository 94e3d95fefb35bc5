// fp32 exact-mode FlashAttention forward (no matrix cores, no reduced precision).
//
// Same schedule and arithmetic as the reference's scalar kernel
// (src/runtime/cuda_flash.rs:53-141): one thread per query row, BQ = 64 rows per
// workgroup (one wave64), BK = 32 keys per step broadcast from LDS, fp32 FMA dot
// products in channel order, `expf`, finite sentinel -1e30 for masked keys,
// acc * (l > 0 ? 1/l : 0) at the end.  head_dim and scale are parameters here.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace arhip {

constexpr int FLASH_F32_BQ = 64;
constexpr int FLASH_F32_BK = 32;
constexpr int FLASH_F32_THREADS = 64;

struct FlashF32Params {
    const float *q, *k, *v;
    float *o;
    const float *mask;      // additive [N,N] or null
    const int32_t *kv_len;  // [B] or null
    int Hq, Hkv, N, nq;
    float scale;
};

template <int D, bool CAUSAL>
__global__ void __launch_bounds__(FLASH_F32_THREADS) flash_f32_kernel(const FlashF32Params p)
{
    constexpr int BQ = FLASH_F32_BQ, BKK = FLASH_F32_BK;
    __shared__ __attribute__((aligned(16))) float ks[BKK][D];
    __shared__ __attribute__((aligned(16))) float vs[BKK][D];

    const int t = threadIdx.x;
    const int bh = blockIdx.x / p.nq;
    const int qblk = (blockIdx.x - bh * p.nq) * BQ;
    const int row = qblk + t;
    const int b = bh / p.Hq;
    const int head = bh - b * p.Hq;
    const int kv_bh = b * p.Hkv + head / (p.Hq / p.Hkv);
    const int N = p.N;
    const float *qp = p.q + ((size_t)bh * N + (row < N ? row : 0)) * D;
    const float *kp = p.k + (size_t)kv_bh * N * D;
    const float *vp = p.v + (size_t)kv_bh * N * D;

    int kvl = N;
    if (p.kv_len) {
        kvl = p.kv_len[b];
        kvl = kvl < 0 ? 0 : (kvl > N ? N : kvl);
    }
    int kend = kvl;
    if (CAUSAL) kend = min(kend, min(N, qblk + BQ));

    float qr[D];
#pragma unroll
    for (int d = 0; d < D; d += 4) {
        float4 x = *(const float4 *)(qp + d);
        if (row >= N) x = make_float4(0.f, 0.f, 0.f, 0.f);
        qr[d] = x.x; qr[d + 1] = x.y; qr[d + 2] = x.z; qr[d + 3] = x.w;
    }
    float acc[D];
#pragma unroll
    for (int d = 0; d < D; ++d) acc[d] = 0.f;
    float m = -1e30f, l = 0.f;

    for (int k0 = 0; k0 < kend; k0 += BKK) {
        __syncthreads();
        for (int i = t; i < BKK * D / 4; i += FLASH_F32_THREADS) {
            const int r = i / (D / 4), c = (i % (D / 4)) * 4;
            const int gr = k0 + r;
            float4 kx = make_float4(0.f, 0.f, 0.f, 0.f), vx = kx;
            if (gr < kend) {
                kx = *(const float4 *)(kp + (size_t)gr * D + c);
                vx = *(const float4 *)(vp + (size_t)gr * D + c);
            }
            *(float4 *)&ks[r][c] = kx;
            *(float4 *)&vs[r][c] = vx;
        }
        __syncthreads();

        float s[BKK];
        float mnew = m;
#pragma unroll
        for (int j = 0; j < BKK; ++j) {
            const int gj = k0 + j;
            float dot = 0.f;
#pragma unroll
            for (int d = 0; d < D; ++d) dot = fmaf(qr[d], ks[j][d], dot);
            dot *= p.scale;
            if (p.mask != nullptr && row < N && gj < N) dot += p.mask[(size_t)row * N + gj];
            if (gj >= kend || (CAUSAL && gj > row)) dot = -1e30f;
            s[j] = dot;
            mnew = fmaxf(mnew, dot);
        }
        const float alpha = expf(m - mnew);
        float sum = 0.f;
#pragma unroll
        for (int j = 0; j < BKK; ++j) {
            s[j] = expf(s[j] - mnew);
            sum += s[j];
        }
        l = l * alpha + sum;
#pragma unroll
        for (int d = 0; d < D; ++d) acc[d] *= alpha;
#pragma unroll
        for (int j = 0; j < BKK; ++j)
#pragma unroll
            for (int d = 0; d < D; ++d) acc[d] = fmaf(s[j], vs[j][d], acc[d]);
        m = mnew;
    }

    if (row < N) {
        const float inv = (l > 0.f) ? 1.f / l : 0.f;
        float *op = p.o + ((size_t)bh * N + row) * D;
#pragma unroll
        for (int d = 0; d < D; d += 4)
            *(float4 *)(op + d) = make_float4(acc[d] * inv, acc[d + 1] * inv, acc[d + 2] * inv, acc[d + 3] * inv);
    }
}

}  // namespace arhip
