// fp32 FlashAttention backward: the softmax-backward row scalar, dQ, and dK/dV.
//
// Semantics of the reference's training kernels (src/runtime/cuda_flash_train.rs:145-309):
//   prep   D[bh, i]  = sum_d O[i, d] dO[i, d]
//   dQ     s = (q_i . k_j) scale (+ mask[i, j]);  p = lse_i > -5e29 ? exp(s - lse_i) : 0;
//          dp = dO_i . v_j;  ds = p (dp - D_i) scale;  dQ_i = sum_j ds k_j
//   dK/dV  dK_j = sum_{g, i} ds q_i;  dV_j = sum_{g, i} p dO_i   (g over the GQA group of the K/V head,
//          in a fixed order: no atomics, bit-reproducible)
// Keys past the diagonal (causal) or past kv_len contribute p = 0.  head_dim and scale are parameters
// here (the reference hard-codes 64 and 0.125).
//
// All contractions run on v_mfma_f32_32x32x2_f32 (fp32 in, fp32 accumulate) with the decomposition of
// the forward kernel (flash_f32.h): one row of the "resident" operand per lane.
//   dQ kernel   a wave owns 32 queries (lane = query): S^T = K Q^T and dP^T = V dO^T leave, per lane,
//               16 keys of one query, so lse_i and D_i are per-lane scalars and dS^T is already the B
//               operand of dQ^T += K^T dS^T.  K and V tiles of 32 keys are staged in LDS.
//   dK/dV kernel  a wave owns 32 keys (lane = key): S = Q K^T and dP = dO V^T leave, per lane, 16
//               queries of one key; P and dS are the B operands of dV^T += dO^T P and dK^T += Q^T dS.
//               Q and dO tiles of 32 queries (with their lse and D) are staged in LDS.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "flash_f32.h"

namespace arhip {

struct FlashBwdParams {
    const float *q, *k, *v, *dout, *lse, *delta, *mask;
    const int32_t *kv_len;  // [B] or null
    float *dq, *dk, *dv;
    int Hq, Hkv, N;
    int nt;  // tiles per head: query tiles (dQ kernel) or key tiles (dK/dV kernel)
    int total_q, total_kv;  // workgroups in the dQ grid (nt * B * Hq) and in the dK/dV grid (nt * B * Hkv)
    int lpt_q, lpt_kv;  // causal: B * Hq / B * Hkv, and the grids run longest tile first over all heads; else 0
    float scale;
};

typedef float f32x4_t __attribute__((ext_vector_type(4)));

constexpr float BWD_LSE_FLOOR = -5e29f;  // lse at or below: the row saw no key (cuda_flash_train.rs:206)
constexpr float BWD_LOG2E = 1.44269504088896340736f;

// D[bh, i] = O[i] . dO[i]; one wave per row group: lane l of a wave sums channels l, l + 64, ...
// in increasing order, then the 64 partial sums are added by a fixed butterfly.
template <int D>
__device__ __forceinline__ void bwd_prep_body(const float *o, const float *dout, float *delta, long rows, long row0)
{
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const long row = row0 + wave;
    if (row >= rows) return;
    float s = 0.f;
#pragma unroll
    for (int c = lane; c < D; c += 64) s += o[row * D + c] * dout[row * D + c];
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) s += __shfl_xor(s, off);
    if (lane == 0) delta[row] = s;
}

// LDS floats of the dQ and dK/dV bodies: two padded 32-row tiles and 64 row statistics (one such slab
// per wave with SPLIT)
template <int D, int NW = 1, bool SPLIT = false>
constexpr int bwd_lds_floats()
{
    return (SPLIT ? NW : 1) * (2 * F32_BK * (D + 4) + 64);
}

// dQ.  lds: bwd_lds_floats<D, NW, SPLIT>() floats.  Workgroup wg_linear in [0, nt * B * Hq): 32 NW queries
// of one head.  SPLIT (few, short heads: one wave per workgroup would leave each SIMD a long chain of
// matrix instructions and most of the chip idle): the NW waves share the same 32 queries and deal the
// key tiles out between them (wave w takes tiles w, w + NW, ...), each staging its tiles in its own
// LDS slab with no workgroup barrier; the partial dQ of the waves are added through LDS in wave order.
template <int D, int NW, bool CAUSAL, bool SPLIT = false>
__device__ __forceinline__ void bwd_dq_body(const FlashBwdParams &p, float *lds, int wg_linear)
{
    constexpr int T = SPLIT ? 64 : NW * 64;   // threads staging one tile
    constexpr int BQ = SPLIT ? 32 : NW * 32;
    constexpr int HALF = D / 2;
    constexpr int ROW = D + 4;  // padded row: conflict-free 128-bit row reads
    constexpr int DB = D / 32;
    constexpr int CHUNKS = F32_BK * D / 4;
    constexpr int PER_THREAD = CHUNKS / T;
    static_assert(CHUNKS % T == 0, "tile staging must divide evenly");

    constexpr int SLAB = 2 * F32_BK * ROW + 64;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    float *ks = lds + (SPLIT ? wave * SLAB : 0);
    float *vs = ks + F32_BK * ROW;
    const int stid = SPLIT ? lane : tid;      // index among the threads staging a tile
    const int i32 = lane & 31, h = lane >> 5;
    // every XCD (consecutive workgroups go to different ones) gets a contiguous range of heads
    const int wg_x = (p.total_q > 0 && (p.total_q & 7) == 0) ? (wg_linear & 7) * (p.total_q >> 3) + (wg_linear >> 3) : wg_linear;
    int bh = wg_x / p.nt;
    int qt = wg_x - bh * p.nt;
    if (CAUSAL) qt = p.nt - 1 - qt;  // the longest query tiles first, within a head ...
    if (CAUSAL && p.lpt_q > 0) {     // ... or over the whole grid
        qt = p.nt - 1 - wg_linear / p.lpt_q;
        bh = wg_linear % p.lpt_q;
    }
    const int b = bh / p.Hq, head = bh - b * p.Hq;
    const int N = p.N;
    const int qblk = qt * BQ;
    const int wq0 = qblk + (SPLIT ? 0 : wave * 32);
    const int q_row = wq0 + i32;
    const int rr = min(q_row, N - 1);
    int kvl = N;
    if (p.kv_len) {
        kvl = p.kv_len[b];
        kvl = kvl < 0 ? 0 : (kvl > N ? N : kvl);
    }
    int kend = kvl;
    if (CAUSAL) kend = min(kend, min(N, qblk + BQ));
    const int ntiles = (kend + F32_BK - 1) / F32_BK;
    const int my_tiles = CAUSAL ? min(ntiles, (wq0 + 31) / F32_BK + 1) : ntiles;
    const int kvh = head / (p.Hq / p.Hkv);
    const float *kp = p.k + ((size_t)b * p.Hkv + kvh) * (size_t)N * D;
    const float *vp = p.v + ((size_t)b * p.Hkv + kvh) * (size_t)N * D;
    const size_t qoff = ((size_t)bh * N + rr) * D + h * HALF;

    float qr[HALF], dor[HALF];
#pragma unroll
    for (int s = 0; s < HALF; s += 4) {
        const float4 x = *(const float4 *)(p.q + qoff + s);
        const float4 y = *(const float4 *)(p.dout + qoff + s);
        qr[s] = x.x; qr[s + 1] = x.y; qr[s + 2] = x.z; qr[s + 3] = x.w;
        dor[s] = y.x; dor[s + 1] = y.y; dor[s + 2] = y.z; dor[s + 3] = y.w;
    }
    const float lse = p.lse[(size_t)bh * N + rr];
    const float di = p.delta[(size_t)bh * N + rr];
    const bool row_live = lse > BWD_LSE_FLOOR;
    // P = exp(x - lse) as v_exp_f32 (base 2) of x * log2(e) - lse * log2(e)
    const float c2 = p.scale * BWD_LOG2E, lse2 = lse * BWD_LOG2E;

    f32x16_t acc[DB];
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[db][r] = 0.f;

    float4 kx[PER_THREAD], vx[PER_THREAD];
    auto fetch = [&](int tile) __attribute__((always_inline)) {
        if (tile * F32_BK + F32_BK <= kend) {  // a full tile: no row tests, no zero fill
#pragma unroll
            for (int j = 0; j < PER_THREAD; ++j) {
                const int c = stid + j * T;
                const int row = c / (D / 4), col = (c % (D / 4)) * 4;
                const size_t off = (size_t)(tile * F32_BK + row) * D + col;
                kx[j] = *(const float4 *)(kp + off);
                vx[j] = *(const float4 *)(vp + off);
            }
            return;
        }
#pragma unroll
        for (int j = 0; j < PER_THREAD; ++j) {
            const int c = stid + j * T;
            const int row = c / (D / 4), col = (c % (D / 4)) * 4;
            const int gr = tile * F32_BK + row;
            kx[j] = vx[j] = make_float4(0.f, 0.f, 0.f, 0.f);
            if (gr < kend) {
                kx[j] = *(const float4 *)(kp + (size_t)gr * D + col);
                vx[j] = *(const float4 *)(vp + (size_t)gr * D + col);
            }
        }
    };
    constexpr int STEP = SPLIT ? NW : 1;
    const int first = SPLIT ? wave : 0;
    if (first < ntiles) fetch(first);
    for (int it = first; it < ntiles; it += STEP) {
        const int k0 = it * F32_BK;
        if (!SPLIT) __syncthreads();
#pragma unroll
        for (int j = 0; j < PER_THREAD; ++j) {
            const int c = stid + j * T;
            const int row = c / (D / 4), col = (c % (D / 4)) * 4;
            *(float4 *)&ks[row * ROW + col] = kx[j];
            *(float4 *)&vs[row * ROW + col] = vx[j];
        }
        if (it + STEP < ntiles) fetch(it + STEP);
        if (!SPLIT) __syncthreads();
        if (it >= my_tiles) continue;

        // S^T = K Q^T and dP^T = V dO^T: lane = query, register r = key 8 (r / 4) + 4 h + r % 4
        f32x16_t s, dp;
#pragma unroll
        for (int r = 0; r < 16; ++r) s[r] = dp[r] = 0.f;
        const float *krow = &ks[i32 * ROW + h * HALF];
        const float *vrow = &vs[i32 * ROW + h * HALF];
#pragma unroll
        for (int st = 0; st < HALF; st += 4) {
            const float4 a = *(const float4 *)(krow + st);
            const float4 c = *(const float4 *)(vrow + st);
            s = __builtin_amdgcn_mfma_f32_32x32x2f32(a.x, qr[st + 0], s, 0, 0, 0);
            dp = __builtin_amdgcn_mfma_f32_32x32x2f32(c.x, dor[st + 0], dp, 0, 0, 0);
            s = __builtin_amdgcn_mfma_f32_32x32x2f32(a.y, qr[st + 1], s, 0, 0, 0);
            dp = __builtin_amdgcn_mfma_f32_32x32x2f32(c.y, dor[st + 1], dp, 0, 0, 0);
            s = __builtin_amdgcn_mfma_f32_32x32x2f32(a.z, qr[st + 2], s, 0, 0, 0);
            dp = __builtin_amdgcn_mfma_f32_32x32x2f32(c.z, dor[st + 2], dp, 0, 0, 0);
            s = __builtin_amdgcn_mfma_f32_32x32x2f32(a.w, qr[st + 3], s, 0, 0, 0);
            dp = __builtin_amdgcn_mfma_f32_32x32x2f32(c.w, dor[st + 3], dp, 0, 0, 0);
        }
        float ds[16];
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int key = k0 + 8 * (r >> 2) + 4 * h + (r & 3);
            float xv = fmaf(s[r], c2, -lse2);
            if (p.mask != nullptr && key < N) xv = fmaf(p.mask[(size_t)rr * N + key], BWD_LOG2E, xv);
            const bool dead = key >= kend || (CAUSAL && key > q_row) || !row_live;
            const float pr = dead ? 0.f : __builtin_amdgcn_exp2f(xv);
            ds[r] = pr * (dp[r] - di) * p.scale;
        }
        // dQ^T += K^T dS^T: step (g, t) multiplies key 8 g + 4 h + t
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const float *kcol = &ks[(8 * (r >> 2) + 4 * h + (r & 3)) * ROW + i32];
#pragma unroll
            for (int db = 0; db < DB; ++db)
                acc[db] = __builtin_amdgcn_mfma_f32_32x32x2f32(kcol[db * 32], ds[r], acc[db], 0, 0, 0);
        }
    }
    if constexpr (SPLIT) {
        // the waves' partial sums, each as [32 queries][ROW] in its own slab (its tiles are consumed)
        float *ow = lds + wave * SLAB;
#pragma unroll
        for (int db = 0; db < DB; ++db)
#pragma unroll
            for (int g = 0; g < 4; ++g)
                *(float4 *)&ow[i32 * ROW + db * 32 + 8 * g + 4 * h] =
                    make_float4(acc[db][4 * g], acc[db][4 * g + 1], acc[db][4 * g + 2], acc[db][4 * g + 3]);
        __syncthreads();
        // thread t: query t % 32, channels [cg * CPT, cg * CPT + CPT)
        constexpr int CPT = D / (NW * 2);
        static_assert(CPT % 4 == 0, "whole float4s per thread");
        const int q = tid & 31, cg = tid >> 5;
        if (qblk + q < N) {
            float *op = p.dq + ((size_t)bh * N + qblk + q) * D + cg * CPT;
#pragma unroll
            for (int c = 0; c < CPT; c += 4) {
                float4 sum = *(const float4 *)&lds[q * ROW + cg * CPT + c];
#pragma unroll
                for (int w = 1; w < NW; ++w) {
                    const float4 x = *(const float4 *)&lds[w * SLAB + q * ROW + cg * CPT + c];
                    sum.x += x.x; sum.y += x.y; sum.z += x.z; sum.w += x.w;
                }
                *(float4 *)(op + c) = sum;
            }
        }
        return;
    }
    if (q_row < N) {
        float *op = p.dq + ((size_t)bh * N + q_row) * D;
#pragma unroll
        for (int db = 0; db < DB; ++db)
#pragma unroll
            for (int g = 0; g < 4; ++g)
                *(float4 *)(op + db * 32 + 8 * g + 4 * h) =
                    make_float4(acc[db][4 * g], acc[db][4 * g + 1], acc[db][4 * g + 2], acc[db][4 * g + 3]);
    }
}

// dK and dV.  Workgroup wg_linear in [0, nt * B * Hkv): 32 NW keys of one K/V head.  SPLIT: the NW waves
// share the same 32 keys and deal the (head of the group, query tile) steps out between them, each in
// its own LDS slab; the partial dK and dV of the waves are added through LDS in wave order.
template <int D, int NW, bool CAUSAL, bool SPLIT = false>
__device__ __forceinline__ void bwd_dkv_body(const FlashBwdParams &p, float *lds, int wg_linear)
{
    constexpr int T = SPLIT ? 64 : NW * 64;   // threads staging one tile
    constexpr int BKW = SPLIT ? 32 : NW * 32;  // keys per workgroup
    constexpr int HALF = D / 2;
    constexpr int ROW = D + 4;
    constexpr int DB = D / 32;
    constexpr int CHUNKS = F32_BK * D / 4;
    constexpr int PER_THREAD = CHUNKS / T;
    static_assert(CHUNKS % T == 0, "tile staging must divide evenly");

    constexpr int SLAB = 2 * F32_BK * ROW + 64;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    float *qs = lds + (SPLIT ? wave * SLAB : 0);
    float *dos = qs + F32_BK * ROW;
    float *stat = qs + 2 * F32_BK * ROW;  // lse[32], D[32] of the staged queries
    const int stid = SPLIT ? lane : tid;      // index among the threads staging a tile
    const int i32 = lane & 31, h = lane >> 5;
    const int wg_x = (p.total_kv > 0 && (p.total_kv & 7) == 0) ? (wg_linear & 7) * (p.total_kv >> 3) + (wg_linear >> 3) : wg_linear;
    int kv_bh = wg_x / p.nt;
    int kt = wg_x - kv_bh * p.nt;  // causal: the first key tiles see the most queries
    if (CAUSAL && p.lpt_kv > 0) {       // the longest over the whole grid first
        kt = wg_linear / p.lpt_kv;
        kv_bh = wg_linear % p.lpt_kv;
    }
    const int b = kv_bh / p.Hkv, kvh = kv_bh - b * p.Hkv;
    const int group = p.Hq / p.Hkv;
    const int N = p.N;
    const int kblk = kt * BKW;
    const int wk0 = kblk + (SPLIT ? 0 : wave * 32);
    const int key = wk0 + i32;
    const int jj = min(key, N - 1);
    int kvl = N;
    if (p.kv_len) {
        kvl = p.kv_len[b];
        kvl = kvl < 0 ? 0 : (kvl > N ? N : kvl);
    }
    const bool key_live = key < kvl;
    const float c2 = p.scale * BWD_LOG2E;

    float kr[HALF], vr[HALF];
    {
        const size_t off = ((size_t)kv_bh * N + jj) * D + h * HALF;
#pragma unroll
        for (int s = 0; s < HALF; s += 4) {
            const float4 x = *(const float4 *)(p.k + off + s);
            const float4 y = *(const float4 *)(p.v + off + s);
            kr[s] = x.x; kr[s + 1] = x.y; kr[s + 2] = x.z; kr[s + 3] = x.w;
            vr[s] = y.x; vr[s + 1] = y.y; vr[s + 2] = y.z; vr[s + 3] = y.w;
        }
    }
    f32x16_t dk[DB], dv[DB];
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int r = 0; r < 16; ++r) dk[db][r] = dv[db][r] = 0.f;

    // queries before the workgroup's first key see none of its keys under the causal mask
    const int qt0 = CAUSAL ? kblk / F32_BK : 0;
    const int qtiles = (N + F32_BK - 1) / F32_BK;
    const int steps = group * (qtiles - qt0);  // (head of the group, query tile) pairs, head-major

    f32x4_t qx[PER_THREAD], dx[PER_THREAD];
    float st_l = 0.f, st_d = 0.f;
    auto fetch = [&](int step) __attribute__((always_inline)) {
        const int g = step / (qtiles - qt0);
        const int q0 = (qt0 + step - g * (qtiles - qt0)) * F32_BK;
        const size_t bh = (size_t)b * p.Hq + (size_t)kvh * group + g;
        // Rows past the last query repeat it: whatever they hold is multiplied by P = dS = 0 (finite values, not
        // zeros, are all that takes).  One path without a branch, and native vectors (typed loads and stores): both
        // keep the staged tile in registers at D = 128.
#pragma unroll
        for (int j = 0; j < PER_THREAD; ++j) {
            const int c = stid + j * T;
            const int row = c / (D / 4), col = (c % (D / 4)) * 4;
            const size_t off = (bh * N + min(q0 + row, N - 1)) * D + col;
            qx[j] = *(const f32x4_t *)(p.q + off);
            dx[j] = *(const f32x4_t *)(p.dout + off);
        }
        if (stid < F32_BK) {
            const int gr = q0 + stid;
            st_l = gr < N ? p.lse[bh * N + gr] : -1e30f;
            st_d = gr < N ? p.delta[bh * N + gr] : 0.f;
        }
    };
    constexpr int STEP = SPLIT ? NW : 1;
    const int first = SPLIT ? wave : 0;
    if (first < steps) fetch(first);
    // the staged tile of the previous step goes to LDS, the next one is requested
    auto stage = [&](int step) __attribute__((always_inline)) {
        if (!SPLIT) __syncthreads();
#pragma unroll
        for (int j = 0; j < PER_THREAD; ++j) {
            const int c = stid + j * T;
            const int row = c / (D / 4), col = (c % (D / 4)) * 4;
            *(f32x4_t *)&qs[row * ROW + col] = qx[j];
            *(f32x4_t *)&dos[row * ROW + col] = dx[j];
        }
        if (stid < F32_BK) {
            stat[stid] = st_l * BWD_LOG2E;   // base-2 units: P = 2^(x log2(e) - lse log2(e))
            stat[32 + stid] = st_d;
        }
        if (step + STEP < steps) fetch(step + STEP);
        if (!SPLIT) __syncthreads();
    };
    auto compute = [&](int step) __attribute__((always_inline)) {
        const int g = step / (qtiles - qt0);
        const int q0 = (qt0 + step - g * (qtiles - qt0)) * F32_BK;

        // S = Q K^T and dP = dO V^T: lane = key, register r = query 8 (r / 4) + 4 h + r % 4 of the tile
        f32x16_t s, dp;
#pragma unroll
        for (int r = 0; r < 16; ++r) s[r] = dp[r] = 0.f;
        const float *qrow = &qs[i32 * ROW + h * HALF];
        const float *drow = &dos[i32 * ROW + h * HALF];
#pragma unroll
        for (int st = 0; st < HALF; st += 4) {
            const float4 a = *(const float4 *)(qrow + st);
            const float4 c = *(const float4 *)(drow + st);
            s = __builtin_amdgcn_mfma_f32_32x32x2f32(a.x, kr[st + 0], s, 0, 0, 0);
            dp = __builtin_amdgcn_mfma_f32_32x32x2f32(c.x, vr[st + 0], dp, 0, 0, 0);
            s = __builtin_amdgcn_mfma_f32_32x32x2f32(a.y, kr[st + 1], s, 0, 0, 0);
            dp = __builtin_amdgcn_mfma_f32_32x32x2f32(c.y, vr[st + 1], dp, 0, 0, 0);
            s = __builtin_amdgcn_mfma_f32_32x32x2f32(a.z, kr[st + 2], s, 0, 0, 0);
            dp = __builtin_amdgcn_mfma_f32_32x32x2f32(c.z, vr[st + 2], dp, 0, 0, 0);
            s = __builtin_amdgcn_mfma_f32_32x32x2f32(a.w, kr[st + 3], s, 0, 0, 0);
            dp = __builtin_amdgcn_mfma_f32_32x32x2f32(c.w, vr[st + 3], dp, 0, 0, 0);
        }
        float pr[16], ds[16];
        const int kq = key - q0 - 4 * h;  // causal: query 8 gq + 4 h + t of the tile sees this lane's key iff kq <= 8 gq + t
#pragma unroll
        for (int gq = 0; gq < 4; ++gq) {
            const float4 l4 = *(const float4 *)&stat[8 * gq + 4 * h];
            const float4 d4 = *(const float4 *)&stat[32 + 8 * gq + 4 * h];
            const float lv[4] = {l4.x, l4.y, l4.z, l4.w}, dvv[4] = {d4.x, d4.y, d4.z, d4.w};
#pragma unroll
            for (int t = 0; t < 4; ++t) {
                const int r = 4 * gq + t;
                const int qi = q0 + 8 * gq + 4 * h + t;
                float xv = fmaf(s[r], c2, -lv[t]);
                if (p.mask != nullptr && qi < N) xv = fmaf(p.mask[(size_t)qi * N + jj], BWD_LOG2E, xv);
                const bool dead = qi >= N || !key_live || (CAUSAL && kq > 8 * gq + t) || !(lv[t] > BWD_LSE_FLOOR);
                pr[r] = dead ? 0.f : __builtin_amdgcn_exp2f(xv);
                ds[r] = pr[r] * (dp[r] - dvv[t]) * p.scale;
            }
        }
        // dV^T += dO^T P and dK^T += Q^T dS: step (g, t) multiplies query 8 g + 4 h + t of the tile
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int qi = 8 * (r >> 2) + 4 * h + (r & 3);
            const float *dcol = &dos[qi * ROW + i32];
            const float *qcol = &qs[qi * ROW + i32];
#pragma unroll
            for (int db = 0; db < DB; ++db) {
                dv[db] = __builtin_amdgcn_mfma_f32_32x32x2f32(dcol[db * 32], pr[r], dv[db], 0, 0, 0);
                dk[db] = __builtin_amdgcn_mfma_f32_32x32x2f32(qcol[db * 32], ds[r], dk[db], 0, 0, 0);
            }
        }
    };
    if constexpr (CAUSAL && !SPLIT) {
        // Every query of the first `wave` tiles of a head precedes this wave's keys: those tiles are staged (all
        // waves pass the same barriers) and not computed.  Two plain loops instead of a branch around the matrix
        // work, which costs the register allocator the accumulators twice.
        const int tiles = qtiles - qt0, nskip = min(wave, tiles);
        for (int g = 0; g < group; ++g) {
            for (int t = 0; t < nskip; ++t) stage(g * tiles + t);
            for (int t = nskip; t < tiles; ++t) {
                stage(g * tiles + t);
                compute(g * tiles + t);
            }
        }
    } else {
        // (SPLIT: the tiles start at the workgroup's first key, so none lies wholly before its keys)
        for (int step = first; step < steps; step += STEP) {
            stage(step);
            compute(step);
        }
    }
    if constexpr (SPLIT) {
        // the waves' partial sums: dK as [32 keys][ROW] in the first tile of the slab, dV in the second
        float *ow = lds + wave * SLAB;
#pragma unroll
        for (int db = 0; db < DB; ++db)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const int d = db * 32 + 8 * g + 4 * h;
                *(float4 *)&ow[i32 * ROW + d] = make_float4(dk[db][4 * g], dk[db][4 * g + 1], dk[db][4 * g + 2], dk[db][4 * g + 3]);
                *(float4 *)&ow[(F32_BK + i32) * ROW + d] = make_float4(dv[db][4 * g], dv[db][4 * g + 1], dv[db][4 * g + 2], dv[db][4 * g + 3]);
            }
        __syncthreads();
        // thread t: key t % 32, channels [cg * CPT, cg * CPT + CPT) of dK and of dV
        constexpr int CPT = D / (NW * 2);
        static_assert(CPT % 4 == 0, "whole float4s per thread");
        const int kq = tid & 31, cg = tid >> 5;
        if (kblk + kq < N) {
            const size_t orow = ((size_t)kv_bh * N + kblk + kq) * D + cg * CPT;
#pragma unroll
            for (int half = 0; half < 2; ++half) {
                float *op = (half ? p.dv : p.dk) + orow;
#pragma unroll
                for (int c = 0; c < CPT; c += 4) {
                    float4 sum = *(const float4 *)&lds[(half * F32_BK + kq) * ROW + cg * CPT + c];
#pragma unroll
                    for (int w = 1; w < NW; ++w) {
                        const float4 x = *(const float4 *)&lds[w * SLAB + (half * F32_BK + kq) * ROW + cg * CPT + c];
                        sum.x += x.x; sum.y += x.y; sum.z += x.z; sum.w += x.w;
                    }
                    *(float4 *)(op + c) = sum;
                }
            }
        }
        return;
    }
    if (key < N) {
        float *okp = p.dk + ((size_t)kv_bh * N + key) * D;
        float *ovp = p.dv + ((size_t)kv_bh * N + key) * D;
#pragma unroll
        for (int db = 0; db < DB; ++db)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const int d = db * 32 + 8 * g + 4 * h;
                *(float4 *)(okp + d) = make_float4(dk[db][4 * g], dk[db][4 * g + 1], dk[db][4 * g + 2], dk[db][4 * g + 3]);
                *(float4 *)(ovp + d) = make_float4(dv[db][4 * g], dv[db][4 * g + 1], dv[db][4 * g + 2], dv[db][4 * g + 3]);
            }
    }
}

template <int D>
__global__ void __launch_bounds__(256) bwd_prep_kernel(const float *o, const float *dout, float *delta, long rows)
{
    bwd_prep_body<D>(o, dout, delta, rows, (long)blockIdx.x * 4);
}

// D = 64: registers held to 256 per lane so that a SIMD holds two waves (the split dK/dV variant would
// spill at that limit and keeps one)
template <int D, int NW, bool CAUSAL, bool SPLIT>
__global__ void __launch_bounds__(NW * 64, (D == 64 ? 2 : 1)) bwd_dq_kernel(const FlashBwdParams p)
{
    __shared__ __attribute__((aligned(16))) float lds[bwd_lds_floats<D, NW, SPLIT>()];
    bwd_dq_body<D, NW, CAUSAL, SPLIT>(p, lds, (int)blockIdx.x);
}

template <int D, int NW, bool CAUSAL, bool SPLIT>
__global__ void __launch_bounds__(NW * 64, (D == 64 && !SPLIT ? 2 : 1)) bwd_dkv_kernel(const FlashBwdParams p)
{
    __shared__ __attribute__((aligned(16))) float lds[bwd_lds_floats<D, NW, SPLIT>()];
    bwd_dkv_body<D, NW, CAUSAL, SPLIT>(p, lds, (int)blockIdx.x);
}

}  // namespace arhip
