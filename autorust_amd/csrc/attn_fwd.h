// Fused attention forward for gfx950 (CDNA4): one kernel template for the bf16
// FlashAttention path and the int8 (SageAttention-style) path.
//
// Work decomposition
//   grid  : one workgroup per (batch*head, tile of BQ = 32*NW queries)
//   wave  : 32 queries; the wave computes S^T = K . Q^T, so that in the MFMA
//           result layout every lane owns ONE query (column lane%32) and 16 of
//           the 32 keys of a block.  Row max / row sum are then per-lane
//           reductions plus one exchange with lane^32, and the probabilities
//           are already in the operand layout the second product needs:
//           O^T = V^T . P^T, again with one query per lane.
//   tiles : BK = 64 keys per step, K and V^T staged through LDS by the whole
//           workgroup (128-bit global loads issued one tile ahead into
//           registers, written to the other LDS buffer after the math).
//
// MFMA shapes (wave64):
//   v_mfma_f32_32x32x16_bf16  A[32 x 16] . B[16 x 32]   lane: row/col = lane%32,
//                             k = 8*(lane/32) + 0..7    (8 bf16 = 16 bytes)
//   v_mfma_i32_32x32x32_i8    lane: k = 16*(lane/32) + 0..15 (16 bytes)
//   result C[32 x 32]: lane holds column lane%32 and rows
//                             8*(r/4) + 4*(lane/32) + r%4,  r = 0..15
//
// Key order inside a 16-key step of P.V: the B operand wants, in lane half h,
// keys "8h + t" (t = 0..7) of the step, while the S^T result gives half h the
// keys 8*(t/4) + 4h + t%4.  A sum over keys does not care about their order,
// so V^T is simply stored in LDS with the two middle groups of four keys of
// every 16 swapped, and P is used exactly as the first MFMA produced it.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace arhip {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(4))) int i32x4;
typedef __attribute__((ext_vector_type(16))) int i32x16;

constexpr int MODE_BF16 = 0;  // q, k bf16
constexpr int MODE_I8 = 1;    // q, k int8 with block scales
constexpr int BK = 64;        // keys per tile
constexpr float NEG_SENTINEL = -1e30f;  // src/runtime/cuda_flash_bf16.rs:106 (AR_NEG)
constexpr float LOG2E = 1.4426950408889634f;

struct AttnParams {
    const void *q;
    const void *k;
    const uint16_t *v;  // bf16 bits
    void *o;
    const float *mask;       // additive [N,N] or null
    const int32_t *kv_len;   // [B] or null
    const float *sq;         // MODE_I8: [B,Hq,ceil(N/bq)]
    const float *sk;         // MODE_I8: [B,Hkv,ceil(N/bk)]
    int32_t *dbg;            // MODE_I8 debug: [32][64] raw logits
    int dbg_bh, dbg_qt, dbg_kt;
    int Hq, Hkv, N;
    int bq, bk;
    int nq;     // query tiles per head
    int total;  // workgroups
    float scale;
};

__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi)
{
    typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
    bf16x2 p = {(__bf16)lo, (__bf16)hi};  // round-to-nearest-even
    return __builtin_bit_cast(uint32_t, p);
}

// max over both lane halves (lane and lane^32 hold the same query)
__device__ __forceinline__ float xhalf_max(float x)
{
    return fmaxf(x, __shfl_xor(x, 32));
}
__device__ __forceinline__ float xhalf_sum(float x)
{
    return x + __shfl_xor(x, 32);
}

// byte offset of V^T element (d, pos) in a [D][64] bf16 tile whose 16-byte
// chunks are XOR-swizzled per row so that both the transposing 8-byte writes
// and the 16-byte operand reads spread over the LDS banks.
__device__ __forceinline__ int vt_off(int d, int pos)
{
    const int chunk = pos >> 3;
    const int sw = (d ^ (d >> 3)) & 7;
    return d * 128 + ((chunk ^ sw) << 4) + ((pos & 7) << 1);
}

template <int D, int NW, bool CAUSAL, bool HAS_MASK, int MODE, bool OUT_F32, bool DBG>
__global__ void __launch_bounds__(NW * 64) attn_fwd_kernel(const AttnParams p)
{
    constexpr int T = NW * 64;
    constexpr int BQ = NW * 32;
    constexpr int QK_BYTES = (MODE == MODE_I8) ? 1 : 2;       // bytes per q/k element
    constexpr int KROW = D * QK_BYTES + 16;                    // padded K row in LDS
    constexpr int K_TILE = BK * KROW;
    constexpr int V_TILE = D * 128;
    constexpr int STAGE = K_TILE + V_TILE;
    constexpr int K_CPR = D * QK_BYTES / 16;                   // 16-byte chunks per K row
    constexpr int K_CHUNKS = BK * K_CPR;
    constexpr int K_PER_THREAD = (K_CHUNKS + T - 1) / T;
    constexpr int V_UNITS = (BK / 4) * (D / 8);                // 4 keys x 8 channels each
    constexpr int V_PER_THREAD = (V_UNITS + T - 1) / T;
    constexpr int KSTEPS = (MODE == MODE_I8) ? D / 32 : D / 16;  // MFMA k steps over D
    constexpr int DB = D / 32;                                 // 32-channel output blocks
    static_assert(K_CHUNKS % T == 0 || K_CHUNKS < T, "K staging must divide evenly");
    static_assert(V_UNITS % T == 0 || V_UNITS < T, "V staging must divide evenly");

    __shared__ __attribute__((aligned(16))) unsigned char lds[2 * STAGE];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int i32 = lane & 31;
    const int h = lane >> 5;

    // Workgroup id -> (head, query tile).  Consecutive ids go to different XCDs
    // (8 of them, each with its own L2); give every XCD a contiguous range of
    // heads so that the query tiles sharing one head's K/V hit the same L2.
    int wg = blockIdx.x;
    if ((p.total & 7) == 0) wg = (wg & 7) * (p.total >> 3) + (wg >> 3);
    const int bh = wg / p.nq;
    int qt = wg - bh * p.nq;
    if (CAUSAL) qt = p.nq - 1 - qt;  // longest tiles first
    const int b = bh / p.Hq;
    const int head = bh - b * p.Hq;
    const int kvh = head / (p.Hq / p.Hkv);
    const int kv_bh = b * p.Hkv + kvh;
    const int N = p.N;

    const int qblk = qt * BQ;
    const int wq0 = qblk + wave * 32;  // first query of this wave
    const int q_row = wq0 + i32;

    int kvl = N;
    if (p.kv_len) {
        kvl = p.kv_len[b];
        kvl = kvl < 0 ? 0 : (kvl > N ? N : kvl);
    }
    int kend = kvl;
    if (CAUSAL) kend = min(kend, min(N, qblk + BQ));
    const int ntiles = (kend + BK - 1) / BK;

    const unsigned char *kbase = (const unsigned char *)p.k + (size_t)kv_bh * N * D * QK_BYTES;
    const uint16_t *vbase = p.v + (size_t)kv_bh * N * D;

    // ---- Q operand, resident in registers for the whole kernel ----
    uint4 qreg[KSTEPS];
    {
        const unsigned char *qb = (const unsigned char *)p.q + ((size_t)bh * N + (size_t)(q_row < N ? q_row : 0)) * D * QK_BYTES;
#pragma unroll
        for (int s = 0; s < KSTEPS; ++s) {
            uint4 val = *(const uint4 *)(qb + s * 32 + h * 16);
            if (q_row >= N) val = make_uint4(0, 0, 0, 0);
            qreg[s] = val;
        }
    }

    // ---- staging registers (tile i+1 in flight while tile i is computed) ----
    uint4 kst[K_PER_THREAD];
    uint4 vst[V_PER_THREAD][4];

    auto load_tile = [&](int k0) {
#pragma unroll
        for (int j = 0; j < K_PER_THREAD; ++j) {
            const int c = tid + j * T;
            if (K_CHUNKS >= T || c < K_CHUNKS) {
                const int row = c / K_CPR, col = c % K_CPR;
                const int gr = k0 + row;
                uint4 val = make_uint4(0, 0, 0, 0);
                if (gr < kend) val = *(const uint4 *)(kbase + (size_t)gr * D * QK_BYTES + col * 16);
                kst[j] = val;
            }
        }
#pragma unroll
        for (int j = 0; j < V_PER_THREAD; ++j) {
            const int u = tid + j * T;
            if (V_UNITS >= T || u < V_UNITS) {
                const int m = u / (D / 8), dc = u % (D / 8);
#pragma unroll
                for (int kk = 0; kk < 4; ++kk) {
                    const int gr = k0 + m * 4 + kk;
                    uint4 val = make_uint4(0, 0, 0, 0);
                    if (gr < kend) val = *(const uint4 *)(vbase + (size_t)gr * D + dc * 8);
                    vst[j][kk] = val;
                }
            }
        }
    };

    auto store_tile = [&](int stage) {
        unsigned char *kl = lds + stage * STAGE;
        unsigned char *vl = kl + K_TILE;
#pragma unroll
        for (int j = 0; j < K_PER_THREAD; ++j) {
            const int c = tid + j * T;
            if (K_CHUNKS >= T || c < K_CHUNKS) {
                const int row = c / K_CPR, col = c % K_CPR;
                *(uint4 *)(kl + row * KROW + col * 16) = kst[j];
            }
        }
#pragma unroll
        for (int j = 0; j < V_PER_THREAD; ++j) {
            const int u = tid + j * T;
            if (V_UNITS >= T || u < V_UNITS) {
                const int m = u / (D / 8), dc = u % (D / 8);
                // keys 4m..4m+3 -> position group: swap the middle two groups of every 16 keys
                const int g4 = m & 3;
                const int pos = ((m & ~3) + ((g4 & 1) << 1) + (g4 >> 1)) << 2;
                const uint32_t r0[4] = {vst[j][0].x, vst[j][0].y, vst[j][0].z, vst[j][0].w};
                const uint32_t r1[4] = {vst[j][1].x, vst[j][1].y, vst[j][1].z, vst[j][1].w};
                const uint32_t r2[4] = {vst[j][2].x, vst[j][2].y, vst[j][2].z, vst[j][2].w};
                const uint32_t r3[4] = {vst[j][3].x, vst[j][3].y, vst[j][3].z, vst[j][3].w};
#pragma unroll
                for (int c = 0; c < 4; ++c) {
                    uint2 lo, hi;
                    lo.x = (r0[c] & 0xffffu) | (r1[c] << 16);
                    lo.y = (r2[c] & 0xffffu) | (r3[c] << 16);
                    hi.x = (r0[c] >> 16) | (r1[c] & 0xffff0000u);
                    hi.y = (r2[c] >> 16) | (r3[c] & 0xffff0000u);
                    *(uint2 *)(vl + vt_off(dc * 8 + 2 * c, pos)) = lo;
                    *(uint2 *)(vl + vt_off(dc * 8 + 2 * c + 1, pos)) = hi;
                }
            }
        }
    };

    // ---- accumulators ----
    f32x16 oacc[DB];
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int r = 0; r < 16; ++r) oacc[db][r] = 0.f;
    float m_run = NEG_SENTINEL;  // running max, in the exp2 domain (x * log2e)
    float l_run = 0.f;           // this lane half's part of the running sum

    float sq_lane = 1.f;
    if (MODE == MODE_I8) {
        const int nqb = (N + p.bq - 1) / p.bq;
        sq_lane = p.sq[(size_t)bh * nqb + (q_row < N ? q_row : N - 1) / p.bq];
    }
    const int nkb = (MODE == MODE_I8) ? (N + p.bk - 1) / p.bk : 0;
    const float c_scale = p.scale * LOG2E;

    if (ntiles > 0) {
        load_tile(0);
        store_tile(0);
    }
    __syncthreads();

    for (int it = 0; it < ntiles; ++it) {
        const int k0 = it * BK;
        const int stage = it & 1;
        if (it + 1 < ntiles) load_tile(k0 + BK);

        // a wave whose queries all precede this tile has nothing to do in it
        const bool active = !CAUSAL || (k0 <= wq0 + 31);
        if (active) {
            const unsigned char *kl = lds + stage * STAGE;
            const unsigned char *vl = kl + K_TILE;

            // ---- S^T = K . Q^T : two blocks of 32 keys x 32 queries ----
            float x[2][16];
#pragma unroll
            for (int kb = 0; kb < 2; ++kb) {
                const unsigned char *krow = kl + (kb * 32 + i32) * KROW + h * 16;
                if (MODE == MODE_I8) {
                    i32x16 acc;
#pragma unroll
                    for (int r = 0; r < 16; ++r) acc[r] = 0;
#pragma unroll
                    for (int s = 0; s < KSTEPS; ++s) {
                        const uint4 a = *(const uint4 *)(krow + s * 32);
                        acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(
                            __builtin_bit_cast(i32x4, a), __builtin_bit_cast(i32x4, qreg[s]), acc, 0, 0, 0);
                    }
                    if (DBG) {
                        if (bh == p.dbg_bh && (wq0 >> 5) == p.dbg_qt && it == p.dbg_kt) {
#pragma unroll
                            for (int r = 0; r < 16; ++r) {
                                const int key = kb * 32 + 8 * (r >> 2) + 4 * h + (r & 3);
                                p.dbg[i32 * 64 + key] = acc[r];
                            }
                        }
                    }
                    // s = (float)acc * ((sq * sk) * scale), src/runtime/cuda_flash_sage.rs:315-322
                    if ((p.bk & 31) == 0) {
                        const float skv = p.sk[(size_t)kv_bh * nkb + min(k0 + kb * 32, N - 1) / p.bk];
                        const float f = ((sq_lane * skv) * p.scale) * LOG2E;
#pragma unroll
                        for (int r = 0; r < 16; ++r) x[kb][r] = (float)acc[r] * f;
                    } else {
#pragma unroll
                        for (int r = 0; r < 16; ++r) {
                            const int key = k0 + kb * 32 + 8 * (r >> 2) + 4 * h + (r & 3);
                            const float skv = p.sk[(size_t)kv_bh * nkb + min(key, N - 1) / p.bk];
                            x[kb][r] = (float)acc[r] * (((sq_lane * skv) * p.scale) * LOG2E);
                        }
                    }
                } else {
                    f32x16 acc;
#pragma unroll
                    for (int r = 0; r < 16; ++r) acc[r] = 0.f;
#pragma unroll
                    for (int s = 0; s < KSTEPS; ++s) {
                        const uint4 a = *(const uint4 *)(krow + s * 32);
                        acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(
                            __builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, qreg[s]), acc, 0, 0, 0);
                    }
#pragma unroll
                    for (int r = 0; r < 16; ++r) x[kb][r] = acc[r] * c_scale;
                }
            }

            // ---- additive mask, causal and key-length masking ----
            if (HAS_MASK) {
#pragma unroll
                for (int kb = 0; kb < 2; ++kb)
#pragma unroll
                    for (int r = 0; r < 16; ++r) {
                        const int key = k0 + kb * 32 + 8 * (r >> 2) + 4 * h + (r & 3);
                        if (key < N && q_row < N) x[kb][r] += p.mask[(size_t)q_row * N + key] * LOG2E;
                    }
            }
            const bool edge = (k0 + BK > kend) || (CAUSAL && (k0 + BK - 1 > wq0));
            if (edge) {
#pragma unroll
                for (int kb = 0; kb < 2; ++kb)
#pragma unroll
                    for (int r = 0; r < 16; ++r) {
                        const int key = k0 + kb * 32 + 8 * (r >> 2) + 4 * h + (r & 3);
                        if (key >= kend || (CAUSAL && key > q_row)) x[kb][r] = NEG_SENTINEL;
                    }
            }

            // ---- online softmax, one query per lane ----
            float mx = x[0][0];
#pragma unroll
            for (int r = 1; r < 16; ++r) mx = fmaxf(mx, x[0][r]);
#pragma unroll
            for (int r = 0; r < 16; ++r) mx = fmaxf(mx, x[1][r]);
            mx = xhalf_max(mx);
            const float m_new = fmaxf(m_run, mx);
            const float alpha = __builtin_amdgcn_exp2f(m_run - m_new);
            m_run = m_new;
            float rs = 0.f;
#pragma unroll
            for (int kb = 0; kb < 2; ++kb)
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const float pv = __builtin_amdgcn_exp2f(x[kb][r] - m_new);
                    x[kb][r] = pv;
                    rs += pv;
                }
            l_run = l_run * alpha + rs;

            // rescale the accumulators only when some lane's maximum moved
            if (__any(alpha != 1.0f)) {
#pragma unroll
                for (int db = 0; db < DB; ++db)
#pragma unroll
                    for (int r = 0; r < 16; ++r) oacc[db][r] *= alpha;
            }

            // ---- P (bf16) as the B operand: 4 steps of 16 keys ----
            uint4 pb[4];
#pragma unroll
            for (int ks = 0; ks < 4; ++ks) {
                const int kb = ks >> 1, r0 = (ks & 1) * 8;
                pb[ks].x = pack_bf16x2(x[kb][r0 + 0], x[kb][r0 + 1]);
                pb[ks].y = pack_bf16x2(x[kb][r0 + 2], x[kb][r0 + 3]);
                pb[ks].z = pack_bf16x2(x[kb][r0 + 4], x[kb][r0 + 5]);
                pb[ks].w = pack_bf16x2(x[kb][r0 + 6], x[kb][r0 + 7]);
            }

            // ---- O^T += V^T . P^T ----
#pragma unroll
            for (int db = 0; db < DB; ++db) {
                const int d = db * 32 + i32;
#pragma unroll
                for (int ks = 0; ks < 4; ++ks) {
                    const uint4 a = *(const uint4 *)(vl + vt_off(d, ks * 16 + h * 8));
                    oacc[db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(
                        __builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, pb[ks]), oacc[db], 0, 0, 0);
                }
            }
        }

        if (it + 1 < ntiles) store_tile(stage ^ 1);
        __syncthreads();
    }

    // ---- normalise and store: acc * (l > 0 ? 1/l : 0), cuda_flash_bf16.rs:414-426 ----
    const float l_tot = xhalf_sum(l_run);
    const float inv = (l_tot > 0.f) ? 1.f / l_tot : 0.f;
    if (q_row < N) {
        const size_t obase = ((size_t)bh * N + q_row) * D;
#pragma unroll
        for (int db = 0; db < DB; ++db)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const int d = db * 32 + 8 * g + 4 * h;
                const float o0 = oacc[db][4 * g + 0] * inv, o1 = oacc[db][4 * g + 1] * inv;
                const float o2 = oacc[db][4 * g + 2] * inv, o3 = oacc[db][4 * g + 3] * inv;
                if (OUT_F32) {
                    *(float4 *)((float *)p.o + obase + d) = make_float4(o0, o1, o2, o3);
                } else {
                    uint2 w;
                    w.x = pack_bf16x2(o0, o1);
                    w.y = pack_bf16x2(o2, o3);
                    *(uint2 *)((uint16_t *)p.o + obase + d) = w;
                }
            }
    }
}

}  // namespace arhip
