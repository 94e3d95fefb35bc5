// Fused attention forward for gfx950 (CDNA4): one kernel template for the bf16
// FlashAttention path and the int8 (SageAttention-style) path.
//
// Work decomposition
//   grid  : one workgroup per (batch*head, tile of BQ = 32*QG*NW queries)
//   wave  : 32*QG queries.  The wave computes S^T = K . Q^T, so that in the
//           MFMA result layout every lane owns ONE query per group (column
//           lane%32) and 16 of the 32 keys of a block.  Row max / row sum are
//           per-lane reductions plus one exchange with lane^32, and the
//           probabilities are already in the operand layout the second product
//           needs: O^T = V^T . P^T, again with one query per lane.  With QG = 2
//           every K / V^T fragment read from LDS feeds two MFMAs.
//   tiles : BK = 64 keys per step, K and V^T staged through LDS by the whole
//           workgroup: 128-bit global loads issued one tile ahead into
//           registers, written to the other LDS buffer after the math.
//   blocks: inside a tile the online softmax advances in blocks of 32 keys and
//           Q.K^T of the next block is issued before the softmax of the current
//           one, so that the matrix pipe works while the vector ALU exponentiates.
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
// so V^T is stored in LDS with the two middle groups of four keys of every 16
// swapped, and P is used exactly as the first MFMA produced it.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <type_traits>

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

// lane and lane^32 hold the same query: combine their partial results
__device__ __forceinline__ float xhalf_other(float x)
{
#if ARHIP_NO_PERMLANE_SWAP
    return __shfl_xor(x, 32);
#else
    // v_permlane32_swap exchanges the upper half of the first operand with the
    // lower half of the second: (x, x) -> ({lo,lo}, {hi,hi})
    const uint32_t u = __float_as_uint(x);
    const auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
    const int h = (threadIdx.x >> 5) & 1;
    return __uint_as_float(h ? r[0] : r[1]);
#endif
}
__device__ __forceinline__ float xhalf_max(float x)
{
#if ARHIP_NO_PERMLANE_SWAP
    return fmaxf(x, __shfl_xor(x, 32));
#else
    const uint32_t u = __float_as_uint(x);
    const auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
    return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
#endif
}
__device__ __forceinline__ float xhalf_sum(float x)
{
#if ARHIP_NO_PERMLANE_SWAP
    return x + __shfl_xor(x, 32);
#else
    const uint32_t u = __float_as_uint(x);
    const auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
    return __uint_as_float(r[0]) + __uint_as_float(r[1]);
#endif
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

// s_waitcnt vmcnt(0): all outstanding global loads of this wave have landed.
__device__ __forceinline__ void wait_vmem() { __builtin_amdgcn_s_waitcnt(0x0F70); }

template <int D, int NW, int QG, bool CAUSAL, bool HAS_MASK, int MODE, bool PER_KEY, bool OUT_F32, bool DBG>
__global__ void __launch_bounds__(NW * 64) attn_fwd_kernel(const AttnParams p)
{
    constexpr int T = NW * 64;
    constexpr int WQ = 32 * QG;                                // queries per wave
    constexpr int BQ = NW * WQ;
    constexpr int QK_BYTES = (MODE == MODE_I8) ? 1 : 2;        // bytes per q/k element
    constexpr int KROW = D * QK_BYTES + 16;                    // padded K row in LDS
    constexpr int K_TILE = BK * KROW;
    constexpr int V_TILE = D * 128;
    constexpr int S_TILE = PER_KEY ? BK * 4 : 0;               // per-key scales of the tile
    constexpr int STAGE = K_TILE + V_TILE + S_TILE;
    constexpr int K_CPR = D * QK_BYTES / 16;                   // 16-byte chunks per K row
    constexpr int K_CHUNKS = BK * K_CPR;
    constexpr int K_PER_THREAD = (K_CHUNKS + T - 1) / T;
    constexpr int V_UNITS = (BK / 4) * (D / 8);                // 4 keys x 8 channels each
    constexpr int V_PER_THREAD = (V_UNITS + T - 1) / T;
    constexpr int KSTEPS = (MODE == MODE_I8) ? D / 32 : D / 16;  // MFMA k steps over D
    constexpr int DB = D / 32;                                 // 32-channel output blocks
    static_assert(K_CHUNKS % T == 0 || K_CHUNKS < T, "K staging must divide evenly");
    static_assert(V_UNITS % T == 0 || V_UNITS < T, "V staging must divide evenly");
    static_assert(!PER_KEY || MODE == MODE_I8, "per-key scales belong to the int8 path");

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
    const int wq0 = qblk + wave * WQ;  // first query of this wave

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

    // ---- Q operand, resident in registers for the whole kernel.  Rows past N
    // read row N-1: their results are never stored. ----
    uint4 qreg[QG][KSTEPS];
    int q_row[QG];
#pragma unroll
    for (int g = 0; g < QG; ++g) {
        q_row[g] = wq0 + g * 32 + i32;
        const unsigned char *qb =
            (const unsigned char *)p.q + ((size_t)bh * N + (size_t)min(q_row[g], N - 1)) * D * QK_BYTES;
#pragma unroll
        for (int s = 0; s < KSTEPS; ++s) qreg[g][s] = *(const uint4 *)(qb + s * 32 + h * 16);
    }

    // ---- staging registers (tile i+1 in flight while tile i is computed) ----
    uint4 kst[K_PER_THREAD];
    uint4 vst[V_PER_THREAD][4];
    float sst = 0.f;
    const int nkb = (MODE == MODE_I8) ? (N + p.bk - 1) / p.bk : 0;

    auto load_tile = [&](int k0) {
        const bool full = k0 + BK <= kend;  // uniform: the common case has no bounds logic
#pragma unroll
        for (int j = 0; j < K_PER_THREAD; ++j) {
            const int c = tid + j * T;
            if (K_CHUNKS >= T || c < K_CHUNKS) {
                const int row = c / K_CPR, col = c % K_CPR;
                const int gr = k0 + row;
                if (full) {
                    kst[j] = *(const uint4 *)(kbase + (size_t)gr * (D * QK_BYTES) + col * 16);
                } else {
                    uint4 val = *(const uint4 *)(kbase + (size_t)min(gr, kend - 1) * (D * QK_BYTES) + col * 16);
                    if (gr >= kend) val = make_uint4(0, 0, 0, 0);
                    kst[j] = val;
                }
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
                    if (full) {
                        vst[j][kk] = *(const uint4 *)(vbase + (size_t)gr * D + dc * 8);
                    } else {
                        uint4 val = *(const uint4 *)(vbase + (size_t)min(gr, kend - 1) * D + dc * 8);
                        if (gr >= kend) val = make_uint4(0, 0, 0, 0);
                        vst[j][kk] = val;
                    }
                }
            }
        }
        if (PER_KEY && tid < BK) sst = p.sk[(size_t)kv_bh * nkb + min(k0 + tid, N - 1) / p.bk];
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
        if (PER_KEY && tid < BK) *(float *)(vl + V_TILE + tid * 4) = sst;
    };

    // ---- accumulators and softmax state, one query per lane and group ----
    f32x16 oacc[QG][DB];
    float m_run[QG], l_run[QG], sq_lane[QG];
#pragma unroll
    for (int g = 0; g < QG; ++g) {
#pragma unroll
        for (int db = 0; db < DB; ++db)
#pragma unroll
            for (int r = 0; r < 16; ++r) oacc[g][db][r] = 0.f;
        m_run[g] = NEG_SENTINEL;  // running max in the exp2 domain (x * log2e)
        l_run[g] = 0.f;           // this lane half's part of the running sum
        sq_lane[g] = 1.f;
        if (MODE == MODE_I8) {
            const int nqb = (N + p.bq - 1) / p.bq;
            sq_lane[g] = p.sq[(size_t)bh * nqb + min(q_row[g], N - 1) / p.bq];
        }
    }
    const float c_scale = p.scale * LOG2E;

    if (ntiles > 0) {
        load_tile(0);
        store_tile(0);
    }
    wait_vmem();  // Q and the first tile have landed: nothing is pending at loop entry
    __syncthreads();

    // S^T block: 32 keys x 32 queries for every query group, raw accumulators
    typedef typename std::conditional<MODE == MODE_I8, i32x16, f32x16>::type acc_t;
    auto qk_block = [&](const unsigned char *kl, int blk, acc_t (&s)[QG]) {
        const unsigned char *krow = kl + (blk * 32 + i32) * KROW + h * 16;
#pragma unroll
        for (int g = 0; g < QG; ++g)
#pragma unroll
            for (int r = 0; r < 16; ++r) s[g][r] = 0;
#pragma unroll
        for (int st = 0; st < KSTEPS; ++st) {
            const uint4 a = *(const uint4 *)(krow + st * 32);
#pragma unroll
            for (int g = 0; g < QG; ++g) {
                if constexpr (MODE == MODE_I8)
                    s[g] = __builtin_amdgcn_mfma_i32_32x32x32_i8(__builtin_bit_cast(i32x4, a),
                                                                 __builtin_bit_cast(i32x4, qreg[g][st]), s[g], 0, 0, 0);
                else
                    s[g] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a),
                                                                   __builtin_bit_cast(bf16x8, qreg[g][st]), s[g], 0, 0, 0);
            }
        }
    };

    int sk_idx = 0, sk_fill = 0;
    for (int it = 0; it < ntiles; ++it) {
        const int k0 = it * BK;
        const int stage = it & 1;
        if (it + 1 < ntiles) load_tile(k0 + BK);

        // a wave whose queries all precede this tile has nothing to do in it
        const bool active = !CAUSAL || (k0 <= wq0 + WQ - 1);
        if (active) {
            const unsigned char *kl = lds + stage * STAGE;
            const unsigned char *vl = kl + K_TILE;

            // tile-uniform K scale (block sizes that are multiples of the tile)
            float f_tile = c_scale;
            if (MODE == MODE_I8 && !PER_KEY) f_tile = p.sk[(size_t)kv_bh * nkb + sk_idx];

            acc_t sacc[2][QG];
            qk_block(kl, 0, sacc[0]);
#pragma unroll
            for (int blk = 0; blk < 2; ++blk) {
                if (blk == 0) qk_block(kl, 1, sacc[1]);
                const int kb0 = k0 + blk * 32;  // first key of the block

                uint4 pb[QG][2];
#pragma unroll
                for (int g = 0; g < QG; ++g) {
                    acc_t &s = sacc[blk][g];
                    if (DBG) {
                        if (bh == p.dbg_bh && ((wq0 >> 5) + g) == p.dbg_qt && it == p.dbg_kt) {
#pragma unroll
                            for (int r = 0; r < 16; ++r)
                                p.dbg[i32 * 64 + blk * 32 + 8 * (r >> 2) + 4 * h + (r & 3)] = (int32_t)s[r];
                        }
                    }
                    float x[16];
                    float m_new;
                    const bool edge = (kb0 + 32 > kend) || (CAUSAL && (kb0 + 31 > wq0 + g * 32));
                    if (!HAS_MASK && !PER_KEY && !edge) {
                        // fast path: max over the raw accumulators, scale folded into the exponent
                        // s = (float)acc * ((sq * sk) * scale), src/runtime/cuda_flash_sage.rs:315-322
                        const float c = (MODE == MODE_I8) ? ((sq_lane[g] * f_tile) * p.scale) * LOG2E : c_scale;
#pragma unroll
                        for (int r = 0; r < 16; ++r) x[r] = (float)s[r];
                        float mx = fmaxf(x[0], x[1]);
#pragma unroll
                        for (int r = 2; r < 16; r += 2) mx = fmaxf(mx, fmaxf(x[r], x[r + 1]));
                        mx = xhalf_max(mx);
                        m_new = fmaxf(m_run[g], mx * c);
#pragma unroll
                        for (int r = 0; r < 16; ++r) x[r] = __builtin_amdgcn_exp2f(__builtin_fmaf(x[r], c, -m_new));
                    } else {
#pragma unroll
                        for (int r = 0; r < 16; ++r) {
                            const int key = kb0 + 8 * (r >> 2) + 4 * h + (r & 3);
                            float c = c_scale;
                            if (MODE == MODE_I8) {
                                const float skv = PER_KEY ? *(const float *)(vl + V_TILE + (key - k0) * 4) : f_tile;
                                c = ((sq_lane[g] * skv) * p.scale) * LOG2E;
                            }
                            float xv = (float)s[r] * c;
                            if (HAS_MASK) {
                                if (key < N && q_row[g] < N) xv += p.mask[(size_t)q_row[g] * N + key] * LOG2E;
                            }
                            if (key >= kend || (CAUSAL && key > q_row[g])) xv = NEG_SENTINEL;
                            x[r] = xv;
                        }
                        float mx = fmaxf(x[0], x[1]);
#pragma unroll
                        for (int r = 2; r < 16; r += 2) mx = fmaxf(mx, fmaxf(x[r], x[r + 1]));
                        mx = xhalf_max(mx);
                        m_new = fmaxf(m_run[g], mx);
#pragma unroll
                        for (int r = 0; r < 16; ++r) x[r] = __builtin_amdgcn_exp2f(x[r] - m_new);
                    }
                    const float alpha = __builtin_amdgcn_exp2f(m_run[g] - m_new);
                    m_run[g] = m_new;
                    float rs = (x[0] + x[1]) + (x[2] + x[3]);
#pragma unroll
                    for (int r = 4; r < 16; r += 4) rs += (x[r] + x[r + 1]) + (x[r + 2] + x[r + 3]);
                    l_run[g] = l_run[g] * alpha + rs;
                    // rescale the accumulators only when some lane's maximum moved
                    if (__any(alpha != 1.0f)) {
#pragma unroll
                        for (int db = 0; db < DB; ++db)
#pragma unroll
                            for (int r = 0; r < 16; ++r) oacc[g][db][r] *= alpha;
                    }
                    // P (bf16) as the B operand: 2 steps of 16 keys
#pragma unroll
                    for (int ks = 0; ks < 2; ++ks) {
                        pb[g][ks].x = pack_bf16x2(x[ks * 8 + 0], x[ks * 8 + 1]);
                        pb[g][ks].y = pack_bf16x2(x[ks * 8 + 2], x[ks * 8 + 3]);
                        pb[g][ks].z = pack_bf16x2(x[ks * 8 + 4], x[ks * 8 + 5]);
                        pb[g][ks].w = pack_bf16x2(x[ks * 8 + 6], x[ks * 8 + 7]);
                    }
                }

                // ---- O^T += V^T . P^T for the 32 keys of the block ----
#pragma unroll
                for (int db = 0; db < DB; ++db) {
                    const int d = db * 32 + i32;
#pragma unroll
                    for (int ks = 0; ks < 2; ++ks) {
                        const uint4 a = *(const uint4 *)(vl + vt_off(d, blk * 32 + ks * 16 + h * 8));
#pragma unroll
                        for (int g = 0; g < QG; ++g)
                            oacc[g][db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(
                                __builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, pb[g][ks]), oacc[g][db], 0, 0, 0);
                    }
                }
            }
        }

        if (it + 1 < ntiles) store_tile(stage ^ 1);
        __syncthreads();
        if (MODE == MODE_I8 && !PER_KEY) {  // advance the K-block index without dividing
            sk_fill += BK;
            if (sk_fill >= p.bk) {
                sk_fill = 0;
                ++sk_idx;
            }
        }
    }

    // ---- normalise and store: acc * (l > 0 ? 1/l : 0), cuda_flash_bf16.rs:414-426 ----
#pragma unroll
    for (int g = 0; g < QG; ++g) {
        const float l_tot = xhalf_sum(l_run[g]);
        const float inv = (l_tot > 0.f) ? 1.f / l_tot : 0.f;
        if (q_row[g] < N) {
            const size_t obase = ((size_t)bh * N + q_row[g]) * D;
#pragma unroll
            for (int db = 0; db < DB; ++db)
#pragma unroll
                for (int gg = 0; gg < 4; ++gg) {
                    const int d = db * 32 + 8 * gg + 4 * h;
                    const float o0 = oacc[g][db][4 * gg + 0] * inv, o1 = oacc[g][db][4 * gg + 1] * inv;
                    const float o2 = oacc[g][db][4 * gg + 2] * inv, o3 = oacc[g][db][4 * gg + 3] * inv;
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
}

}  // namespace arhip
