// fp32 exact-mode FlashAttention forward: no reduced precision anywhere.
//
// Semantics of the reference's scalar kernel (src/runtime/cuda_flash.rs:53-141): fp32 products
// and sums, fp32 exponentials, finite sentinel -1e30 for masked keys, acc * (l > 0 ? 1/l : 0) at
// the end; head_dim and scale are parameters here (the reference hard-codes 64 and 0.125).  The
// exponential is v_exp_f32 (base 2, 1 ulp) on logits scaled by scale * log2(e), where the reference
// calls expf on logits scaled by scale: the same function to a few ulp.
//
// The two contractions run on the fp32 matrix instruction v_mfma_f32_32x32x2_f32 (fp32 in,
// fp32 accumulate) with the same decomposition as the bf16 kernel: a wave owns 32 queries and
// computes S^T = K . Q^T, so each lane owns one query (column lane%32) and 16 of a block's 32
// keys; O^T = V^T . P^T keeps one query per lane, and the online-softmax state is per lane.
//   A[32 x 2] . B[2 x 32]: lane holds A[lane%32][lane/32] and B[lane/32][lane%32]
//   result C[32 x 32]: lane holds column lane%32, rows 8*(r/4) + 4*(lane/32) + r%4
// The order of the channels inside Q.K^T is free as long as Q and K agree, so MFMA step s of
// lane half h multiplies channel h*D/2 + s: every lane reads its K row as D/2 consecutive
// floats.  For P.V the step (g, t) multiplies key 8g + 4h + t, which is exactly the key the
// S^T result left in register 4g + t of that lane.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <type_traits>

namespace arhip {

typedef __attribute__((ext_vector_type(16))) float f32x16_t;

constexpr int F32_BK = 32;  // keys per tile

struct FlashF32Params {
    const float *q, *k, *v;
    float *o;
    const float *mask;      // additive [N,N] or null
    const int32_t *kv_len;  // [B] or null
    float *lse;             // optional [B,Hq,N]: m + log(l), src/runtime/cuda_flash_train.rs:141
    int Hq, Hkv, N, nq;
    int lpt_heads;  // causal: B * Hq, and the grid runs longest query tile first over all heads; else 0
    int total;      // workgroups in the grid (nq * B * Hq)
    long qs[3], ks[3], os[3];  // element strides [batch, head, token] of q / k,v / o (channel stride 1)
    float scale;
};

// LDS floats flash_f32_body needs: one padded K tile and one V tile (one pair per wave with SPLITK)
template <int D, int NW = 1, bool SPLITK = false>
constexpr int flash_f32_lds_floats()
{
    return (SPLITK ? NW : 1) * (F32_BK * (D + 4) + F32_BK * D);
}

// The kernel body.  lds: flash_f32_lds_floats<D, NW, SPLITK>() floats of workgroup memory, 16-byte
// aligned; wg_linear: this workgroup's index in [0, nq * B * Hq).
//
// SPLITK (few, short heads: the launch would otherwise leave most SIMDs idle behind one wave's
// chain of matrix instructions): the NW waves of a workgroup share the same 32 queries and deal
// the key tiles out between them (wave w takes tiles w, w + NW, ...), each staging its own tiles
// in its own LDS slab with no workgroup barrier; at the end the partial (m, l, O) of the waves are
// merged through LDS: m = max m_w, l = sum l_w e^(m_w - m), O = sum O_w e^(m_w - m).
template <int D, int NW, bool CAUSAL, bool SPLITK = false>
__device__ __forceinline__ void flash_f32_body(const FlashF32Params &p, float *lds, int wg_linear)
{
    constexpr int T = SPLITK ? 64 : NW * 64;      // threads staging one tile
    constexpr int BQ = SPLITK ? 32 : NW * 32;
    constexpr int HALF = D / 2;          // channels per lane half
    constexpr int KROW = D + 4;          // padded K row (floats): conflict-free 128-bit row reads
    constexpr int DB = D / 32;
    constexpr int CHUNKS = F32_BK * D / 4;             // float4 chunks per K (or V) tile
    constexpr int PER_THREAD = (CHUNKS + T - 1) / T;
    static_assert(CHUNKS % T == 0, "tile staging must divide evenly");

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);   // a scalar: tile indices and K/V tile addresses stay scalar
    constexpr int SLAB = F32_BK * KROW + F32_BK * D;
    float *ks = lds + (SPLITK ? wave * SLAB : 0);  // [F32_BK][KROW]
    float *vs = ks + F32_BK * KROW;                // [F32_BK][D]
    const int stid = SPLITK ? lane : tid;          // index among the threads staging a tile
    const int i32 = lane & 31, h = lane >> 5;
    // causal: the longest query tiles first over the whole grid, so that no head's long tiles are left for the end
    // (these kernels are bound by the matrix pipe at any grid size: every workgroup may stream its own K/V)
    // Consecutive workgroups go to different XCDs (8, each with its own L2): every XCD gets a contiguous range of
    // heads, so that the query tiles sharing a head's K/V meet in one L2 and, under the causal mask, every XCD gets
    // tiles of every length.
    const int wg_x = (p.total > 0 && (p.total & 7) == 0) ? (wg_linear & 7) * (p.total >> 3) + (wg_linear >> 3) : wg_linear;
    int bh = wg_x / p.nq;
    int qt = wg_x - bh * p.nq;
    if (CAUSAL) qt = p.nq - 1 - qt;
    if (CAUSAL && p.lpt_heads > 0) {
        qt = p.nq - 1 - wg_linear / p.lpt_heads;
        bh = wg_linear % p.lpt_heads;
    }
    const int b = bh / p.Hq, head = bh - b * p.Hq;
    const int N = p.N;
    const int qblk = qt * BQ;
    const int wq0 = qblk + (SPLITK ? 0 : wave * 32);
    const int q_row = wq0 + i32;

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
    const size_t kv_off = (size_t)b * p.ks[0] + (size_t)kvh * p.ks[1];
    const size_t k_rs = (size_t)p.ks[2];
    const char *kp = (const char *)(p.k + kv_off);
    const char *vp = (const char *)(p.v + kv_off);

    // Q: this lane's half of its query row (rows past N read row N-1; never stored)
    float qr[HALF];
    {
        const float *qp = p.q + (size_t)b * p.qs[0] + (size_t)head * p.qs[1] + (size_t)min(q_row, N - 1) * p.qs[2] + h * HALF;
#pragma unroll
        for (int s = 0; s < HALF; s += 4) {
            const float4 x = *(const float4 *)(qp + s);
            qr[s] = x.x; qr[s + 1] = x.y; qr[s + 2] = x.z; qr[s + 3] = x.w;
        }
    }

    f32x16_t oacc[DB];
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int r = 0; r < 16; ++r) oacc[db][r] = 0.f;
    // The softmax runs on base-2 exponentials: logits are scaled by scale * log2(e) and the running
    // maximum is kept in those units (one multiply-add and one v_exp_f32 per logit).
    constexpr float LOG2E = 1.44269504088896340736f, LN2 = 0.69314718055994530942f;
    const float c2 = p.scale * LOG2E;
    float m_run = -1e30f, l_run = 0.f;

    // The global loads of a tile are issued one tile ahead of its use, into registers, so that
    // their latency is spent under the matrix instructions of the tile before.  Thread t stages
    // rows t / (D/4) + j * RPJ, 16 bytes at column 4 * (t % (D/4)): a per-thread byte offset on top
    // of a scalar address per (tile, j).
    constexpr int RPJ = T / (D / 4);
    const int row0 = stid / (D / 4), col0 = (stid % (D / 4)) * 4;
    const size_t voff = ((size_t)row0 * k_rs + col0) * sizeof(float);
    float4 kx[PER_THREAD], vx[PER_THREAD];
    auto fetch = [&](int tile) __attribute__((always_inline)) {
        const size_t t0 = (size_t)tile * F32_BK * k_rs * sizeof(float);
        if (tile * F32_BK + F32_BK <= kend) {
#pragma unroll
            for (int j = 0; j < PER_THREAD; ++j) {
                const size_t so = t0 + (size_t)j * RPJ * k_rs * sizeof(float);
                kx[j] = *(const float4 *)(kp + so + voff);
                vx[j] = *(const float4 *)(vp + so + voff);
            }
        } else {
#pragma unroll
            for (int j = 0; j < PER_THREAD; ++j) {
                const size_t so = t0 + (size_t)j * RPJ * k_rs * sizeof(float);
                kx[j] = vx[j] = make_float4(0.f, 0.f, 0.f, 0.f);
                if (tile * F32_BK + row0 + j * RPJ < kend) {
                    kx[j] = *(const float4 *)(kp + so + voff);
                    vx[j] = *(const float4 *)(vp + so + voff);
                }
            }
        }
    };

    // one key tile; GENERIC: additive mask, keys past the end or hidden by the causal mask, or a
    // negative scale (the plain path takes the maximum before scaling)
    auto tile_body = [&](auto generic, int k0) __attribute__((always_inline)) {
        constexpr bool GENERIC = decltype(generic)::value;
        // ---- S^T = K . Q^T ----
        f32x16_t s;
#pragma unroll
        for (int r = 0; r < 16; ++r) s[r] = 0.f;
        const float *krow = &ks[i32 * KROW + h * HALF];
#pragma unroll
        for (int st = 0; st < HALF; st += 4) {
            const float4 kq = *(const float4 *)(krow + st);
            s = __builtin_amdgcn_mfma_f32_32x32x2f32(kq.x, qr[st + 0], s, 0, 0, 0);
            s = __builtin_amdgcn_mfma_f32_32x32x2f32(kq.y, qr[st + 1], s, 0, 0, 0);
            s = __builtin_amdgcn_mfma_f32_32x32x2f32(kq.z, qr[st + 2], s, 0, 0, 0);
            s = __builtin_amdgcn_mfma_f32_32x32x2f32(kq.w, qr[st + 3], s, 0, 0, 0);
        }

        // ---- scale, masks, online softmax ----
        float x[16];
        float m_new;
        if constexpr (GENERIC) {
            float mx = -1e30f;
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int key = k0 + 8 * (r >> 2) + 4 * h + (r & 3);
                float xv = s[r] * c2;
                if (p.mask != nullptr && key < N && q_row < N) xv = fmaf(p.mask[(size_t)q_row * N + key], LOG2E, xv);
                if (key >= kend || (CAUSAL && key > q_row)) xv = -1e30f;
                x[r] = xv;
                mx = fmaxf(mx, xv);
            }
            mx = fmaxf(mx, __shfl_xor(mx, 32));
            m_new = fmaxf(m_run, mx);
#pragma unroll
            for (int r = 0; r < 16; ++r) x[r] = __builtin_amdgcn_exp2f(x[r] - m_new);
        } else {
            float mx = fmaxf(s[0], s[1]);
#pragma unroll
            for (int r = 2; r < 16; ++r) mx = fmaxf(mx, s[r]);
            mx = fmaxf(mx, __shfl_xor(mx, 32));
            m_new = fmaxf(m_run, mx * c2);   // c2 >= 0 here: the largest logit is the largest product
#pragma unroll
            for (int r = 0; r < 16; ++r) x[r] = __builtin_amdgcn_exp2f(fmaf(s[r], c2, -m_new));
        }
        const float alpha = __builtin_amdgcn_exp2f(m_run - m_new);
        m_run = m_new;
        float rs = 0.f;
#pragma unroll
        for (int r = 0; r < 16; ++r) rs += x[r];
        l_run = l_run * alpha + rs;
        if (__any(alpha != 1.0f)) {
#pragma unroll
            for (int db = 0; db < DB; ++db)
#pragma unroll
                for (int r = 0; r < 16; ++r) oacc[db][r] *= alpha;
        }

        // ---- O^T += V^T . P^T : step (g, t) uses key 8g + 4h + t ----
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const float *vrow = &vs[(8 * (r >> 2) + 4 * h + (r & 3)) * D + i32];
#pragma unroll
            for (int db = 0; db < DB; ++db)
                oacc[db] = __builtin_amdgcn_mfma_f32_32x32x2f32(vrow[db * 32], x[r], oacc[db], 0, 0, 0);
        }
    };

    const bool always_generic = p.mask != nullptr || !(c2 >= 0.f);
    constexpr int STEP = SPLITK ? NW : 1;
    const int first = SPLITK ? wave : 0;
    if (first < ntiles) fetch(first);
    for (int it = first; it < ntiles; it += STEP) {
        const int k0 = it * F32_BK;
        if (!SPLITK) __syncthreads();  // the previous tile has been consumed
#pragma unroll
        for (int j = 0; j < PER_THREAD; ++j) {
            *(float4 *)&ks[(row0 + j * RPJ) * KROW + col0] = kx[j];
            *(float4 *)&vs[(row0 + j * RPJ) * D + col0] = vx[j];
        }
        if (it + STEP < ntiles) fetch(it + STEP);
        if (!SPLITK) __syncthreads();
        if (it >= my_tiles) continue;  // under the causal mask this wave is done (it still helps staging)
        if (always_generic || k0 + F32_BK > kend || (CAUSAL && k0 + F32_BK - 1 > wq0))
            tile_body(std::true_type{}, k0);
        else
            tile_body(std::false_type{}, k0);
    }

    const float l_tot = l_run + __shfl_xor(l_run, 32);
    if constexpr (SPLITK) {
        // ---- merge the waves' partial results ----
        // slab of wave w, reused: O_w as [32 queries][D + 4], then m_w[32], l_w[32]
        constexpr int OROW = D + 4;
        static_assert(32 * OROW + 64 <= SLAB, "merge buffers fit the staging slab");
        float *ow = lds + wave * SLAB;
#pragma unroll
        for (int db = 0; db < DB; ++db)
#pragma unroll
            for (int g = 0; g < 4; ++g)
                *(float4 *)&ow[i32 * OROW + db * 32 + 8 * g + 4 * h] =
                    make_float4(oacc[db][4 * g], oacc[db][4 * g + 1], oacc[db][4 * g + 2], oacc[db][4 * g + 3]);
        if (h == 0) {
            ow[32 * OROW + i32] = m_run;
            ow[32 * OROW + 32 + i32] = l_tot;
        }
        __syncthreads();
        // thread t: query t % 32, channels [cg * CPT, cg * CPT + CPT)
        constexpr int CPT = D / (NW * 2);
        static_assert(CPT % 4 == 0, "whole float4s per thread");
        const int q = tid & 31, cg = tid >> 5;
        const int row = qblk + q;
        float m = -1e30f;
#pragma unroll
        for (int w = 0; w < NW; ++w) m = fmaxf(m, lds[w * SLAB + 32 * OROW + q]);
        float l = 0.f, acc[CPT];
#pragma unroll
        for (int c = 0; c < CPT; ++c) acc[c] = 0.f;
#pragma unroll
        for (int w = 0; w < NW; ++w) {
            const float f = __builtin_amdgcn_exp2f(lds[w * SLAB + 32 * OROW + q] - m);
            l += lds[w * SLAB + 32 * OROW + 32 + q] * f;
#pragma unroll
            for (int c = 0; c < CPT; c += 4) {
                const float4 x = *(const float4 *)&lds[w * SLAB + q * OROW + cg * CPT + c];
                acc[c] += x.x * f; acc[c + 1] += x.y * f; acc[c + 2] += x.z * f; acc[c + 3] += x.w * f;
            }
        }
        const float inv = (l > 0.f) ? 1.f / l : 0.f;
        if (row < N) {
            if (p.lse != nullptr && cg == 0) p.lse[(size_t)bh * N + row] = (l > 0.f) ? m * LN2 + logf(l) : -1e30f;
            float *op = p.o + (size_t)b * p.os[0] + (size_t)head * p.os[1] + (size_t)row * p.os[2] + cg * CPT;
#pragma unroll
            for (int c = 0; c < CPT; c += 4)
                *(float4 *)(op + c) = make_float4(acc[c] * inv, acc[c + 1] * inv, acc[c + 2] * inv, acc[c + 3] * inv);
        }
        return;
    }
    const float inv = (l_tot > 0.f) ? 1.f / l_tot : 0.f;
    if (p.lse != nullptr && h == 0 && q_row < N)
        p.lse[(size_t)bh * N + q_row] = (l_tot > 0.f) ? m_run * LN2 + logf(l_tot) : -1e30f;
    if (q_row < N) {
        float *op = p.o + (size_t)b * p.os[0] + (size_t)head * p.os[1] + (size_t)q_row * p.os[2];
#pragma unroll
        for (int db = 0; db < DB; ++db)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const int d = db * 32 + 8 * g + 4 * h;
                *(float4 *)(op + d) = make_float4(oacc[db][4 * g] * inv, oacc[db][4 * g + 1] * inv,
                                                  oacc[db][4 * g + 2] * inv, oacc[db][4 * g + 3] * inv);
            }
    }
}

// D = 64: two waves per SIMD (registers held to 256 per lane); D = 128 needs more than that
template <int D, int NW, bool CAUSAL, bool SPLITK = false>
__global__ void __launch_bounds__(NW * 64, (D == 64 ? 2 : 1)) flash_f32_kernel(const FlashF32Params p)
{
    __shared__ __attribute__((aligned(16))) float lds[flash_f32_lds_floats<D, NW, SPLITK>()];
    flash_f32_body<D, NW, CAUSAL, SPLITK>(p, lds, (int)blockIdx.x);
}

}  // namespace arhip
