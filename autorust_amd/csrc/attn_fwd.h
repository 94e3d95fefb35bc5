// Fused attention forward for gfx950 (CDNA4): one kernel template for the bf16
// FlashAttention path and the int8 (SageAttention-style) path.
//
// Work decomposition
//   grid  : one workgroup per (batch*head, tile of BQ = 32*NW queries)
//   wave  : 32 queries.  The wave computes S^T = K . Q^T, so that in the MFMA
//           result layout every lane owns ONE query (column lane%32) and 16 of
//           the 32 keys of a block.  Row max / row sum are per-lane reductions
//           plus one exchange with lane^32, and the probabilities are already in
//           the operand layout the second product needs: O^T = V^T . P^T, again
//           with one query per lane (the softmax rescale is a per-lane scalar).
//   tiles : BK = 64 keys per step, K and V staged through LDS by the whole
//           workgroup (two stages, one barrier per tile) and two tiles ahead of
//           the math: in the middle of the iteration that computes tile i, tile
//           i+1 goes from registers to the stage tile i-1 vacated, and the
//           128-bit global loads of tile i+2 are issued.
//   blocks: inside a tile the online softmax advances 32 keys at a time and the
//           wave alternates between the matrix pipe and the vector ALU; every
//           LDS fragment is requested one phase before the MFMAs that use it.
//           With 8 waves per workgroup each SIMD holds two waves, and one of
//           them can exponentiate while the other multiplies.
//   lazy  : the exponent reference only moves (and the accumulators are only
//           rescaled) when a row maximum outgrows it by 2^60; softmax does not
//           depend on the reference, so the result is the same function.
//
// MFMA shapes (wave64):
//   v_mfma_f32_32x32x16_bf16  A[32 x 16] . B[16 x 32]   lane: row/col = lane%32,
//                             k = 8*(lane/32) + 0..7    (8 bf16 = 16 bytes)
//   v_mfma_i32_32x32x32_i8    lane: k = 16*(lane/32) + 0..15 (16 bytes)
//   result C[32 x 32]: lane holds column lane%32 and rows
//                             8*(r/4) + 4*(lane/32) + r%4,  r = 0..15
//
// V^T operand without a transpose pass: V sits in LDS row-major like K, and
// ds_read_b64_tr_b16 hands every lane four keys of ONE channel (within 16 lanes,
// result element e of lane i is element i%4 of the 8 bytes lane 4e + i/4 pointed
// at).  The S^T result gives lane half h the keys 8*(t/4) + 4h + t%4 of a 16-key
// step as B-operand elements t = 0..7, so the two transposing reads of a step
// simply fetch keys 4h..4h+3 and 8+4h..8+4h+3: P is used exactly as the first
// MFMA produced it and nothing is shuffled.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <type_traits>

namespace arhip {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(4))) int i32x4;
typedef __attribute__((ext_vector_type(16))) int i32x16;
typedef __attribute__((ext_vector_type(4))) short s16x4;

constexpr int MODE_BF16 = 0;  // q, k bf16
constexpr int MODE_I8 = 1;    // q, k int8 with block scales
constexpr int MODE_FP8 = 2;   // q, k FP8 E4M3 (OCP) with block scales: the reference's AR_FP8 branch, cuda_flash_sage.rs:92-147
constexpr int BK = 64;        // keys per tile
constexpr float NEG_SENTINEL = -1e30f;  // src/runtime/cuda_flash_bf16.rs:106 (AR_NEG)
constexpr float LOG2E = 1.4426950408889634f;
constexpr float LAZY_TAU = 60.0f;    // log2 units the running maximum may outgrow the exponent reference
constexpr float LAZY_LIMIT = 1152921504606846976.0f;  // = 2^LAZY_TAU: the largest probability the lazy reference lets through

struct AttnParams {
    const void *q;
    const void *k;
    const uint16_t *v;  // bf16 bits
    void *o;
    const float *mask;       // additive [N,N] or null
    const int32_t *kv_len;   // [B] or null
    const float *sq;         // MODE_I8: [B,Hq,ceil(N/bq)]
    const float *sk;         // MODE_I8: [B,Hkv,ceil(N/bk)]
    float *lse;              // optional [B,Hq,N]: log-sum-exp of the scaled, masked logits (natural log)
    float *sq_out;           // fused Q quantiser: optional [B,Hq,ceil(N/128)] scales it derived
    int8_t *q8_out;          // fused Q quantiser: optional [B,Hq,N,D] codes it derived
    int32_t *dbg;            // MODE_I8 debug: [32][64] raw logits
    int dbg_bh, dbg_qt, dbg_kt;
    int Hq, Hkv, N;
    // element strides of q / k / o (and v, below): [batch, head, token]; the channel stride is 1.
    // Dense [B,H,N,D] is {H*N*D, N*D, D}; token-major [B,N,H,D] is {N*H*D, D, H*D}.
    long qs[3], ks[3], os[3];
    long vs[3];    // V's own strides (the int8 path reads a dense K8 next to a V that may be strided)
    int bq, bk;
    int bk_tile_shift;  // log2(bk / 64) when the K scales are tile-uniform
    int bk_key_shift;   // log2(bk) for the pipelined kernel's per-key form (bk a power of two below 64)
    int out_f32;        // pipelined 8-bit kernels: store f32 instead of bf16
    int nq;        // query tiles per head
    int total;     // workgroups
    int lpt;       // causal: order the whole grid longest-tile-first (small grids)
    float scale;
};

__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi)
{
    typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
    bf16x2 p = {(__bf16)lo, (__bf16)hi};  // round-to-nearest-even
    return __builtin_bit_cast(uint32_t, p);
}

// v_max3_f32 (the generic fmaxf spends an extra instruction per operand on NaN quieting).
// Never hand it the raw result registers of a matrix instruction: the compiler pads the wait
// between an MFMA and the first vector read of its result only for instructions it generated,
// not for inline assembly, and an early read returns a partial sum.  Operands must have passed
// through an ordinary vector instruction (a scale, a convert) first.
__device__ __forceinline__ float max3(float a, float b, float c)
{
    float r;
    asm("v_max3_f32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "v"(c));
    return r;
}

// lane and lane^32 hold the same query: combine their partial results.
// v_permlane32_swap exchanges the upper half of its first operand with the lower
// half of its second: (x, x) -> ({lo,lo}, {hi,hi}).
__device__ __forceinline__ float xhalf_max(float x)
{
    const uint32_t u = __float_as_uint(x);
    const auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
    return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float xhalf_sum(float x)
{
    const uint32_t u = __float_as_uint(x);
    const auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
    return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}

// Four keys of one channel: the transposing LDS read described above.
__device__ __forceinline__ uint2 lds_read_tr16(const unsigned char *p)
{
    const s16x4 v = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4 *)p);
    return __builtin_bit_cast(uint2, v);
}

// Scheduling fence: the compiler may reorder freely inside a phase, not across this line.
#define ARHIP_FENCE() __builtin_amdgcn_sched_barrier(0)

// s_waitcnt vmcnt(0): all outstanding global loads of this wave have landed.
__device__ __forceinline__ void wait_vmem() { __builtin_amdgcn_s_waitcnt(0x0F70); }

// LDS bytes attn_fwd_body needs for a tiling variant
template <int D, int NW, int MODE, bool PER_KEY>
constexpr int attn_fwd_lds_bytes()
{
    constexpr int QKB = (MODE != MODE_BF16) ? 1 : 2;
    return 2 * (BK * (D * QKB + 16) + BK * (D * 2 + 64) + (PER_KEY ? BK * 4 : 0));
}

// The kernel body.  lds: attn_fwd_lds_bytes<...>() bytes of workgroup memory, 16-byte aligned;
// wg_linear: this workgroup's index in [0, p.total) (the entry points below and the named entry
// points of the loadable code object derive it from their grids).
template <int D, int NW, bool CAUSAL, bool HAS_MASK, int MODE, bool PER_KEY, bool OUT_F32, bool DBG>
__device__ __forceinline__ void attn_fwd_body(const AttnParams &p, unsigned char *lds, int wg_linear)
{
    constexpr int QW = NW;      // waves of a workgroup, each with 32 queries of its own
    constexpr int NSTAGE = 2;
    constexpr int NSLOT = 1;    // register sets for tiles in flight
    constexpr int T = NW * 64;
    constexpr int BQ = QW * 32;
    constexpr int QK_BYTES = (MODE != MODE_BF16) ? 1 : 2;        // bytes per q/k element
    constexpr int KROW = D * QK_BYTES + 16;                    // padded K row in LDS
    constexpr int K_TILE = BK * KROW;
    constexpr int VROW = D * 2 + 64;                           // V row in LDS: 4 rows fill the 64 banks
    constexpr int V_TILE = BK * VROW;
    constexpr int S_TILE = PER_KEY ? BK * 4 : 0;               // per-key scales of the tile
    constexpr int STAGE = K_TILE + V_TILE + S_TILE;
    constexpr int K_CPR = D * QK_BYTES / 16;                   // 16-byte chunks per K row
    constexpr int K_CHUNKS = BK * K_CPR;
    constexpr int K_PER_THREAD = (K_CHUNKS + T - 1) / T;
    constexpr int V_CPR = D * 2 / 16;                          // 16-byte chunks per V row
    constexpr int V_CHUNKS = BK * V_CPR;
    constexpr int V_PER_THREAD = (V_CHUNKS + T - 1) / T;
    constexpr int KSTEPS = (MODE != MODE_BF16) ? D / 32 : D / 16;  // MFMA k steps over D
    constexpr int DB = D / 32;                                 // 32-channel output blocks
    static_assert(K_CHUNKS % T == 0 || K_CHUNKS < T, "K staging must divide evenly");
    static_assert(V_CHUNKS % T == 0 || V_CHUNKS < T, "V staging must divide evenly");
    static_assert(!PER_KEY || MODE != MODE_BF16, "per-key scales belong to the 8-bit paths");
    static_assert(!DBG || MODE == MODE_I8, "the logits export is int32");

    static_assert(NSTAGE * STAGE == attn_fwd_lds_bytes<D, NW, MODE, PER_KEY>(), "LDS size bookkeeping");

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int i32 = lane & 31;
    const int h = lane >> 5;

    // Workgroup id -> (head, query tile).  Consecutive ids go to different XCDs
    // (8 of them, each with its own L2); give every XCD a contiguous range of
    // heads so that the query tiles sharing one head's K/V hit the same L2.
    int wg = wg_linear;
    int bh, qt;
    if (CAUSAL && p.lpt) {
        // Few workgroups per CU and very unequal ones (causal): longest-first over the whole
        // grid, so that no long tile is left for the end.  K/V of all heads then share the L2s
        // and the chip-wide cache instead of one XCD's L2.
        const int nbh = p.total / p.nq;
        qt = p.nq - 1 - wg / nbh;
        bh = wg % nbh;
    } else {
        if ((p.total & 7) == 0) wg = (wg & 7) * (p.total >> 3) + (wg >> 3);
        bh = wg / p.nq;
        qt = wg - bh * p.nq;
        if (CAUSAL) qt = p.nq - 1 - qt;  // longest tiles first within a head
    }
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
    // tiles this wave takes part in: under the causal mask, none past its last query
    const int my_tiles = CAUSAL ? min(ntiles, (wq0 + 31) / BK + 1) : ntiles;

    const size_t kv_off = (size_t)b * p.ks[0] + (size_t)kvh * p.ks[1];
    const size_t k_rs = (size_t)p.ks[2];  // elements between consecutive tokens of K / V
    const unsigned char *kbase = (const unsigned char *)p.k + kv_off * QK_BYTES;
    const uint16_t *vbase = p.v + (size_t)b * p.vs[0] + (size_t)kvh * p.vs[1];
    const size_t v_rs = (size_t)p.vs[2];

    // ---- Q operand, resident in registers for the whole kernel.  Rows past N
    // read row N-1: their results are never stored. ----
    uint4 qreg[KSTEPS];
    {
        const unsigned char *qb = (const unsigned char *)p.q +
                                  ((size_t)b * p.qs[0] + (size_t)head * p.qs[1] + (size_t)min(q_row, N - 1) * p.qs[2]) * QK_BYTES;
#pragma unroll
        for (int s = 0; s < KSTEPS; ++s) qreg[s] = *(const uint4 *)(qb + s * 32 + h * 16);
    }

    // ---- staging registers (tile i+1 in flight while tile i is computed) ----
    uint4 kst[NSLOT][K_PER_THREAD];
    uint4 vst[NSLOT][V_PER_THREAD];
    float sst = 0.f;
    const int nkb = (MODE != MODE_BF16) ? (N + p.bk - 1) / p.bk : 0;

    auto load_tile = [&](int k0, int slot = 0) __attribute__((always_inline)) {
        const bool full = k0 + BK <= kend;  // uniform: the common case has no bounds logic
#pragma unroll
        for (int j = 0; j < K_PER_THREAD; ++j) {
            const int c = tid + j * T;
            if (K_CHUNKS >= T || c < K_CHUNKS) {
                const int row = c / K_CPR, col = c % K_CPR;
                const int gr = k0 + row;
                if (full) {
                    kst[slot][j] = *(const uint4 *)(kbase + (size_t)gr * k_rs * QK_BYTES + col * 16);
                } else {
                    // rows past the last visible key are zeros and cost no memory transaction
                    uint4 val = make_uint4(0, 0, 0, 0);
                    if (gr < kend) val = *(const uint4 *)(kbase + (size_t)gr * k_rs * QK_BYTES + col * 16);
                    kst[slot][j] = val;
                }
            }
        }
#pragma unroll
        for (int j = 0; j < V_PER_THREAD; ++j) {
            const int c = tid + j * T;
            if (V_CHUNKS >= T || c < V_CHUNKS) {
                const int row = c / V_CPR, col = c % V_CPR;
                const int gr = k0 + row;
                if (full) {
                    vst[slot][j] = *(const uint4 *)(vbase + (size_t)gr * v_rs + col * 8);
                } else {
                    uint4 val = make_uint4(0, 0, 0, 0);
                    if (gr < kend) val = *(const uint4 *)(vbase + (size_t)gr * v_rs + col * 8);
                    vst[slot][j] = val;
                }
            }
        }
        if (PER_KEY && tid < BK) sst = p.sk[(size_t)kv_bh * nkb + min(k0 + tid, N - 1) / p.bk];
    };

    auto store_tile = [&](int stage, int slot = 0) __attribute__((always_inline)) {
        unsigned char *kl = lds + stage * STAGE;
        unsigned char *vl = kl + K_TILE;
#pragma unroll
        for (int j = 0; j < K_PER_THREAD; ++j) {
            const int c = tid + j * T;
            if (K_CHUNKS >= T || c < K_CHUNKS) {
                const int row = c / K_CPR, col = c % K_CPR;
                *(uint4 *)(kl + row * KROW + col * 16) = kst[slot][j];
            }
        }
#pragma unroll
        for (int j = 0; j < V_PER_THREAD; ++j) {
            const int c = tid + j * T;
            if (V_CHUNKS >= T || c < V_CHUNKS) {
                const int row = c / V_CPR, col = c % V_CPR;
                *(uint4 *)(vl + row * VROW + col * 16) = vst[slot][j];
            }
        }
        if (PER_KEY && tid < BK) *(float *)(vl + V_TILE + tid * 4) = sst;
    };

    // ---- accumulators and softmax state, one query per lane ----
    typedef typename std::conditional<MODE == MODE_I8, i32x16, f32x16>::type acc_t;
    f32x16 oacc[DB];
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int r = 0; r < 16; ++r) oacc[db][r] = 0.f;
    float m_run = NEG_SENTINEL;  // running max in the exp2 domain (x * log2e)
    float l_run = 0.f;           // this lane half's part of the running sum
    float sq_lane = 1.f;
    if (MODE != MODE_BF16) {
        const int nqb = (N + p.bq - 1) / p.bq;
        sq_lane = p.sq[(size_t)bh * nqb + min(q_row, N - 1) / p.bq];
    }
    const float c_scale = p.scale * LOG2E;
    const float sq_c = (sq_lane * p.scale) * LOG2E;  // per-key scales: the query's share of the exponent factor
    // ---- per-block pipeline ----------------------------------------------------------
    // A tile is two blocks of 32 keys.  For every block the wave alternates between the
    // matrix pipe and the vector ALU, and every LDS fragment is requested one phase before
    // the MFMAs that consume it, so that no MFMA waits for LDS latency:
    //   P1  request V^T fragments of the block;  S^T = K . Q^T   (K fragments already here)
    //   P2  online softmax of the block (vector ALU)
    //   P3  request K fragments of the next block;  O^T += V^T . P^T
    // The other wave of the SIMD is in a different phase most of the time, which is what
    // keeps both pipes busy; the fences stop the compiler from merging the phases.
    uint4 kf[KSTEPS];   // K fragments of the block about to be multiplied
    uint2 vf[DB][2][2]; // V^T fragments of the block about to be added: [channel block][16-key step][4+4 keys]

    auto load_kf = [&](const unsigned char *kl, int blk) __attribute__((always_inline)) {
        const unsigned char *krow = kl + (blk * 32 + i32) * KROW + h * 16;
#pragma unroll
        for (int st = 0; st < KSTEPS; ++st) kf[st] = *(const uint4 *)(krow + st * 32);
    };
    auto load_vf = [&](const unsigned char *vl, int blk) __attribute__((always_inline)) {
        // this lane's corner of the transposing reads: key row 4h + (lane%16)/4, channels
        // 16*((lane/16)%2) + 4*(lane%4) .. +3 of a 32-channel block
        const unsigned char *vrd = vl + (blk * 32 + 4 * h + ((lane & 15) >> 2)) * VROW + (((lane >> 4) & 1) * 16 + (lane & 3) * 4) * 2;
#pragma unroll
        for (int db = 0; db < DB; ++db)
#pragma unroll
            for (int ks = 0; ks < 2; ++ks) {
                vf[db][ks][0] = lds_read_tr16(vrd + (ks * 16) * VROW + db * 64);
                vf[db][ks][1] = lds_read_tr16(vrd + (ks * 16 + 8) * VROW + db * 64);
            }
    };
    auto mfma_qk = [&]() __attribute__((always_inline)) -> acc_t {
        acc_t s;
#pragma unroll
        for (int r = 0; r < 16; ++r) s[r] = 0;
#pragma unroll
        for (int st = 0; st < KSTEPS; ++st) {
            if constexpr (MODE == MODE_I8) {
                s = __builtin_amdgcn_mfma_i32_32x32x32_i8(__builtin_bit_cast(i32x4, kf[st]), __builtin_bit_cast(i32x4, qreg[st]), s, 0, 0, 0);
            } else if constexpr (MODE == MODE_FP8) {
                // same 16-byte fragments as int8; the FP8 instruction contracts 8 bytes per lane, so a
                // fragment is two steps (low halves, then high halves: any order Q and K agree on)
                s = __builtin_amdgcn_mfma_f32_32x32x16_fp8_fp8((long)(kf[st].x | ((uint64_t)kf[st].y << 32)),
                                                               (long)(qreg[st].x | ((uint64_t)qreg[st].y << 32)), s, 0, 0, 0);
                s = __builtin_amdgcn_mfma_f32_32x32x16_fp8_fp8((long)(kf[st].z | ((uint64_t)kf[st].w << 32)),
                                                               (long)(qreg[st].z | ((uint64_t)qreg[st].w << 32)), s, 0, 0, 0);
            } else {
                s = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, kf[st]), __builtin_bit_cast(bf16x8, qreg[st]), s, 0, 0, 0);
            }
        }
        return s;
    };
    auto mfma_pv = [&](const uint4 (&pb)[2]) __attribute__((always_inline)) {
#pragma unroll
        for (int db = 0; db < DB; ++db)
#pragma unroll
            for (int ks = 0; ks < 2; ++ks) {
                const uint4 a = make_uint4(vf[db][ks][0].x, vf[db][ks][0].y, vf[db][ks][1].x, vf[db][ks][1].y);
                oacc[db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a),
                                                                   __builtin_bit_cast(bf16x8, pb[ks]), oacc[db], 0, 0, 0);
            }
    };

    // GENERIC handles everything (additive mask, causal and key-length masking, per-key
    // scales); the other instantiation is for tiles in which no key is masked for this wave.
    auto tile_body = [&](auto generic_c, int it, auto &&mid_tile) __attribute__((always_inline)) {
        constexpr bool GENERIC = decltype(generic_c)::value;
        const int k0 = it * BK;
        const unsigned char *kl = lds + (it % NSTAGE) * STAGE;
        const unsigned char *vl = kl + K_TILE;
        float f_tile = 1.f;
        if (MODE != MODE_BF16 && !PER_KEY) f_tile = p.sk[(size_t)kv_bh * nkb + (it >> p.bk_tile_shift)];
        // online softmax of one 32-key block: raw accumulators in, probabilities (bf16, B-operand
        // layout) out; updates the running reference / sum and, rarely, rescales the accumulators
        auto softmax_block = [&](int blk, const acc_t &s, uint4 (&pb)[2]) __attribute__((always_inline)) {
            if (DBG) {
                if (bh == p.dbg_bh && (wq0 >> 5) == p.dbg_qt && it == p.dbg_kt) {
#pragma unroll
                    for (int r = 0; r < 16; ++r) p.dbg[i32 * 64 + blk * 32 + 8 * (r >> 2) + 4 * h + (r & 3)] = (int32_t)s[r];
                }
            }
            // The exponent reference m_run is lazy: it only moves when a row maximum outgrows it by
            // 2^LAZY_TAU (then the accumulators are rescaled).  Softmax does not depend on the
            // reference, so the result is the same function with almost no rescaling.
            float x[16];
            float rs;
            auto move_reference = [&](float mx) __attribute__((always_inline)) {
                const float m_new = fmaxf(m_run, mx);
                const float alpha = __builtin_amdgcn_exp2f(m_run - m_new);
                m_run = m_new;
                l_run *= alpha;
#pragma unroll
                for (int db = 0; db < DB; ++db)
#pragma unroll
                    for (int r = 0; r < 16; ++r) oacc[db][r] *= alpha;
            };
            auto row_sum = [&]() __attribute__((always_inline)) {
                // over the unrounded probabilities (src/runtime/cuda_flash_bf16.rs:365-377)
                float rs0 = (x[0] + x[1]) + (x[2] + x[3]), rs1 = (x[8] + x[9]) + (x[10] + x[11]);
                rs0 += (x[4] + x[5]) + (x[6] + x[7]);
                rs1 += (x[12] + x[13]) + (x[14] + x[15]);
                return rs0 + rs1;
            };
            if (!GENERIC) {
                // Unmasked block: exponentiate against the current reference straight away, the scale
                // folded into the exponent: s = (float)acc * ((sq * sk) * scale),
                // src/runtime/cuda_flash_sage.rs:315-322.  The row sum bounds the largest probability
                // (max <= sum <= 16 max), so only a sum that is too large (or not finite: the very first
                // block, or a jump of the maximum) sends the wave to the exact path below.
                if constexpr (PER_KEY) {
                    // one factor per key (the reference's own granularity, src/runtime/cuda_flash_sage.rs:264-268,
                    // 315-322): the tile's K scales sit in LDS, and element r of a lane is key
                    // 8 (r / 4) + 4 h + r % 4 of the block, so four 16-byte reads fetch the lane's sixteen
                    // (the query's part of the factor, (sq scale) log2 e, is a per-lane constant: one multiply per
                    // key instead of three; against (sq sk) scale the factor moves by two units in the last place)
                    float cr[16];
#pragma unroll
                    for (int g = 0; g < 4; ++g) {
                        const float4 sk4 = *(const float4 *)(vl + V_TILE + (blk * 32 + 8 * g + 4 * h) * 4);
                        cr[4 * g + 0] = sq_c * sk4.x;
                        cr[4 * g + 1] = sq_c * sk4.y;
                        cr[4 * g + 2] = sq_c * sk4.z;
                        cr[4 * g + 3] = sq_c * sk4.w;
                    }
#pragma unroll
                    for (int r = 0; r < 16; ++r) x[r] = __builtin_amdgcn_exp2f(__builtin_fmaf((float)s[r], cr[r], -m_run));
                    rs = row_sum();
                    if (__any(!(rs <= 16.0f * LAZY_LIMIT))) {
                        float y[16];
#pragma unroll
                        for (int r = 0; r < 16; ++r) y[r] = (float)s[r] * cr[r];
                        float mx = max3(y[0], y[1], y[2]);
#pragma unroll
                        for (int r = 3; r < 15; r += 2) mx = max3(mx, y[r], y[r + 1]);
                        mx = xhalf_max(fmaxf(mx, y[15]));
                        move_reference(mx);
#pragma unroll
                        for (int r = 0; r < 16; ++r) x[r] = __builtin_amdgcn_exp2f(__builtin_fmaf((float)s[r], cr[r], -m_run));
                        rs = row_sum();
                    }
                } else {
                const float c = (MODE != MODE_BF16) ? ((sq_lane * f_tile) * p.scale) * LOG2E : c_scale;
#pragma unroll
                for (int r = 0; r < 16; ++r) x[r] = __builtin_amdgcn_exp2f(__builtin_fmaf((float)s[r], c, -m_run));
                rs = row_sum();
                if (__any(!(rs <= 16.0f * LAZY_LIMIT))) {
                    // (s has been read by the vector instructions above, so max3 may take it as it is)
                    float mx = max3((float)s[0], (float)s[1], (float)s[2]);
#pragma unroll
                    for (int r = 3; r < 15; r += 2) mx = max3(mx, (float)s[r], (float)s[r + 1]);
                    mx = xhalf_max(fmaxf(mx, (float)s[15])) * c;
                    move_reference(mx);
#pragma unroll
                    for (int r = 0; r < 16; ++r) x[r] = __builtin_amdgcn_exp2f(__builtin_fmaf((float)s[r], c, -m_run));
                    rs = row_sum();
                }
                }
            } else {
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int kt = blk * 32 + 8 * (r >> 2) + 4 * h + (r & 3);  // key within the tile
                    const int key = k0 + kt;
                    float cc = c_scale;
                    if (MODE != MODE_BF16) {
                        const float skv = PER_KEY ? *(const float *)(vl + V_TILE + kt * 4) : f_tile;
                        cc = ((sq_lane * skv) * p.scale) * LOG2E;
                    }
                    float xv = (float)s[r] * cc;
                    if (HAS_MASK) {
                        if (key < N && q_row < N) xv += p.mask[(size_t)q_row * N + key] * LOG2E;
                    }
                    if (key >= kend || (CAUSAL && key > q_row)) xv = NEG_SENTINEL;
                    x[r] = xv;
                }
                float mx = max3(x[0], x[1], x[2]);
#pragma unroll
                for (int r = 3; r < 15; r += 2) mx = max3(mx, x[r], x[r + 1]);
                mx = xhalf_max(fmaxf(mx, x[15]));
                if (__any(mx > m_run + LAZY_TAU)) move_reference(mx);
#pragma unroll
                for (int r = 0; r < 16; ++r) x[r] = __builtin_amdgcn_exp2f(x[r] - m_run);
                rs = row_sum();
            }
            l_run += rs;
#pragma unroll
            for (int ks = 0; ks < 2; ++ks) {
                pb[ks].x = pack_bf16x2(x[ks * 8 + 0], x[ks * 8 + 1]);
                pb[ks].y = pack_bf16x2(x[ks * 8 + 2], x[ks * 8 + 3]);
                pb[ks].z = pack_bf16x2(x[ks * 8 + 4], x[ks * 8 + 5]);
                pb[ks].w = pack_bf16x2(x[ks * 8 + 6], x[ks * 8 + 7]);
            }
        };

        load_kf(kl, 0);
#pragma unroll
        for (int blk = 0; blk < 2; ++blk) {
            // a second block whose keys are all hidden from every query of the wave (past the key length,
            // or above the causal diagonal) contributes exact zeros and leaves the reference alone
            if (GENERIC && blk == 1 && (k0 + 32 >= kend || (CAUSAL && k0 + 32 > wq0 + 31))) break;
            uint4 pb[2];
            // ---- P1 ----
            load_vf(vl, blk);
            acc_t s = mfma_qk();
            ARHIP_FENCE();
            // ---- P2 ----
            softmax_block(blk, s, pb);
            ARHIP_FENCE();
            // ---- P3 ----
            if (blk == 0) load_kf(kl, 1);
            mfma_pv(pb);
            ARHIP_FENCE();
            if (blk == 0) {
                mid_tile();  // staging of the tiles ahead, issued while the matrix pipe has work queued
                ARHIP_FENCE();
            }
        }
    };

    // Staging runs two tiles ahead of the math with one set of registers: in the middle of the
    // iteration that computes tile i, tile i+1 (loaded during iteration i-1) goes from registers
    // to the LDS stage that tile i-1 vacated at the last barrier, and the loads of tile i+2 are
    // issued; they have a whole iteration to land before anybody waits for them.
    if (ntiles > 0) {
        load_tile(0);
        store_tile(0);
    }
    if (ntiles > 1) load_tile(BK);
    __syncthreads();
    auto nothing = [] {};

    if constexpr (!CAUSAL && !HAS_MASK) {
        // only the last tile can hold masked keys: keep it out of the loop
        const int nfull = kend / BK;
#pragma clang loop unroll(disable)
        for (int it = 0; it < nfull; ++it) {
            auto stage_ahead = [&]() __attribute__((always_inline)) {
                if (it + 1 < ntiles) store_tile((it + 1) % NSTAGE);
                if (it + 2 < ntiles) load_tile((it + 2) * BK);
            };
            tile_body(std::false_type{}, it, stage_ahead);
            __syncthreads();
        }
        if (nfull < ntiles) tile_body(std::true_type{}, nfull, nothing);
    } else {
#pragma clang loop unroll(disable)
        for (int it = 0; it < ntiles; ++it) {
            auto stage_ahead = [&]() __attribute__((always_inline)) {
                if (it + 1 < ntiles) store_tile((it + 1) % NSTAGE);
                if (it + 2 < ntiles) load_tile((it + 2) * BK);
            };
            if (it < my_tiles) {
                const int k0 = it * BK;
                const bool masked = (k0 + BK > kend) || (CAUSAL && (k0 + BK - 1 > wq0));
                if (HAS_MASK || masked) tile_body(std::true_type{}, it, stage_ahead);
                else tile_body(std::false_type{}, it, stage_ahead);
            } else {
                stage_ahead();
            }
            __syncthreads();
        }
    }

    // ---- normalise and store: acc * (l > 0 ? 1/l : 0), cuda_flash_bf16.rs:414-426 ----
    const float l_tot = xhalf_sum(l_run);
    const float inv = (l_tot > 0.f) ? 1.f / l_tot : 0.f;
    if (p.lse != nullptr && h == 0 && q_row < N) {
        // LSE = m + log(l) in natural units (src/runtime/cuda_flash_train.rs:141); m_run is kept in
        // the exp2 domain, so LSE = (m_run + log2 l) * ln 2
        p.lse[(size_t)bh * N + q_row] = (l_tot > 0.f) ? (m_run + __builtin_amdgcn_logf(l_tot)) * 0.6931471805599453f : NEG_SENTINEL;
    }
    if (q_row < N) {
        const size_t obase =(size_t)b * p.os[0] + (size_t)head * p.os[1] + (size_t)q_row * p.os[2];
#pragma unroll
        for (int db = 0; db < DB; ++db)
#pragma unroll
            for (int gg = 0; gg < 4; ++gg) {
                const int d = db * 32 + 8 * gg + 4 * h;
                const float o0 = oacc[db][4 * gg + 0] * inv, o1 = oacc[db][4 * gg + 1] * inv;
                const float o2 = oacc[db][4 * gg + 2] * inv, o3 = oacc[db][4 * gg + 3] * inv;
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

template <int D, int NW, bool CAUSAL, bool HAS_MASK, int MODE, bool PER_KEY, bool OUT_F32, bool DBG>
__global__ void __launch_bounds__(NW * 64, (NW == 4 ? 2 : 1)) attn_fwd_kernel(const AttnParams p)
{
    __shared__ __attribute__((aligned(16))) unsigned char lds[attn_fwd_lds_bytes<D, NW, MODE, PER_KEY>()];
    attn_fwd_body<D, NW, CAUSAL, HAS_MASK, MODE, PER_KEY, OUT_F32, DBG>(p, lds, (int)blockIdx.x);
}

}  // namespace arhip
