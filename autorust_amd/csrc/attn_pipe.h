// Fused attention forward on gfx950: the software-pipelined kernel, which serves every launch without an
// additive mask or the logits export (attn_fwd_kernel, attn_fwd.h, keeps those), bf16, int8 and FP8 E4M3
// operands, K scales over whole 64-key tiles or per key (PER_KEY), the Q quantiser of the int8 path inside its
// prologue on request (QFUSE).  Same arithmetic and MFMA decomposition as attn_fwd_kernel (S^T = K . Q^T, one
// query per lane, O^T += V^T . P^T), different plumbing:
//
//   HBM -> LDS   K and V tiles of 64 keys go straight to LDS (buffer_load ... lds, 16 bytes per
//                lane, no registers in between), four stages deep, so a tile is requested three
//                iterations before the one that computes on it (two before the look-ahead
//                first touches it).  Rows past the last visible key come back as
//                zeros from the buffer bounds check; nothing is clamped or branched on.
//   LDS layout   A transfer writes 64 x 16 bytes to consecutive addresses, so rows cannot be padded.
//                Rows are cut into 64-byte pieces and stored [piece][row][64 B]; inside a block of
//                16 rows the four 16-byte chunks of a row are permuted with chunk ^= (row / 4) % 4.
//                The permutation is applied to the SOURCE address a lane fetches, and the operand
//                reads (ds_read_b128 for K, ds_read_b64_tr_b16 for V^T) then hit 16 distinct
//                16-byte bank groups per 16 lanes.
//   wave stream  A wave issues in order, and a matrix instruction keeps the matrix pipe busy for
//                8 passes during which the wave may issue independent vector instructions.  The
//                instruction stream therefore interleaves the two pipes itself, one 32-key block
//                ahead:
//                  R1(j)  S(j+1) = K(j+1) . Q^T    (MFMA)  |  second part of the softmax of S(j)  (VALU)
//                  R2(j)  O^T += V(j)^T . P(j)^T   (MFMA)  |  first part of the softmax of S(j+1)
//                softmax = exp2(S c - m), row sum, bf16 pack, dealt out one instruction at a time
//                Every fragment register is refilled right after the MFMA that read it: K(j+2)
//                behind the S^T MFMAs of R1(j), V(j+1) behind the O^T MFMAs of R2(j).
//                Carried from block to block: the logits S(j) with their softmax half done, the
//                K(j+1) and V(j) fragments.
//   reference    lazy exponent reference as in attn_fwd.h; it is checked between R1 and R2 (the
//                rare case recomputes the block's logits from K, which is still in LDS).
//   masked tiles (causal diagonal, key-length edge) run the same pipeline with the mask applied inside
//                the softmax instructions; a wave past its last query only keeps feeding the
//                transfers and barriers.
//
// 8 waves of 32 queries per workgroup, two waves per SIMD.
//
// NW = 4 is the variant for launches whose workgroups see few tiles (short or causal sequences): 128
// queries per workgroup and at most 80 KB of LDS, so that a compute unit holds two workgroups and one's
// prologue and epilogue (first transfers, output store, the gap to the next workgroup) run under the
// other's tiles.  K and V then live in rings of their own (attn_pipe_rings), K two tiles deep and V three: while tile t is
// computed the wave reads K(t+1), V(t) and V(t+1) from LDS (K(t) went into registers during tile t-1),
// and tile t+2 is on its way.  The rare reference move takes the block's logits from their registers
// instead of recomputing them from K(t), which this ring no longer holds.
#pragma once

#include "attn_fwd.h"

// 1: the int8 pipeline reads its int32 logit accumulators as biased floats (no conversions)
#ifndef ARHIP_PIPE_INT_BIAS
#define ARHIP_PIPE_INT_BIAS 1
#endif

namespace arhip {

typedef __attribute__((address_space(3))) void *lds_ptr_t;

// s_waitcnt vmcnt(n) only (gfx9 encoding: vmcnt[3:0] | expcnt[6:4] | lgkmcnt[11:8] | vmcnt[5:4] << 14)
template <int N>
__device__ __forceinline__ void wait_vmem_le()
{
    __builtin_amdgcn_s_waitcnt((N & 15) | ((N >> 4) << 14) | (7 << 4) | (15 << 8));
}

// f(integral_constant<int, A>) ... f(integral_constant<int, B - 1>), unrolled at compile time
template <int A, int B, typename F>
__device__ __forceinline__ void static_for(F &&f)
{
    if constexpr (A < B) {
        f(std::integral_constant<int, A>{});
        static_for<A + 1, B>(f);
    }
}

// The 4-wave form keeps K and V in rings of their own (two and three tiles) so that two workgroups fit a compute
// unit at D = 128; with 8-bit operands at D = 64 four whole stages fit twice as well (48 KB each), and with them the
// four-tiles-per-trip loop and one more tile of latency cover: int8 B4 H32 N = 2048 / 8192 -7 / -5 %, causal -4 / -5 %,
// per-key scales -7 / -5 %, B8 H6 N789 -4 %, same bits (bf16 at D = 64 gains nothing and loses 6 % on short causal shapes).
template <int D, int MODE, int NW>
constexpr bool attn_pipe_rings()
{
    return NW == 4 && !(D == 64 && MODE != MODE_BF16);
}

// LDS bytes attn_pipe_body needs: [piece][64 rows][64 B] K and V tiles, four stages of both, or a
// ring of two K tiles and one of three V tiles (attn_pipe_rings).  PER_KEY (a scale per key, or per block of fewer than
// 64 keys): behind the tiles, a ring of four times 64 raw key scales and, per wave, two times 64 pairs of
// derived factors.
// QFUSE (Q is quantised in the prologue): with scales over blocks of 128 queries, 256 bytes for the exchange of the
// waves' maxima.
template <int D, int MODE, int NW = 8, bool PER_KEY = false, bool QFUSE = false>
constexpr int attn_pipe_lds_bytes()
{
    constexpr bool R = attn_pipe_rings<D, MODE, NW>();
    return 4096 * ((R ? 2 : 4) * (D * ((MODE != MODE_BF16) ? 1 : 2) / 64) + (R ? 3 : 4) * (D * 2 / 64)) +
           (PER_KEY ? 1024 + NW * 1024 : 0) + ((QFUSE && !PER_KEY) ? 256 : 0);
}

// workgroup index -> (batch * heads + head, query tile of 256), as in attn_fwd_kernel
template <bool CAUSAL>
__device__ __forceinline__ void pipe_work_item(const AttnParams &p, int wg, int &bh, int &qt)
{
    if (CAUSAL && p.lpt) {
        const int nbh = p.total / p.nq;
        qt = p.nq - 1 - wg / nbh;
        bh = wg % nbh;
    } else {
        if ((p.total & 7) == 0) wg = (wg & 7) * (p.total >> 3) + (wg >> 3);
        bh = wg / p.nq;
        qt = wg - bh * p.nq;
        if (CAUSAL) qt = p.nq - 1 - qt;
    }
}

// The kernel body.  lds: attn_pipe_lds_bytes<D, MODE>() bytes of workgroup memory, 1024-byte
// aligned; wg_linear: this workgroup's index in [0, p.total).  BIAS (int8 only): see s_init below.
// QFUSE (int8, FP8): the prologue is the quantiser of sage_quant_kernels.h for this workgroup's queries, operation for
// operation (absmax, scale = absmax / 127 or 1, x8 = clamp(rint(x * (1 / scale)), +-127); FP8: absmax / 448 and the
// saturating E4M3 conversion of x * (1 / scale)), so the result is bit for bit
// that of quantising first; p.sq_out / p.q8_out, where not null, receive the scales and the codes.  Two forms: with K
// scales over whole tiles, p.q holds bf16 values and a scale covers a block of 128 queries; with PER_KEY, p.q holds
// f32 values and every query has its own scale (the reference's convention, src/runtime/cuda_flash_sage.rs:201-223).
template <int D, bool CAUSAL, int MODE, bool OUT_F32, bool BIAS, int NW = 8, bool PER_KEY = false, bool QFUSE = false>
__device__ __forceinline__ void attn_pipe_impl(const AttnParams &p, unsigned char *lds, int wg_linear)
{
    static_assert(!QFUSE || MODE != MODE_BF16, "the fused Q quantiser produces 8-bit operands");
    static_assert(!QFUSE || BIAS || MODE == MODE_FP8, "int8 with the fused Q quantiser runs on biased logits");
    static_assert(!(QFUSE && PER_KEY && MODE == MODE_FP8), "rows form: int8 only");
    constexpr bool QROWS = QFUSE && PER_KEY;  // f32 queries, a scale per query
    static_assert(!BIAS || MODE == MODE_I8, "biased accumulators are an int8 device");
    static_assert(!PER_KEY || BIAS || MODE == MODE_FP8, "per-key scales: int8 (on the biased accumulators) and FP8");
    static_assert(NW == 8 || NW == 4, "8 waves (one workgroup per CU) or 4 (two)");
    constexpr bool RINGS = attn_pipe_rings<D, MODE, NW>();  // K and V in rings of their own, two and three tiles deep
    constexpr int BQ = NW * 32;
    constexpr int QK_BYTES = (MODE != MODE_BF16) ? 1 : 2;
    constexpr int KP = D * QK_BYTES / 64;  // 64-byte pieces per K row
    constexpr int VP = D * 2 / 64;         // 64-byte pieces per V row
    constexpr int K_TILE = KP * 4096;      // [piece][64 rows][64 B]
    constexpr int V_TILE = VP * 4096;
    constexpr int STAGE = K_TILE + V_TILE;
    constexpr int NSTAGE = 4;
    constexpr int AHEAD = RINGS ? 2 : 3;          // a tile is requested this many iterations before the one that computes on it
    constexpr int LDS_BYTES = attn_pipe_lds_bytes<D, MODE, NW>();  // the tiles (PER_KEY: the scale areas follow)
    constexpr int SK_RAW = LDS_BYTES;          // PER_KEY: [4][64] raw scales of the tiles in flight
    constexpr int SK_OWN = LDS_BYTES + 1024;   // PER_KEY: [wave][2][2][64] factors of the current and the next tile
    constexpr int QF_RED = LDS_BYTES;          // QFUSE: [wave] largest |q| of the wave's 32 queries
    constexpr int XFERS = (KP + VP) * 4;          // 1 KB transfers per tile
    constexpr int XPW = (XFERS + NW - 1) / NW;    // at most this many per wave
    constexpr int XPW_MIN = XFERS / NW;           // at least this many per wave
    constexpr int KSTEPS = (MODE != MODE_BF16) ? D / 32 : D / 16;
    constexpr int DB = D / 32;
    static_assert(KP >= 1 && XFERS >= NW, "tile too small for 8 waves");

    static_assert(RINGS ? (2 * K_TILE + 3 * V_TILE == LDS_BYTES) : (NSTAGE * STAGE == LDS_BYTES), "LDS size bookkeeping");
    // where the K and the V part of tile t live (byte offsets into lds)
    auto k_base = [](int t) __attribute__((always_inline)) -> int { return RINGS ? (t & 1) * K_TILE : (t & 3) * STAGE; };
    auto v_base = [](int t) __attribute__((always_inline)) -> int {
        return RINGS ? 2 * K_TILE + (t % 3) * V_TILE : (t & 3) * STAGE + K_TILE;
    };

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int i32 = lane & 31;
    const int h = lane >> 5;

    int bh, qt;
    pipe_work_item<CAUSAL>(p, wg_linear, bh, qt);
    const int b = bh / p.Hq;
    const int head = bh - b * p.Hq;
    const int kvh = head / (p.Hq / p.Hkv);
    const int kv_bh = b * p.Hkv + kvh;
    const int N = p.N;
    const int qblk = qt * BQ;
    const int wq0 = qblk + wave * 32;
    const int q_row = wq0 + i32;

    int kvl = N;
    if (p.kv_len) {
        kvl = p.kv_len[b];
        kvl = kvl < 0 ? 0 : (kvl > N ? N : kvl);
    }
    int kend = kvl;
    if (CAUSAL) kend = min(kend, min(N, qblk + BQ));
    const int ntiles = (kend + BK - 1) / BK;
    // key `key` is masked for this lane's query iff key > min(q_row, kend - 1) (causal) or
    // key > kend - 1.  Element r of a block whose first key is kb0 is key kb0 + 4 h + 8 (r / 4) + r % 4,
    // so with rel = lim4h - kb0 the test is 8 (r / 4) + r % 4 > rel.
    const int lim4h = (CAUSAL ? min(q_row, kend - 1) : kend - 1) - 4 * h;

    // ---- buffer resources over this head's K and V: offsets past kend rows read as zero ----
    const size_t kv_off = (size_t)b * p.ks[0] + (size_t)kvh * p.ks[1];
    const uint32_t k_rowb = (uint32_t)p.ks[2] * QK_BYTES;  // bytes between consecutive keys
    const uint32_t v_rowb = (uint32_t)p.vs[2] * 2;
    // raw buffer descriptor: base address, stride 0, size in bytes, 32-bit untyped data
    auto make_rsrc = [](const void *base, uint32_t bytes) __attribute__((always_inline)) -> i32x4 {
        const uint64_t a = (uint64_t)(uintptr_t)base;
        i32x4 r;
        r[0] = __builtin_amdgcn_readfirstlane((int)(uint32_t)a);
        r[1] = __builtin_amdgcn_readfirstlane((int)(uint32_t)(a >> 32) & 0xffff);
        r[2] = __builtin_amdgcn_readfirstlane((int)bytes);
        r[3] = 0x00020000;
        return r;
    };
    const i32x4 k_rsrc = make_rsrc((const unsigned char *)p.k + kv_off * QK_BYTES, (uint32_t)kend * k_rowb);
    const i32x4 v_rsrc = make_rsrc(p.v + (size_t)b * p.vs[0] + (size_t)kvh * p.vs[1], (uint32_t)kend * v_rowb);
    // PER_KEY: this head's key scales, one per block of 1 << bk_key_shift keys
    i32x4 sk_rsrc = k_rsrc;
    if constexpr (PER_KEY) {
        const int nkeyb = (N + p.bk - 1) >> p.bk_key_shift;
        sk_rsrc = make_rsrc(p.sk + (size_t)kv_bh * nkeyb, (uint32_t)nkeyb * 4);
    }

    // transfer x of a tile (x = wave + 8 j): rows 16 g .. 16 g + 15 of piece pc of K (x < 4 KP) or V;
    // lane l fetches row 16 g + l / 4, chunk (l % 4) ^ ((l / 16) % 4) of that piece
    uint32_t xoff[XPW];
#pragma unroll
    for (int j = 0; j < XPW; ++j) {
        const int x = wave + NW * j;
        const bool is_k = x < KP * 4;
        const int xl = is_k ? x : x - KP * 4;
        const int pc = xl >> 2, g = xl & 3;
        const int r = lane >> 2;
        const int c = (lane & 3) ^ ((r >> 2) & 3);
        xoff[j] = (uint32_t)(16 * g + r) * (is_k ? k_rowb : v_rowb) + pc * 64 + c * 16;
    }
    // The transfers are written as inline assembly on purpose: the compiler makes every LDS read
    // wait for all outstanding transfers it knows of (it cannot tell the stages apart), which
    // would put the whole memory latency in front of every tile.  Here the waits are explicit
    // (wait_vmem_le before the barrier that publishes a tile).  m0 holds the LDS destination; one
    // wait state is required between writing m0 and the transfer, and five between a vector
    // instruction writing a scalar register (v_readfirstlane of the descriptors, a scalar register
    // reloaded from a spill lane) and a memory instruction reading it: the compiler pads neither
    // for inline assembly, so the assembly carries the wait states itself (s_mov + s_nop 3).
    auto issue_tile = [&](int tile) __attribute__((always_inline)) {
        // RINGS waits for everything in flight at the end of every tile: a transfer past the last tile (which would
        // deliver zeros) is a memory round trip the last two tiles of a workgroup would wait for
        if (RINGS && tile >= ntiles) return;
        const uint32_t lds0 = (uint32_t)(uintptr_t)(lds_ptr_t)lds;
        const uint32_t dst_k = lds0 + k_base(tile), dst_v = lds0 + v_base(tile);
        if constexpr (PER_KEY) {
            // the scales of the tile's 64 keys, 4 bytes per lane, by one wave; first, so that a wait that leaves
            // the newest XPW_MIN transfers of a wave in flight covers it as it covers the tile before
            if (wave == 0) {
                const uint32_t off = (uint32_t)((tile * BK + lane) >> p.bk_key_shift) * 4;
                asm volatile("s_mov_b32 m0, %0\n\ts_nop 3\n\tbuffer_load_dword %1, %2, 0 offen lds"
                             :
                             : "s"(lds0 + SK_RAW + (RINGS ? tile % 3 : tile & 3) * 256), "v"(off), "s"(sk_rsrc)
                             : "memory", "m0");
            }
        }
#pragma unroll
        for (int j = 0; j < XPW; ++j) {
            const int x = wave + NW * j;
            if (XFERS % NW == 0 || x < XFERS) {
                // the tile offset goes into the per-lane offset: the scalar offset operand of a
                // buffer access is not covered by the bounds check
                const bool is_k = x < KP * 4;
                const uint32_t off = xoff[j] + (uint32_t)tile * BK * (is_k ? k_rowb : v_rowb);
                const i32x4 rsrc = is_k ? k_rsrc : v_rsrc;
                asm volatile("s_mov_b32 m0, %0\n\ts_nop 3\n\tbuffer_load_dwordx4 %1, %2, 0 offen lds"
                             :
                             : "s"(is_k ? dst_k + x * 1024 : dst_v + (x - KP * 4) * 1024), "v"(off), "s"(rsrc)
                             : "memory", "m0");
            }
        }
    };

    uint4 qreg[KSTEPS];  // Q operand (loaded in the prologue below)

    // ---- LDS operand addresses (relative to a stage) ----
    // K fragment of step st: row 32 blk + i32, bytes 32 st + 16 h .. +15, i.e. piece st / 2, chunk
    // 2 (st % 2) + h, stored at chunk position (2 (st % 2) + h) ^ ((i32 / 4) % 4)
    const int k_t = h ^ ((i32 >> 2) & 3);
    const int k_row = (i32 & 15) * 64 + (i32 >> 4) * 1024;
    const int k_addr[2] = {k_row + k_t * 16, k_row + (k_t ^ 2) * 16};
    // V^T fragment: this lane's corner of the transposing reads is key row 4 h + (lane % 16) / 4
    // (+ 8 for the second read), channels 16 ((lane / 16) % 2) + 4 (lane % 4) .. + 3 of a 32-channel
    // block, i.e. chunk 2 ((lane / 16) % 2) + (lane % 4) / 2, byte 8 (lane % 2) inside it
    const int v_r0 = 4 * h + ((lane & 15) >> 2);
    const int v_c = ((lane >> 4) & 1) * 2 + ((lane & 3) >> 1);
    const int v_addr[2] = {v_r0 * 64 + (v_c ^ h) * 16 + (lane & 1) * 8,
                           (v_r0 + 8) * 64 + (v_c ^ (h + 2)) * 16 + (lane & 1) * 8};
    // The offset field of an LDS read has 16 bits and the four stages of the 8-wave form span 96 KB: where the
    // stage of a tile is a compile-time constant (the four-tiles-per-trip loop), reads of stages 2 and 3 go
    // through a second set of address registers that already contain 2 STAGE, so that what is left fits the
    // field and no read needs an address computation of its own: 10 vector instructions fewer per tile, Sage
    // B4 H32 S8192 -2 %.  (The compiler would rebuild a register it can derive from the first set, hence the
    // empty assembly.)
    constexpr int HI_BASE = 2 * STAGE;
    int k_addr_hi[2] = {k_addr[0] + HI_BASE, k_addr[1] + HI_BASE};
    int v_addr_hi[2] = {v_addr[0] + HI_BASE, v_addr[1] + HI_BASE};
    asm("" : "+v"(k_addr_hi[0]), "+v"(k_addr_hi[1]), "+v"(v_addr_hi[0]), "+v"(v_addr_hi[1]));

    typedef typename std::conditional<MODE == MODE_I8, i32x16, f32x16>::type acc_t;
    f32x16 oacc[DB];
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int r = 0; r < 16; ++r) oacc[db][r] = 0.f;
    float m_run = NEG_SENTINEL;
    float l_run = 0.f;
    // int8: the int32 accumulators start at 0x4B400000, the bit pattern of the float 12582912 = 1.5 * 2^23,
    // whose unit in the last place is 1: with |sum| <= 128 * 128^2 = 2^21 < 2^22 the accumulator's bits,
    // read as a float, ARE the value 12582912 + sum, so no int -> float conversion is needed; the softmax
    // subtracts m_bias = m_run + 12582912 c instead of m_run (one fused multiply-add per block), and
    // fma(12582912 + sum, c, -m_bias) rounds the same real number sum c - m_run as
    // fma((float)sum, c, -m_run) does PROVIDED m_bias is exact.  Two things make it exact: c is
    // rounded to 21 significant bits (so that 12582912 c = 3 c 2^22 has at most 23), and m_run only
    // ever takes multiples of m_grid, a power of two that no unit in the last place of any
    // 12582912 c + m_run this workgroup can meet exceeds (the prologue derives it from the largest
    // scales).  Where m_run outweighs 12582912 c (tiny scales) the sum may still round, by at most
    // half a unit in the last place of m_run: 2^-16 for references below 256.
    constexpr float BIAS_F = 12582912.0f;
    acc_t s_init;
#pragma unroll
    for (int r = 0; r < 16; ++r) s_init[r] = 0;
    if constexpr (BIAS) {
#pragma unroll
        for (int r = 0; r < 16; ++r) s_init[r] = 0x4B400000;
        asm volatile("" : "+v"(s_init));  // a register block of its own: the matrix instruction's C operand
    }
    float m_bias = NEG_SENTINEL;  // what the pipelined softmax subtracts for the block it works on
    auto set_bias = [&](float c) __attribute__((always_inline)) {
        m_bias = (BIAS && !PER_KEY) ? __builtin_fmaf(BIAS_F, c, m_run) : m_run;
    };
    float m_grid = 1.0f, m_grid_inv = 1.0f;  // set in the prologue (BIAS only)
    // a logit accumulator as a float (before the factor c)
    auto as_logit = [&](const acc_t &a, int r) __attribute__((always_inline)) -> float {
        if constexpr (BIAS) return __builtin_bit_cast(float, (int)a[r]);
        else return (float)a[r];
    };
    float sq_lane = 1.f;
    const int nkb = (MODE != MODE_BF16) ? (N + p.bk - 1) / p.bk : 0;
    if (MODE != MODE_BF16 && !QFUSE) {
        const int nqb = (N + p.bq - 1) / p.bq;
        sq_lane = p.sq[(size_t)bh * nqb + min(q_row, N - 1) / p.bq];
    }
    const float c_scale = p.scale * LOG2E;
    const int last_tile = (N - 1) / BK;
    // int8: the K scales of 64 consecutive tiles sit in one register (lane l holds tile 64 g + l),
    // for the current group of tiles and the next one; a tile's scale is then a v_readlane away.
    // (A scalar load per tile would share its counter with the LDS reads and, returning out of
    // order, force every LDS wait in the loop down to "everything has returned".)
    float skv_cur = 1.f, skv_nxt = 1.f;
    auto load_sk_group = [&](int g) __attribute__((always_inline)) -> float {
        const int t = min(g * 64 + lane, last_tile);
        return p.sk[(size_t)kv_bh * nkb + (t >> p.bk_tile_shift)];
    };
    // exponent factor of the keys of tile t (in the group of tile `it` or the next one): scale log2(e),
    // times sq sk for int8 (s = (float)acc * ((sq * sk) * scale), src/runtime/cuda_flash_sage.rs:315-322)
    // PER_KEY: the keys' own scales are applied per logit (see convert_sk); what is left is the lane's factor
    float sq_c = (sq_lane * p.scale) * LOG2E;  // (QFUSE: set again once the prologue has the scale)
    auto tile_c = [&](int t, int it) __attribute__((always_inline)) -> float {
        if constexpr (PER_KEY) {
            return sq_c;
        } else if constexpr (MODE != MODE_BF16) {
            const int a = __builtin_amdgcn_readlane(__float_as_int(skv_cur), t & 63);
            const int bnext = __builtin_amdgcn_readlane(__float_as_int(skv_nxt), t & 63);
            const float f = __int_as_float(((t >> 6) == (it >> 6)) ? a : bnext);
            const float c = ((sq_lane * f) * p.scale) * LOG2E;
            // BIAS: to 21 significant bits, round to nearest (a relative change of at most 2^-21)
            return BIAS ? __uint_as_float((__float_as_uint(c) + 4u) & ~7u) : c;
        } else {
            return c_scale;
        }
    };
    // called at the top of iteration it: moves to the next group of 64 tiles when it begins.  The
    // wait makes the new vector's arrival explicit (once per 64 tiles) so that no wait for it is
    // left at its uses.
    auto advance_sk_group = [&](int it) __attribute__((always_inline)) {
        if constexpr (MODE != MODE_BF16 && !PER_KEY) {
            if ((it & 63) == 0 && it > 0) {
                skv_cur = skv_nxt;
                skv_nxt = load_sk_group((it >> 6) + 1);
                wait_vmem_le<0>();
            }
        }
    };

    // PER_KEY.  A logit is acc sk_j (sq_i scale log2 e) - m.  The accumulator, read as a float, is 12582912 + acc, so
    //   t = fma(12582912 + acc, ck_j, -12582912 ck_j)    (exactly fl(acc ck_j): ck_j is sk_j cut to 21 bits, so the
    //                                                      second product is exact and the fma rounds once)
    //   x = fma(t, sq_c, -m)
    // costs one instruction per logit more than a per-tile scale, provided ck_j and -12582912 ck_j come from
    // somewhere: every wave derives them from the raw scales of a tile (lane = key) one tile ahead, into its own
    // two slots of LDS (no other wave reads them, LDS operations of a wave complete in order: no barrier), and
    // reads them back four keys at a time in the order its lanes hold the logits.
    float *const sk_own = (float *)(lds + SK_OWN + wave * 1024);
    auto convert_sk = [&](int tile) __attribute__((always_inline)) {
        if constexpr (PER_KEY) {
            const float raw = *(const float *)(lds + SK_RAW + (RINGS ? tile % 3 : tile & 3) * 256 + lane * 4);
            // (FP8: fp32 accumulators, t = acc sk_j needs neither the cut nor the bias product)
            const float ck = BIAS ? __uint_as_float((__float_as_uint(raw) + 4u) & ~7u) : raw;
            float *dst = sk_own + (tile & 1) * 128;
            dst[lane] = ck;
            if constexpr (BIAS) dst[64 + lane] = -BIAS_F * ck;
        }
    };
    // factors of block blk of tile t as this lane's registers want them: keys 4 h + 8 G .. + 3 at [8 G], their
    // negated bias products 64 floats further on
    auto key_factors = [&](int t, int blk) __attribute__((always_inline)) -> const float * {
        return PER_KEY ? sk_own + (t & 1) * 128 + blk * 32 + 4 * h : nullptr;
    };
    float kc[8], kn[8];  // ck_j and -12582912 ck_j of the half block the softmax list works on next
    auto load_factors = [&](const float *kp, int G, int part) __attribute__((always_inline)) {
        // part 0 / 1: ck of group G / G + 1 into kc[0..3] / kc[4..7]; 2 / 3: their bias products into kn likewise
        const float4 v = *(const float4 *)(kp + (part >= 2 ? 64 : 0) + 8 * (G + (part & 1)));
        float *d = (part >= 2 ? kn : kc) + 4 * (part & 1);
        d[0] = v.x; d[1] = v.y; d[2] = v.z; d[3] = v.w;
    };

    uint4 kf[KSTEPS];
    uint2 vf[DB][2][2];
    auto load_kf = [&](const unsigned char *st, int blk) __attribute__((always_inline)) {
#pragma unroll
        for (int s = 0; s < KSTEPS; ++s)
            kf[s] = *(const uint4 *)(st + k_addr[s & 1] + (s >> 1) * 4096 + blk * 2048);
    };
    auto load_vf = [&](const unsigned char *st, int blk) __attribute__((always_inline)) {
#pragma unroll
        for (int db = 0; db < DB; ++db)
#pragma unroll
            for (int ks = 0; ks < 2; ++ks) {
                vf[db][ks][0] = lds_read_tr16(st + v_addr[0] + db * 4096 + (blk * 2 + ks) * 1024);
                vf[db][ks][1] = lds_read_tr16(st + v_addr[1] + db * 4096 + (blk * 2 + ks) * 1024);
            }
    };
    // One step of S^T += K-fragment . Q-fragment.  int8: v_mfma_i32_32x32x32_i8 on the 16-byte
    // fragments of step st.  FP8 (E4M3): the same fragments, two steps at a time, on
    // v_mfma_f32_32x32x64_f8f6f4 (32 bytes per lane, the int8 rate): the call for an even step does
    // nothing, the call for the odd step multiplies the fragments of both (the contraction order is
    // free as long as Q and K agree).  bf16: v_mfma_f32_32x32x16_bf16.
    auto qk_step = [&](auto si, acc_t &acc, const uint4 &a_prev, const uint4 &a, const uint4 &b_prev, const uint4 &b)
                       __attribute__((always_inline)) {
        constexpr int st = decltype(si)::value;
        if constexpr (MODE == MODE_I8) {
            acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(__builtin_bit_cast(i32x4, a), __builtin_bit_cast(i32x4, b), acc, 0, 0, 0);
        } else if constexpr (MODE == MODE_FP8) {
            if constexpr (st % 2 == 1) {
                typedef __attribute__((ext_vector_type(8))) int i32x8;
                const i32x8 av = {(int)a_prev.x, (int)a_prev.y, (int)a_prev.z, (int)a_prev.w, (int)a.x, (int)a.y, (int)a.z, (int)a.w};
                const i32x8 bv = {(int)b_prev.x, (int)b_prev.y, (int)b_prev.z, (int)b_prev.w, (int)b.x, (int)b.y, (int)b.z, (int)b.w};
                acc = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(av, bv, acc, 0, 0, 0, 0, 0, 0);
            }
        } else {
            acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), acc, 0, 0, 0);
        }
    };
    static_assert(MODE != MODE_FP8 || KSTEPS % 2 == 0, "FP8 steps come in pairs");
    auto mfma_qk = [&]() __attribute__((always_inline)) -> acc_t {
        acc_t s = s_init;
        static_for<0, KSTEPS>([&](auto si) __attribute__((always_inline)) {
            constexpr int st = decltype(si)::value;
            constexpr int pv = st > 0 ? st - 1 : 0;
            qk_step(si, s, kf[pv], kf[st], qreg[pv], qreg[st]);
        });
        return s;
    };
    auto move_reference = [&](float mx) __attribute__((always_inline)) {
        float m_new = fmaxf(m_run, mx);
        // BIAS: up to the next multiple of m_grid (softmax does not depend on the reference; a row
        // with no visible key yet keeps the sentinel)
        if (BIAS && !PER_KEY && m_new > -1e29f) m_new = __builtin_ceilf(m_new * m_grid_inv) * m_grid;
        const float alpha = __builtin_amdgcn_exp2f(m_run - m_new);
        m_run = m_new;
        l_run *= alpha;
#pragma unroll
        for (int db = 0; db < DB; ++db)
#pragma unroll
            for (int r = 0; r < 16; ++r) oacc[db][r] *= alpha;
    };
    // probabilities of an unmasked block against the current reference, the scale folded into the
    // exponent; row sum over the unrounded values (src/runtime/cuda_flash_bf16.rs:365-377); bf16
    // pack in the B-operand layout.  Done in two halves of 8 keys so that only 8 values are live.
    // (PER_KEY: y holds the logits already multiplied by their keys' factors)
    auto exp_pack = [&](const acc_t &s, const float (&y)[16], float c, uint4 (&pb)[2], float &rs) __attribute__((always_inline)) {
        float half[2];
#pragma unroll
        for (int ks = 0; ks < 2; ++ks) {
            float x[8];
#pragma unroll
            for (int r = 0; r < 8; ++r)
                x[r] = __builtin_amdgcn_exp2f(__builtin_fmaf(PER_KEY ? y[ks * 8 + r] : (float)s[ks * 8 + r], c, -m_run));
            half[ks] = ((x[0] + x[1]) + (x[2] + x[3])) + ((x[4] + x[5]) + (x[6] + x[7]));
            pb[ks].x = pack_bf16x2(x[0], x[1]);
            pb[ks].y = pack_bf16x2(x[2], x[3]);
            pb[ks].z = pack_bf16x2(x[4], x[5]);
            pb[ks].w = pack_bf16x2(x[6], x[7]);
        }
        rs = half[0] + half[1];
    };
    // The row sum bounds the largest probability (max <= sum <= 16 max): a sum that is too large, or
    // not finite (the first block, or a jump of the maximum), moves the reference and redoes the
    // block.  Rare, so the raw logits are not kept for it: they are recomputed from the K block,
    // which is still in LDS (block blk of stage st).
    // (RINGS: K of the block is gone from LDS by now; its logits are still in their registers, s_blk, as
    // the matrix instructions left them, i.e. with the bias in the int8 case.)
    auto fix_reference = [&](auto masked, const unsigned char *st, int blk, const acc_t &s_blk, float c, int rel, uint4 (&pb)[2],
                             float &rs, const float *kp) __attribute__((always_inline)) {
        constexpr bool M = decltype(masked)::value;
        acc_t s;
        if constexpr (RINGS) {
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                if constexpr (BIAS) s[r] = s_blk[r] - 0x4B400000;  // integer subtraction: exactly the sum
                else s[r] = s_blk[r];
            }
        } else {
#pragma unroll
            for (int r = 0; r < 16; ++r) s[r] = 0;
            uint4 kt[KSTEPS];
#pragma unroll
            for (int q = 0; q < KSTEPS; ++q) kt[q] = *(const uint4 *)(st + k_addr[q & 1] + (q >> 1) * 4096 + blk * 2048);
            static_for<0, KSTEPS>([&](auto qi) __attribute__((always_inline)) {
                constexpr int q = decltype(qi)::value;
                constexpr int pv = q > 0 ? q - 1 : 0;
                qk_step(qi, s, kt[pv], kt[q], qreg[pv], qreg[q]);
            });
        }
        // max3 is inline assembly, which the compiler leaves out when it pads the distance between a
        // matrix instruction and the first vector read of its result: the scaled copies below are
        // ordinary vector instructions, so the result has landed by the time max3 runs
        float x[16], y[16];
        if constexpr (PER_KEY) {
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const float4 f = *(const float4 *)(kp + 8 * g);
                y[4 * g + 0] = (float)s[4 * g + 0] * f.x;   // the same fl(acc ck) as the pipelined fma
                y[4 * g + 1] = (float)s[4 * g + 1] * f.y;
                y[4 * g + 2] = (float)s[4 * g + 2] * f.z;
                y[4 * g + 3] = (float)s[4 * g + 3] * f.w;
            }
        }
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            x[r] = (PER_KEY ? y[r] : (float)s[r]) * c;
            if (M && 8 * (r >> 2) + (r & 3) > rel) x[r] = NEG_SENTINEL;
        }
        float mx = max3(x[0], x[1], x[2]);
#pragma unroll
        for (int r = 3; r < 15; r += 2) mx = max3(mx, x[r], x[r + 1]);
        mx = xhalf_max(fmaxf(mx, x[15]));
        move_reference(mx);
        if constexpr (M) {
            // masked keys contribute exactly 0 whatever the reference is
            float half[2];
#pragma unroll
            for (int ks = 0; ks < 2; ++ks) {
                float e[8];
#pragma unroll
                for (int r = 0; r < 8; ++r) {
                    const int rr = ks * 8 + r;
                    e[r] = (8 * (rr >> 2) + (rr & 3) > rel) ? 0.f : __builtin_amdgcn_exp2f(x[rr] - m_run);
                }
                half[ks] = ((e[0] + e[1]) + (e[2] + e[3])) + ((e[4] + e[5]) + (e[6] + e[7]));
                pb[ks].x = pack_bf16x2(e[0], e[1]);
                pb[ks].y = pack_bf16x2(e[2], e[3]);
                pb[ks].z = pack_bf16x2(e[4], e[5]);
                pb[ks].w = pack_bf16x2(e[6], e[7]);
            }
            rs = half[0] + half[1];
        } else {
            exp_pack(s, y, c, pb, rs);
        }
    };

    // P (bf16, B-operand layout) of two consecutive blocks: while the O^T MFMAs of block j read one,
    // the softmax of block j+1 fills the other
    uint4 p_a[2], p_b[2];
    float rs = 0.f;  // its row sum
    // The softmax of an unmasked block as a list of single vector instructions, so that they can be
    // dealt out between the matrix instructions by hand.  Per half of 8 keys: [convert (int8 only)]
    // 8 x fma(s, c, -m), 8 x exp2, 7 adds (row sum of the unrounded values), 4 bf16 packs.
    // PER_KEY: 8 x fma(s, ck, -12582912 ck) first, then 4 LDS reads that refill kc / kn for the NEXT half block
    // (the second half of this block, or the first half of the next one, whose factors start at kpn), so that
    // they have the rest of the list to arrive; kp are this block's factors.
    constexpr int SM_CVT = (MODE == MODE_I8 && !BIAS) ? 8 : 0;
    constexpr int SM_KEY = PER_KEY ? (BIAS ? 12 : 10) : 0;
    constexpr int SM_PRE = SM_CVT + SM_KEY;
    constexpr int SM_HALF = SM_PRE + 8 + 8 + 7 + 4;
    constexpr int SM_OPS = 2 * SM_HALF;
    float sm_t[8], sm_x[8], sm_a[6], sm_half[2];
    auto sm_op = [&](auto masked, auto ic, const acc_t &s, float c, int rel, uint4 (&pn)[2], const float *kp, const float *kpn)
                     __attribute__((always_inline)) {
        constexpr bool M = decltype(masked)::value;
        constexpr int i = decltype(ic)::value;
        constexpr int ks = i / SM_HALF, k = i % SM_HALF;
        if constexpr (k < SM_CVT) {
            sm_t[k] = (float)s[ks * 8 + k];
        } else if constexpr (PER_KEY && k < 8) {
            if constexpr (BIAS) sm_t[k] = __builtin_fmaf(as_logit(s, ks * 8 + k), kc[k], kn[k]);
            else sm_t[k] = (float)s[ks * 8 + k] * kc[k];
        } else if constexpr (PER_KEY && k < SM_KEY) {
            load_factors(ks == 0 ? kp : kpn, ks == 0 ? 2 : 0, k - 8);
        } else if constexpr (k < SM_PRE + 8) {
            constexpr int r = k - SM_PRE;
            sm_t[r] = __builtin_fmaf((SM_CVT || PER_KEY) ? sm_t[r] : as_logit(s, ks * 8 + r), c, -m_bias);
            // a masked key: exp2 of the sentinel is exactly 0
            if (M && 8 * ((ks * 8 + r) >> 2) + (r & 3) > rel) sm_t[r] = NEG_SENTINEL;
        } else if constexpr (k < SM_PRE + 16) {
            constexpr int r = k - SM_PRE - 8;
            sm_x[r] = __builtin_amdgcn_exp2f(sm_t[r]);
        } else if constexpr (k < SM_PRE + 23) {
            constexpr int a = k - SM_PRE - 16;  // ((x0+x1)+(x2+x3)) + ((x4+x5)+(x6+x7))
            if constexpr (a < 4) sm_a[a] = sm_x[2 * a] + sm_x[2 * a + 1];
            else if constexpr (a < 6) sm_a[a] = sm_a[2 * (a - 4)] + sm_a[2 * (a - 4) + 1];
            else sm_half[ks] = sm_a[4] + sm_a[5];
        } else {
            constexpr int j = k - SM_PRE - 23;
            const uint32_t w = pack_bf16x2(sm_x[2 * j], sm_x[2 * j + 1]);
            if constexpr (j == 0) pn[ks].x = w;
            else if constexpr (j == 1) pn[ks].y = w;
            else if constexpr (j == 2) pn[ks].z = w;
            else pn[ks].w = w;
        }
    };

    // One pipelined block j.  On entry kf holds the K(j+1) fragments and vf the V(j) fragments (both
    // requested during block j-1), s_old the logits of block j with the first SM_SPLIT softmax
    // instructions already done.
    //   R1  S^T(j+1) = K(j+1) . Q^T into s_new     |  rest of the softmax of block j  -> P(j), row sum
    //   --  reference check for block j (rare: recompute P(j) from K(j), block cb of stage sc)
    //   R2  O^T += V(j)^T . P(j)^T                  |  first SM_SPLIT softmax instructions of block j+1
    // Every fragment register is refilled right after the MFMA that read it: K(j+2) (block kb of
    // stage sk) in R1, V(j+1) (block vb of stage sv) in R2, so each LDS read has a whole region to
    // arrive.  c_cur / c_next are the exponent factors of blocks j and j+1.  The instruction order
    // below IS the schedule: the fences keep the compiler from moving anything across them, and
    // the wave issues in order.  Past the last pipelined block the look-ahead works on whatever
    // the next LDS stage holds; those results are never used.
    constexpr int R2_SLOTS = DB * 2 - 2;  // S is not ready under the first two O^T MFMAs
    constexpr int SM_SPLIT = (MODE != MODE_BF16) ? (SM_OPS * R2_SLOTS) / (R2_SLOTS + KSTEPS) : SM_HALF;
    // mc / mn: block j / block j+1 has masked keys (causal diagonal, key-length edge); rel_cur /
    // rel_next are their mask offsets (see lim4h).  sc and sk point at K tiles, sv at a V tile.
    // chi / vhi / khi: the pointer sc / sv / sk is short of its tile by HI_BASE and the read adds it back through
    // the second set of address registers.
    auto pipe_block = [&](auto mc, auto mn, acc_t &s_old, acc_t &s_new, uint4 (&p_cur)[2], uint4 (&p_nxt)[2],
                          const unsigned char *sc, int cb,
                          const unsigned char *sv, int vb, const unsigned char *sk, int kb, float c_cur, float c_next,
                          int rel_cur, int rel_next, auto chi, auto vhi, auto khi, const float *kp0, const float *kp1,
                          const float *kp2) __attribute__((always_inline)) {
        // kp0 / kp1 / kp2: the key factors of blocks j, j+1, j+2 (PER_KEY)
        const int *ka = decltype(khi)::value ? k_addr_hi : k_addr;
        const int *va = decltype(vhi)::value ? v_addr_hi : v_addr;
        // ---- R1 ----
        s_new = s_init;
        ARHIP_FENCE();
        static_for<0, KSTEPS>([&](auto si) __attribute__((always_inline)) {
            constexpr int st = decltype(si)::value;
            constexpr int pv = st > 0 ? st - 1 : 0;
            qk_step(si, s_new, kf[pv], kf[st], qreg[pv], qreg[st]);
            ARHIP_FENCE();
            constexpr int lo = SM_SPLIT + st * (SM_OPS - SM_SPLIT) / KSTEPS, hi = SM_SPLIT + (st + 1) * (SM_OPS - SM_SPLIT) / KSTEPS;
            static_for<lo, hi>([&](auto ic) __attribute__((always_inline)) { sm_op(mc, ic, s_old, c_cur, rel_cur, p_cur, kp0, kp1); });
            // refill behind the MFMA that read the fragment (FP8: behind the odd step, both halves)
            if constexpr (MODE == MODE_FP8) {
                if constexpr (st % 2 == 1) {
                    kf[st - 1] = *(const uint4 *)(sk + ka[(st - 1) & 1] + ((st - 1) >> 1) * 4096 + kb * 2048);
                    kf[st] = *(const uint4 *)(sk + ka[st & 1] + (st >> 1) * 4096 + kb * 2048);
                }
            } else {
                kf[st] = *(const uint4 *)(sk + ka[st & 1] + (st >> 1) * 4096 + kb * 2048);
            }
            ARHIP_FENCE();
        });
        rs = sm_half[0] + sm_half[1];
        if (__builtin_expect(__any(!(rs <= 16.0f * LAZY_LIMIT)), 0))
            fix_reference(mc, sc + (decltype(chi)::value ? HI_BASE : 0), cb, s_old, c_cur, rel_cur, p_cur, rs, kp0);
        l_run += rs;
        set_bias(c_next);  // the reference is final for block j+1 from here to the end of its softmax
        ARHIP_FENCE();
        // ---- R2 ----
        static_for<0, DB * 2>([&](auto gi) __attribute__((always_inline)) {
            constexpr int g = decltype(gi)::value;
            constexpr int db = g / 2, ks = g % 2;
            const uint4 a = make_uint4(vf[db][ks][0].x, vf[db][ks][0].y, vf[db][ks][1].x, vf[db][ks][1].y);
            oacc[db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a),
                                                               __builtin_bit_cast(bf16x8, p_cur[ks]), oacc[db], 0, 0, 0);
            ARHIP_FENCE();
            if constexpr (g >= 2) {
                constexpr int lo = (g - 2) * SM_SPLIT / R2_SLOTS, hi = (g - 1) * SM_SPLIT / R2_SLOTS;
                static_for<lo, hi>([&](auto ic) __attribute__((always_inline)) { sm_op(mn, ic, s_new, c_next, rel_next, p_nxt, kp1, kp2); });
            }
            if constexpr (ks == 1) {
#pragma unroll
                for (int k2 = 0; k2 < 2; ++k2) {
                    vf[db][k2][0] = lds_read_tr16(sv + va[0] + db * 4096 + (vb * 2 + k2) * 1024);
                    vf[db][k2][1] = lds_read_tr16(sv + va[1] + db * 4096 + (vb * 2 + k2) * 1024);
                }
            }
            ARHIP_FENCE();
        });
    };

    // ---- prologue: tiles 0..2 on their way, tiles 0 and 1 visible ----
    // Tiles [0, nfull) have no masked key for this wave (all full tiles; under the causal mask those
    // before the wave's first query); the remaining ones (the one on the wave's causal diagonal, or the
    // last partial one) run the same pipeline with the mask applied inside the softmax.  Every wave
    // passes one barrier per tile and requests its share of every tile's transfers, whichever form of
    // the tile it runs.
    const int nfull = CAUSAL ? min(kend / BK, wq0 / BK) : kend / BK;
    static_for<0, AHEAD>([&](auto ti) __attribute__((always_inline)) { issue_tile(decltype(ti)::value); });
    // Q operand, resident in registers.  Everything in flight is awaited here once, Q included, so
    // that no wait for a global load is left inside the loops.
    // QFUSE: the 16 values (bf16: 2 x 16 bytes, f32: 4 x 16 bytes) behind each 16-byte piece of the operand
    uint4 qraw[QFUSE ? KSTEPS : 1][QROWS ? 4 : 2];
    if constexpr (QROWS) {
        const float *qb = (const float *)p.q + (size_t)b * p.qs[0] + (size_t)head * p.qs[1] + (size_t)min(q_row, N - 1) * p.qs[2];
#pragma unroll
        for (int s = 0; s < KSTEPS; ++s)
#pragma unroll
            for (int c = 0; c < 4; ++c) qraw[s][c] = *(const uint4 *)(qb + s * 32 + h * 16 + c * 4);
    } else if constexpr (QFUSE) {
        const uint16_t *qb = (const uint16_t *)p.q + (size_t)b * p.qs[0] + (size_t)head * p.qs[1] + (size_t)min(q_row, N - 1) * p.qs[2];
#pragma unroll
        for (int s = 0; s < KSTEPS; ++s) {
            qraw[s][0] = *(const uint4 *)(qb + s * 32 + h * 16);
            qraw[s][1] = *(const uint4 *)(qb + s * 32 + h * 16 + 8);
        }
    } else {
        const unsigned char *qb = (const unsigned char *)p.q +
                                  ((size_t)b * p.qs[0] + (size_t)head * p.qs[1] + (size_t)min(q_row, N - 1) * p.qs[2]) * QK_BYTES;
#pragma unroll
        for (int s = 0; s < KSTEPS; ++s) qreg[s] = *(const uint4 *)(qb + s * 32 + h * 16);
    }

    if constexpr (MODE != MODE_BF16 && !PER_KEY) {
        skv_cur = load_sk_group(0);
        skv_nxt = load_sk_group(1);
    }
    // BIAS: the largest Q scale of the workgroup's queries and the largest K scale of the head, read
    // behind the transfers issued above so that their latency is spent under them
    float mq = 0.f, mk = 0.f;
    if constexpr (BIAS && !PER_KEY) {
        const int nqb = (N + p.bq - 1) / p.bq, nkb = (N + p.bk - 1) / p.bk;
        const int qb0 = qblk / p.bq, qb1 = min(qblk + BQ - 1, N - 1) / p.bq;
        if constexpr (!QFUSE)
            for (int i = qb0 + lane; i <= qb1; i += 64) mq = fmaxf(mq, fabsf(p.sq[(size_t)bh * nqb + i]));
        for (int i = lane; i < nkb; i += 64) mk = fmaxf(mk, fabsf(p.sk[(size_t)kv_bh * nkb + i]));
    }
    wait_vmem_le<0>();
    __syncthreads();
    if constexpr (QFUSE) {
        // bf16 -> f32 is a shift; the quantiser's own operations from there on
        auto val = [&](int s, int e) __attribute__((always_inline)) -> float {
            if constexpr (QROWS) {
                const uint4 w = qraw[s][e >> 2];
                return __uint_as_float((e & 3) == 0 ? w.x : (e & 3) == 1 ? w.y : (e & 3) == 2 ? w.z : w.w);
            } else {
                const uint4 w = qraw[s][e >> 3];
                const uint32_t u = (e & 7) < 2 ? w.x : (e & 7) < 4 ? w.y : (e & 7) < 6 ? w.z : w.w;
                return __uint_as_float((e & 1) ? (u & 0xffff0000u) : (u << 16));
            }
        };
        float mx = 0.f;
#pragma unroll
        for (int s = 0; s < KSTEPS; ++s)
#pragma unroll
            for (int e = 0; e < 16; ++e) mx = fmaxf(mx, fabsf(val(s, e)));
        mx = xhalf_max(mx);  // the two lanes of a query
        float *red = (float *)(lds + QF_RED);
        if constexpr (!QROWS) {
#pragma unroll
            for (int o = 16; o >= 1; o >>= 1) mx = fmaxf(mx, __shfl_xor(mx, o));
            if (lane == 0) red[wave] = mx;
            __syncthreads();
            // a block of 128 queries is four waves (a block past the last query holds copies of the last row and is
            // neither used nor written back)
            const int w0 = wave & ~3;
            mx = fmaxf(fmaxf(red[w0], red[w0 + 1]), fmaxf(red[w0 + 2], red[w0 + 3]));
        }
        constexpr float QMAX = (MODE == MODE_FP8) ? 448.0f : 127.0f;
        const float scale = (mx > 0.f) ? mx / QMAX : 1.f;
        const float inv = 1.f / scale;
#pragma unroll
        for (int s = 0; s < KSTEPS; ++s) {
            uint32_t w[4] = {0u, 0u, 0u, 0u};
            if constexpr (MODE == MODE_FP8) {
                // E4M3, round to nearest even, saturating: the clamp first, as the pre-pass quantiser does
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    float c[4];
#pragma unroll
                    for (int i = 0; i < 4; ++i) c[i] = fminf(fmaxf(val(s, 4 * j + i) * inv, -448.0f), 448.0f);
                    int r = 0;
                    r = __builtin_amdgcn_cvt_pk_fp8_f32(c[0], c[1], r, false);
                    r = __builtin_amdgcn_cvt_pk_fp8_f32(c[2], c[3], r, true);
                    w[j] = (uint32_t)r;
                }
            } else {
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    int iv = (int)rintf(val(s, e) * inv);
                    iv = iv < -127 ? -127 : (iv > 127 ? 127 : iv);
                    w[e >> 2] |= ((uint32_t)iv & 0xffu) << ((e & 3) * 8);
                }
            }
            qreg[s] = make_uint4(w[0], w[1], w[2], w[3]);
        }
        sq_lane = scale;
        sq_c = (sq_lane * p.scale) * LOG2E;
        if constexpr (QROWS) {
            if (p.sq_out != nullptr && h == 0 && q_row < N) p.sq_out[(size_t)bh * N + q_row] = scale;
        } else {
            // the workgroup's largest Q scale, for the grid below: every wave reads every wave's maximum
            float wg_mx = red[0];
#pragma unroll
            for (int w = 1; w < NW; ++w) wg_mx = fmaxf(wg_mx, red[w]);
            mq = (wg_mx > 0.f) ? wg_mx / QMAX : 1.f;
            const int blk = q_row >> 7, nqb = (N + 127) >> 7;
            if (p.sq_out != nullptr && lane == 0 && (wave & 3) == 0 && blk < nqb) p.sq_out[(size_t)bh * nqb + blk] = scale;
        }
        if (p.q8_out != nullptr && q_row < N) {
            int8_t *dst = p.q8_out + ((size_t)bh * N + q_row) * D;
#pragma unroll
            for (int s = 0; s < KSTEPS; ++s) *(uint4 *)(dst + s * 32 + h * 16) = qreg[s];
        }
    }
    if constexpr (BIAS && !PER_KEY) {
        // The exponent reference stays on a grid no finer than the unit in the last place of
        // 12582912 c for the largest c = sq sk scale log2(e) the workgroup can meet; every wave reduces
        // the same scales, so the grid is uniform over the workgroup.
#pragma unroll
        for (int o = 32; o >= 1; o >>= 1) {
            mq = fmaxf(mq, __shfl_xor(mq, o));
            mk = fmaxf(mk, __shfl_xor(mk, o));
        }
        // 12582912 c_max < 2^(E+1): the sums stay below 2^(E+2) wherever the bias outweighs the
        // reference, so their unit in the last place is at most 2^(E-22); the grid is twice that.
        // (Scales that are not finite, or zero, give a grid of 1: the results are garbage or
        // trivial either way.)
        const float x = 12582912.0f * (((mq * mk) * fabsf(p.scale)) * LOG2E);
        const int e = (int)((__float_as_uint(x) >> 23) & 0xff) - 127;  // floor(log2 x)
        float grid = 1.0f;
        if (x > 0x1p-60f && x < 0x1p100f) grid = __uint_as_float((uint32_t)(e - 21 + 127) << 23);
        m_grid = __uint_as_float(__builtin_amdgcn_readfirstlane(__float_as_uint(grid)));
        m_grid_inv = 1.0f / m_grid;
    }
    float c_carry = tile_c(0, 0);  // exponent factor of the tile the next tile_iter works on
    acc_t s_a, s_b;  // logits of the even / odd block of a tile
#pragma unroll
    for (int r = 0; r < 16; ++r) s_a[r] = s_b[r] = 0;
    constexpr std::false_type PLAIN{};
    constexpr std::true_type MASKED{};
    if (ntiles > 0) {
        convert_sk(0);
        load_kf(lds + k_base(0), 0);
        s_a = mfma_qk();
        load_kf(lds + k_base(0), 1);
        load_vf(lds + v_base(0), 0);
        const float c0 = tile_c(0, 0);
        set_bias(c0);
        const float *f0 = key_factors(0, 0), *f1 = key_factors(0, 1);
        if constexpr (PER_KEY) {
            static_for<0, SM_KEY - 8>([&](auto pi) __attribute__((always_inline)) { load_factors(f0, 0, decltype(pi)::value); });
        }
        if (nfull > 0)
            static_for<0, SM_SPLIT>([&](auto ic) __attribute__((always_inline)) { sm_op(PLAIN, ic, s_a, c0, 0, p_a, f0, f1); });
        else
            static_for<0, SM_SPLIT>([&](auto ic) __attribute__((always_inline)) { sm_op(MASKED, ic, s_a, c0, lim4h, p_a, f0, f1); });
    }

    // one tile: its two blocks; m0 / m1 / m2 say whether the first block, the second block and the
    // first block of the next tile have masked keys
    // stg: the stage of tile `it` where the caller knows it at compile time (it % 4), else -1
    auto tile_iter = [&](auto m0, auto m1, auto m2, int it, auto stg) __attribute__((always_inline)) {
        constexpr int S = decltype(stg)::value, S1 = (S + 1) & 3;
        constexpr bool cur_hi = S >= 2, nxt_hi = S >= 0 && S1 >= 2;
        const unsigned char *k_cur = lds + (S >= 0 ? S * STAGE - (cur_hi ? HI_BASE : 0) : k_base(it));
        const unsigned char *k_nxt = lds + (S >= 0 ? S1 * STAGE - (nxt_hi ? HI_BASE : 0) : k_base(it + 1));
        const unsigned char *v_cur = lds + (S >= 0 ? S * STAGE + K_TILE - (cur_hi ? HI_BASE : 0) : v_base(it));
        const unsigned char *v_nxt = lds + (S >= 0 ? S1 * STAGE + K_TILE - (nxt_hi ? HI_BASE : 0) : v_base(it + 1));
        const std::integral_constant<bool, cur_hi> hc;
        const std::integral_constant<bool, nxt_hi> hn;
        // tile it + 3 goes to the stage tile it - 1 vacated at the last barrier (RINGS: K(it + 2) to where
        // K(it) was, read for the last time before that barrier, V(it + 2) to where V(it - 1) was)
        issue_tile(it + AHEAD);
        advance_sk_group(it);
        convert_sk(it + 1);  // visible since the barrier that ended the last iteration
        const float *f00 = key_factors(it, 0), *f01 = key_factors(it, 1), *f10 = key_factors(it + 1, 0), *f11 = key_factors(it + 1, 1);
        // (tile_iter runs on consecutive tiles from 0 on: this tile's factor is last iteration's c_nxt)
        const float c_cur = c_carry, c_nxt = tile_c(it + 1, it);
        c_carry = c_nxt;
        const int rel0 = lim4h - it * BK;
        pipe_block(m0, m1, s_a, s_b, p_a, p_b, k_cur, 0, v_cur, 1, k_nxt, 0, c_cur, c_cur, rel0, rel0 - 32, hc, hc, hn, f00, f01, f10);
        pipe_block(m1, m2, s_b, s_a, p_b, p_a, k_cur, 1, v_nxt, 0, k_nxt, 1, c_cur, c_nxt, rel0 - 32, rel0 - 64, hc, hn, hn, f01, f10, f11);
        wait_vmem_le<RINGS ? 0 : XPW_MIN>();  // tile it + 2 has landed (tile it + 3 may still be in flight)
        __syncthreads();
    };
    // RINGS: the first iteration requests K(2) into the place of K(0), which the lines above have just
    // read: every wave's reads must have returned first
    if constexpr (RINGS) __syncthreads();
    // the last unmasked tile hands a masked block to the look-ahead: it is peeled off
    const int nplain = (nfull < ntiles) ? max(nfull - 1, 0) : nfull;
    // Four tiles per trip, so that the stage of a tile (it % 4) and with it every LDS offset and transfer
    // destination is a constant (int8: 15 vector and 23 scalar instructions fewer per tile, Sage B4 H32 S8192
    // 3.05 -> 2.96 ms; bf16, once no offset needs a register of its own: S8192 -1.8 %).
    const int nplain4 = !RINGS ? (nplain & ~3) : 0;
#pragma clang loop unroll(disable)
    for (int it = 0; it < nplain4; it += 4) {
        tile_iter(PLAIN, PLAIN, PLAIN, it, std::integral_constant<int, 0>());
        tile_iter(PLAIN, PLAIN, PLAIN, it + 1, std::integral_constant<int, 1>());
        tile_iter(PLAIN, PLAIN, PLAIN, it + 2, std::integral_constant<int, 2>());
        tile_iter(PLAIN, PLAIN, PLAIN, it + 3, std::integral_constant<int, 3>());
    }
    const std::integral_constant<int, -1> any_stage;
#pragma clang loop unroll(disable)
    for (int it = nplain4; it < nplain; ++it) tile_iter(PLAIN, PLAIN, PLAIN, it, any_stage);
    if (nplain < nfull) tile_iter(PLAIN, PLAIN, MASKED, nplain, any_stage);
    // under the causal mask a wave is done once the tiles start past its last query; it keeps
    // feeding the transfers and the barriers the other waves rely on
    const int my_tiles = CAUSAL ? min(ntiles, (wq0 + 31) / BK + 1) : ntiles;
    // (two loops rather than a branch inside one: the accumulators would be copied at the join)
#pragma clang loop unroll(disable)
    for (int it = nfull; it < my_tiles; ++it) tile_iter(MASKED, MASKED, MASKED, it, any_stage);
#pragma clang loop unroll(disable)
    for (int it = max(nfull, my_tiles); it < ntiles; ++it) {
        issue_tile(it + AHEAD);
        wait_vmem_le<RINGS ? 0 : XPW_MIN>();
        __syncthreads();
    }

    // ---- normalise and store: acc * (l > 0 ? 1/l : 0), cuda_flash_bf16.rs:414-426 ----
    const float l_tot = xhalf_sum(l_run);
    const float inv = (l_tot > 0.f) ? 1.f / l_tot : 0.f;
    if (p.lse != nullptr && h == 0 && q_row < N) {
        p.lse[(size_t)bh * N + q_row] = (l_tot > 0.f) ? (m_run + __builtin_amdgcn_logf(l_tot)) * 0.6931471805599453f : NEG_SENTINEL;
    }
    // (f32 or bf16 output is the launch's choice, not a variant of the kernel: the two stores are a few lines at the
    // end, and every variant of the kernel is minutes of compilation)
    if (OUT_F32 || (MODE != MODE_BF16 && p.out_f32)) {
        if (q_row < N) {
            const size_t obase = (size_t)b * p.os[0] + (size_t)head * p.os[1] + (size_t)q_row * p.os[2];
#pragma unroll
            for (int db = 0; db < DB; ++db)
#pragma unroll
                for (int gg = 0; gg < 4; ++gg) {
                    const int d = db * 32 + 8 * gg + 4 * h;
                    *(float4 *)((float *)p.o + obase + d) = make_float4(oacc[db][4 * gg + 0] * inv, oacc[db][4 * gg + 1] * inv,
                                                                        oacc[db][4 * gg + 2] * inv, oacc[db][4 * gg + 3] * inv);
                }
        }
    } else {
        // bf16 output.  In the accumulator layout a lane holds one query's channels 4 at a time, so
        // storing from there writes 8 bytes per lane to 32 different rows per instruction (measured:
        // the output stores cost 5.5 us per workgroup, 11 % of a B4 H32 S2048 causal launch).  The
        // wave's 32 x D tile is turned around in LDS instead (its own slab of the tile stages, which
        // are free once every wave is past the last tile and the transfers requested beyond it have
        // landed) and leaves as whole rows, 16 bytes per lane, 4 rows per instruction.
        constexpr int OROW = D * 2 + 16;  // bytes; 16-byte aligned rows
        static_assert(NW * 32 * OROW <= LDS_BYTES, "output staging fits the tile stages");
        wait_vmem_le<0>();
        __syncthreads();
        unsigned char *ob = lds + wave * 32 * OROW;
#pragma unroll
        for (int db = 0; db < DB; ++db)
#pragma unroll
            for (int gg = 0; gg < 4; ++gg) {
                uint2 w;
                w.x = pack_bf16x2(oacc[db][4 * gg + 0] * inv, oacc[db][4 * gg + 1] * inv);
                w.y = pack_bf16x2(oacc[db][4 * gg + 2] * inv, oacc[db][4 * gg + 3] * inv);
                *(uint2 *)(ob + i32 * OROW + (db * 32 + 8 * gg + 4 * h) * 2) = w;
            }
        // the wave reads back only what it wrote: LDS operations of a wave complete in order
        constexpr int LPR = D * 2 / 16;        // lanes per row
        constexpr int RPI = 64 / LPR;          // rows per store instruction
        const int rl = lane / LPR, cl = lane % LPR;
        uint16_t *obase = (uint16_t *)p.o + (size_t)b * p.os[0] + (size_t)head * p.os[1];
#pragma unroll
        for (int k = 0; k < 32 / RPI; ++k) {
            const int r = k * RPI + rl;
            const uint4 w = *(const uint4 *)(ob + r * OROW + cl * 16);
            if (wq0 + r < N) *(uint4 *)(obase + (size_t)(wq0 + r) * p.os[2] + cl * 8) = w;
        }
    }
}

// int8 uses the biased accumulators (see s_init); bf16 and FP8 the plain ones.
template <int D, bool CAUSAL, int MODE, bool OUT_F32, int NW = 8, bool PER_KEY = false, bool QFUSE = false>
__device__ __forceinline__ void attn_pipe_body(const AttnParams &p, unsigned char *lds, int wg_linear)
{
    attn_pipe_impl<D, CAUSAL, MODE, OUT_F32, (MODE == MODE_I8 && ARHIP_PIPE_INT_BIAS), NW, PER_KEY, QFUSE>(p, lds, wg_linear);
}

template <int D, bool CAUSAL, int MODE, bool OUT_F32, int NW = 8, bool PER_KEY = false, bool QFUSE = false>
__global__ void __launch_bounds__(NW * 64, NW == 4 ? 2 : 1) attn_pipe_kernel(const AttnParams p)
{
    __shared__ __attribute__((aligned(1024))) unsigned char lds[attn_pipe_lds_bytes<D, MODE, NW, PER_KEY, QFUSE>()];
    attn_pipe_body<D, CAUSAL, MODE, OUT_F32, NW, PER_KEY, QFUSE>(p, lds, (int)blockIdx.x);
}

}  // namespace arhip
