// arhip_flash_fwd / arhip_sage_fwd: argument checks, kernel selection, launch.
//
// Mirrors the reference's launch wrappers: cuda_flash::run_ex
// (src/runtime/cuda_flash.rs:203-254), cuda_flash_bf16::run_ex
// (src/runtime/cuda_flash_bf16.rs:495-548) and cuda_flash_sage::run_ex
// (src/runtime/cuda_flash_sage.rs:452-485).
#include "arhip_internal.h"
#include "attn_fwd.h"
#include "pipe_launch.h"
#include "flash_bwd_f32.h"
#include "flash_f32.h"

#include <algorithm>


using namespace arhip;

extern "C" int arhip_attn_supported(int kind, int64_t n, int64_t d, int dtype)
{
    if (n <= 0 || n > (int64_t)1 << 24) return 0;
    if (d != 64 && d != 128) return 0;
    switch (kind) {
    case ARHIP_ATTN_FLASH: return dtype == ARHIP_F32 || dtype == ARHIP_BF16;
    case ARHIP_ATTN_SAGE: return dtype == ARHIP_F32 || dtype == ARHIP_BF16;
    default: return 0;  // SDPA is the caller's general path
    }
}

static int check_common(const char *fn, arhip_device *dev, const void *q, const void *k, const void *v, const void *o,
                        const float *mask, int64_t B, int64_t Hq, int64_t Hkv, int64_t N, int64_t D)
{
    ARHIP_REQUIRE(dev != nullptr, "%s: null device", fn);
    ARHIP_REQUIRE(q && k && v && o, "%s: null tensor pointer", fn);
    ARHIP_REQUIRE(B > 0 && Hq > 0 && Hkv > 0 && N > 0, "%s: empty shape B=%lld Hq=%lld Hkv=%lld N=%lld", fn,
                  (long long)B, (long long)Hq, (long long)Hkv, (long long)N);
    ARHIP_REQUIRE(Hq % Hkv == 0, "%s: Hq=%lld is not a multiple of Hkv=%lld", fn, (long long)Hq, (long long)Hkv);
    if (D != 64 && D != 128) return arhip_fail(ARHIP_EUNSUPPORTED, "%s: head_dim %lld (64 or 128)", fn, (long long)D);
    // workgroup ids, tile counts and row indices are 32-bit in the kernels
    if (N > ((int64_t)1 << 24) || B * Hq > ((int64_t)1 << 24) || B * Hq * ((N + 31) / 32) > ((int64_t)1 << 30))
        return arhip_fail(ARHIP_EUNSUPPORTED, "%s: shape too large for 32-bit tile indices", fn);
    ARHIP_REQUIRE(arhip_aligned16(q) && arhip_aligned16(k) && arhip_aligned16(v) && arhip_aligned16(o),
                  "%s: q/k/v/o must be 16-byte aligned", fn);
    ARHIP_REQUIRE(mask == nullptr || (reinterpret_cast<uintptr_t>(mask) & 3u) == 0, "%s: mask must be 4-byte aligned", fn);
    return ARHIP_OK;
}

// CAUSAL / HAS_MASK dispatch for one tiling variant.
template <int D, int NW, int MODE, bool PER_KEY, bool OUT_F32, bool DBG, bool MASKS>
static void launch_attn(hipStream_t stream, const AttnParams &p, bool causal, bool has_mask)
{
    const dim3 grid((unsigned)p.total), block(NW * 64);
    if constexpr (MASKS) {
        if (has_mask) {
            if (causal)
                hipLaunchKernelGGL((attn_fwd_kernel<D, NW, true, true, MODE, PER_KEY, OUT_F32, DBG>), grid, block, 0, stream, p);
            else
                hipLaunchKernelGGL((attn_fwd_kernel<D, NW, false, true, MODE, PER_KEY, OUT_F32, DBG>), grid, block, 0, stream, p);
            return;
        }
    }
    if (causal)
        hipLaunchKernelGGL((attn_fwd_kernel<D, NW, true, false, MODE, PER_KEY, OUT_F32, DBG>), grid, block, 0, stream, p);
    else
        hipLaunchKernelGGL((attn_fwd_kernel<D, NW, false, false, MODE, PER_KEY, OUT_F32, DBG>), grid, block, 0, stream, p);
}

// The software-pipelined kernel (no additive mask): 8 waves per workgroup, or 4 (two workgroups per compute
// unit) where a workgroup sees few tiles.  Its variants are compiled in translation units of their own
// (pipe_launch.h).
// Which of the two: 128 queries per workgroup hide a workgroup's prologue and epilogue under its
// neighbour's tiles and fill the chip with fewer heads, but request every K/V tile twice as often and
// keep only one tile in flight.  Two workgroups of equal length that start together stay in step and
// hide nothing, so the gain is in few or unequal workgroups.  Measured at D = 128, bf16 (B4 H32 unless
// noted; 4 waves against 8): causal N = 512 / 1024 / 2048 -15 / -7 / -5 %, B1 H16 N = 2048 causal -25 %,
// B2 H16 N = 1024 -22 %, N = 1024 -4 %; N = 2048 equal; N = 2048 causal with key lengths in [N/2, N]
// (many equal workgroups) +3 %; N = 8192 +3 %, causal N = 32768 +4.5 %.
// At D = 64 (B4 H32): N = 2048 -8 %, N = 8192 -2 %, causal N = 2048 -16 %, causal N = 8192 -4 %: always 4 waves.
// (Three such workgroups per compute unit fit at D = 64, 154 registers and 40 KB of LDS each, and run no
// faster than two.)
static bool pipe_wants_4_waves(arhip_device *dev, int64_t heads, int64_t N, int64_t D, bool causal, bool has_len)
{
    if (dev->attn_waves == 8 || dev->attn_waves == 40) return dev->attn_waves == 40;
    if (D == 64) return true;
    if (heads * ((N + 255) / 256) < 2 * (int64_t)dev->cus) return true;
    return N <= 1024 || (N <= 2048 && causal && !has_len);
}

// The pipelined kernel addresses K and V through 32-bit buffer offsets (rows of one head, plus the
// tiles it requests past the end).
static bool pipe_addressable(int64_t N, int64_t kv_token_stride, int64_t elem_bytes)
{
    return (N + 5 * 64) * kv_token_stride * elem_bytes < ((int64_t)1 << 31);
}

// Which kernel.  Launches without an additive mask, per-key scales or the logits export take the
// software-pipelined kernel (returned as 8; whether it runs with 8 or 4 waves per workgroup is
// pipe_wants_4_waves' choice): with its 4-wave form it is the fastest kernel down to the shortest sequences
// (bf16, against the kernels that used to serve them: B8 H12 N197 D64 7.8 -> 7.0 us, B4 H16 N256 D128 11.8 ->
// 9.0 us, B32 H12 N64 D64 9.1 -> 5.6 us, B8 H12 N400 D64 27.8 -> 12.9 us).  The others take the general
// kernel with 4 waves of 32 queries, or 1 at D = 64 when that still leaves compute units idle.
static int pick_waves(arhip_device *dev, int64_t heads, int64_t N, int64_t D, bool special)
{
    const int64_t cus = dev->cus, wg128 = heads * ((N + 127) / 128);
    int nw;
    if (!special) nw = 8;
    else if (D == 64 && wg128 < 2 * cus) nw = 1;
    else nw = 4;
    // ARHIP_ATTN_WAVES (read once when the device is opened) is a tuning aid; results do not depend on it
    // (1, 4: the general kernel with that many waves; 8, 40: the pipelined kernel with 8 / 4 waves)
    const int w = dev->attn_waves;
    if ((w == 1 || w == 4 || w == 8) && !special && (w != 1 || D == 64)) nw = w;
    if (w == 40 && !special) nw = 8;
    return nw;
}

static void dense_strides(long s[3], int64_t H, int64_t N, int64_t D)
{
    s[0] = (long)(H * N * D);
    s[1] = (long)(N * D);
    s[2] = (long)D;
}

extern "C" int arhip_flash_fwd(arhip_device *dev, const void *q, const void *k, const void *v, void *o,
                               const float *mask, const int32_t *kv_len,
                               int64_t B, int64_t Hq, int64_t Hkv, int64_t N, int64_t D,
                               int causal, int dtype, float scale, int wait, double *secs)
{
    long qs[3], ks[3];
    dense_strides(qs, Hq, N, D);
    dense_strides(ks, Hkv, N, D);
    const int64_t q64[3] = {qs[0], qs[1], qs[2]}, k64[3] = {ks[0], ks[1], ks[2]};
    return arhip_flash_fwd_strided(dev, q, k, v, o, q64, k64, q64, mask, kv_len, B, Hq, Hkv, N, D, causal, dtype, scale,
                                   wait, secs);
}

extern "C" int arhip_flash_fwd_strided(arhip_device *dev, const void *q, const void *k, const void *v, void *o,
                                       const int64_t q_strides[3], const int64_t kv_strides[3], const int64_t o_strides[3],
                                       const float *mask, const int32_t *kv_len,
                                       int64_t B, int64_t Hq, int64_t Hkv, int64_t N, int64_t D,
                                       int causal, int dtype, float scale, int wait, double *secs)
{
    return arhip_flash_fwd_lse(dev, q, k, v, o, nullptr, q_strides, kv_strides, o_strides, mask, kv_len, B, Hq, Hkv, N, D,
                               causal, dtype, scale, wait, secs);
}

extern "C" int arhip_flash_fwd_lse(arhip_device *dev, const void *q, const void *k, const void *v, void *o, float *lse,
                                   const int64_t q_strides[3], const int64_t kv_strides[3], const int64_t o_strides[3],
                                   const float *mask, const int32_t *kv_len,
                                   int64_t B, int64_t Hq, int64_t Hkv, int64_t N, int64_t D,
                                   int causal, int dtype, float scale, int wait, double *secs)
{
    if (int rc = check_common("arhip_flash_fwd", dev, q, k, v, o, mask, B, Hq, Hkv, N, D)) return rc;
    ARHIP_REQUIRE(lse == nullptr || (reinterpret_cast<uintptr_t>(lse) & 3u) == 0, "arhip_flash_fwd_lse: lse must be 4-byte aligned");
    ARHIP_REQUIRE(dtype == ARHIP_F32 || dtype == ARHIP_BF16, "arhip_flash_fwd: dtype %d", dtype);
    ARHIP_REQUIRE(q_strides && kv_strides && o_strides, "arhip_flash_fwd_strided: null strides");
    {
        // rows must stay 16-byte aligned and must not overlap: every stride a multiple of 8 elements,
        // the token stride at least D
        const int64_t *all[3] = {q_strides, kv_strides, o_strides};
        for (int t = 0; t < 3; ++t)
            for (int i = 0; i < 3; ++i)
                ARHIP_REQUIRE(all[t][i] >= 0 && all[t][i] % 8 == 0 && (i != 2 || all[t][i] >= D) && (t != 2 || all[t][i] > 0),
                              "arhip_flash_fwd_strided: stride %lld (multiples of 8 elements, token stride >= D, output "
                              "strides > 0 so that output rows cannot alias)",
                              (long long)all[t][i]);
    }
    ARHIP_HIP(hipSetDevice(dev->ordinal));
    arhip_call_timer t{dev, wait, secs};
    t.kernel = (dtype == ARHIP_F32) ? ARHIP_K_FLASH_F32 : ARHIP_K_FLASH_BF16;

    if (dtype == ARHIP_F32) {
        FlashF32Params fp;
        fp.q = (const float *)q; fp.k = (const float *)k; fp.v = (const float *)v; fp.o = (float *)o;
        fp.mask = mask; fp.kv_len = kv_len; fp.lse = lse;
        fp.Hq = (int)Hq; fp.Hkv = (int)Hkv; fp.N = (int)N;
        for (int i = 0; i < 3; ++i) {
            fp.qs[i] = (long)q_strides[i];
            fp.ks[i] = (long)kv_strides[i];
            fp.os[i] = (long)o_strides[i];
        }
        // 128 queries per workgroup of 4 waves when that still fills the chip, else 32 queries whose key
        // tiles are dealt out between the waves of the workgroup: 4 waves, or 2 when that lets every
        // workgroup be resident at once (8 waves per CU) and 4 would need a second round
        const bool splitk = B * Hq * ((N + 127) / 128) < 2 * (int64_t)dev->cus;
        const int bq = splitk ? 32 : 128;
        fp.nq = (int)((N + bq - 1) / bq);
        fp.scale = scale;
        const int64_t wgs = fp.nq * B * Hq;
        fp.total = (int)wgs;
        fp.lpt_heads = causal ? (int)(B * Hq) : 0;  // causal: longest query tile first over all heads
        const bool two = splitk && D == 64 && wgs > 2 * (int64_t)dev->cus && wgs <= 4 * (int64_t)dev->cus;
        if (int rc = t.begin()) return rc;
        const dim3 grid((unsigned)wgs), block(two ? 128 : 256);
#define F32_LAUNCH(DD, NWW, SK)                                                                         \
    do {                                                                                              \
        if (causal) hipLaunchKernelGGL((flash_f32_kernel<DD, NWW, true, SK>), grid, block, 0, dev->stream, fp);  \
        else hipLaunchKernelGGL((flash_f32_kernel<DD, NWW, false, SK>), grid, block, 0, dev->stream, fp); \
    } while (0)
        if (D == 64) {
            if (two) F32_LAUNCH(64, 2, true); else if (splitk) F32_LAUNCH(64, 4, true); else F32_LAUNCH(64, 4, false);
        } else {
            if (splitk) F32_LAUNCH(128, 4, true); else F32_LAUNCH(128, 4, false);
        }
#undef F32_LAUNCH
        arhip_note_selected(ARHIP_K_FLASH_F32);
        return t.end();
    }

    AttnParams p = {};
    p.q = q; p.k = k; p.v = (const uint16_t *)v; p.o = o;
    p.mask = mask; p.kv_len = kv_len; p.lse = lse;
    p.Hq = (int)Hq; p.Hkv = (int)Hkv; p.N = (int)N;
    for (int i = 0; i < 3; ++i) {
        p.qs[i] = (long)q_strides[i];
        p.ks[i] = (long)kv_strides[i];
        p.vs[i] = (long)kv_strides[i];
        p.os[i] = (long)o_strides[i];
    }
    p.bq = p.bk = 1;
    p.scale = scale;
    const bool c = causal != 0, hm = mask != nullptr;
    int nw = pick_waves(dev, B * Hq, N, D, hm);
    if (nw == 8 && !pipe_addressable(N, kv_strides[2], 2)) nw = 4;
    const bool pipe = nw == 8;  // the software-pipelined kernel; how many waves it runs with is its own choice
    if (pipe && pipe_wants_4_waves(dev, B * Hq, N, D, causal != 0, kv_len != nullptr)) nw = 4;
    p.nq = (int)((N + nw * 32 - 1) / (nw * 32));
    p.total = (int)(p.nq * B * Hq);
    p.lpt = p.total <= 16 * dev->cus;  // few workgroups per CU: balance them globally
    if (int rc = t.begin()) return rc;
    if (pipe) {
        launch_pipe_bf16(dev->stream, p, (int)D, c, nw);
    } else if (D == 64) {
        if (nw == 1) launch_attn<64, 1, MODE_BF16, false, false, false, true>(dev->stream, p, c, hm);
        else launch_attn<64, 4, MODE_BF16, false, false, false, true>(dev->stream, p, c, hm);
    } else {
        launch_attn<128, 4, MODE_BF16, false, false, false, true>(dev->stream, p, c, hm);
    }
    arhip_note_selected(ARHIP_K_FLASH_BF16);
    return t.end();
}

extern "C" int arhip_sage_fwd(arhip_device *dev, const int8_t *q8, const int8_t *k8,
                              const float *sq, const float *sk, const uint16_t *v, void *o,
                              const float *mask, const int32_t *kv_len,
                              int64_t B, int64_t Hq, int64_t Hkv, int64_t N, int64_t D,
                              int64_t bq, int64_t bk, int causal, int out_dtype, float scale,
                              int32_t *dbg_logits, const int32_t dbg_sel[3],
                              int wait, double *secs)
{
    return arhip_sage_fwd_strided(dev, q8, k8, sq, sk, v, o, nullptr, nullptr, mask, kv_len, B, Hq, Hkv, N, D, bq, bk, causal,
                                  out_dtype, scale, dbg_logits, dbg_sel, wait, secs);
}

static int sage_fwd_impl(arhip_device *dev, const int8_t *q8, const int8_t *k8,
                         const float *sq, const float *sk, const uint16_t *v, void *o,
                         const int64_t v_strides[3], const int64_t o_strides[3],
                         const float *mask, const int32_t *kv_len,
                         int64_t B, int64_t Hq, int64_t Hkv, int64_t N, int64_t D,
                         int64_t bq, int64_t bk, int causal, int out_dtype, float scale,
                         int32_t *dbg_logits, const int32_t dbg_sel[3], int wait, double *secs, bool fp8)
{
    if (int rc = check_common("arhip_sage_fwd", dev, q8, k8, v, o, mask, B, Hq, Hkv, N, D)) return rc;
    ARHIP_REQUIRE(sq && sk, "arhip_sage_fwd: null scale pointer");
    ARHIP_REQUIRE(bq >= 1 && bk >= 1, "arhip_sage_fwd: block sizes bq=%lld bk=%lld", (long long)bq, (long long)bk);
    ARHIP_REQUIRE(out_dtype == ARHIP_F32 || out_dtype == ARHIP_BF16, "arhip_sage_fwd: out_dtype %d", out_dtype);
    ARHIP_REQUIRE(dbg_logits == nullptr || dbg_sel != nullptr, "arhip_sage_fwd: dbg_logits without dbg_sel");
    ARHIP_REQUIRE(dbg_logits == nullptr || mask == nullptr, "arhip_sage_fwd: the logits export does not take a mask");
    for (int t = 0; t < 2; ++t) {
        const int64_t *st = t == 0 ? v_strides : o_strides;
        if (!st) continue;
        for (int i = 0; i < 3; ++i)
            ARHIP_REQUIRE(st[i] >= 0 && st[i] % 8 == 0 && (i != 2 || st[i] >= D) && (t == 0 || st[i] > 0),
                          "arhip_sage_fwd_strided: stride %lld (multiples of 8 elements, token stride >= D, output strides > 0)",
                          (long long)st[i]);
    }
    ARHIP_HIP(hipSetDevice(dev->ordinal));

    AttnParams p = {};
    p.q = q8; p.k = k8; p.v = v; p.o = o;
    p.mask = mask; p.kv_len = kv_len;
    p.sq = sq; p.sk = sk;
    p.Hq = (int)Hq; p.Hkv = (int)Hkv; p.N = (int)N;
    dense_strides(p.qs, Hq, N, D);
    dense_strides(p.ks, Hkv, N, D);
    dense_strides(p.vs, Hkv, N, D);
    dense_strides(p.os, Hq, N, D);
    for (int i = 0; i < 3; ++i) {
        if (v_strides) p.vs[i] = (long)v_strides[i];
        if (o_strides) p.os[i] = (long)o_strides[i];
    }
    p.bq = (int)bq; p.bk = (int)bk;
    p.scale = scale;
    const bool dbg = dbg_logits != nullptr;
    ARHIP_REQUIRE(!(fp8 && dbg), "arhip_sage_fwd_fp8: the logits export is an int8 facility");
    const bool c = causal != 0, hm = mask != nullptr, f32o = out_dtype == ARHIP_F32;
    p.out_f32 = f32o;
    // K scales that are uniform over a 64-key tile (bk = 64 * 2^n) take the fast kernel; anything
    // else, including the reference's per-key scales (bk == 1), stages the tile's scales in LDS
    int shift = 0;
    while (((int64_t)64 << shift) < bk) ++shift;
    const bool per_key = ((int64_t)64 << shift) != bk;
    p.bk_tile_shift = shift;
    // ... in the general kernel; scales over a power of two of keys below 64 (the reference's bk = 1 among them)
    // have a form of the pipelined kernel that applies them per logit
    int key_shift = 0;
    while (((int64_t)1 << key_shift) < bk) ++key_shift;
    const bool pipe_keys = per_key && ((int64_t)1 << key_shift) == bk;
    p.bk_key_shift = pipe_keys ? key_shift : -1;
    int nw = pick_waves(dev, B * Hq, N, D, hm || (per_key && !pipe_keys) || dbg);
    if (nw == 1) nw = 4;
    if (nw == 8 && !pipe_addressable(N, std::max<int64_t>(D, v_strides ? v_strides[2] : D), 2)) nw = 4;
    const bool pipe = nw == 8 && (!per_key || pipe_keys) && !dbg;
    const bool pipe4 = pipe && pipe_wants_4_waves(dev, B * Hq, N, D, causal != 0, kv_len != nullptr);
    if (pipe4) nw = 4;
    p.nq = (int)((N + nw * 32 - 1) / (nw * 32));
    p.total = (int)(p.nq * B * Hq);
    p.lpt = p.total <= 16 * dev->cus;
    if (dbg) {
        p.dbg = dbg_logits;
        p.dbg_bh = dbg_sel[0]; p.dbg_qt = dbg_sel[1]; p.dbg_kt = dbg_sel[2];
        ARHIP_REQUIRE(p.dbg_bh >= 0 && p.dbg_bh < B * Hq && p.dbg_qt >= 0 && (int64_t)p.dbg_qt * 32 < N &&
                          p.dbg_kt >= 0 && (int64_t)p.dbg_kt * 64 < N,
                      "arhip_sage_fwd: debug tile selector out of range");
    }
    arhip_call_timer t{dev, wait, secs};
    t.kernel = ARHIP_K_SAGE;
    if (int rc = t.begin()) return rc;
#define SAGE_V(DD, NWW, PK, DB_, MK)                                                                   \
    do {                                                                                               \
        if (f32o) launch_attn<DD, NWW, MODE_I8, PK, true, DB_, MK>(dev->stream, p, c, hm);             \
        else launch_attn<DD, NWW, MODE_I8, PK, false, DB_, MK>(dev->stream, p, c, hm);                 \
    } while (0)
#define SAGE_D(DD)                                                                                     \
    do {                                                                                               \
        if (dbg) {                                                                                     \
            if (per_key) SAGE_V(DD, 4, true, true, false);                                             \
            else SAGE_V(DD, 4, false, true, false);                                                    \
        } else if (pipe && pipe_keys) launch_pipe_i8_keys(dev->stream, p, DD, c, nw);                  \
        else if (per_key) SAGE_V(DD, 4, true, false, true);                                            \
        else if (pipe) launch_pipe_i8(dev->stream, p, DD, c, nw);                                      \
        else SAGE_V(DD, 4, false, false, true);                                                        \
    } while (0)
#define SAGE_F(DD, PK)                                                                                 \
    do {                                                                                               \
        if (f32o) launch_attn<DD, 4, MODE_FP8, PK, true, false, true>(dev->stream, p, c, hm);          \
        else launch_attn<DD, 4, MODE_FP8, PK, false, false, true>(dev->stream, p, c, hm);              \
    } while (0)
    if (fp8 && pipe) {
        if (pipe_keys) launch_pipe_fp8_keys(dev->stream, p, (int)D, c, nw);
        else launch_pipe_fp8(dev->stream, p, (int)D, c, nw);
    } else if (fp8) {
        if (D == 64) { if (per_key) SAGE_F(64, true); else SAGE_F(64, false); }
        else { if (per_key) SAGE_F(128, true); else SAGE_F(128, false); }
    } else if (D == 64) SAGE_D(64);
    else SAGE_D(128);
#undef SAGE_F
#undef SAGE_D
#undef SAGE_V
    arhip_note_selected(ARHIP_K_SAGE);
    return t.end();
}

// Q quantised inside the attention kernel (as the reference does, src/runtime/cuda_flash_sage.rs:201-223): the
// pipelined int8 (FP8) kernel with bf16 queries, scales over blocks of 128 queries.
static int sage_fwd_qfused_impl(const char *who, bool fp8, arhip_device *dev, const uint16_t *q, const int8_t *k8, const float *sk,
                               const uint16_t *v, void *o, float *sq_out, int8_t *q8_out, const int32_t *kv_len,
                               int64_t B, int64_t Hq, int64_t Hkv, int64_t N, int64_t D, int64_t bk,
                               int causal, int out_dtype, float scale, int wait, double *secs)
{
    if (int rc = check_common(who, dev, q, k8, v, o, nullptr, B, Hq, Hkv, N, D)) return rc;
    ARHIP_REQUIRE(sk, "%s: null scale pointer", who);
    ARHIP_REQUIRE(out_dtype == ARHIP_F32 || out_dtype == ARHIP_BF16, "%s: out_dtype %d", who, out_dtype);
    int shift = 0;
    while (((int64_t)64 << shift) < bk) ++shift;
    ARHIP_REQUIRE(((int64_t)64 << shift) == bk, "%s: K scales over whole 64-key tiles (bk = 64 * 2^j), got bk = %lld", who,
                  (long long)bk);
    ARHIP_REQUIRE(pipe_addressable(N, D, 2), "%s: (N + 320) * D * 2 must stay below 2^31 (N = %lld)", who, (long long)N);
    ARHIP_REQUIRE(q8_out == nullptr || arhip_aligned16(q8_out), "%s: q8_out must be 16-byte aligned", who);
    ARHIP_HIP(hipSetDevice(dev->ordinal));
    AttnParams p = {};
    p.q = q; p.k = k8; p.v = v; p.o = o;
    p.kv_len = kv_len;
    p.sk = sk;
    p.sq_out = sq_out; p.q8_out = q8_out;
    p.Hq = (int)Hq; p.Hkv = (int)Hkv; p.N = (int)N;
    dense_strides(p.qs, Hq, N, D);
    dense_strides(p.ks, Hkv, N, D);
    dense_strides(p.vs, Hkv, N, D);
    dense_strides(p.os, Hq, N, D);
    p.bq = 128; p.bk = (int)bk;
    p.bk_tile_shift = shift;
    p.bk_key_shift = -1;
    p.scale = scale;
    const bool c = causal != 0;
    p.out_f32 = out_dtype == ARHIP_F32;
    const int nw = pipe_wants_4_waves(dev, B * Hq, N, D, c, kv_len != nullptr) ? 4 : 8;
    p.nq = (int)((N + nw * 32 - 1) / (nw * 32));
    p.total = (int)(p.nq * B * Hq);
    p.lpt = p.total <= 16 * dev->cus;
    arhip_call_timer t{dev, wait, secs};
    t.kernel = ARHIP_K_SAGE;
    if (int rc = t.begin()) return rc;
    if (fp8) launch_pipe_fp8_qf(dev->stream, p, (int)D, c, nw);
    else launch_pipe_i8_qf(dev->stream, p, (int)D, c, nw);
    arhip_note_selected(ARHIP_K_SAGE);
    return t.end();
}

extern "C" int arhip_sage_fwd_qfused(arhip_device *dev, const uint16_t *q, const int8_t *k8, const float *sk,
                                     const uint16_t *v, void *o, float *sq_out, int8_t *q8_out, const int32_t *kv_len,
                                     int64_t B, int64_t Hq, int64_t Hkv, int64_t N, int64_t D, int64_t bk,
                                     int causal, int out_dtype, float scale, int wait, double *secs)
{
    return sage_fwd_qfused_impl("arhip_sage_fwd_qfused", false, dev, q, k8, sk, v, o, sq_out, q8_out, kv_len, B, Hq, Hkv, N, D, bk,
                                causal, out_dtype, scale, wait, secs);
}

// The same on E4M3 codes (k8 from arhip_sage_quant_fp8; the kernel derives E4M3 codes of Q with scale = absmax / 448).
extern "C" int arhip_sage_fwd_fp8_qfused(arhip_device *dev, const uint16_t *q, const uint8_t *k8, const float *sk,
                                         const uint16_t *v, void *o, float *sq_out, uint8_t *q8_out, const int32_t *kv_len,
                                         int64_t B, int64_t Hq, int64_t Hkv, int64_t N, int64_t D, int64_t bk,
                                         int causal, int out_dtype, float scale, int wait, double *secs)
{
    return sage_fwd_qfused_impl("arhip_sage_fwd_fp8_qfused", true, dev, q, (const int8_t *)k8, sk, v, o, sq_out, (int8_t *)q8_out,
                                kv_len, B, Hq, Hkv, N, D, bk, causal, out_dtype, scale, wait, secs);
}

// The reference's own convention in one attention launch: f32 queries quantised row by row inside the kernel
// (src/runtime/cuda_flash_sage.rs:201-223), K scales per key (or per power of two of keys below 64).
extern "C" int arhip_sage_fwd_qfused_rows(arhip_device *dev, const float *q, const int8_t *k8, const float *sk,
                                          const uint16_t *v, void *o, float *sq_out, int8_t *q8_out, const int32_t *kv_len,
                                          int64_t B, int64_t Hq, int64_t Hkv, int64_t N, int64_t D, int64_t bk,
                                          int causal, int out_dtype, float scale, int wait, double *secs)
{
    if (int rc = check_common("arhip_sage_fwd_qfused_rows", dev, q, k8, v, o, nullptr, B, Hq, Hkv, N, D)) return rc;
    ARHIP_REQUIRE(sk, "arhip_sage_fwd_qfused_rows: null scale pointer");
    ARHIP_REQUIRE(out_dtype == ARHIP_F32 || out_dtype == ARHIP_BF16, "arhip_sage_fwd_qfused_rows: out_dtype %d", out_dtype);
    int key_shift = 0;
    while (((int64_t)1 << key_shift) < bk) ++key_shift;
    ARHIP_REQUIRE(bk >= 1 && bk < 64 && ((int64_t)1 << key_shift) == bk,
                  "arhip_sage_fwd_qfused_rows: K scales over a power of two of keys below 64 (bk = 1 ... 32), got bk = %lld", (long long)bk);
    ARHIP_REQUIRE(pipe_addressable(N, D, 2), "arhip_sage_fwd_qfused_rows: (N + 320) * D * 2 must stay below 2^31 (N = %lld)", (long long)N);
    ARHIP_REQUIRE(q8_out == nullptr || arhip_aligned16(q8_out), "arhip_sage_fwd_qfused_rows: q8_out must be 16-byte aligned");
    ARHIP_HIP(hipSetDevice(dev->ordinal));
    AttnParams p = {};
    p.q = q; p.k = k8; p.v = v; p.o = o;
    p.kv_len = kv_len;
    p.sk = sk;
    p.sq_out = sq_out; p.q8_out = q8_out;
    p.Hq = (int)Hq; p.Hkv = (int)Hkv; p.N = (int)N;
    dense_strides(p.qs, Hq, N, D);
    dense_strides(p.ks, Hkv, N, D);
    dense_strides(p.vs, Hkv, N, D);
    dense_strides(p.os, Hq, N, D);
    p.bq = 1; p.bk = (int)bk;
    p.bk_tile_shift = 0;
    p.bk_key_shift = key_shift;
    p.scale = scale;
    const bool c = causal != 0;
    p.out_f32 = out_dtype == ARHIP_F32;
    const int nw = pipe_wants_4_waves(dev, B * Hq, N, D, c, kv_len != nullptr) ? 4 : 8;
    p.nq = (int)((N + nw * 32 - 1) / (nw * 32));
    p.total = (int)(p.nq * B * Hq);
    p.lpt = p.total <= 16 * dev->cus;
    arhip_call_timer t{dev, wait, secs};
    t.kernel = ARHIP_K_SAGE;
    if (int rc = t.begin()) return rc;
    launch_pipe_i8_keys_qf(dev->stream, p, (int)D, c, nw);
    arhip_note_selected(ARHIP_K_SAGE);
    return t.end();
}

extern "C" int arhip_sage_fwd_strided(arhip_device *dev, const int8_t *q8, const int8_t *k8,
                                      const float *sq, const float *sk, const uint16_t *v, void *o,
                                      const int64_t v_strides[3], const int64_t o_strides[3],
                                      const float *mask, const int32_t *kv_len,
                                      int64_t B, int64_t Hq, int64_t Hkv, int64_t N, int64_t D,
                                      int64_t bq, int64_t bk, int causal, int out_dtype, float scale,
                                      int32_t *dbg_logits, const int32_t dbg_sel[3], int wait, double *secs)
{
    return sage_fwd_impl(dev, q8, k8, sq, sk, v, o, v_strides, o_strides, mask, kv_len, B, Hq, Hkv, N, D, bq, bk, causal,
                         out_dtype, scale, dbg_logits, dbg_sel, wait, secs, false);
}

extern "C" int arhip_sage_fwd_fp8(arhip_device *dev, const uint8_t *q8, const uint8_t *k8,
                                  const float *sq, const float *sk, const uint16_t *v, void *o,
                                  const float *mask, const int32_t *kv_len,
                                  int64_t B, int64_t Hq, int64_t Hkv, int64_t N, int64_t D,
                                  int64_t bq, int64_t bk, int causal, int out_dtype, float scale,
                                  int wait, double *secs)
{
    return sage_fwd_impl(dev, (const int8_t *)q8, (const int8_t *)k8, sq, sk, v, o, nullptr, nullptr, mask, kv_len, B, Hq, Hkv,
                         N, D, bq, bk, causal, out_dtype, scale, nullptr, nullptr, wait, secs, true);
}

extern "C" int arhip_flash_bwd(arhip_device *dev, const float *q, const float *k, const float *v, const float *o,
                               const float *lse, const float *dout, float *dq, float *dk, float *dv, float *delta,
                               const float *mask, const int32_t *kv_len,
                               int64_t B, int64_t Hq, int64_t Hkv, int64_t N, int64_t D,
                               int causal, float scale, int wait, double *secs)
{
    if (int rc = check_common("arhip_flash_bwd", dev, q, k, v, o, mask, B, Hq, Hkv, N, D)) return rc;
    ARHIP_REQUIRE(lse && dout && dq && dk && dv && delta, "arhip_flash_bwd: null tensor pointer");
    ARHIP_REQUIRE(arhip_aligned16(dout) && arhip_aligned16(dq) && arhip_aligned16(dk) && arhip_aligned16(dv),
                  "arhip_flash_bwd: dout/dq/dk/dv must be 16-byte aligned");
    ARHIP_REQUIRE(((reinterpret_cast<uintptr_t>(lse) | reinterpret_cast<uintptr_t>(delta)) & 3u) == 0,
                  "arhip_flash_bwd: lse/delta must be 4-byte aligned");
    ARHIP_HIP(hipSetDevice(dev->ordinal));
    arhip_call_timer t{dev, wait, secs};
    t.kernel = ARHIP_K_FLASH_BWD;
    FlashBwdParams p = {};
    p.q = q; p.k = k; p.v = v; p.dout = dout; p.lse = lse; p.delta = delta; p.mask = mask; p.kv_len = kv_len;
    p.dq = dq; p.dk = dk; p.dv = dv;
    p.Hq = (int)Hq; p.Hkv = (int)Hkv; p.N = (int)N;
    p.scale = scale;
    if (int rc = t.begin()) return rc;
    const long rows = (long)(B * Hq * N);
    // 4 waves per workgroup: 128 queries / keys when that still fills the chip, else the same 32
    // queries / keys with the tiles of the other side dealt out between the waves
    const bool split = B * Hkv * ((N + 127) / 128) < 2 * (int64_t)dev->cus;
    const int rows_wg = split ? 32 : 128;
    const int nt = (int)((N + rows_wg - 1) / rows_wg);
    const dim3 block(256), grid_prep((unsigned)((rows + 3) / 4)), grid_q((unsigned)(nt * B * Hq)),
        grid_kv((unsigned)(nt * B * Hkv));
    p.nt = nt;
    // causal: longest tile first over all heads, so that no head's long tiles are left for the end
    p.total_q = (int)(nt * B * Hq);
    p.total_kv = (int)(nt * B * Hkv);
    p.lpt_q = causal ? (int)(B * Hq) : 0;
    p.lpt_kv = causal ? (int)(B * Hkv) : 0;
#define BWD_LAUNCH(DD, SP)                                                                              \
    do {                                                                                                \
        hipLaunchKernelGGL((bwd_prep_kernel<DD>), grid_prep, dim3(256), 0, dev->stream, o, dout, delta, rows); \
        if (causal) {                                                                                   \
            hipLaunchKernelGGL((bwd_dq_kernel<DD, 4, true, SP>), grid_q, block, 0, dev->stream, p);     \
            hipLaunchKernelGGL((bwd_dkv_kernel<DD, 4, true, SP>), grid_kv, block, 0, dev->stream, p);   \
        } else {                                                                                        \
            hipLaunchKernelGGL((bwd_dq_kernel<DD, 4, false, SP>), grid_q, block, 0, dev->stream, p);    \
            hipLaunchKernelGGL((bwd_dkv_kernel<DD, 4, false, SP>), grid_kv, block, 0, dev->stream, p);  \
        }                                                                                               \
    } while (0)
    if (D == 64) { if (split) BWD_LAUNCH(64, true); else BWD_LAUNCH(64, false); }
    else { if (split) BWD_LAUNCH(128, true); else BWD_LAUNCH(128, false); }
#undef BWD_LAUNCH
    arhip_note_selected(ARHIP_K_FLASH_BWD);
    return t.end();
}
