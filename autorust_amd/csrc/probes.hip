// MFMA lane-layout probes, launched through the generic host-kernel seam
// (arhip_module_load + arhip_launch).  They are to this build what
// tests/sage_layout_probe.rs is to the reference: a known-answer check that
// pins the matrix-instruction operand/result layouts the attention kernel
// relies on.
//
// Every probe multiplies A[M x K] (row-major) by B[K x N] (row-major) with ONE
// MFMA, loading operands with the lane mapping the attention kernel assumes and
// scattering the result with the assumed result layout.  If the assumed layouts
// are right, C == A.B exactly (small integers).
#include <hip/hip_runtime.h>
#include <stdint.h>

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(4))) int i32x4;
typedef __attribute__((ext_vector_type(16))) int i32x16;

// A int8 [32 x 32], B int8 [32 x 32] (k rows), C int32 [32 x 32]
extern "C" __global__ void probe_i8_32x32x32(const int8_t *A, const int8_t *B, int32_t *C)
{
    const int lane = threadIdx.x, i = lane & 31, h = lane >> 5;
    int8_t a[16], b[16];
    for (int t = 0; t < 16; ++t) {
        a[t] = A[i * 32 + 16 * h + t];        // row i, k = 16h + t
        b[t] = B[(16 * h + t) * 32 + i];      // k = 16h + t, column i
    }
    i32x4 av, bv;
    __builtin_memcpy(&av, a, 16);
    __builtin_memcpy(&bv, b, 16);
    i32x16 acc;
    for (int r = 0; r < 16; ++r) acc[r] = 0;
    acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(av, bv, acc, 0, 0, 0);
    for (int r = 0; r < 16; ++r) C[(8 * (r >> 2) + 4 * h + (r & 3)) * 32 + i] = acc[r];
}

// A bf16 bits [32 x 16], B bf16 bits [16 x 32], C f32 [32 x 32]
extern "C" __global__ void probe_bf16_32x32x16(const uint16_t *A, const uint16_t *B, float *C)
{
    const int lane = threadIdx.x, i = lane & 31, h = lane >> 5;
    uint16_t a[8], b[8];
    for (int t = 0; t < 8; ++t) {
        a[t] = A[i * 16 + 8 * h + t];
        b[t] = B[(8 * h + t) * 32 + i];
    }
    bf16x8 av, bv;
    __builtin_memcpy(&av, a, 16);
    __builtin_memcpy(&bv, b, 16);
    f32x16 acc;
    for (int r = 0; r < 16; ++r) acc[r] = 0.f;
    acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(av, bv, acc, 0, 0, 0);
    for (int r = 0; r < 16; ++r) C[(8 * (r >> 2) + 4 * h + (r & 3)) * 32 + i] = acc[r];
}

// The reference's own known answer (tests/sage_layout_probe.rs:73-84):
// A int8 [16 x 32], B int8 [32 x 8], C int32 [16 x 8], here computed with the
// 32x32x32 instruction on zero-padded operands.
extern "C" __global__ void probe_i8_16x8_padded(const int8_t *A, const int8_t *B, int32_t *C)
{
    const int lane = threadIdx.x, i = lane & 31, h = lane >> 5;
    int8_t a[16], b[16];
    for (int t = 0; t < 16; ++t) {
        a[t] = (i < 16) ? A[i * 32 + 16 * h + t] : (int8_t)0;
        b[t] = (i < 8) ? B[(16 * h + t) * 8 + i] : (int8_t)0;
    }
    i32x4 av, bv;
    __builtin_memcpy(&av, a, 16);
    __builtin_memcpy(&bv, b, 16);
    i32x16 acc;
    for (int r = 0; r < 16; ++r) acc[r] = 0;
    acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(av, bv, acc, 0, 0, 0);
    for (int r = 0; r < 16; ++r) {
        const int row = 8 * (r >> 2) + 4 * h + (r & 3);
        if (row < 16 && i < 8) C[row * 8 + i] = acc[r];
    }
}

// The trivial kernel of tests/host_kernel.rs:28-61: y[i] = x[i] * 3 + 1.
extern "C" __global__ void probe_axpb(const float *x, float *y, int n)
{
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) y[i] = x[i] * 3.0f + 1.0f;
}

// Plain streaming copy of n 16-byte words: the calibration kernel for the HBM traffic
// counters (its traffic is known: n*16 bytes read, n*16 bytes written).
extern "C" __global__ void probe_copy(const uint4 *src, uint4 *dst, long n)
{
    const long stride = (long)gridDim.x * blockDim.x;
    for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) dst[i] = src[i];
}

// Sustained rate of the bf16 matrix instruction on operands taken from memory, with the shader
// clock it ran at: 8 waves per workgroup issue independent 32x32x16 MFMAs back to back (8 distinct
// A and B operands, 4 accumulators) and lane 0 of every workgroup records the shader-clock and
// 100 MHz real-time ticks of the loop.  On random operands the chip lowers its clock to stay
// inside its power limit, so this is the matrix rate a kernel can reach at best on real data.
extern "C" __global__ void __launch_bounds__(512) probe_mfma_rate(const uint4 *src, float *out, long long *ticks, int iters)
{
    bf16x8 a[8], b[8];
    for (int j = 0; j < 8; ++j) {
        a[j] = __builtin_bit_cast(bf16x8, src[(threadIdx.x * 16 + j) & 8191]);
        b[j] = __builtin_bit_cast(bf16x8, src[(threadIdx.x * 16 + 8 + j) & 8191]);
    }
    f32x16 o[4];
    for (int n = 0; n < 4; ++n)
        for (int r = 0; r < 16; ++r) o[n][r] = 0.f;
    const long long t0 = __builtin_readcyclecounter(), r0 = __builtin_amdgcn_s_memrealtime();
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int j = 0; j < 8; ++j) o[j & 3] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[j], b[j], o[j & 3], 0, 0, 0);
    }
    const long long t1 = __builtin_readcyclecounter(), r1 = __builtin_amdgcn_s_memrealtime();
    float r = 0.f;
    for (int n = 0; n < 4; ++n)
        for (int i = 0; i < 16; ++i) r += o[n][i];
    out[blockIdx.x * blockDim.x + threadIdx.x] = r;
    if (threadIdx.x == 0) {
        ticks[blockIdx.x * 2] = t1 - t0;
        ticks[blockIdx.x * 2 + 1] = r1 - r0;
    }
}

// Shader-clock sampler: one wave that, `samples` times, sleeps for a few microseconds and records
// the shader-clock and real-time (100 MHz) ticks that went by.  Launched on a second stream next
// to the kernel under test, it reports the clock that kernel actually ran at.
extern "C" __global__ void probe_clock_sampler(long long *ticks, int samples, int naps)
{
    if (threadIdx.x != 0) return;
    for (int i = 0; i < samples; ++i) {
        const long long t0 = __builtin_readcyclecounter(), r0 = __builtin_amdgcn_s_memrealtime();
        for (int k = 0; k < naps; ++k) __builtin_amdgcn_s_sleep(127);
        const long long t1 = __builtin_readcyclecounter(), r1 = __builtin_amdgcn_s_memrealtime();
        ticks[2 * i] = t1 - t0;
        ticks[2 * i + 1] = r1 - r0;
    }
}

// What the vector ALU can still issue beside the matrix pipe: every wave runs `iters` times
// { 1 matrix instruction (bf16 32x32x16 or int8 32x32x32, four accumulators in turn); K independent
// vector instructions (v_fma_f32 or v_exp_f32) } and records the shader-clock ticks (s_memtime) and
// the real-time (100 MHz) ticks of its loop: ticks[2 w] and ticks[2 w + 1] for wave w of the grid.
// The workgroup size sets the waves per SIMD (256 threads: one, 512: two like the attention kernels,
// 768: three).  With K = 0 the loop runs at the matrix rate; the growth with K is what the softmax
// instructions between the matrix instructions of an attention block cost, and the shader-clock
// figures separate an issue limit from a clock (power) limit.  One kernel per (matrix type, vector
// instruction, K).
template <int K, bool EXP, bool I8>
__device__ __forceinline__ void probe_issue_mix_body(const uint4 *src, float *out, long long *ticks, int iters)
{
    float d[8], a = threadIdx.x * 0.001f, b = 1.0001f;
    for (int i = 0; i < 8; ++i) d[i] = i * 0.5f;
    uint4 fa[4], fb[4];
    for (int j = 0; j < 4; ++j) {
        fa[j] = src[(threadIdx.x * 8 + j) & 8191];
        fb[j] = src[(threadIdx.x * 8 + 4 + j) & 8191];
    }
    f32x16 o[4];
    i32x16 oi[4];
    for (int n = 0; n < 4; ++n)
        for (int r = 0; r < 16; ++r) {
            o[n][r] = 0.f;
            oi[n][r] = 0;
        }
    const long long c0 = __builtin_readcyclecounter(), r0 = __builtin_amdgcn_s_memrealtime();
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            if constexpr (I8)
                oi[j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(__builtin_bit_cast(i32x4, fa[j]), __builtin_bit_cast(i32x4, fb[j]), oi[j], 0, 0, 0);
            else
                o[j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, fa[j]), __builtin_bit_cast(bf16x8, fb[j]), o[j], 0, 0, 0);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int i = 0; i < K; ++i) {
                if constexpr (EXP) asm volatile("v_exp_f32 %0, %1" : "+v"(d[i & 7]) : "v"(a));
                else asm volatile("v_fma_f32 %0, %1, %2, %0" : "+v"(d[i & 7]) : "v"(a), "v"(b));
            }
            __builtin_amdgcn_sched_barrier(0);
        }
    }
    const long long c1 = __builtin_readcyclecounter(), r1 = __builtin_amdgcn_s_memrealtime();
    float r = 0.f;
    for (int i = 0; i < 8; ++i) r += d[i];
    for (int n = 0; n < 4; ++n)
        for (int i = 0; i < 16; ++i) r += o[n][i] + (float)oi[n][i];
    out[blockIdx.x * blockDim.x + threadIdx.x] = r;
    if ((threadIdx.x & 63) == 0) {
        const int w = blockIdx.x * (blockDim.x / 64) + threadIdx.x / 64;
        ticks[2 * w] = c1 - c0;
        ticks[2 * w + 1] = r1 - r0;
    }
}
#define PROBE_ISSUE_MIX(NAME, K, EXP, I8)                                                                              \
    extern "C" __global__ void __launch_bounds__(768) NAME(const uint4 *src, float *out, long long *ticks, int iters)  \
    {                                                                                                                  \
        probe_issue_mix_body<K, EXP, I8>(src, out, ticks, iters);                                                      \
    }
#define PROBE_ISSUE_MIX_KS(PREFIX, EXP, I8)     \
    PROBE_ISSUE_MIX(PREFIX##_k0, 0, EXP, I8)    \
    PROBE_ISSUE_MIX(PREFIX##_k2, 2, EXP, I8)    \
    PROBE_ISSUE_MIX(PREFIX##_k4, 4, EXP, I8)    \
    PROBE_ISSUE_MIX(PREFIX##_k6, 6, EXP, I8)    \
    PROBE_ISSUE_MIX(PREFIX##_k8, 8, EXP, I8)    \
    PROBE_ISSUE_MIX(PREFIX##_k10, 10, EXP, I8)  \
    PROBE_ISSUE_MIX(PREFIX##_k14, 14, EXP, I8)  \
    PROBE_ISSUE_MIX(PREFIX##_k18, 18, EXP, I8)
PROBE_ISSUE_MIX_KS(probe_mix_bf16_fma, false, false)
PROBE_ISSUE_MIX_KS(probe_mix_bf16_exp, true, false)
PROBE_ISSUE_MIX_KS(probe_mix_i8_fma, false, true)
PROBE_ISSUE_MIX_KS(probe_mix_i8_exp, true, true)

// The same loop with 8 v_fma_f32 and S scalar instructions (s_add_u32) per matrix instruction: what a scalar
// instruction costs the SIMD's instruction issue.  ticks as above.
template <int S>
__device__ __forceinline__ void probe_issue_salu_body(const uint4 *src, float *out, long long *ticks, int iters)
{
    float d[8], a = threadIdx.x * 0.001f, b = 1.0001f;
    for (int i = 0; i < 8; ++i) d[i] = i * 0.5f;
    const uint4 fa = src[threadIdx.x & 1023], fb = src[(threadIdx.x + 512) & 1023];
    f32x16 o[4];
    for (int n = 0; n < 4; ++n)
        for (int r = 0; r < 16; ++r) o[n][r] = 0.f;
    int sacc = 0;
    const long long c0 = __builtin_readcyclecounter(), r0 = __builtin_amdgcn_s_memrealtime();
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            o[j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, fa), __builtin_bit_cast(bf16x8, fb), o[j], 0, 0, 0);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int i = 0; i < 8; ++i) asm volatile("v_fma_f32 %0, %1, %2, %0" : "+v"(d[i & 7]) : "v"(a), "v"(b));
#pragma unroll
            for (int i = 0; i < S; ++i) asm volatile("s_add_u32 %0, %0, 1" : "+s"(sacc));
            __builtin_amdgcn_sched_barrier(0);
        }
    }
    const long long c1 = __builtin_readcyclecounter(), r1 = __builtin_amdgcn_s_memrealtime();
    float r = (float)sacc;
    for (int i = 0; i < 8; ++i) r += d[i];
    for (int n = 0; n < 4; ++n)
        for (int i = 0; i < 16; ++i) r += o[n][i];
    out[blockIdx.x * blockDim.x + threadIdx.x] = r;
    if ((threadIdx.x & 63) == 0) {
        const int w = blockIdx.x * (blockDim.x / 64) + threadIdx.x / 64;
        ticks[2 * w] = c1 - c0;
        ticks[2 * w + 1] = r1 - r0;
    }
}
#define PROBE_ISSUE_SALU(NAME, S)                                                                                      \
    extern "C" __global__ void __launch_bounds__(768) NAME(const uint4 *src, float *out, long long *ticks, int iters)  \
    {                                                                                                                  \
        probe_issue_salu_body<S>(src, out, ticks, iters);                                                              \
    }
PROBE_ISSUE_SALU(probe_mix_salu_s0, 0)
PROBE_ISSUE_SALU(probe_mix_salu_s2, 2)
PROBE_ISSUE_SALU(probe_mix_salu_s4, 4)
PROBE_ISSUE_SALU(probe_mix_salu_s8, 8)

// How exactly the 8-bit floating-point matrix instructions add up their products: the dot product of
// two vectors of 64 E4M3 codes, once with the 64-deep scaled instruction and once with four 16-deep
// ones (every lane half takes the same bytes of both operands, so every element of the result is the
// same dot product whatever the operand layout is).  out[0] = 64-deep, out[1] = 4 x 16-deep.
extern "C" __global__ void probe_fp8_dot64(const unsigned char *a, const unsigned char *b, float *out)
{
    typedef __attribute__((ext_vector_type(8))) int i32x8;
    const int h = threadIdx.x >> 5;
    i32x8 av, bv;
    for (int j = 0; j < 8; ++j) {
        av[j] = ((const int *)(a + 32 * h))[j];
        bv[j] = ((const int *)(b + 32 * h))[j];
    }
    f32x16 acc;
    for (int r = 0; r < 16; ++r) acc[r] = 0.f;
    acc = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(av, bv, acc, 0, 0, 0, 0, 0, 0);
    f32x16 acc2;
    for (int r = 0; r < 16; ++r) acc2[r] = 0.f;
    for (int s = 0; s < 4; ++s) {
        const long a8 = *(const long *)(a + 16 * s + 8 * h), b8 = *(const long *)(b + 16 * s + 8 * h);
        acc2 = __builtin_amdgcn_mfma_f32_32x32x16_fp8_fp8(a8, b8, acc2, 0, 0, 0);
    }
    if (threadIdx.x == 37) {
        out[0] = acc[5];
        out[1] = acc2[5];
    }
}
