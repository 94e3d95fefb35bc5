// Sage pre-pass: K mean (smoothing), per-block symmetric int8 quantisation,
// and the f32 -> bf16 cast of V.  All of it is HBM-bound streaming work.
//
// The quantisation rule is the reference's (src/runtime/cuda_flash_sage.rs):
//   scale = absmax > 0 ? absmax / 127 : 1      (:209-213, :264-268)
//   inv   = 1 / scale                          (:218, :273)
//   x8    = clamp(rint(x * inv), -127, 127)    (:124-137), rint = nearest-even
// hoisted out of the attention kernel (the reference re-quantises K for every
// query block, :248-278) and applied to blocks of tokens instead of single
// rows.  Every fp32 operation is a single IEEE operation in a fixed order, so
// the int8 tensors and scales are bit-reproducible on the CPU.
#include "arhip_internal.h"

#include <mutex>

#pragma clang fp contract(off)

// Scratch of arhip_sage_quant_static, resident on the device: the partial channel sums of the K
// mean.  Each GPU the library runs on holds its own copy until the process ends.
constexpr size_t STATIC_SCRATCH_FLOATS = (size_t)4 << 20;  // 16 MiB
static __device__ __align__(256) float scratch[STATIC_SCRATCH_FLOATS];

// Device address of `scratch` per GPU ordinal, resolved once per device in
// arhip_static_scratch_setup.  In host code the array's name is only a stand-in for the symbol,
// not a device address: kernels, copies and fills always get the resolved pointer.
constexpr int MAX_DEVICES = 64;
static float *g_scratch_ptr[MAX_DEVICES];
static std::mutex g_scratch_mutex;

namespace {

constexpr int MEAN_CHUNK = 64;  // tokens per partial sum


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
__global__ void __launch_bounds__(256) k_mean_partial_kernel(const T *x, float *part, int N, int D, int nchunk)
{
    const int gpr = D / 8;                       // 8-channel groups per row
    const int cpb = 256 / gpr;                   // chunks per workgroup
    const int c = blockIdx.x * cpb + threadIdx.x / gpr;
    const int g = threadIdx.x % gpr, bh = blockIdx.y;
    if (c >= nchunk) return;
    const int j0 = c * MEAN_CHUNK;
    const int j1 = min(N, j0 + MEAN_CHUNK);
    const size_t base = (size_t)bh * N * D + g * 8;
    float s[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    for (int j = j0; j < j1; ++j) {
        float v[8];
        ld8(x, base + (size_t)j * D, v);
#pragma unroll
        for (int i = 0; i < 8; ++i) s[i] += v[i];
    }
    float *o = part + ((size_t)bh * nchunk + c) * D + g * 8;
    *(float4 *)o = make_float4(s[0], s[1], s[2], s[3]);
    *(float4 *)(o + 4) = make_float4(s[4], s[5], s[6], s[7]);
}

// mean[bh][d] = (part[0] + part[1] + ...) / N in chunk order (loads batched, adds in order)
__global__ void k_mean_final_kernel(const float *part, float *mean, int N, int D, int nchunk)
{
    const int bh = blockIdx.x, d = threadIdx.x;
    const float *p = part + (size_t)bh * nchunk * D + d;
    float tot = 0.f;
    int c = 0;
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

// One workgroup per (block of `blk` tokens, head).  Blocks of up to 256*64 elements are kept
// in registers between the absmax pass and the quantising pass (one trip to memory); larger
// ones are read twice.
template <typename T, bool SMOOTH>
__global__ void __launch_bounds__(256) quant_blocks_kernel(const T *x, int8_t *x8, float *scales, const float *mean,
                                                           int N, int D, int blk, int nblk)
{
    constexpr int KEEP = 8;  // 8-element groups a thread can hold
    __shared__ float red[4];
    const int bi = blockIdx.x, bh = blockIdx.y, tid = threadIdx.x;
    const int r0 = bi * blk;
    const int r1 = min(N, r0 + blk);
    const size_t base = ((size_t)bh * N + r0) * D;
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
                ld8(x, base + e, held[it]);
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
            ld8(x, base + e, v);
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

    const float scale = (mx > 0.f) ? mx / 127.0f : 1.f;
    const float inv = 1.f / scale;
    if (tid == 0) scales[(size_t)bh * nblk + bi] = scale;

    auto quant8 = [&](const float (&v)[8]) {
        uint32_t w[2] = {0u, 0u};
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            int iv = (int)rintf(v[i] * inv);
            iv = iv < -127 ? -127 : (iv > 127 ? 127 : iv);
            w[i >> 2] |= ((uint32_t)iv & 0xffu) << ((i & 3) * 8);
        }
        return make_uint2(w[0], w[1]);
    };
    if (keep) {
#pragma unroll
        for (int it = 0; it < KEEP; ++it) {
            const int e = (it * 256 + tid) * 8;
            if (e < nelem) *(uint2 *)(x8 + base + e) = quant8(held[it]);
        }
    } else {
        for (int e = tid * 8; e < nelem; e += 256 * 8) {
            float v[8];
            ld8(x, base + e, v);
            const int d = e % D;
            if (SMOOTH) {
#pragma unroll
                for (int i = 0; i < 8; ++i) v[i] = v[i] - mu[d + i];
            }
            *(uint2 *)(x8 + base + e) = quant8(v);
        }
    }
}

// The reference's own granularity, one scale per token row (block == 1): D/8 lanes share a row,
// so a workgroup of 256 threads quantises 256/(D/8) rows and the absmax is a shuffle reduction
// inside the lane group.  Same arithmetic, same order of operations per element.
template <typename T, bool SMOOTH>
__global__ void __launch_bounds__(256) quant_rows_kernel(const T *x, int8_t *x8, float *scales, const float *mean,
                                                         int N, int D, long rows_total)
{
    const int gpr = D / 8;                                   // lanes per row (8 or 16)
    const long row = (long)blockIdx.x * (256 / gpr) + threadIdx.x / gpr;   // global row over [B*H*N]
    const int g = threadIdx.x % gpr;
    const bool live = row < rows_total;
    float v[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    if (live) {
        ld8(x, (size_t)row * D + g * 8, v);
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
    const float scale = (mx > 0.f) ? mx / 127.0f : 1.f;
    const float inv = 1.f / scale;
    if (live) {
        if (g == 0) scales[row] = scale;
        uint32_t w[2] = {0u, 0u};
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            int iv = (int)rintf(v[i] * inv);
            iv = iv < -127 ? -127 : (iv > 127 ? 127 : iv);
            w[i >> 2] |= ((uint32_t)iv & 0xffu) << ((i & 3) * 8);
        }
        *(uint2 *)(x8 + (size_t)row * D + g * 8) = make_uint2(w[0], w[1]);
    }
}

__global__ void __launch_bounds__(256) cast_bf16_kernel(const float *x, uint16_t *y, size_t n)
{
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
        const __bf16 b = (__bf16)x[i];  // round-to-nearest-even
        y[i] = __builtin_bit_cast(uint16_t, b);
    }
}

}  // namespace

extern "C" size_t arhip_sage_quant_workspace(int64_t B, int64_t H, int64_t N, int64_t D)
{
    if (B <= 0 || H <= 0 || N <= 0 || D <= 0) return 0;
    const int64_t nchunk = (N + MEAN_CHUNK - 1) / MEAN_CHUNK;
    return (size_t)(B * H * nchunk * D) * sizeof(float);
}

// Called by arhip_open with the device current: resolves this GPU's copy of `scratch`.
int arhip_static_scratch_setup(int ordinal)
{
    ARHIP_REQUIRE(ordinal >= 0 && ordinal < MAX_DEVICES, "device ordinal %d beyond %d", ordinal, MAX_DEVICES);
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (g_scratch_ptr[ordinal] != nullptr) return ARHIP_OK;
    float *ptr = nullptr;
    ARHIP_HIP(hipGetSymbolAddress((void **)&ptr, HIP_SYMBOL(scratch)));
    ARHIP_REQUIRE(ptr != nullptr, "hipGetSymbolAddress returned a null scratch address for device %d", ordinal);
    g_scratch_ptr[ordinal] = ptr;
    return ARHIP_OK;
}

static int sage_quant_impl(arhip_device *dev, const void *x, int8_t *x8, float *scales, float *mean,
                           void *workspace, int64_t B, int64_t H, int64_t N, int64_t D,
                           int64_t block, int dtype, int smooth, int wait, double *secs, int prof_kernel)
{
    ARHIP_REQUIRE(dev != nullptr, "arhip_sage_quant: null device");
    ARHIP_REQUIRE(x && x8 && scales, "arhip_sage_quant: null pointer");
    ARHIP_REQUIRE(B > 0 && H > 0 && N > 0 && block > 0, "arhip_sage_quant: empty shape");
    if (D != 64 && D != 128) return arhip_fail(ARHIP_EUNSUPPORTED, "arhip_sage_quant: head_dim %lld (64 or 128)", (long long)D);
    ARHIP_REQUIRE(dtype == ARHIP_F32 || dtype == ARHIP_BF16, "arhip_sage_quant: dtype %d", dtype);
    ARHIP_REQUIRE(B * H <= 65535, "arhip_sage_quant: B*H = %lld exceeds the grid limit", (long long)(B * H));
    ARHIP_REQUIRE(arhip_aligned16(x) && (reinterpret_cast<uintptr_t>(x8) & 7u) == 0,
                  "arhip_sage_quant: x must be 16-byte and x8 8-byte aligned");
    ARHIP_REQUIRE(!smooth || (mean && workspace), "arhip_sage_quant: smoothing needs mean and workspace buffers");
    ARHIP_HIP(hipSetDevice(dev->ordinal));
    const int nblk = (int)((N + block - 1) / block);
    const int nchunk = (int)((N + MEAN_CHUNK - 1) / MEAN_CHUNK);
    const dim3 qgrid((unsigned)nblk, (unsigned)(B * H));
    arhip_call_timer t{dev, wait, secs};
    t.kernel = prof_kernel;
    if (int rc = t.begin()) return rc;
    if (smooth) {
        const int cpb = 256 / (int)(D / 8);  // chunks per workgroup
        const dim3 pgrid((unsigned)((nchunk + cpb - 1) / cpb), (unsigned)(B * H));
        if (dtype == ARHIP_F32)
            hipLaunchKernelGGL(k_mean_partial_kernel<float>, pgrid, dim3(256), 0, dev->stream,
                               (const float *)x, (float *)workspace, (int)N, (int)D, nchunk);
        else
            hipLaunchKernelGGL(k_mean_partial_kernel<uint16_t>, pgrid, dim3(256), 0, dev->stream,
                               (const uint16_t *)x, (float *)workspace, (int)N, (int)D, nchunk);
        hipLaunchKernelGGL(k_mean_final_kernel, dim3((unsigned)(B * H)), dim3((unsigned)D), 0, dev->stream,
                           (const float *)workspace, mean, (int)N, (int)D, nchunk);
    }
    if (block == 1) {  // scales [B,H,N]: one per row
        const long rows = (long)(B * H * N);
        const int rpb = 256 / (int)(D / 8);
        const dim3 rgrid((unsigned)((rows + rpb - 1) / rpb));
        if (smooth) {
            if (dtype == ARHIP_F32)
                hipLaunchKernelGGL((quant_rows_kernel<float, true>), rgrid, dim3(256), 0, dev->stream,
                                   (const float *)x, x8, scales, mean, (int)N, (int)D, rows);
            else
                hipLaunchKernelGGL((quant_rows_kernel<uint16_t, true>), rgrid, dim3(256), 0, dev->stream,
                                   (const uint16_t *)x, x8, scales, mean, (int)N, (int)D, rows);
        } else {
            if (dtype == ARHIP_F32)
                hipLaunchKernelGGL((quant_rows_kernel<float, false>), rgrid, dim3(256), 0, dev->stream,
                                   (const float *)x, x8, scales, nullptr, (int)N, (int)D, rows);
            else
                hipLaunchKernelGGL((quant_rows_kernel<uint16_t, false>), rgrid, dim3(256), 0, dev->stream,
                                   (const uint16_t *)x, x8, scales, nullptr, (int)N, (int)D, rows);
        }
    } else if (smooth) {
        if (dtype == ARHIP_F32)
            hipLaunchKernelGGL((quant_blocks_kernel<float, true>), qgrid, dim3(256), 0, dev->stream,
                               (const float *)x, x8, scales, mean, (int)N, (int)D, (int)block, nblk);
        else
            hipLaunchKernelGGL((quant_blocks_kernel<uint16_t, true>), qgrid, dim3(256), 0, dev->stream,
                               (const uint16_t *)x, x8, scales, mean, (int)N, (int)D, (int)block, nblk);
    } else {
        if (dtype == ARHIP_F32)
            hipLaunchKernelGGL((quant_blocks_kernel<float, false>), qgrid, dim3(256), 0, dev->stream,
                               (const float *)x, x8, scales, nullptr, (int)N, (int)D, (int)block, nblk);
        else
            hipLaunchKernelGGL((quant_blocks_kernel<uint16_t, false>), qgrid, dim3(256), 0, dev->stream,
                               (const uint16_t *)x, x8, scales, nullptr, (int)N, (int)D, (int)block, nblk);
    }
    arhip_note_selected(ARHIP_K_SAGE_QUANT);
    return t.end();
}

extern "C" int arhip_sage_quant(arhip_device *dev, const void *x, int8_t *x8, float *scales, float *mean,
                                void *workspace, int64_t B, int64_t H, int64_t N, int64_t D,
                                int64_t block, int dtype, int smooth, int wait, double *secs)
{
    return sage_quant_impl(dev, x, x8, scales, mean, workspace, B, H, N, D, block, dtype, smooth, wait, secs,
                           ARHIP_K_SAGE_QUANT);
}

extern "C" size_t arhip_sage_quant_static_limit(void) { return STATIC_SCRATCH_FLOATS * sizeof(float); }

// The same kernels with the partial sums in the library's own device array: no allocation here,
// none asked of the caller.  The launches are not entered in the per-kernel profile log, which
// would create events.  Every chunk the final reduction reads is written by the partial-sum
// kernel of the same call first, so nothing has to be cleared between calls; two calls that
// overlap on one GPU (different streams or handles) race on the array.
extern "C" int arhip_sage_quant_static(arhip_device *dev, const void *x, int8_t *x8, float *scales, float *mean,
                                       int64_t B, int64_t H, int64_t N, int64_t D,
                                       int64_t block, int dtype, int smooth, int wait, double *secs)
{
    ARHIP_REQUIRE(dev != nullptr, "arhip_sage_quant_static: null device");
    float *ws = nullptr;
    if (smooth) {
        const size_t need = arhip_sage_quant_workspace(B, H, N, D);
        if (need > STATIC_SCRATCH_FLOATS * sizeof(float))
            return arhip_fail(ARHIP_EINVAL,
                              "arhip_sage_quant_static: B*H*ceil(N/64)*D*4 = %zu bytes of partial sums exceed the "
                              "built-in %zu-byte scratch; use arhip_sage_quant with a caller workspace",
                              need, STATIC_SCRATCH_FLOATS * sizeof(float));
        ARHIP_REQUIRE(dev->ordinal >= 0 && dev->ordinal < MAX_DEVICES && g_scratch_ptr[dev->ordinal] != nullptr,
                      "arhip_sage_quant_static: the scratch address of device %d was not resolved at open", dev->ordinal);
        ws = g_scratch_ptr[dev->ordinal];
    }
    return sage_quant_impl(dev, x, x8, scales, mean, ws, B, H, N, D, block, dtype, smooth, wait, secs, -1);
}

extern "C" int arhip_cast_bf16(arhip_device *dev, const float *x, uint16_t *y, int64_t n, int wait, double *secs)
{
    ARHIP_REQUIRE(dev != nullptr, "arhip_cast_bf16: null device");
    ARHIP_REQUIRE(n >= 0 && (n == 0 || (x && y)), "arhip_cast_bf16: null pointer");
    ARHIP_HIP(hipSetDevice(dev->ordinal));
    arhip_call_timer t{dev, wait, secs};
    if (int rc = t.begin()) return rc;
    if (n > 0) {
        size_t blocks = ((size_t)n + 255) / 256;
        if (blocks > 16384) blocks = 16384;
        hipLaunchKernelGGL(cast_bf16_kernel, dim3((unsigned)blocks), dim3(256), 0, dev->stream, x, y, (size_t)n);
    }
    return t.end();
}
