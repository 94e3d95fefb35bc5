// arhip_sage_quant / arhip_cast_bf16: argument checks and launches of the Sage pre-pass
// (kernels in sage_quant_kernels.h), and the entry point that allocates nothing.
#include "arhip_internal.h"
#include "sage_quant_kernels.h"

#include <algorithm>
#include <mutex>

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

using namespace arhip;

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

// block == 1: one scale per row (scales [B,H,N]); otherwise one workgroup per (block, head)
template <typename T, bool SMOOTH, bool FP8>
static void launch_quant(arhip_device *dev, const void *x, int8_t *x8, float *scales, const float *mean, int64_t N, int64_t D,
                         int64_t block, int nblk, long rows, int64_t heads, const XLayout &lay)
{
    if (block == 1) {
        const int rpb = 256 / (int)(D / 8);
        hipLaunchKernelGGL((quant_rows_kernel<T, SMOOTH, FP8>), dim3((unsigned)((rows + rpb - 1) / rpb)), dim3(256), 0,
                           dev->stream, (const T *)x, x8, scales, mean, (int)N, (int)D, rows, lay);
    } else {
        hipLaunchKernelGGL((quant_blocks_kernel<T, SMOOTH, FP8>), dim3((unsigned)nblk, (unsigned)heads), dim3(256), 0,
                           dev->stream, (const T *)x, x8, scales, mean, (int)N, (int)D, (int)block, nblk, lay);
    }
}

static int sage_quant_impl(arhip_device *dev, const void *x, const int64_t x_strides[3], int8_t *x8, float *scales, float *mean,
                           void *workspace, int64_t B, int64_t H, int64_t N, int64_t D,
                           int64_t block, int dtype, int smooth, int wait, double *secs, int prof_kernel, bool fp8 = false)
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
    XLayout lay = XLayout::dense((int)H, (int)N, (int)D);
    if (x_strides) {
        // rows stay 16-byte aligned and do not overlap: multiples of 8 elements, token stride >= D
        for (int i = 0; i < 3; ++i)
            ARHIP_REQUIRE(x_strides[i] >= 0 && x_strides[i] % 8 == 0 && (i != 2 || x_strides[i] >= D),
                          "arhip_sage_quant_strided: stride %lld (multiples of 8 elements, token stride >= D)",
                          (long long)x_strides[i]);
        lay = XLayout{(long)x_strides[0], (long)x_strides[1], (long)x_strides[2], (int)H};
    }
    ARHIP_HIP(hipSetDevice(dev->ordinal));
    const int nblk = (int)((N + block - 1) / block);
    const int nchunk = (int)((N + MEAN_CHUNK - 1) / MEAN_CHUNK);
    arhip_call_timer t{dev, wait, secs};
    t.kernel = prof_kernel;
    if (int rc = t.begin()) return rc;
    if (smooth) {
        const int cpb = 256 / (int)(D / 8);  // chunks per workgroup
        const dim3 pgrid((unsigned)((nchunk + cpb - 1) / cpb), (unsigned)(B * H));
        if (dtype == ARHIP_F32)
            hipLaunchKernelGGL(k_mean_partial_kernel<float>, pgrid, dim3(256), 0, dev->stream,
                               (const float *)x, (float *)workspace, (int)N, (int)D, nchunk, lay);
        else
            hipLaunchKernelGGL(k_mean_partial_kernel<uint16_t>, pgrid, dim3(256), 0, dev->stream,
                               (const uint16_t *)x, (float *)workspace, (int)N, (int)D, nchunk, lay);
        hipLaunchKernelGGL(k_mean_final_kernel, dim3((unsigned)(B * H)), dim3((unsigned)D), 0, dev->stream,
                           (const float *)workspace, mean, (int)N, (int)D, nchunk);
    }
    const long rows = (long)(B * H * N);
    if (dtype == ARHIP_F32) {
        if (smooth) fp8 ? launch_quant<float, true, true>(dev, x, x8, scales, mean, N, D, block, nblk, rows, B * H, lay)
                        : launch_quant<float, true, false>(dev, x, x8, scales, mean, N, D, block, nblk, rows, B * H, lay);
        else fp8 ? launch_quant<float, false, true>(dev, x, x8, scales, nullptr, N, D, block, nblk, rows, B * H, lay)
                 : launch_quant<float, false, false>(dev, x, x8, scales, nullptr, N, D, block, nblk, rows, B * H, lay);
    } else {
        if (smooth) fp8 ? launch_quant<uint16_t, true, true>(dev, x, x8, scales, mean, N, D, block, nblk, rows, B * H, lay)
                        : launch_quant<uint16_t, true, false>(dev, x, x8, scales, mean, N, D, block, nblk, rows, B * H, lay);
        else fp8 ? launch_quant<uint16_t, false, true>(dev, x, x8, scales, nullptr, N, D, block, nblk, rows, B * H, lay)
                 : launch_quant<uint16_t, false, false>(dev, x, x8, scales, nullptr, N, D, block, nblk, rows, B * H, lay);
    }
    arhip_note_selected(ARHIP_K_SAGE_QUANT);
    return t.end();
}

extern "C" int arhip_sage_quant(arhip_device *dev, const void *x, int8_t *x8, float *scales, float *mean,
                                void *workspace, int64_t B, int64_t H, int64_t N, int64_t D,
                                int64_t block, int dtype, int smooth, int wait, double *secs)
{
    return sage_quant_impl(dev, x, nullptr, x8, scales, mean, workspace, B, H, N, D, block, dtype, smooth, wait, secs,
                           ARHIP_K_SAGE_QUANT);
}

extern "C" int arhip_sage_quant_strided(arhip_device *dev, const void *x, const int64_t x_strides[3], int8_t *x8,
                                        float *scales, float *mean, void *workspace, int64_t B, int64_t H, int64_t N,
                                        int64_t D, int64_t block, int dtype, int smooth, int wait, double *secs)
{
    ARHIP_REQUIRE(x_strides != nullptr, "arhip_sage_quant_strided: null strides");
    return sage_quant_impl(dev, x, x_strides, x8, scales, mean, workspace, B, H, N, D, block, dtype, smooth, wait, secs,
                           ARHIP_K_SAGE_QUANT);
}

extern "C" int arhip_sage_quant_fp8(arhip_device *dev, const void *x, uint8_t *x8, float *scales, float *mean,
                                    void *workspace, int64_t B, int64_t H, int64_t N, int64_t D,
                                    int64_t block, int dtype, int smooth, int wait, double *secs)
{
    return sage_quant_impl(dev, x, nullptr, (int8_t *)x8, scales, mean, workspace, B, H, N, D, block, dtype, smooth, wait, secs,
                           ARHIP_K_SAGE_QUANT, true);
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
    return sage_quant_impl(dev, x, nullptr, x8, scales, mean, ws, B, H, N, D, block, dtype, smooth, wait, secs, -1);
}

extern "C" int arhip_sage_prep_kv_rows(arhip_device *dev, const float *k, int8_t *k8, float *sk, const float *v, uint16_t *vb,
                                       int64_t B, int64_t Hkv, int64_t N, int64_t D, int wait, double *secs)
{
    ARHIP_REQUIRE(dev != nullptr, "arhip_sage_prep_kv_rows: null device");
    ARHIP_REQUIRE(k && k8 && sk && v && vb, "arhip_sage_prep_kv_rows: null pointer");
    ARHIP_REQUIRE(B > 0 && Hkv > 0 && N > 0 && (D == 64 || D == 128), "arhip_sage_prep_kv_rows: shape B=%lld Hkv=%lld N=%lld D=%lld",
                  (long long)B, (long long)Hkv, (long long)N, (long long)D);
    ARHIP_REQUIRE(arhip_aligned16(k) && arhip_aligned16(k8) && arhip_aligned16(v) && arhip_aligned16(vb),
                  "arhip_sage_prep_kv_rows: tensors must be 16-byte aligned");
    ARHIP_HIP(hipSetDevice(dev->ordinal));
    const long rows = (long)(B * Hkv * N), nv = rows * (long)D;
    const int rpb = 256 / (int)(D / 8);
    const long row_blocks = (rows + rpb - 1) / rpb;
    const long cast_blocks = std::min<long>((nv + 255) / 256, 16384);
    ARHIP_REQUIRE(row_blocks + cast_blocks < ((long)1 << 31), "arhip_sage_prep_kv_rows: too many rows");
    arhip_call_timer t{dev, wait, secs};
    t.kernel = ARHIP_K_SAGE_QUANT;
    if (int rc = t.begin()) return rc;
    hipLaunchKernelGGL(quant_rows_cast_kernel, dim3((unsigned)(row_blocks + cast_blocks)), dim3(256), 0, dev->stream, k, k8, sk, v, vb,
                       (int)N, (int)D, rows, nv, (int)row_blocks);
    return t.end();
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
