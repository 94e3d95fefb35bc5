// Device handle, memory, timing and the generic host-kernel launch of libarhip.
//
// Stands in for the reference's CUDA device (src/runtime/ops_cuda.rs): context
// and stream (:140-174), allocator (:595-685), module load and argument
// encoding (:888-1019).  One stream per handle, default priority.
#include "arhip_internal.h"

#include <algorithm>
#include <atomic>
#include <cstdlib>
#include <cstring>

static thread_local std::string g_last_error;

int arhip_fail(int code, const char *fmt, ...)
{
    char buf[1024];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof(buf), fmt, ap);
    va_end(ap);
    g_last_error = buf;
    return code;
}

extern "C" const char *arhip_last_error(void) { return g_last_error.c_str(); }

static std::atomic<uint64_t> g_selected[ARHIP_K_COUNT];

void arhip_note_selected(int kernel)
{
    if (kernel >= 0 && kernel < ARHIP_K_COUNT) g_selected[kernel].fetch_add(1, std::memory_order_relaxed);
}

extern "C" uint64_t arhip_selections(int kernel)
{
    if (kernel < 0 || kernel >= ARHIP_K_COUNT) return 0;
    return g_selected[kernel].load(std::memory_order_relaxed);
}

static int prof_event(arhip_device *dev, hipEvent_t *e)
{
    if (!dev->prof_pool.empty()) {
        *e = dev->prof_pool.back();
        dev->prof_pool.pop_back();
        return ARHIP_OK;
    }
    ARHIP_HIP(hipEventCreate(e));
    return ARHIP_OK;
}

int arhip_call_timer::begin()
{
    if (dev->capturing) {
        if (wait) return arhip_fail(ARHIP_EINVAL, "a launch that waits cannot be recorded into a graph (pass wait = 0)");
        return ARHIP_OK;
    }
    if (dev->prof && kernel >= 0) {
        if (int rc = prof_event(dev, &p0)) return rc;
        if (int rc = prof_event(dev, &p1)) return rc;
        ARHIP_HIP(hipEventRecord(p0, dev->stream));
    }
    if (wait) ARHIP_HIP(hipEventRecord(dev->ev0, dev->stream));
    return ARHIP_OK;
}

int arhip_call_timer::end()
{
    ARHIP_HIP(hipGetLastError());
    if (dev->capturing) return ARHIP_OK;
    if (p0) {
        ARHIP_HIP(hipEventRecord(p1, dev->stream));
        dev->prof_log.push_back({kernel, p0, p1});
    }
    if (wait) {
        ARHIP_HIP(hipEventRecord(dev->ev1, dev->stream));
        ARHIP_HIP(hipEventSynchronize(dev->ev1));
        float ms = 0.f;
        ARHIP_HIP(hipEventElapsedTime(&ms, dev->ev0, dev->ev1));
        if (secs) *secs = (double)ms * 1e-3;
    }
    return ARHIP_OK;
}

extern "C" int arhip_device_count(int *count)
{
    ARHIP_REQUIRE(count, "arhip_device_count: null out pointer");
    int n = 0;
    hipError_t e = hipGetDeviceCount(&n);
    if (e != hipSuccess) {
        (void)hipGetLastError();
        n = 0;
    }
    *count = n;
    return ARHIP_OK;
}

extern "C" int arhip_open(int ordinal, arhip_device **out)
{
    ARHIP_REQUIRE(out, "arhip_open: null out pointer");
    *out = nullptr;
    int n = 0;
    if (hipGetDeviceCount(&n) != hipSuccess || n <= 0) {
        (void)hipGetLastError();
        return arhip_fail(ARHIP_ENODEVICE, "arhip_open: no HIP device is visible");
    }
    if (ordinal < 0 || ordinal >= n)
        return arhip_fail(ARHIP_ENODEVICE, "arhip_open: ordinal %d out of range (%d devices)", ordinal, n);
    hipDeviceProp_t prop;
    ARHIP_HIP(hipGetDeviceProperties(&prop, ordinal));
    std::string arch = prop.gcnArchName;  // e.g. "gfx950:sramecc+:xnack-"
    arch = arch.substr(0, arch.find(':'));
    if (arch != "gfx950")
        return arhip_fail(ARHIP_ENODEVICE, "arhip_open: device %d is %s; the kernels are built for gfx950 only",
                          ordinal, arch.c_str());
    ARHIP_HIP(hipSetDevice(ordinal));
    arhip_device *d = new arhip_device();
    d->ordinal = ordinal;
    d->arch = arch;
    d->cus = prop.multiProcessorCount;
    if (const char *e = getenv("ARHIP_ATTN_WAVES")) d->attn_waves = atoi(e);
    hipError_t e = hipStreamCreateWithFlags(&d->stream, hipStreamNonBlocking);
    if (e == hipSuccess) e = hipEventCreate(&d->ev0);
    if (e == hipSuccess) e = hipEventCreate(&d->ev1);
    if (e == hipSuccess) e = hipEventCreate(&d->tm0);
    if (e == hipSuccess) e = hipEventCreate(&d->tm1);
    if (e != hipSuccess) {
        delete d;
        return arhip_fail(ARHIP_EHIP, "arhip_open: stream/event creation failed: %s", hipGetErrorString(e));
    }
    if (int rc = arhip_static_scratch_setup(ordinal)) {
        (void)arhip_close(d);
        return rc;
    }
    *out = d;
    return ARHIP_OK;
}

extern "C" int arhip_close(arhip_device *dev)
{
    if (!dev) return ARHIP_OK;
    (void)hipSetDevice(dev->ordinal);
    (void)hipStreamSynchronize(dev->stream);
    for (auto &kv : dev->modules) {
        for (hipModule_t m : kv.second->mods) (void)hipModuleUnload(m);
        delete kv.second;
    }
    for (auto &e : dev->prof_log) {
        (void)hipEventDestroy(e.e0);
        (void)hipEventDestroy(e.e1);
    }
    for (auto e : dev->prof_pool) (void)hipEventDestroy(e);
    (void)hipEventDestroy(dev->ev0);
    (void)hipEventDestroy(dev->ev1);
    (void)hipEventDestroy(dev->tm0);
    (void)hipEventDestroy(dev->tm1);
    (void)hipStreamDestroy(dev->stream);
    delete dev;
    return ARHIP_OK;
}

extern "C" const char *arhip_arch(arhip_device *dev) { return dev ? dev->arch.c_str() : ""; }
extern "C" int arhip_compute_units(arhip_device *dev) { return dev ? dev->cus : 0; }
extern "C" void *arhip_stream(arhip_device *dev) { return dev ? (void *)dev->stream : nullptr; }

#define ARHIP_DEV(dev)                                              \
    do {                                                            \
        ARHIP_REQUIRE((dev) != nullptr, "%s: null device", __func__); \
        ARHIP_HIP(hipSetDevice((dev)->ordinal));                    \
    } while (0)

extern "C" int arhip_alloc(arhip_device *dev, size_t bytes, void **dptr)
{
    ARHIP_DEV(dev);
    ARHIP_REQUIRE(dptr, "arhip_alloc: null out pointer");
    *dptr = nullptr;
    if (bytes == 0) return ARHIP_OK;  // zero-size buffers have no storage (src/runtime/device.rs:128-203)
    ARHIP_HIP(hipMalloc(dptr, bytes));
    return ARHIP_OK;
}

extern "C" int arhip_free(arhip_device *dev, void *dptr)
{
    ARHIP_DEV(dev);
    if (!dptr) return ARHIP_OK;
    ARHIP_HIP(hipStreamSynchronize(dev->stream));
    ARHIP_HIP(hipFree(dptr));
    return ARHIP_OK;
}

extern "C" int arhip_copyin(arhip_device *dev, void *dst, const void *host, size_t bytes)
{
    ARHIP_DEV(dev);
    if (bytes == 0) return ARHIP_OK;
    ARHIP_REQUIRE(dst && host, "arhip_copyin: null pointer");
    ARHIP_HIP(hipMemcpyAsync(dst, host, bytes, hipMemcpyHostToDevice, dev->stream));
    ARHIP_HIP(hipStreamSynchronize(dev->stream));  // the host buffer may be reused on return
    return ARHIP_OK;
}

extern "C" int arhip_copyout(arhip_device *dev, void *host, const void *src, size_t bytes)
{
    ARHIP_DEV(dev);
    if (bytes == 0) return ARHIP_OK;
    ARHIP_REQUIRE(host && src, "arhip_copyout: null pointer");
    ARHIP_HIP(hipMemcpyAsync(host, src, bytes, hipMemcpyDeviceToHost, dev->stream));
    ARHIP_HIP(hipStreamSynchronize(dev->stream));
    return ARHIP_OK;
}

extern "C" int arhip_copy_d2d(arhip_device *dev, void *dst, const void *src, size_t bytes)
{
    ARHIP_DEV(dev);
    if (bytes == 0) return ARHIP_OK;
    ARHIP_REQUIRE(dst && src, "arhip_copy_d2d: null pointer");
    ARHIP_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice, dev->stream));
    return ARHIP_OK;
}

__global__ void __launch_bounds__(256) arhip_fill_zero_kernel(uint32_t *p, size_t words, uint8_t *tail, int tail_bytes)
{
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < words; i += stride) p[i] = 0u;
    if (blockIdx.x == 0 && (int)threadIdx.x < tail_bytes) tail[threadIdx.x] = 0;
}

extern "C" int arhip_fill_zero(arhip_device *dev, void *dst, size_t bytes)
{
    ARHIP_DEV(dev);
    if (bytes == 0) return ARHIP_OK;
    ARHIP_REQUIRE(dst && (reinterpret_cast<uintptr_t>(dst) & 3u) == 0, "arhip_fill_zero: dst must be 4-byte aligned");
    const size_t words = bytes / 4;
    const int tail = (int)(bytes % 4);
    size_t blocks = (words + 255) / 256;
    if (blocks > 4096) blocks = 4096;
    if (blocks == 0) blocks = 1;
    hipLaunchKernelGGL(arhip_fill_zero_kernel, dim3((unsigned)blocks), dim3(256), 0, dev->stream,
                       (uint32_t *)dst, words, (uint8_t *)dst + words * 4, tail);
    ARHIP_HIP(hipGetLastError());
    return ARHIP_OK;
}

extern "C" int arhip_mem_info(arhip_device *dev, size_t *free_bytes, size_t *total_bytes)
{
    ARHIP_DEV(dev);
    size_t f = 0, t = 0;
    ARHIP_HIP(hipMemGetInfo(&f, &t));
    if (free_bytes) *free_bytes = f;
    if (total_bytes) *total_bytes = t;
    return ARHIP_OK;
}

extern "C" int arhip_sync(arhip_device *dev)
{
    ARHIP_DEV(dev);
    ARHIP_HIP(hipStreamSynchronize(dev->stream));
    return ARHIP_OK;
}

extern "C" int arhip_timer_start(arhip_device *dev)
{
    ARHIP_DEV(dev);
    ARHIP_HIP(hipEventRecord(dev->tm0, dev->stream));
    return ARHIP_OK;
}

extern "C" int arhip_timer_stop(arhip_device *dev, double *secs)
{
    ARHIP_DEV(dev);
    ARHIP_HIP(hipEventRecord(dev->tm1, dev->stream));
    ARHIP_HIP(hipEventSynchronize(dev->tm1));
    float ms = 0.f;
    ARHIP_HIP(hipEventElapsedTime(&ms, dev->tm0, dev->tm1));
    if (secs) *secs = (double)ms * 1e-3;
    return ARHIP_OK;
}

// Per-kernel device time, the counterpart of the reference's AUTORUST_KPROF
// (src/runtime/ops_cuda.rs:1004-1016), without a sync per launch: every typed
// launch is bracketed by two events on the stream while profiling is on.
extern "C" int arhip_kprof_enable(arhip_device *dev, int on)
{
    ARHIP_DEV(dev);
    dev->prof = on != 0;
    return ARHIP_OK;
}

extern "C" int arhip_kprof_collect(arhip_device *dev, int kernel, double *total_secs, uint64_t *launches)
{
    return arhip_kprof_collect_stats(dev, kernel, total_secs, launches, nullptr, nullptr);
}

extern "C" int arhip_kprof_collect_stats(arhip_device *dev, int kernel, double *total_secs, uint64_t *launches,
                                         double *min_secs, double *median_secs)
{
    ARHIP_DEV(dev);
    ARHIP_HIP(hipStreamSynchronize(dev->stream));
    double tot = 0.0;
    uint64_t n = 0;
    std::vector<double> each;
    std::vector<arhip_device::prof_entry> keep;
    for (auto &e : dev->prof_log) {
        if (e.kernel != kernel) {
            keep.push_back(e);
            continue;
        }
        float ms = 0.f;
        ARHIP_HIP(hipEventElapsedTime(&ms, e.e0, e.e1));
        tot += (double)ms * 1e-3;
        each.push_back((double)ms * 1e-3);
        ++n;
        dev->prof_pool.push_back(e.e0);
        dev->prof_pool.push_back(e.e1);
    }
    dev->prof_log.swap(keep);
    if (total_secs) *total_secs = tot;
    if (launches) *launches = n;
    std::sort(each.begin(), each.end());
    if (min_secs) *min_secs = each.empty() ? 0.0 : each.front();
    if (median_secs) *median_secs = each.empty() ? 0.0 : 0.5 * (each[(each.size() - 1) / 2] + each[each.size() / 2]);
    return ARHIP_OK;
}

// Launch graphs: the device-side counterpart of the reference's captured replay (Session capture
// + `Jit::replay`, src/engine/jit.rs:186-195).  Typed launches issued with wait = 0 between begin
// and end are recorded from the handle's stream into a HIP graph instead of running; launching
// the graph replays them in order with one submission.  Nothing in this library records a
// memset into a graph (buffers are cleared with a fill kernel).
extern "C" int arhip_graph_begin(arhip_device *dev)
{
    ARHIP_DEV(dev);
    ARHIP_REQUIRE(!dev->capturing, "arhip_graph_begin: a capture is already open");
    ARHIP_HIP(hipStreamSynchronize(dev->stream));
    ARHIP_HIP(hipStreamBeginCapture(dev->stream, hipStreamCaptureModeThreadLocal));
    dev->capturing = true;
    return ARHIP_OK;
}

extern "C" int arhip_graph_end(arhip_device *dev, void **graph_exec)
{
    ARHIP_DEV(dev);
    ARHIP_REQUIRE(dev->capturing && graph_exec, "arhip_graph_end: no capture is open (or null out pointer)");
    dev->capturing = false;
    hipGraph_t g = nullptr;
    ARHIP_HIP(hipStreamEndCapture(dev->stream, &g));
    hipGraphExec_t ex = nullptr;
    hipError_t e = hipGraphInstantiate(&ex, g, nullptr, nullptr, 0);
    (void)hipGraphDestroy(g);
    if (e != hipSuccess) {
        (void)hipGetLastError();
        return arhip_fail(ARHIP_EHIP, "hipGraphInstantiate failed: %s", hipGetErrorString(e));
    }
    *graph_exec = ex;
    return ARHIP_OK;
}

extern "C" int arhip_graph_launch(arhip_device *dev, void *graph_exec, int wait, double *secs)
{
    ARHIP_DEV(dev);
    ARHIP_REQUIRE(graph_exec && !dev->capturing, "arhip_graph_launch: null graph or capture still open");
    arhip_call_timer t{dev, wait, secs};
    if (int rc = t.begin()) return rc;
    ARHIP_HIP(hipGraphLaunch((hipGraphExec_t)graph_exec, dev->stream));
    return t.end();
}

extern "C" int arhip_graph_destroy(arhip_device *dev, void *graph_exec)
{
    ARHIP_DEV(dev);
    if (!graph_exec) return ARHIP_OK;
    ARHIP_HIP(hipStreamSynchronize(dev->stream));
    ARHIP_HIP(hipGraphExecDestroy((hipGraphExec_t)graph_exec));
    return ARHIP_OK;
}

// ---------------------------------------------------------------------------
// Generic launch: the `run_host_kernel` seam (src/runtime/device.rs:383-402).

static uint64_t fnv1a(const void *p, size_t n)
{
    const uint8_t *b = (const uint8_t *)p;
    uint64_t h = 1469598103934665603ull;
    for (size_t i = 0; i < n; ++i) {
        h ^= b[i];
        h *= 1099511628211ull;
    }
    return h ^ (uint64_t)n;
}

extern "C" int arhip_module_load(arhip_device *dev, const void *image, size_t len, void **module)
{
    ARHIP_DEV(dev);
    ARHIP_REQUIRE(image && len > 0 && module, "arhip_module_load: null image or out pointer");
    const uint64_t key = fnv1a(image, len);
    auto it = dev->modules.find(key);
    if (it != dev->modules.end()) {
        *module = it->second;
        return ARHIP_OK;
    }
    // An image is one code object (an ELF file), or a container of several that the build compiles side by side
    // and that are looked up as one: "ARHIPKO1", uint32 count, uint32 0, then per part uint64 size and the part's
    // bytes padded to a multiple of 16.
    std::vector<std::pair<const char *, size_t>> parts;
    const char *bytes = (const char *)image;
    if (len >= 16 && memcmp(bytes, "ARHIPKO1", 8) == 0) {
        uint32_t count;
        memcpy(&count, bytes + 8, 4);
        size_t at = 16;
        for (uint32_t i = 0; i < count; ++i) {
            uint64_t sz = 0;
            ARHIP_REQUIRE(at + 8 <= len, "arhip_module_load: truncated container (part %u of %u)", i, count);
            memcpy(&sz, bytes + at, 8);
            at += 8;
            ARHIP_REQUIRE(sz > 0 && sz <= len - at, "arhip_module_load: truncated container (part %u of %u)", i, count);
            parts.emplace_back(bytes + at, (size_t)sz);
            at += (size_t)((sz + 15) & ~(uint64_t)15);
        }
        ARHIP_REQUIRE(!parts.empty(), "arhip_module_load: empty container");
    } else {
        parts.emplace_back(bytes, len);
    }
    // Keep a private copy of every part alive for as long as its module is loaded.
    arhip_module_entry *e = new arhip_module_entry();
    for (auto &pt : parts) {
        e->images.emplace_back(pt.first, pt.first + pt.second);
        hipModule_t mod = nullptr;
        hipError_t err = hipModuleLoadData(&mod, e->images.back().data());
        if (err != hipSuccess) {
            for (hipModule_t m : e->mods) (void)hipModuleUnload(m);
            delete e;
            return arhip_fail(ARHIP_EHIP, "hipModuleLoadData failed: %s", hipGetErrorString(err));
        }
        e->mods.push_back(mod);
    }
    dev->modules[key] = e;
    *module = e;
    return ARHIP_OK;
}

// What the attention entry points of attn_kernels.hsaco (include/arhip_kernels.h) require of a launch.
// Given anything else they return without writing (or, with a wrong workgroup shape, compute on
// partly loaded tiles), and the caller's output is uninitialised memory with rc 0: a launch by one of
// these names is therefore checked here first.  Other names (probes, a host's own kernels) are not.
namespace {
struct named_entry {
    const char *name;
    int nbufs;        // device pointers
    int nvals;        // 32-bit scalars: n, head_dim, causal, has_mask, hq, hkv [, bq, bk [, out_f32]]
    unsigned block;   // workgroup size
    int rows;         // queries (keys for dK/dV) per workgroup: grid.x = ceil(n / rows)
    bool d64_only;    // head_dim must be 64
    bool no_mask;     // has_mask must be 0
    bool pipelined;   // 32-bit K/V offsets, bk = 64 * 2^j
    int max_n;        // 0 = any
    bool kv_grid;     // grid.y counts kv heads (dK/dV)
};
const named_entry NAMED[] = {
    {"ar_flash_f32", 5, 6, 256, 128, false, false, false, 0, false},
    {"ar_flash_f32_lens", 6, 6, 256, 128, false, false, false, 0, false},
    {"ar_flash_f32_short", 5, 6, 256, 32, true, false, false, 0, false},
    {"ar_flash_bf16", 5, 6, 256, 128, false, false, false, 0, false},
    {"ar_flash_bf16_lens", 6, 6, 256, 128, false, false, false, 0, false},
    {"ar_flash_bf16_long", 5, 6, 512, 256, false, true, true, 0, false},
    {"ar_flash_bf16_long_lens", 6, 6, 512, 256, false, true, true, 0, false},
    {"ar_flash_bf16_mid", 5, 6, 256, 128, false, true, true, 0, false},
    {"ar_flash_bf16_mid_lens", 6, 6, 256, 128, false, true, true, 0, false},
    {"ar_flash_sage", 7, 8, 256, 128, false, false, false, 0, false},
    {"ar_flash_sage_lens", 8, 8, 256, 128, false, false, false, 0, false},
    {"ar_flash_sage_fp8", 7, 8, 256, 128, false, false, false, 0, false},
    {"ar_flash_sage_fp8_lens", 8, 8, 256, 128, false, false, false, 0, false},
    {"ar_flash_sage_long", 7, 9, 512, 256, false, true, true, 0, false},
    {"ar_flash_sage_long_lens", 8, 9, 512, 256, false, true, true, 0, false},
    {"ar_flash_sage_mid", 7, 9, 256, 128, false, true, true, 0, false},
    {"ar_flash_sage_mid_lens", 8, 9, 256, 128, false, true, true, 0, false},
    {"ar_flash_sage_qf_long", 7, 9, 512, 256, false, true, true, 0, false},
    {"ar_flash_sage_qf_long_lens", 8, 9, 512, 256, false, true, true, 0, false},
    {"ar_flash_sage_qf_mid", 7, 9, 256, 128, false, true, true, 0, false},
    {"ar_flash_sage_qf_mid_lens", 8, 9, 256, 128, false, true, true, 0, false},
    {"ar_flash_sage_fp8_qf_long", 7, 9, 512, 256, false, true, true, 0, false},
    {"ar_flash_sage_fp8_qf_long_lens", 8, 9, 512, 256, false, true, true, 0, false},
    {"ar_flash_sage_fp8_qf_mid", 7, 9, 256, 128, false, true, true, 0, false},
    {"ar_flash_sage_fp8_qf_mid_lens", 8, 9, 256, 128, false, true, true, 0, false},
    {"ar_flash_sage_qr_long", 7, 9, 512, 256, false, true, true, 0, false},
    {"ar_flash_sage_qr_long_lens", 8, 9, 512, 256, false, true, true, 0, false},
    {"ar_flash_sage_qr_mid", 7, 9, 256, 128, false, true, true, 0, false},
    {"ar_flash_sage_qr_mid_lens", 8, 9, 256, 128, false, true, true, 0, false},
    {"ar_flash_sage_fp8_mid", 7, 9, 256, 128, false, true, true, 0, false},
    {"ar_flash_sage_fp8_mid_lens", 8, 9, 256, 128, false, true, true, 0, false},
    {"ar_flash_sage_fp8_long", 7, 9, 512, 256, false, true, true, 0, false},
    {"ar_flash_sage_fp8_long_lens", 8, 9, 512, 256, false, true, true, 0, false},
    {"ar_fl_fwd", 6, 6, 256, 128, false, false, false, 0, false},
    {"ar_fl_fwd_short", 6, 6, 256, 32, true, false, false, 0, false},
    {"ar_fl_bwd_dq", 8, 6, 256, 128, false, false, false, 0, false},
    {"ar_fl_bwd_dq_short", 8, 6, 256, 32, true, false, false, 0, false},
    {"ar_fl_bwd_dkv", 9, 6, 256, 128, false, false, false, 0, true},
    {"ar_fl_bwd_dkv_short", 9, 6, 256, 32, true, false, false, 0, true},
};

int check_named_entry(const char *name, const unsigned grid[3], const unsigned block[3], int nbufs, const int64_t *vals,
                      int nvals)
{
    const named_entry *e = nullptr;
    for (const named_entry &c : NAMED)
        if (std::strcmp(c.name, name) == 0) e = &c;
    if (!e) return ARHIP_OK;
    ARHIP_REQUIRE(nbufs == e->nbufs && nvals == e->nvals, "arhip_launch: %s takes %d buffers and %d scalars, got %d and %d", name,
                  e->nbufs, e->nvals, nbufs, nvals);
    ARHIP_REQUIRE(block[0] == e->block && block[1] == 1 && block[2] == 1, "arhip_launch: %s runs with block [%u,1,1], got [%u,%u,%u]",
                  name, e->block, block[0], block[1], block[2]);
    const int64_t n = vals[0], d = vals[1], has_mask = vals[3], hq = vals[4], hkv = vals[5];
    ARHIP_REQUIRE(n > 0 && n <= ((int64_t)1 << 24), "arhip_launch: %s: n = %lld", name, (long long)n);
    ARHIP_REQUIRE(d == 64 || (d == 128 && !e->d64_only), "arhip_launch: %s: head_dim %lld (%s)", name, (long long)d,
                  e->d64_only ? "64 only" : "64 or 128");
    ARHIP_REQUIRE(hq > 0 && hkv > 0 && hq % hkv == 0, "arhip_launch: %s: hq = %lld, hkv = %lld", name, (long long)hq, (long long)hkv);
    ARHIP_REQUIRE(!(e->no_mask && has_mask), "arhip_launch: %s takes no additive mask (has_mask must be 0)", name);
    ARHIP_REQUIRE(e->max_n == 0 || n <= e->max_n, "arhip_launch: %s: n = %lld exceeds %d", name, (long long)n, e->max_n);
    ARHIP_REQUIRE((int64_t)grid[0] == (n + e->rows - 1) / e->rows && grid[2] == 1,
                  "arhip_launch: %s: grid [%u,%u,%u], expected [ceil(n/%d) = %lld, B*h, 1]", name, grid[0], grid[1], grid[2], e->rows,
                  (long long)((n + e->rows - 1) / e->rows));
    ARHIP_REQUIRE(grid[1] % (unsigned)(e->kv_grid ? hkv : hq) == 0, "arhip_launch: %s: grid.y = %u is not a multiple of %s = %lld", name,
                  grid[1], e->kv_grid ? "hkv" : "hq", (long long)(e->kv_grid ? hkv : hq));
    if (e->nvals >= 8) ARHIP_REQUIRE(vals[6] >= 1 && vals[7] >= 1, "arhip_launch: %s: block sizes bq = %lld, bk = %lld", name,
                                     (long long)vals[6], (long long)vals[7]);
    if (e->pipelined) {
        ARHIP_REQUIRE((n + 320) * d * 2 < ((int64_t)1 << 31), "arhip_launch: %s addresses K/V with 32-bit offsets: (n + 320) * head_dim * 2 "
                      "must stay below 2^31", name);
        if (e->nvals >= 8) {
            // any power of two (below 64 keys the kernel applies the scales per logit)
            const int64_t bk = vals[7];
            ARHIP_REQUIRE((bk & (bk - 1)) == 0, "arhip_launch: %s needs K scales over a power of two of keys (bk = 2^j), got bk = %lld",
                          name, (long long)bk);
            if (strstr(name, "_qr_") != nullptr)
                ARHIP_REQUIRE(vals[6] == 1 && bk < 64, "arhip_launch: %s quantises Q row by row and takes K scales over "
                              "a power of two of keys below 64, got bq = %lld, bk = %lld", name, (long long)vals[6], (long long)bk);
            if (strstr(name, "_qf_") != nullptr)
                ARHIP_REQUIRE(vals[6] == 128 && bk >= 64, "arhip_launch: %s quantises Q over blocks of 128 queries and takes K scales "
                              "over whole 64-key tiles, got bq = %lld, bk = %lld", name, (long long)vals[6], (long long)bk);
        }
    }
    return ARHIP_OK;
}
}  // namespace

extern "C" int arhip_launch(arhip_device *dev, void *module, const char *name,
                            const unsigned grid[3], const unsigned block[3],
                            void *const *bufs, int nbufs,
                            const int64_t *vals, const int *val_bits, int nvals,
                            int wait, double *secs)
{
    ARHIP_DEV(dev);
    ARHIP_REQUIRE(module && name && grid && block, "arhip_launch: null argument");
    ARHIP_REQUIRE(nbufs >= 0 && nvals >= 0 && nbufs + nvals <= 64, "arhip_launch: too many arguments");
    ARHIP_REQUIRE(nvals == 0 || (vals && val_bits), "arhip_launch: scalar values without widths");
    arhip_module_entry *m = (arhip_module_entry *)module;
    hipFunction_t fn;
    auto it = m->fns.find(name);
    if (it == m->fns.end()) {
        hipError_t err = hipErrorNotFound;
        for (hipModule_t mod : m->mods) {
            err = hipModuleGetFunction(&fn, mod, name);
            if (err == hipSuccess) break;
        }
        (void)hipGetLastError();  // a miss in an earlier part of a container is not an error of this launch
        if (err != hipSuccess) {
            return arhip_fail(ARHIP_EHIP, "arhip_launch: no kernel named %s in the module: %s", name, hipGetErrorString(err));
        }
        m->fns[name] = fn;
    } else {
        fn = it->second;
    }
    // A zero-sized grid is a no-op (the reference clamps negatives to 0, session.rs:241-251).
    if (grid[0] == 0 || grid[1] == 0 || grid[2] == 0) {
        if (secs) *secs = 0.0;
        return ARHIP_OK;
    }
    ARHIP_REQUIRE(block[0] * block[1] * block[2] >= 1 && block[0] * block[1] * block[2] <= 1024,
                  "arhip_launch: block of %u threads", block[0] * block[1] * block[2]);
    if (int rc = check_named_entry(name, grid, block, nbufs, vals, nvals)) return rc;
    void *ptrs[64];
    int32_t v32[64];
    int64_t v64[64];
    void *params[64];
    int na = 0;
    for (int i = 0; i < nbufs; ++i, ++na) {
        ptrs[na] = bufs[i];
        params[na] = &ptrs[na];
    }
    for (int i = 0; i < nvals; ++i, ++na) {
        if (val_bits[i] == 32) {
            v32[na] = (int32_t)vals[i];
            params[na] = &v32[na];
        } else if (val_bits[i] == 64) {
            v64[na] = vals[i];
            params[na] = &v64[na];
        } else {
            return arhip_fail(ARHIP_EINVAL, "arhip_launch: scalar %d has width %d (32 or 64)", i, val_bits[i]);
        }
    }
    arhip_call_timer t{dev, wait, secs};
    if (int rc = t.begin()) return rc;
    ARHIP_HIP(hipModuleLaunchKernel(fn, grid[0], grid[1], grid[2], block[0], block[1], block[2], 0,
                                    dev->stream, params, nullptr));
    return t.end();
}
