// Implementation of the C++ mirror of the reference's attention interface (autorust_host.h).
// Everything computes through libarhip's C ABI; nothing here touches HIP directly.
#include "autorust_host.h"

#include <dlfcn.h>

#include <atomic>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <fstream>
#include <mutex>

namespace autorust {

const char *name(AttentionKind k)
{
    switch (k) {
    case AttentionKind::Sdpa: return "sdpa";
    case AttentionKind::Flash: return "flash";
    default: return "sage";
    }
}

AttentionKind attention_kind_from_str(const std::string &s)
{
    if (s == "sdpa") return AttentionKind::Sdpa;
    if (s == "sage") return AttentionKind::Sage;
    return AttentionKind::Flash;  // the default, also for unknown values (settings.rs:209-213)
}

static bool env_flag(const char *n, bool dflt)
{
    const char *v = getenv(n);
    if (!v || !*v) return dflt;
    return !(v[0] == '0' || v[0] == 'f' || v[0] == 'F' || v[0] == 'n' || v[0] == 'N');
}

Settings Settings::from_env()
{
    Settings s;
    if (const char *a = getenv("AUTORUST_ATTN")) s.attention = attention_kind_from_str(a);
    s.tensor_cores = env_flag("AUTORUST_TENSOR_CORES", env_flag("AUTORUST_TC", true));
    s.async_pipeline = env_flag("AUTORUST_ASYNC", true);
    if (const char *f = getenv("AUTORUST_SAGE_FP8")) s.sage_fp8 = f[0] == '1';
    if (const char *m = getenv("AUTORUST_MATH")) {
        if (std::string(m) == "exact") {  // settings.rs:202-208: exact mode turns the matrix units off
            s.math_exact = true;
            s.tensor_cores = false;
        }
    }
    return s;
}

// ---- device ---------------------------------------------------------------------------

void Device::check(int rc) const
{
    if (rc != ARHIP_OK) throw std::runtime_error(std::string("TGERR: arhip ") + std::to_string(rc) + ": " + arhip_last_error());
}

Device::Device(int ordinal) : ordinal_(ordinal)
{
    const int rc = arhip_open(ordinal, &dev_);
    if (rc != ARHIP_OK) throw std::runtime_error(std::string("TGERR: arhip ") + std::to_string(rc) + ": " + arhip_last_error());
}

Device::~Device()
{
    for (auto &kv : free_)
        for (void *p : kv.second) arhip_free(dev_, p);
    arhip_close(dev_);
}

int Device::compute_units() const { return arhip_compute_units(dev_); }

std::string attention_kernels_src()
{
    if (const char *e = getenv("AUTORUST_HIP_KERNELS")) return e;
    Dl_info info;
    if (dladdr((const void *)&attention_kernels_src, &info) && info.dli_fname) {
        std::string p = info.dli_fname;
        const size_t slash = p.rfind('/');
        return (slash == std::string::npos ? std::string(".") : p.substr(0, slash)) + "/attn_kernels.hsaco";
    }
    return "attn_kernels.hsaco";
}

std::optional<double> Device::run_host_kernel(const std::string &src, const std::string &name,
                                              const std::vector<std::pair<int64_t, DType>> &signature,
                                              const std::vector<void *> &bufs, const int64_t global[3],
                                              const std::optional<std::array<int64_t, 3>> &local,
                                              const std::vector<int64_t> &vals, bool wait)
{
    // compile_cached: one load per code object and device (device.rs:239-251; the image itself is
    // cached by content inside arhip_module_load as well)
    auto it = modules_.find(src);
    if (it == modules_.end()) {
        std::ifstream f(src, std::ios::binary);
        if (!f) throw std::runtime_error("TGERR: run_host_kernel: cannot read the code object " + src);
        const std::vector<char> image((std::istreambuf_iterator<char>(f)), std::istreambuf_iterator<char>());
        void *mod = nullptr;
        check(arhip_module_load(dev_, image.data(), image.size(), &mod));
        it = modules_.emplace(src, mod).first;
        uint64_t key = 1469598103934665603ull;  // content hash of the compiled artifact (FNV-1a), printed by KPROF
        for (char c : image) key = (key ^ (unsigned char)c) * 1099511628211ull;
        module_keys_[src] = key;
        if (getenv("AUTORUST_KERNEL_INFO"))  // ops_cuda.rs:902-918 prints per-kernel resources at load
            std::fprintf(stderr, "[hip] loaded %s (%zu bytes) for %s\n", src.c_str(), image.size(), this->name().c_str());
    }
    if (!local) throw std::runtime_error("TGERR: run_host_kernel: " + name + " needs an explicit workgroup shape");
    const size_t nb = bufs.size();
    if (signature.size() != nb + vals.size())
        throw std::runtime_error("TGERR: run_host_kernel: " + name + ": signature does not match bufs + vals");
    std::vector<void *> ptrs(nb);
    std::vector<int64_t> sv(vals.size());
    std::vector<int> bits(vals.size());
    for (size_t i = 0; i < signature.size(); ++i) {
        const int64_t slot = signature[i].first;
        if (slot < 0 || (size_t)slot >= signature.size() || (size_t)slot != i)
            throw std::runtime_error("TGERR: run_host_kernel: " + name + ": slots must be 0..n-1 in order");
        if (i < nb) {
            ptrs[i] = bufs[i];
        } else {
            sv[i - nb] = vals[i - nb];
            bits[i - nb] = signature[i].second == DType::Int64 ? 64 : 32;  // narrowed like ops_cuda.rs:943-990
        }
    }
    unsigned g[3], l[3];
    for (int i = 0; i < 3; ++i) {
        g[i] = (unsigned)std::max<int64_t>(global[i], 0);       // negatives clamp to 0 (session.rs:241-251)
        l[i] = (unsigned)std::max<int64_t>((*local)[i], 0);
    }
    // AUTORUST_KPROF (src/runtime/ops_cuda.rs:879-885, 1004-1012): a launch that would not wait is
    // synchronised and reported as `KPROF <name> <secs> <content key>` on stderr; it serialises the
    // stream, so it is a profiling aid, not a benchmark mode.
    const bool kprof = !wait && getenv("AUTORUST_KPROF") != nullptr;
    double secs = 0.0;
    check(arhip_launch(dev_, it->second, name.c_str(), g, l, ptrs.data(), (int)nb, sv.data(), bits.data(), (int)sv.size(),
                       (wait || kprof) ? 1 : 0, &secs));
    if (kprof) {
        std::fprintf(stderr, "KPROF\t%s\t%.6f\t%016llx\n", name.c_str(), secs, (unsigned long long)module_keys_[src]);
        return secs;
    }
    if (wait) return secs;
    return std::nullopt;
}

void *Device::alloc(size_t bytes)
{
    if (bytes == 0) return nullptr;
    auto it = free_.find(bytes);
    if (it != free_.end() && !it->second.empty()) {
        void *p = it->second.back();
        it->second.pop_back();
        return p;
    }
    void *p = nullptr;
    check(arhip_alloc(dev_, bytes, &p));
    ++raw_allocs_;
    return p;
}

void Device::release(void *p, size_t bytes)
{
    if (!p) return;
    auto &v = free_[bytes];
    if (v.size() < 32) {  // device.rs:128-203: at most 32 cached blocks per size
        v.push_back(p);
    } else {
        arhip_free(dev_, p);
    }
}

Storage::~Storage()
{
    if (dev && ptr) dev->release(ptr, bytes);
}

// ---- tensors --------------------------------------------------------------------------

static size_t esize(DType d)
{
    switch (d) {
    case DType::BFloat16: return 2;
    case DType::Int8: return 1;
    case DType::Int64: return 8;
    default: return 4;
    }
}

size_t Tensor::nbytes() const { return (size_t)numel() * esize(dtype_); }

int64_t Tensor::numel() const
{
    int64_t n = 1;
    for (auto s : shape_) n *= s;
    return n;
}

Tensor Tensor::empty(const std::shared_ptr<Device> &dev, const std::vector<int64_t> &shape, DType dtype)
{
    Tensor t;
    t.shape_ = shape;
    t.dtype_ = dtype;
    t.st_ = std::make_shared<Storage>();
    t.st_->dev = dev;
    t.st_->bytes = (size_t)t.numel() * esize(dtype);
    t.st_->ptr = dev->alloc(t.st_->bytes);
    return t;
}

Tensor Tensor::from_slice(const std::shared_ptr<Device> &dev, const float *data, const std::vector<int64_t> &shape, DType dtype)
{
    if (dtype == DType::Other) throw std::runtime_error("TGERR: from_slice: only f32 and bf16 tensors exist on this device");
    Tensor t = empty(dev, shape, dtype);
    const int64_t n = t.numel();
    if (n == 0) return t;
    if (dtype == DType::Float32) {
        dev->check(arhip_copyin(dev->handle(), t.ptr(), data, (size_t)n * 4));
    } else {
        // cast on the device (round to nearest even, dtype/mod.rs:973-981) through an f32 staging buffer
        void *tmp = dev->alloc((size_t)n * 4);
        dev->check(arhip_copyin(dev->handle(), tmp, data, (size_t)n * 4));
        dev->check(arhip_cast_bf16(dev->handle(), (const float *)tmp, (uint16_t *)t.ptr(), n, 1, nullptr));
        dev->release(tmp, (size_t)n * 4);
    }
    return t;
}

Tensor Tensor::from_i32(const std::shared_ptr<Device> &dev, const int32_t *data, const std::vector<int64_t> &shape)
{
    Tensor t = empty(dev, shape, DType::Int32);
    if (t.numel() > 0) dev->check(arhip_copyin(dev->handle(), t.ptr(), data, (size_t)t.numel() * 4));
    return t;
}

Tensor Tensor::reshape(const std::vector<int64_t> &shape) const
{
    int64_t n = 1;
    for (auto s : shape) n *= s;
    if (n != numel()) throw std::runtime_error("TGERR: reshape: element count differs");
    Tensor t = *this;
    t.shape_ = shape;
    return t;
}

std::vector<float> Tensor::to_list() const
{
    const int64_t n = numel();
    std::vector<float> out((size_t)n);
    if (n == 0) return out;
    auto &dev = st_->dev;
    if (dtype_ == DType::Float32) {
        dev->check(arhip_copyout(dev->handle(), out.data(), ptr(), (size_t)n * 4));
    } else {
        std::vector<uint16_t> raw((size_t)n);
        dev->check(arhip_copyout(dev->handle(), raw.data(), ptr(), (size_t)n * 2));
        for (int64_t i = 0; i < n; ++i) {
            const uint32_t bits = (uint32_t)raw[(size_t)i] << 16;
            std::memcpy(&out[(size_t)i], &bits, 4);
        }
    }
    return out;
}

// ---- dispatcher -----------------------------------------------------------------------

static void note_once(std::once_flag &flag, const char *msg)
{
    std::call_once(flag, [msg] { std::fprintf(stderr, "%s\n", msg); });
}

Kernel plan_fused(const std::vector<int64_t> &q, const std::vector<int64_t> &k, const std::vector<int64_t> &v,
                  DType qd, DType kd, DType vd, const std::vector<int64_t> *mask_shape, DType mask_dtype,
                  bool enable_gqa, bool quantized, const Settings &st, bool *sage_declined)
{
    if (sage_declined) *sage_declined = false;
    if (q.size() != 4 || k.size() != 4 || v.size() != 4) return Kernel::None;            // :358-369
    const int64_t b = q[0], h = q[1], n = q[2], d = q[3];
    const int64_t hk = k[1], nk = k[2], dk = k[3], hv = v[1], nv = v[2], dv = v[3];
    if (k[0] != b || v[0] != b) return Kernel::None;
    if (nk != n || nv != n || dk != d || dv != d || hk != hv) return Kernel::None;       // :372-374
    if (enable_gqa) {
        if (hk <= 0 || h % hk != 0) return Kernel::None;                                 // :375-378
    } else if (hk != h) {
        return Kernel::None;                                                             // :379-381
    }
    if (qd != DType::Float32 && qd != DType::BFloat16) return Kernel::None;              // :382-385
    if (kd != qd || vd != qd) return Kernel::None;                                       // :386-388
    if (mask_shape) {  // dense additive f32 [n, n] only (:391-396)
        if (mask_dtype != DType::Float32 || mask_shape->size() != 2 || (*mask_shape)[0] != n || (*mask_shape)[1] != n)
            return Kernel::None;
    }
    // the launch grid is [query tiles, b*h, 1]: b*h must fit the y dimension of a grid
    if (b <= 0 || h <= 0 || n <= 0 || b * h > 65535) return Kernel::None;
    const int dt = qd == DType::BFloat16 ? ARHIP_BF16 : ARHIP_F32;
    // Sage: the reference takes f32 tensors only (:411-414); bf16 tensors are accepted here too.
    const bool sage = quantized && st.tensor_cores && arhip_attn_supported(ARHIP_ATTN_SAGE, n, d, dt);
    if (quantized && !sage && sage_declined) *sage_declined = true;                      // :420-422
    if (sage) return Kernel::Sage;
    if (!arhip_attn_supported(ARHIP_ATTN_FLASH, n, d, dt)) return Kernel::None;
    if (qd == DType::BFloat16) return st.tensor_cores ? Kernel::FlashBf16 : Kernel::None;  // :427-429, bf16 needs the matrix units
    // f32 tensors: the reference prefers its TF32 kernel; CDNA4 has no such MFMA, so f32 runs exact
    return Kernel::FlashF32;                                                             // :451
}

bool wants_fused(std::optional<AttentionKind> force, const Settings &st, double dropout_p, bool has_session, bool *quantized)
{
    const AttentionKind requested = force.value_or(st.attention);     // explicit calls are never overridden
    if (quantized) *quantized = requested == AttentionKind::Sage;
    return effective(requested) != AttentionKind::Sdpa && dropout_p == 0.0 && has_session;
}

static std::atomic<uint64_t> g_selected[3];

uint64_t selections(Kernel k) { return k == Kernel::None ? 0 : g_selected[(int)k].load(std::memory_order_relaxed); }

// Record a dispatch; one-time line under AUTORUST_ATTN_DEBUG (cuda_flash_bf16.rs:446-456,
// cuda_flash_sage.rs:417-436).
static void note_selected(Kernel k)
{
    static std::once_flag once[3];
    static const char *what[3] = {"[attention] flash: fp32 exact, fp32 MFMA (gfx950)",
                                  "[attention] flash: bf16 MFMA, software-pipelined for long sequences (gfx950)",
                                  "[attention] sage: int8 MFMA for q.k^T, bf16 MFMA for p.v, K smoothing + block scales (gfx950)"};
    g_selected[(int)k].fetch_add(1, std::memory_order_relaxed);
    if (getenv("AUTORUST_ATTN_DEBUG")) note_once(once[(int)k], what[(int)k]);
}

void HostCall::exec() const
{
    if (bufs.empty()) throw std::runtime_error("TGERR: HostCall::exec: no buffers");
    const auto &dev = bufs.front().device();   // the reference resolves `device` by name (session.rs:232)
    if (dev->name() != device) throw std::runtime_error("TGERR: HostCall::exec: buffers live on " + dev->name() + ", not " + device);
    std::vector<void *> ptrs;
    for (const auto &b : bufs) ptrs.push_back(b.ptr());
    dev->run_host_kernel(src, name, signature, ptrs, global, local, vals, true);
}

std::optional<Tensor> fused_attention(const Tensor &q, const Tensor &k, const Tensor &v, Session &sess, const Settings &st)
{
    return fused_attention_ex(q, k, v, nullptr, false, false, false, sess, st);
}

std::optional<Tensor> fused_attention_kind(const Tensor &q, const Tensor &k, const Tensor &v, AttentionKind kind,
                                           Session &sess, const Settings &st)
{
    return fused_attention_ex(q, k, v, nullptr, false, false, kind == AttentionKind::Sage, sess, st);
}

namespace {

using Sig = std::vector<std::pair<int64_t, DType>>;

// bufs first, then 32-bit scalars (64-bit where wide[i] is set)
Sig make_sig(const std::vector<DType> &buf_types, size_t nvals, const std::vector<size_t> &wide = {})
{
    Sig s;
    for (size_t i = 0; i < buf_types.size(); ++i) s.emplace_back((int64_t)i, buf_types[i]);
    for (size_t i = 0; i < nvals; ++i) {
        DType t = DType::Int32;
        for (size_t w : wide)
            if (w == i) t = DType::Int64;
        s.emplace_back((int64_t)(buf_types.size() + i), t);
    }
    return s;
}

HostCall make_call(const std::shared_ptr<Device> &dev, const char *name, const std::vector<Tensor> &bufs,
                   const std::vector<DType> &buf_types, std::array<int64_t, 3> global, std::array<int64_t, 3> local,
                   const std::vector<int64_t> &vals, const std::vector<size_t> &wide = {})
{
    HostCall c;
    c.device = dev->name();
    c.src = attention_kernels_src();
    c.name = name;
    c.signature = make_sig(buf_types, vals.size(), wide);
    c.bufs = bufs;
    for (int i = 0; i < 3; ++i) c.global[i] = global[(size_t)i];
    c.local = local;
    c.vals = vals;
    return c;
}

// The software-pipelined kernels serve every launch without an additive mask whose K/V they can address
// with 32-bit byte offsets ...
bool long_variant(int64_t n, int64_t d)
{
    return (n + 320) * d * 2 < ((int64_t)1 << 31);
}

// ... and run with 4 waves / 128 queries per workgroup (the `_mid` entry points, two workgroups per compute
// unit) where a workgroup sees few tiles: the rule of arhip_flash_fwd / arhip_sage_fwd
bool mid_variant(const std::shared_ptr<Device> &dev, int64_t b, int64_t h, int64_t n, int64_t d, bool causal, bool has_lens)
{
    if (d == 64) return true;
    if (b * h * ((n + 255) / 256) < 2 * (int64_t)dev->compute_units()) return true;
    return n <= 1024 || (n <= 2048 && causal && !has_lens);
}

}  // namespace

// The fp32 kernels: 128 queries (keys) per workgroup when that still fills the chip, else 32
static bool short_f32(const std::shared_ptr<Device> &dev, int64_t b, int64_t heads, int64_t n)
{
    return b * heads * ((n + 127) / 128) < 2 * (int64_t)dev->compute_units();
}

std::vector<HostCall> attention_host_calls(const Tensor &q, const Tensor &k, const Tensor &v, const Tensor *attn_mask,
                                           const Tensor &out, bool is_causal, Kernel kern, const Settings &st,
                                           const Tensor *key_lengths)
{
    const int64_t b = q.shape()[0], h = q.shape()[1], n = q.shape()[2], d = q.shape()[3], hk = k.shape()[1];
    const auto dev = q.device();
    const DType F = DType::Float32, BF = DType::BFloat16, I8 = DType::Int8;
    const bool has_mask = attn_mask != nullptr;
    // the mask slot always holds a buffer; without a mask it is `out` (cuda_flash.rs:233-240)
    const Tensor mslot = has_mask ? *attn_mask : out;
    const std::vector<int64_t> vals = {n, d, (int64_t)is_causal, (int64_t)has_mask, h, hk};  // cuda_flash_bf16.rs:550-561
    std::vector<HostCall> calls;
    // the attention kernel itself: with key lengths it is the `_lens` twin, whose argument list has the
    // lengths ([b] int32) right after the mask slot (slot 4 in every forward entry)
    auto attn_call = [&](const std::string &name, std::vector<Tensor> bufs, std::vector<DType> types, std::array<int64_t, 3> global,
                         std::array<int64_t, 3> local, const std::vector<int64_t> &scalars) {
        if (!key_lengths) return make_call(dev, name.c_str(), bufs, types, global, local, scalars);
        bufs.insert(bufs.begin() + 5, *key_lengths);
        types.insert(types.begin() + 5, DType::Int32);
        return make_call(dev, (name + "_lens").c_str(), bufs, types, global, local, scalars);
    };

    if (kern == Kernel::FlashF32) {
        // few, short heads: 32 queries per workgroup instead of 128 (the rule of arhip_flash_fwd)
        if (d == 64 && short_f32(dev, b, h, n) && !key_lengths)
            calls.push_back(make_call(dev, "ar_flash_f32_short", {q, k, v, out, mslot}, {F, F, F, F, F},
                                      {(n + 31) / 32, b * h, 1}, {256, 1, 1}, vals));
        else
            calls.push_back(attn_call("ar_flash_f32", {q, k, v, out, mslot}, {F, F, F, F, F}, {(n + 127) / 128, b * h, 1},
                                      {256, 1, 1}, vals));
        return calls;
    }
    if (kern == Kernel::FlashBf16) {
        if (!has_mask && long_variant(n, d) && mid_variant(dev, b, h, n, d, is_causal, key_lengths != nullptr))
            calls.push_back(attn_call("ar_flash_bf16_mid", {q, k, v, out, mslot}, {BF, BF, BF, BF, F},
                                      {(n + 127) / 128, b * h, 1}, {256, 1, 1}, vals));
        else if (!has_mask && long_variant(n, d))
            calls.push_back(attn_call("ar_flash_bf16_long", {q, k, v, out, mslot}, {BF, BF, BF, BF, F},
                                      {(n + 255) / 256, b * h, 1}, {512, 1, 1}, vals));
        else
            calls.push_back(attn_call("ar_flash_bf16", {q, k, v, out, mslot}, {BF, BF, BF, BF, F},
                                      {(n + 127) / 128, b * h, 1}, {256, 1, 1}, vals));
        return calls;
    }

    // ---- Sage: quantise Q, smooth + quantise K, (cast V), attention; scratch tensors ride in the
    // HostCalls, so a replay finds them again and nothing is allocated then ----
    const bool bf16_in = q.dtype() == DType::BFloat16;
    const char *sfx = bf16_in ? "bf16" : "f32";
    const DType X = bf16_in ? BF : F;
    const int64_t bq = st.sage_block_q, bk = st.sage_block_k;
    const int64_t nqb = (n + bq - 1) / bq, nkb = (n + bk - 1) / bk, nchunk = (n + 63) / 64;
    Tensor q8 = Tensor::empty(dev, {b, h, n, d}, I8), k8 = Tensor::empty(dev, {b, hk, n, d}, I8);
    Tensor sq = Tensor::empty(dev, {b, h, nqb}, F), sk = Tensor::empty(dev, {b, hk, nkb}, F);
    Tensor mean = Tensor::empty(dev, {b, hk, d}, F);
    const std::string part_name = std::string("ar_sage_kmean_partial_") + sfx;
    const std::string q8fmt = st.sage_fp8 ? "fp8_" : "";
    const std::string rows_name = "ar_sage_quant_rows_" + q8fmt + sfx, blocks_name = "ar_sage_quant_blocks_" + q8fmt + sfx;
    const char *general = st.sage_fp8 ? "ar_flash_sage_fp8" : "ar_flash_sage";
    auto quant = [&](const Tensor &x, const Tensor &x8, const Tensor &sc, int64_t heads, int64_t blk, int64_t nblk, bool smooth) {
        if (blk == 1) {
            const int64_t rows = b * heads * n, rpb = 256 / (d / 8);
            calls.push_back(make_call(dev, rows_name.c_str(), {x, x8, sc, mean}, {X, I8, F, F}, {(rows + rpb - 1) / rpb, 1, 1},
                                      {256, 1, 1}, {n, d, rows, (int64_t)smooth}, {2}));
        } else {
            calls.push_back(make_call(dev, blocks_name.c_str(), {x, x8, sc, mean}, {X, I8, F, F}, {nblk, b * heads, 1},
                                      {256, 1, 1}, {n, d, blk, nblk, (int64_t)smooth}));
        }
    };
    int shift = 0;
    while (((int64_t)64 << shift) < bk) ++shift;
    const bool tile_uniform = ((int64_t)64 << shift) == bk;
    // scales over a power of two of keys below 64 (the reference's bk = 1) are applied per logit
    const bool key_scales = bk < 64 && (bk & (bk - 1)) == 0;
    const bool pipelined = !has_mask && (tile_uniform || key_scales) && long_variant(n, d);
    // bf16 queries with scales over blocks of 128 are quantised by the attention kernel itself (as the reference's
    // kernel does, cuda_flash_sage.rs:201-223): one launch and one pass over Q fewer
    const bool q_fused = pipelined && tile_uniform && bf16_in && bq == 128;
    // f32 queries with a scale each and K scales per key (the reference's own convention): the same, row by row
    const bool q_rows = pipelined && key_scales && !bf16_in && bq == 1 && !st.sage_fp8;
    if (!q_fused && !q_rows) quant(q, q8, sq, h, bq, nqb, false);
    if (st.sage_smooth_k) {
        Tensor part = Tensor::empty(dev, {b, hk, nchunk, d}, F);
        const int64_t cpb = 256 / (d / 8);
        calls.push_back(make_call(dev, part_name.c_str(), {k, part}, {X, F}, {(nchunk + cpb - 1) / cpb, b * hk, 1}, {256, 1, 1},
                                  {n, d, nchunk}));
        calls.push_back(make_call(dev, "ar_sage_kmean_final", {part, mean}, {F, F}, {b * hk, 1, 1}, {d, 1, 1}, {n, d, nchunk}));
    }
    Tensor vb = v;
    // unsmoothed f32 K with a scale per key and the cast of V are one launch (ar_sage_quant_rows_cast_f32)
    const bool kv_one_launch = !bf16_in && bk == 1 && !st.sage_smooth_k && !st.sage_fp8;
    if (kv_one_launch) {
        vb = Tensor::empty(dev, {b, hk, n, d}, BF);
        const int64_t rows = b * hk * n, rpb = 256 / (d / 8), row_blocks = (rows + rpb - 1) / rpb, nv = rows * d;
        calls.push_back(make_call(dev, "ar_sage_quant_rows_cast_f32", {k, k8, sk, v, vb}, {F, I8, F, F, BF},
                                  {row_blocks + std::min<int64_t>((nv + 255) / 256, 16384), 1, 1}, {256, 1, 1},
                                  {n, d, rows, nv, row_blocks}, {2, 3}));
    } else {
        quant(k, k8, sk, hk, bk, nkb, st.sage_smooth_k);
    }
    if (!bf16_in && !kv_one_launch) {
        vb = Tensor::empty(dev, {b, hk, n, d}, BF);
        const int64_t nv = b * hk * n * d;
        calls.push_back(make_call(dev, "ar_cast_bf16", {v, vb}, {F, BF}, {std::min<int64_t>((nv + 255) / 256, 16384), 1, 1},
                                  {256, 1, 1}, {nv}, {0}));
    }
    std::vector<int64_t> svals = vals;
    svals.push_back(bq);
    svals.push_back(bk);
    if (pipelined) {
        svals.push_back(bf16_in ? 0 : 1);  // out_f32
        const bool mid = mid_variant(dev, b, h, n, d, is_causal, key_lengths != nullptr);
        const std::array<int64_t, 3> grid = {mid ? (n + 127) / 128 : (n + 255) / 256, b * h, 1}, block = {mid ? 256 : 512, 1, 1};
        if (q_fused)   // Q itself in the first slot; the scales slot is written
            calls.push_back(attn_call(st.sage_fp8 ? (mid ? "ar_flash_sage_fp8_qf_mid" : "ar_flash_sage_fp8_qf_long")
                                                  : (mid ? "ar_flash_sage_qf_mid" : "ar_flash_sage_qf_long"),
                                      {q, k8, vb, out, mslot, sq, sk},
                                      {BF, I8, BF, X, F, F, F}, grid, block, svals));
        else if (q_rows)
            calls.push_back(attn_call(mid ? "ar_flash_sage_qr_mid" : "ar_flash_sage_qr_long", {q, k8, vb, out, mslot, sq, sk},
                                      {F, I8, BF, X, F, F, F}, grid, block, svals));
        else if (mid)
            calls.push_back(attn_call(st.sage_fp8 ? "ar_flash_sage_fp8_mid" : "ar_flash_sage_mid", {q8, k8, vb, out, mslot, sq, sk},
                                      {I8, I8, BF, X, F, F, F}, grid, block, svals));
        else
            calls.push_back(attn_call(st.sage_fp8 ? "ar_flash_sage_fp8_long" : "ar_flash_sage_long", {q8, k8, vb, out, mslot, sq, sk},
                                      {I8, I8, BF, X, F, F, F}, grid, block, svals));
    } else if (!bf16_in) {
        calls.push_back(attn_call(general, {q8, k8, vb, out, mslot, sq, sk}, {I8, I8, BF, F, F, F, F},
                                  {(n + 127) / 128, b * h, 1}, {256, 1, 1}, svals));
    } else {
        // ar_flash_sage stores f32 (the reference's convention); bf16 tensors get their bf16 result
        // through one more cast
        Tensor o32 = Tensor::empty(dev, {b, h, n, d}, F);
        const Tensor m2 = has_mask ? *attn_mask : o32;
        calls.push_back(attn_call(general, {q8, k8, vb, o32, m2, sq, sk}, {I8, I8, BF, F, F, F, F},
                                  {(n + 127) / 128, b * h, 1}, {256, 1, 1}, svals));
        const int64_t no = b * h * n * d;
        calls.push_back(make_call(dev, "ar_cast_bf16", {o32, out}, {F, BF}, {std::min<int64_t>((no + 255) / 256, 16384), 1, 1},
                                  {256, 1, 1}, {no}, {0}));
    }
    return calls;
}

std::optional<Tensor> fused_attention_ex(const Tensor &q, const Tensor &k, const Tensor &v, const Tensor *attn_mask,
                                         bool is_causal, bool enable_gqa, bool quantized, Session &sess, const Settings &st,
                                         const Tensor *key_lengths)
{
    static std::once_flag sage_note;
    bool sage_declined = false;
    std::vector<int64_t> mshape;
    if (attn_mask) mshape = attn_mask->shape();
    const Kernel kern = plan_fused(q.shape(), k.shape(), v.shape(), q.dtype(), k.dtype(), v.dtype(),
                                   attn_mask ? &mshape : nullptr, attn_mask ? attn_mask->dtype() : DType::Float32,
                                   enable_gqa, quantized, st, &sage_declined);
    if (sage_declined)
        note_once(sage_note, "[attention] sage: quantized attention is not available for this shape/settings: using the exact kernel");
    if (kern == Kernel::None) return std::nullopt;
    // key lengths: one int32 per batch entry on the same device; anything else is the caller's general path
    if (key_lengths && (key_lengths->dtype() != DType::Int32 || key_lengths->shape() != std::vector<int64_t>{q.shape()[0]} ||
                        key_lengths->device() != q.device()))
        return std::nullopt;

    const int64_t b = q.shape()[0], h = q.shape()[1], n = q.shape()[2], d = q.shape()[3];
    // out: bf16 for bf16 tensors, f32 otherwise (:514-530); no host-side zero fill is needed, the
    // kernels write every element
    Tensor out = Tensor::empty(q.device(), {b, h, n, d}, q.dtype());
    // Record the launches for replay and run them now (flash_attention.rs:696-701).
    for (const HostCall &call : attention_host_calls(q, k, v, attn_mask, out, is_causal, kern, st, key_lengths)) {
        sess.capture_host(call);
        call.exec();
    }
    note_selected(kern);
    return out;
}

// ---- training --------------------------------------------------------------------------

// `train_shape` (flash_attention.rs:760-787): 4-D, same n and d for q/k/v, hk divides h
static bool train_shape(const Tensor &q, const Tensor &k, const Tensor &v, const Tensor *mask)
{
    const auto &qs = q.shape(), &ks = k.shape(), &vs = v.shape();
    if (qs.size() != 4 || ks.size() != 4 || vs.size() != 4) return false;
    if (ks != vs || ks[0] != qs[0] || ks[2] != qs[2] || ks[3] != qs[3]) return false;
    if (ks[1] <= 0 || qs[1] % ks[1] != 0) return false;
    if (qs[2] <= 0 || (qs[3] != 64 && qs[3] != 128)) return false;   // cuda_flash_train.rs:312-314 (d == 64 there)
    if (q.dtype() != DType::Float32 || k.dtype() != DType::Float32 || v.dtype() != DType::Float32) return false;
    if (mask && (mask->dtype() != DType::Float32 || mask->shape() != std::vector<int64_t>{qs[2], qs[2]})) return false;
    return qs[0] * qs[1] <= 65535;
}

std::optional<TrainOut> fused_attention_train(const Tensor &q, const Tensor &k, const Tensor &v, const Tensor *attn_mask,
                                              bool is_causal, Session &sess)
{
    if (!train_shape(q, k, v, attn_mask)) return std::nullopt;
    const int64_t b = q.shape()[0], h = q.shape()[1], n = q.shape()[2], d = q.shape()[3], hk = k.shape()[1];
    const auto dev = q.device();
    const DType F = DType::Float32;
    Tensor out = Tensor::empty(dev, {b, h, n, d}, F), lse = Tensor::empty(dev, {b * h, n}, F);
    const Tensor mslot = attn_mask ? *attn_mask : out;
    const bool shrt = d == 64 && short_f32(dev, b, h, n);
    const HostCall call = make_call(dev, shrt ? "ar_fl_fwd_short" : "ar_fl_fwd", {q, k, v, out, lse, mslot}, {F, F, F, F, F, F},
                                    {(n + (shrt ? 31 : 127)) / (shrt ? 32 : 128), b * h, 1}, {256, 1, 1},
                                    {n, d, (int64_t)is_causal, (int64_t)(attn_mask != nullptr), h, hk});
    sess.capture_host(call);
    call.exec();
    return TrainOut{out, lse};
}

std::optional<Grads> fused_attention_backward(const Tensor &q, const Tensor &k, const Tensor &v, const Tensor &out,
                                              const Tensor &lse, const Tensor &dout, const Tensor *attn_mask,
                                              bool is_causal, Session &sess)
{
    if (!train_shape(q, k, v, attn_mask)) return std::nullopt;
    if (dout.dtype() != DType::Float32 || dout.shape() != q.shape() || out.shape() != q.shape()) return std::nullopt;  // :892-901
    const int64_t b = q.shape()[0], h = q.shape()[1], n = q.shape()[2], d = q.shape()[3], hk = k.shape()[1];
    if (lse.dtype() != DType::Float32 || lse.numel() != b * h * n) return std::nullopt;
    const auto dev = q.device();
    const DType F = DType::Float32;
    Tensor delta = Tensor::empty(dev, {b * h, n}, F);
    Grads g{Tensor::empty(dev, {b, h, n, d}, F), Tensor::empty(dev, {b, hk, n, d}, F), Tensor::empty(dev, {b, hk, n, d}, F)};
    const Tensor mslot = attn_mask ? *attn_mask : g.dq;   // the reference's dummy (cuda_flash_train.rs:442-449)
    const std::vector<int64_t> vals = {n, d, (int64_t)is_causal, (int64_t)(attn_mask != nullptr), h, hk};
    // few, short heads: 32 queries / keys per workgroup (the rule of arhip_flash_bwd)
    const bool shrt = d == 64 && short_f32(dev, b, hk, n);
    const int64_t rows = shrt ? 32 : 128;
    const std::vector<HostCall> calls = {
        make_call(dev, "ar_fl_prep", {out, dout, delta}, {F, F, F}, {(n + 3) / 4, b * h, 1}, {256, 1, 1}, {n, d}),
        make_call(dev, shrt ? "ar_fl_bwd_dq_short" : "ar_fl_bwd_dq", {q, k, v, dout, lse, delta, mslot, g.dq},
                  {F, F, F, F, F, F, F, F}, {(n + rows - 1) / rows, b * h, 1}, {256, 1, 1}, vals),
        make_call(dev, shrt ? "ar_fl_bwd_dkv_short" : "ar_fl_bwd_dkv", {q, k, v, dout, lse, delta, mslot, g.dk, g.dv},
                  {F, F, F, F, F, F, F, F, F}, {(n + rows - 1) / rows, b * hk, 1}, {256, 1, 1}, vals),
    };
    for (const HostCall &call : calls) {
        sess.capture_host(call);
        call.exec();
    }
    return g;
}

// ---- Tensor API -----------------------------------------------------------------------

Tensor Tensor::attention_kind(const Tensor &key, const Tensor &value, const Tensor *mask, double dropout_p, bool is_causal,
                              std::optional<AttentionKind> force, Session *sess, const Settings &st,
                              const Tensor *key_lengths) const
{
    bool quantized = false;
    const bool fused = wants_fused(force, st, dropout_p, sess != nullptr, &quantized);
    // fewer K/V heads than Q heads means GQA (tensor/mod.rs:2185-2195)
    const bool gqa = shape_.size() == 4 && key.shape().size() == 4 && key.shape()[1] != shape_[1];
    if (fused) {
        auto t = fused_attention_ex(*this, key, value, mask, is_causal, gqa, quantized, *sess, st, key_lengths);
        if (t) return *t;
    }
    // tensor/mod.rs:2207: the general scaled_dot_product_attention (generated kernels) runs here in the
    // reference; it is not part of this build, so the fallback is reported instead of being faked
    throw std::runtime_error("TGERR: attention: the fused kernels declined (shape, dtype, mask, dropout or no session); "
                             "the general SDPA path is the caller's");
}

Tensor Tensor::attention(const Tensor &k, const Tensor &v, const Tensor *mask, double dropout_p, bool is_causal) const
{
    return attention_kind(k, v, mask, dropout_p, is_causal, std::nullopt, nullptr, Settings(), nullptr);
}
Tensor Tensor::attention_with(const Tensor &k, const Tensor &v, const Tensor *mask, double dropout_p, bool is_causal,
                              Session &sess, const Settings &st, const Tensor *key_lengths) const
{
    return attention_kind(k, v, mask, dropout_p, is_causal, std::nullopt, &sess, st, key_lengths);
}
Tensor Tensor::flash_attention_with(const Tensor &k, const Tensor &v, const Tensor *mask, double dropout_p, bool is_causal,
                                    Session &sess, const Settings &st, const Tensor *key_lengths) const
{
    return attention_kind(k, v, mask, dropout_p, is_causal, AttentionKind::Flash, &sess, st, key_lengths);
}
Tensor Tensor::sage_attention_with(const Tensor &k, const Tensor &v, const Tensor *mask, double dropout_p, bool is_causal,
                                   Session &sess, const Settings &st, const Tensor *key_lengths) const
{
    return attention_kind(k, v, mask, dropout_p, is_causal, AttentionKind::Sage, &sess, st, key_lengths);
}

}  // namespace autorust
